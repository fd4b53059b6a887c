#!/usr/bin/env python3
"""Benchmark driver.  `python bench.py --gpus 1 --steps K --warmup W` prints ONE JSON line.

Workloads (synthetic weights and inputs, resident in HBM before the timed region):
  decode  (default) batch-1 greedy decode of the Qwen-Next-style A3B hybrid of BASELINE.json configs[4]: 48 layers
          (3 Gated DeltaNet + 1 gated attention per group), 512 routed experts top-10 + 1 shared per layer, vocab
          151936, everything IQ3_S except the bf16 router, 4-bit KV cache behind a --ctx token prompt of random ids.
          One step = one generated token; the whole loop runs on the device without host round trips.
  gemv    one IQ3_S dequant-GEMV of the vocabulary-head shape (151936 x 2048, t = 1) per step, rotating over enough
          distinct weight buffers (> 512 MB) that nothing is served from the 256 MB Infinity Cache.
  gemv0   configs[0]: the single 4096 x 4096 IQ3_S GEMV, rotating over 128 matrices, plus cache-resident rate and call latency.
  sweep   configs[1]: IQ2_XS / IQ3_S / Q4_K / Q8_0 x five shapes x t in 1, 2, 4, 8 (one table under "sweep").
  moe     configs[2]: the MoE FFN step (512 experts top-10 + shared) at t = 1 and 4.
  gdn     configs[3]: the Gated DeltaNet decode step and the 4096-token chunked prefill (kernel durations).
  attn    the attention layer core of configs[4] at --ctx cached positions (kernel durations).
Timed regions are bracketed by HIP events recorded on the library's own stream; per-kernel-class durations come from
the library's event-pair profiler in a second, separately timed pass.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0


class HipEvents:
    """hipEvent timing on an arbitrary stream (torch.cuda.Event only sees torch's current stream)."""

    def __init__(self):
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [C.c_void_p]
        self.hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]

    def event(self):
        e = C.c_void_p()
        assert self.hip.hipEventCreate(C.byref(e)) == 0
        return e

    def record(self, e, stream):
        assert self.hip.hipEventRecord(e, C.c_void_p(stream)) == 0

    def elapsed_ms(self, a, b):
        assert self.hip.hipEventSynchronize(b) == 0
        ms = C.c_float()
        assert self.hip.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return float(ms.value)


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


# ---------------------------------------------------------------------------------------------------------------- gemv
def cpu_baseline_gemv(ty, rows, cols, seed, budget_s=12.0):
    """The oracle's QMat::matmul restatement (row dequant + f32 dot, rows over the host threads) on a bounded row
    sample of the same matrix."""
    import orc
    from pyre_amd import synth
    threads = min(os.cpu_count() or 1, 16)
    el, bs, _ = synth.GEOM[ty]
    sample_rows = 8192
    raw = synth.matrix(ty, sample_rows, cols, seed)
    x = synth.normal((1, cols), 5)
    orc.matmul(ty, raw, sample_rows, cols, x, threads=threads)
    n = 0; t0 = time.perf_counter()
    while True:
        orc.matmul(ty, raw, sample_rows, cols, x, threads=threads); n += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or n >= 200:
            break
    gb_s = n * sample_rows / dt * (cols // el * bs) / 1e9
    return {"value": round(gb_s, 3), "unit": "GB/s of GGUF weight bytes", "cores": threads, "kind": "port",
            "sample": "%d launches of the oracle matmul over the first %d rows x %d cols (IQ3_S), t=1" % (n, sample_rows, cols)}


def bench_gemv(args):
    from pyre_amd import lib, synth
    ev = HipEvents()
    ctx = lib.Context(0)
    names = {"iq3_s": lib.IQ3_S, "iq2_xs": lib.IQ2_XS, "q4_k": lib.Q4_K, "q8_0": lib.Q8_0, "q4_0": lib.Q4_0, "q5_0": lib.Q5_0, "q6_k": lib.Q6_K, "iq2_xxs": lib.IQ2_XXS,
             "iq2_s": lib.IQ2_S, "iq3_xxs": lib.IQ3_XXS, "iq4_nl": lib.IQ4_NL, "iq4_xs": lib.IQ4_XS, "q3_k": lib.Q3_K, "q5_k": lib.Q5_K, "q2_0": lib.Q2_0}
    ty, rows, cols = names[args.fmt], 151936, 2048
    FN = args.fmt.upper()
    el, bs, _ = synth.GEOM[ty]
    nb = rows * cols // el
    nbuf = 5                                    # 5 x 133.7 MB = 668 MB > 512 MB
    mats = []
    for i in range(nbuf):
        dev = ctx.alloc(nb * bs)
        ctx.synth_blocks(ty, nb, 9000 + i, dev_out=dev)
        mats.append(lib.QMat(ctx, ty, rows, cols, dev_blocks=dev, nbytes=nb * bs))
        ctx.free(dev)
    x = ctx.upload(synth.normal((1, cols), 3))
    y = ctx.alloc(rows * 4)
    t = args.t
    if t > 1:
        x = ctx.upload(synth.normal((t, cols), 3)); y = ctx.alloc(t * rows * 4)
    run = lambda m: m.matmul_dev(x, t, y)
    for i in range(args.warmup):
        run(mats[i % nbuf])
    ctx.sync()
    e0, e1 = ev.event(), ev.event()
    ev.record(e0, ctx.stream)
    for i in range(args.steps):
        run(mats[i % nbuf])
    ev.record(e1, ctx.stream)
    per = ev.elapsed_ms(e0, e1) / args.steps
    if args.calib_copy:
        # reference dispatches for scaling rocprofv3's FETCH_SIZE / WRITE_SIZE: plain device copies of a known size
        import torch
        src = torch.empty(args.calib_copy << 20, dtype=torch.uint8, device="cuda"); dst = torch.empty_like(src)
        src.fill_(1); torch.cuda.synchronize()
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        log("calibration: 4 device copies of %d MiB (each reads and writes that many bytes)" % args.calib_copy)
    # second pass: an event pair around every launch, so the dominant kernel's own duration is known beside the step time
    ctx.prof_reset(); ctx.prof_enable(True)
    pn = min(50, args.steps)
    for i in range(pn):
        run(mats[i % nbuf])
    ctx.sync()
    prof = ctx.prof_report(); ctx.prof_enable(False)
    kernels = [{"kernel": k, "launches_per_step": round(v[0] / pn, 2), "avg_launch_us": round(v[1] / v[0] * 1e3, 3)} for k, v in sorted(prof.items(), key=lambda kv: -kv[1][1])]
    dom_us = kernels[0]["avg_launch_us"] if kernels else per * 1e3
    alg_bytes = mats[0].gguf_bytes + 4 * t * cols + 4 * t * rows
    dom_name = kernels[0]["kernel"] if kernels else None
    # which kernel the operator took: one token of an IQ3_S matrix streams the native layout (the file's bits per weight)
    # through integer dot products, a window the matrix-core layout; PYRE_QMATMUL_F32=1 / other block types the lane = row GEMV
    if ty == lib.IQ2_XS and t == 1 and os.environ.get("PYRE_QMATMUL_NATIVE", "1") != "0" and os.environ.get("PYRE_QMATMUL_F32") != "1":
        layout, path = 2, "native-format GEMV (k_gemv_n over 80 bytes per 256 weights: 17-bit codebook-index + sign fields, two signed codebook tables in shared memory, v_dot4_i32_i8), preceded by the activation digits launch k_act_digits_n"
    elif ty == lib.Q4_K and t == 1 and os.environ.get("PYRE_QMATMUL_NATIVE", "1") != "0" and os.environ.get("PYRE_QMATMUL_F32") != "1":
        layout, path = 2, "native-format GEMV (k_gemv_n over the file's 144-byte blocks: nibbles into v_dot4_i32_i8, minima through the digit sums), preceded by the activation digits launch k_act_digits_n"
    elif ty != lib.IQ3_S or os.environ.get("PYRE_QMATMUL_F32") == "1":
        layout, path = 0, "f32 multiply-add GEMV, lane = row (k_gemv)"
    elif t == 1 and os.environ.get("PYRE_QMATMUL_NATIVE", "1") != "0":
        layout, path = 2, "native-format GEMV (k_gemv_n: 13-bit codebook-index + sign fields, signed codebook in shared memory, v_dot4_i32_i8), preceded by the activation digits launch k_act_digits_n"
    else:
        layout, path = 1, "f16 matrix cores (k_gemm_m, preceded by the operand split k_act_split): the kernel the model's projections and head run on a window"
    # HBM bytes per launch and the kernel-trace duration come from the committed counter summary of this very kernel
    # (not from this run); a summary that names another kernel is not quoted
    traffic = None; traffic_source = None; trace_us = None
    prof_file = {0: "gemv_lane_row_iq3s_vocab_head_kernel_stats.txt", 1: "gemm_m_iq3s_vocab_head_kernel_stats.txt", 2: "gemv_n_iq3s_vocab_head_kernel_stats.txt"}[layout]
    if ty == lib.IQ3_S:
        try:
            fields = {}
            for line in open(os.path.join(ROOT, "profiles", prof_file)):
                if ":" in line and not line.startswith(" "):
                    k_, v_ = line.split(":", 1); fields[k_.strip()] = v_.strip()
            if fields.get("profiled_kernel_class") == dom_name and fields.get("tokens_per_launch") == str(t):
                traffic = int(fields["traffic_bytes_per_launch"]) if "traffic_bytes_per_launch" in fields else None
                trace_us = float(fields["kernel_trace_avg_us"]) if "kernel_trace_avg_us" in fields else None
                traffic_source = "profiles/%s: rocprofv3 FETCH_SIZE + WRITE_SIZE and --kernel-trace runs of this command, not this run" % prof_file
        except (OSError, ValueError):
            pass
    gbs = alg_bytes / (per * 1e-3) / 1e9                 # whole step (every launch of the operator call)
    kgbs = alg_bytes / (dom_us * 1e-6) / 1e9             # the dominant kernel alone
    out = {
        "metric": "%s dequant-GEMV achieved HBM GB/s (vocab head 151936x2048, t=%d%s)" % (FN, t, ""), "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(per, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: %s GEMV 2048->151936, batch %d, rotating over %d weight buffers (%.0f MB)" % (FN, t, nbuf, nbuf * mats[0].gguf_bytes / 1e6)},
        "path": path,
        "roofline": {"bound": "hbm", "achieved": round(kgbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(kgbs / HBM_PEAK_GBS, 4),
                     "frac_is": "algorithmic bytes / this run's event-pair duration of the dominant kernel; frac_kernel_trace: the same bytes / the kernel-trace duration in the committed profile",
                     "frac_kernel_trace": round(alg_bytes / (trace_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4) if trace_us else None, "kernel_trace_avg_us": trace_us,
                     "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": dom_name, "device_bytes_per_launch": mats[0].layout_bytes(layout) or mats[0].dev_bytes, "algorithmic_bytes_per_launch": alg_bytes, "avg_launch_us": dom_us},
        "kernels": kernels,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_gemv(ty, rows, cols, 9000)
    return out


# ------------------------------------------------------------------------------------------ the other configurations
def _dev_matrix(ctx, lib, synth, ty, rows, cols, seed):
    el, bs, _ = synth.GEOM[ty]
    nb = rows * (cols // el)
    dev = ctx.alloc(nb * bs)
    ctx.synth_blocks(ty, nb, seed, dev_out=dev)
    m = lib.QMat(ctx, ty, rows, cols, dev_blocks=dev, nbytes=nb * bs)
    ctx.free(dev)
    return m


def _timed(ev, ctx, n, fn):
    e0, e1 = ev.event(), ev.event()
    ctx.sync(); ev.record(e0, ctx.stream)
    for i in range(n):
        fn(i)
    ev.record(e1, ctx.stream)
    return ev.elapsed_ms(e0, e1) / n


def _prof(ctx, n, fn):
    """{kernel class: (launches per step, avg launch us, algorithmic bytes per launch)} from the library's event pairs."""
    ctx.prof_reset(); ctx.prof_enable(True)
    for i in range(n):
        fn(i)
    ctx.sync()
    rep = ctx.prof_report(); ctx.prof_enable(False)
    return {k: (v[0] / n, v[1] / v[0] * 1e3, v[2] / v[0]) for k, v in rep.items()}


def _line(metric, value, unit, args, per_ms, dtype, workload, roofline, extra):
    out = {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(per_ms, 5),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic", "config": {"workload": workload}, "roofline": roofline}
    out.update(extra)
    return out


def bench_gemv0(args):
    """configs[0]: one IQ3_S GEMV, 4096 x 4096, t = 1.  The matrix (7.2 MB) fits the 256 MB Infinity Cache many times over, so
    the timed loop rotates over 128 distinct matrices (923 MB); the cache-resident rate and the latency of one synchronised call
    are reported beside it."""
    from pyre_amd import lib, synth
    ev = HipEvents(); ctx = lib.Context(0)
    rows = cols = 4096; ty = lib.IQ3_S; nbuf = 128
    mats = [_dev_matrix(ctx, lib, synth, ty, rows, cols, 100 + i) for i in range(nbuf)]
    x = ctx.upload(synth.normal((1, cols), 3)); y = ctx.alloc(rows * 4)
    alg = mats[0].gguf_bytes + 4 * cols + 4 * rows
    res = {}
    for name, call in (("operator", lambda m: m.matmul_dev(x, 1, y)), ("f32", lambda m: m.matmul_f32_dev(x, 1, y))):
        for i in range(args.warmup):
            call(mats[i % nbuf])
        per = _timed(ev, ctx, args.steps, lambda i: call(mats[i % nbuf]))
        hot = _timed(ev, ctx, args.steps, lambda i: call(mats[0]))
        pr = _prof(ctx, min(args.steps, 128), lambda i: call(mats[i % nbuf]))
        lat = []
        for i in range(20):
            ctx.sync(); t0 = time.perf_counter(); call(mats[(7 * i) % nbuf]); ctx.sync(); lat.append((time.perf_counter() - t0) * 1e6)
        dom = max(pr.items(), key=lambda kv: kv[1][1] * kv[1][0])
        res[name] = {"us_per_call_rotating": round(per * 1e3, 3), "GBps_rotating": round(alg / (per * 1e-3) / 1e9, 1), "us_per_call_cache_resident": round(hot * 1e3, 3),
                     "GBps_cache_resident": round(alg / (hot * 1e-3) / 1e9, 1), "single_synchronised_call_us_median": round(float(np.median(lat)), 2),
                     "kernels": {k: {"launches_per_call": round(v[0], 2), "avg_launch_us": round(v[1], 3)} for k, v in pr.items()},
                     "dominant_kernel": dom[0], "dominant_kernel_us": round(dom[1][1], 3), "dominant_kernel_GBps": round(alg / (dom[1][1] * 1e-6) / 1e9, 1)}
    op = res["operator"]
    roof = {"bound": "hbm", "achieved": op["dominant_kernel_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(op["dominant_kernel_GBps"] / HBM_PEAK_GBS, 4), "traffic": None,
            "kernel": op["dominant_kernel"], "algorithmic_bytes_per_launch": alg, "device_bytes_per_launch": mats[0].layout_bytes(0), "avg_launch_us": op["dominant_kernel_us"]}
    extra = {"paths": res}
    if not args.no_cpu:
        import orc
        threads = min(os.cpu_count() or 1, 16)
        raw = synth.matrix(ty, rows, cols, 100); xh = synth.normal((1, cols), 3)
        orc.matmul(ty, raw, rows, cols, xh, threads=threads); n = 0; t0 = time.perf_counter()
        while time.perf_counter() - t0 < 10.0 and n < 400:
            orc.matmul(ty, raw, rows, cols, xh, threads=threads); n += 1
        dt = time.perf_counter() - t0
        extra["cpu_baseline"] = {"value": round(n * alg / dt / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
                                 "sample": "%d calls of the oracle matmul (row dequant + f32 dot, rows over %d threads) on the whole 4096 x 4096 IQ3_S matrix, t=1" % (n, threads)}
    return _line("IQ3_S dequant-GEMV achieved HBM GB/s (4096x4096, t=1)", op["GBps_rotating"], "GB/s", args, op["us_per_call_rotating"] / 1e3, "f32",
                 "configs[0]: IQ3_S GEMV 4096x4096, batch 1, rotating over %d weight buffers (%.0f MB); the operator (a single token of a matrix of at most 128 row tiles takes the one-launch lane = row f32 GEMV, the kernel of pyre_qmatmul_f32) and pyre_qmatmul_f32" % (nbuf, nbuf * mats[0].gguf_bytes / 1e6), roof, extra)


def bench_sweep(args):
    """configs[1]: IQ2_XS, IQ3_S, Q4_K, Q8_0 x five shapes x t in 1, 2, 4, 8; every case rotates over enough matrices to exceed
    600 MB (at most 512 of them: the smallest shapes stay partly cache resident, their working set is stated)."""
    from pyre_amd import lib, synth
    ev = HipEvents(); ctx = lib.Context(0)
    fmts = [("IQ2_XS", lib.IQ2_XS), ("IQ3_S", lib.IQ3_S), ("Q4_K", lib.Q4_K), ("Q8_0", lib.Q8_0)]
    shapes = [(4096, 2048), (2048, 4096), (512, 2048), (2048, 512), (151936, 2048)]
    table = []
    steps = max(16, min(args.steps, 200))
    for fname, ty in fmts:
        for rows, cols in shapes:
            el, bs, _ = synth.GEOM[ty]
            gbytes = rows * (cols // el) * bs
            nbuf = int(min(512, max(2, -(-600e6 // gbytes))))
            mats = [_dev_matrix(ctx, lib, synth, ty, rows, cols, 7000 + 31 * i + ty) for i in range(nbuf)]
            x = ctx.upload(synth.normal((8, cols), 5)); y = ctx.alloc(8 * rows * 4)
            for t in (1, 2, 4, 8):
                for i in range(4):
                    mats[i % nbuf].matmul_dev(x, t, y)
                per = _timed(ev, ctx, steps, lambda i: mats[i % nbuf].matmul_dev(x, t, y))
                alg = gbytes + 4 * t * (cols + rows)
                table.append({"fmt": fname, "rows": rows, "cols": cols, "t": t, "us_per_call": round(per * 1e3, 3), "GBps": round(alg / (per * 1e-3) / 1e9, 1),
                              "frac_of_peak": round(alg / (per * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "working_set_MB": round(nbuf * gbytes / 1e6)})
            for m in mats:
                m.close()
            ctx.free(x); ctx.free(y)
        log("sweep: %s done" % fname)
    head = next(r for r in table if r["fmt"] == "IQ3_S" and r["rows"] == 151936 and r["t"] == 1)
    gm = float(np.exp(np.mean([np.log(r["GBps"]) for r in table])))
    roof = {"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": head["frac_of_peak"], "traffic": None,
            "kernel": "operator call (every launch of pyre_qmatmul_dev), IQ3_S 151936x2048 t=1", "avg_launch_us": head["us_per_call"]}
    extra = {"sweep": table, "geometric_mean_GBps": round(gm, 1)}
    if not args.no_cpu:
        extra["cpu_baseline"] = cpu_baseline_gemv(lib.IQ3_S, 151936, 2048, 9000)
    return _line("quant-format GEMV sweep, achieved HBM GB/s per operator call (value: IQ3_S vocab head, t=1)", head["GBps"], "GB/s", args, head["us_per_call"] / 1e3, "f32",
                 "configs[1]: IQ2_XS / IQ3_S / Q4_K / Q8_0 x {4096<-2048, 2048<-4096, 512<-2048, 2048<-512, 151936<-2048} x t in {1,2,4,8}, rotating weight buffers", roof, extra)


def bench_moe(args):
    """configs[2]: the MoE FFN step, 512 routed experts top-10 + 1 shared, d 2048, expert ff 512, IQ3_S, bf16 router, t in 1, 4.
    Two layers' worth of experts (1.4 GB) alternate and the token activations rotate, so the chosen experts are cold."""
    from pyre_amd import lib, synth
    from pyre_amd import modelgen as mg
    ev = HipEvents(); ctx = lib.Context(0)
    c = mg.a3b_config(n_layers=2, full_every=8)
    layers, globals_, raw = mg.build_device(ctx, c, seed=17)
    moes = []
    for L in layers:
        qm = {s: (lib.QMat(ctx, L[s][0], L[s][1], L[s][2], dev_blocks=L[s][3], nbytes=L[s][1] * (L[s][2] // synth.GEOM[L[s][0]][0]) * synth.GEOM[L[s][0]][1]) if not isinstance(L[s][3], np.ndarray)
                  else lib.QMat(ctx, L[s][0], L[s][1], L[s][2], L[s][3])) for s in (mg.ROUTER, mg.GATE_E, mg.UP_E, mg.DOWN_E, mg.SH_GATE, mg.SH_UP, mg.SH_DOWN)}
        moes.append((lib.Moe(ctx, c.top_k, qm[mg.ROUTER], qm[mg.GATE_E], qm[mg.UP_E], qm[mg.DOWN_E], L[mg.SH_GATE_INP][3].view(np.float32), qm[mg.SH_GATE], qm[mg.SH_UP], qm[mg.SH_DOWN]), qm))
    host_raw = None
    if not args.no_cpu:          # the oracle's copy of layer 0, before the raw blocks are freed
        host_raw = {s: ((layers[0][s][0], layers[0][s][1], layers[0][s][2], ctx.download(layers[0][s][3], (layers[0][s][1] * (layers[0][s][2] // synth.GEOM[layers[0][s][0]][0]) * synth.GEOM[layers[0][s][0]][1],), np.uint8))
                        if not isinstance(layers[0][s][3], np.ndarray) else layers[0][s]) for s in (mg.ROUTER, mg.GATE_E, mg.UP_E, mg.DOWN_E, mg.SH_GATE, mg.SH_UP, mg.SH_DOWN, mg.SH_GATE_INP)}
    for p in raw:
        ctx.free(p)
    nx = 64
    xs = synth.normal((nx * 4, c.d), 23)
    xd = ctx.upload(xs); yd = ctx.alloc(4 * c.d * 4)
    el, bs, _ = synth.GEOM[synth.IQ3_S]
    per_expert = (2 * c.ff_exp * (c.d // el) + c.d * (c.ff_exp // el)) * bs
    res = {}
    for t in (1, 4):
        call = lambda i: moes[i % 2][0].ffn_dev(xd + ((i % nx) * 4) * c.d * 4, t, yd)
        for i in range(args.warmup):
            call(i)
        per = _timed(ev, ctx, args.steps, call)
        pr = _prof(ctx, min(args.steps, 64), call)
        alg = c.n_exp * c.d * 2 + (min(t * c.top_k, c.n_exp) + 1) * per_expert + 4 * t * 2 * c.d          # bf16 router + distinct experts (upper bound: all distinct) + shared
        ksum = sum(v[0] * v[1] for v in pr.values())
        res["t%d" % t] = {"us_per_step": round(per * 1e3, 3), "algorithmic_bytes": alg, "GBps": round(alg / (per * 1e-3) / 1e9, 1), "frac_of_peak": round(alg / (per * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                          "kernel_us_per_step": round(ksum, 3), "kernels": {k: {"launches_per_step": round(v[0], 2), "avg_launch_us": round(v[1], 3), "GBps": round(v[2] / (v[1] * 1e-6) / 1e9, 1) if v[2] else None} for k, v in pr.items()}}
    r1 = res["t1"]; dom = max(r1["kernels"].items(), key=lambda kv: kv[1]["avg_launch_us"] * kv[1]["launches_per_step"])
    roof = {"bound": "hbm", "achieved": dom[1]["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round((dom[1]["GBps"] or 0) / HBM_PEAK_GBS, 4), "traffic": None, "kernel": dom[0], "avg_launch_us": dom[1]["avg_launch_us"]}
    extra = {"steps_by_width": res}
    if host_raw is not None:
        import orc
        threads = min(os.cpu_count() or 1, 16)
        T = {s: orc.tensor(*host_raw[s]) for s in (mg.ROUTER, mg.GATE_E, mg.UP_E, mg.DOWN_E, mg.SH_GATE, mg.SH_UP, mg.SH_DOWN)}
        sgi = host_raw[mg.SH_GATE_INP][3].view(np.float32)
        f = lambda i: orc.moe_ffn(c.d, c.n_exp, c.top_k, c.ff_exp, T[mg.ROUTER], T[mg.GATE_E], T[mg.UP_E], T[mg.DOWN_E], sgi, T[mg.SH_GATE], T[mg.SH_UP], T[mg.SH_DOWN], xs[4 * (i % nx):4 * (i % nx) + 1], threads=threads)
        f(0); n = 0; t0 = time.perf_counter()
        while time.perf_counter() - t0 < 10.0 and n < 2000:
            f(n); n += 1
        dt = time.perf_counter() - t0
        extra["cpu_baseline"] = {"value": round(n / dt, 2), "unit": "MoE steps/s (t=1)", "cores": threads, "kind": "port",
                                 "sample": "%d single-token steps of the oracle's moe_ffn on layer 0's tensors (512 experts resident, top-10 + shared)" % n}
    return _line("MoE FFN step (512 experts top-10 + shared, IQ3_S): steps/s at t=1", round(1e3 / r1["us_per_step"] * 1e3, 1), "steps/s", args, r1["us_per_step"] / 1e3, "f32",
                 "configs[2]: MoE FFN step, d 2048, ff 512, 512 experts top-10 + 1 shared, IQ3_S, bf16 router, batch 1 and 4; two layers' experts alternate, 64 activations rotate", roof, extra)


def bench_gdn(args):
    """configs[3]: the Gated DeltaNet layer core, 16 QK / 32 V heads of 128: the decode step at batch 1 and the chunked prefill of
    4096 tokens (chunks of 64).  The block entry points take host buffers, so the figures are the kernels' own durations (event
    pairs on the library's stream around each launch): inputs are in HBM when a timed region starts."""
    from pyre_amd import lib
    ctx = lib.Context(0)
    nk, nv, T = 16, 32, 4096
    ch = 2 * nk * 128 + nv * 128
    g = np.random.Generator(np.random.PCG64(41))
    a = (-np.exp(g.uniform(0.0, np.log(16.0), nv))).astype(np.float32); dt = np.zeros(nv, np.float32)
    conv_w = (0.5 * g.standard_normal(ch * 4)).astype(np.float32); norm_w = (1 + 0.1 * g.standard_normal(128)).astype(np.float32)
    gd = lib.Gdn(ctx, nk, nv, 128, 128, 4, 1e-6, a, dt, conv_w, norm_w)
    S0 = (0.01 * g.standard_normal((nv, 128, 128))).astype(np.float32)
    gd.set_state(None, S0)
    qkv = g.standard_normal((T, ch), dtype=np.float32); z = g.standard_normal((T, nv * 128), dtype=np.float32)
    beta = g.standard_normal((T, nv), dtype=np.float32); alpha = g.standard_normal((T, nv), dtype=np.float32)
    n = max(8, min(args.steps, 128))
    for i in range(args.warmup):
        gd.step(qkv[i:i + 1], z[i:i + 1], beta[i:i + 1], alpha[i:i + 1])
    pr = _prof(ctx, n, lambda i: gd.step(qkv[i:i + 1], z[i:i + 1], beta[i:i + 1], alpha[i:i + 1]))
    step_us = sum(v[0] * v[1] for v in pr.values())
    state_b = 2 * nv * 128 * 128 * 4 + 2 * 3 * ch * 4 + 4 * (ch + nv * 128 + 2 * nv) + 4 * nv * 128
    gd.set_state(None, S0)
    gd.prefill_chunked(qkv, z, beta, alpha)                  # untimed
    gd.set_state(None, S0)
    pp = _prof(ctx, 1, lambda i: gd.prefill_chunked(qkv, z, beta, alpha))
    pre_us = sum(v[0] * v[1] for v in pp.values())
    # fp32 matrix work of the chunked form per (head, chunk of 64): A = K K^T (64x64x128), B-ish products and the state update: ~ 2*(64*64*128*3 + 64*128*128*3) flop
    flop = nv * (T // 64) * 2.0 * (3 * 64 * 64 * 128 + 3 * 64 * 128 * 128)
    res = {"decode_step": {"kernel_us": round(step_us, 3), "algorithmic_bytes": state_b, "GBps": round(state_b / (step_us * 1e-6) / 1e9, 1), "frac_of_hbm_peak": round(state_b / (step_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                           "kernels": {k: {"launches_per_step": round(v[0], 2), "avg_launch_us": round(v[1], 3)} for k, v in pr.items()}},
           "prefill_4096": {"kernel_ms": round(pre_us / 1e3, 3), "us_per_token": round(pre_us / T, 4), "matrix_TFLOPs": round(flop / (pre_us * 1e-6) / 1e12, 2), "frac_of_fp32_mfma_peak": round(flop / (pre_us * 1e-6) / 1e12 / 157.3, 4),
                            "kernels": {k: {"launches": round(v[0], 2), "avg_launch_us": round(v[1], 3)} for k, v in pp.items()}}}
    roof = {"bound": "hbm", "achieved": res["decode_step"]["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": res["decode_step"]["frac_of_hbm_peak"], "traffic": None, "kernel": "gdn_delta", "avg_launch_us": round(step_us, 3)}
    extra = {"gdn": res}
    if not args.no_cpu:
        import orc
        so, co = S0.copy().reshape(-1), np.zeros(3 * ch, np.float32)
        m = 0; t0 = time.perf_counter()
        while time.perf_counter() - t0 < 10.0 and m < T:
            orc.gdn_core(nk, nv, 128, 128, 4, 1e-6, a, dt, conv_w, norm_w, qkv[m:m + 64], z[m:m + 64], beta[m:m + 64], alpha[m:m + 64], co, so); m += 64
        dtc = time.perf_counter() - t0
        extra["cpu_baseline"] = {"value": round(m / dtc, 1), "unit": "tokens/s (sequential recurrence)", "cores": 1, "kind": "port", "sample": "%d tokens of the oracle's linear_core restatement, one thread" % m}
    return _line("Gated DeltaNet decode step (16/32 heads of 128): steps/s by kernel time", round(1e6 / step_us, 1), "steps/s", args, step_us / 1e3, "f32",
                 "configs[3]: Gated DeltaNet layer core, post-projection inputs, conv 4, state N(0,0.01), A_log~U(0,ln16); decode step at batch 1 and chunked prefill of 4096 tokens (chunk 64)", roof, extra)


def bench_attn(args):
    """The gated attention layer core over the 4-bit cache at the metric's context (16 / 2 heads of 256, 32768 positions, newest
    1024 in f32), t = 1: kernel durations from the library's event pairs (the block entry point takes host buffers)."""
    from pyre_amd import lib
    ctx = lib.Context(0)
    nh, nkv, n0 = 16, 2, args.ctx
    row = nkv * 256
    g = np.random.Generator(np.random.PCG64(43))
    att = lib.Attn(ctx, nh, nkv, 256, 64, 1e7, 1e-6, np.ones(256, np.float32), np.ones(256, np.float32), 4, 1024, n0 + 512)
    att.load_cache(g.standard_normal((n0, row), dtype=np.float32), g.standard_normal((n0, row), dtype=np.float32))
    q = g.standard_normal((256, nh * 512), dtype=np.float32); k = g.standard_normal((256, row), dtype=np.float32); v = g.standard_normal((256, row), dtype=np.float32)
    n = max(8, min(args.steps, 128))
    for i in range(args.warmup):
        att.decode(q[i:i + 1], k[i:i + 1], v[i:i + 1])
    pr = _prof(ctx, n, lambda i: att.decode(q[8 + i:9 + i], k[8 + i:9 + i], v[8 + i:9 + i]))
    us = sum(v_[0] * v_[1] for v_ in pr.values())
    nn = n0 + args.warmup + n // 2
    pb = ((nn - 1024) // 64) * 64 if nn > 1024 + 64 else 0
    alg = 2 * row * (pb * 0.625 + (nn - pb) * 4.0)
    dom = max(pr.items(), key=lambda kv: kv[1][0] * kv[1][1])
    roof = {"bound": "hbm", "achieved": round(alg / (dom[1][1] * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(alg / (dom[1][1] * 1e-6) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
            "kernel": dom[0], "algorithmic_bytes_per_launch": round(alg), "avg_launch_us": round(dom[1][1], 3)}
    extra = {"kernels": {k_: {"launches_per_step": round(v_[0], 2), "avg_launch_us": round(v_[1], 3)} for k_, v_ in pr.items()}, "kernel_us_per_step": round(us, 3)}
    return _line("gated attention decode step over the 4-bit KV cache: steps/s by kernel time", round(1e6 / us, 1), "steps/s", args, us / 1e3, "f32",
                 "attention layer core of configs[4]: 16 Q / 2 KV heads of 256, %d cached positions (4-bit below the newest 1024), batch 1" % n0, roof, extra)


# -------------------------------------------------------------------------------------------------------------- decode
def cpu_baseline_decode(cfg, seed, budget_s=20.0):
    """The oracle's token step (the reference's host f32 path restated in C++) on a bounded sample: ONE group of four
    layers (3 Gated DeltaNet + 1 attention, all 512 experts resident) plus the head of the same configuration, decoded
    at a short context; tok/s of the 48-layer model follows from time(4 layers) * 12 + time(head)."""
    import copy
    import orc
    from helpers import orc_model
    from pyre_amd import modelgen as mg
    threads = min(os.cpu_count() or 1, 16)
    c4 = copy.copy(cfg); c4.n_layers = 4
    t0 = time.perf_counter()
    hw = mg.build_host(c4, seed=seed)
    om = orc_model(hw, threads=threads)
    log("cpu baseline: 4-layer host weights in %.1f s" % (time.perf_counter() - t0))
    st = om.new_state()
    g = np.random.Generator(np.random.PCG64(11))
    prompt = g.integers(0, cfg.vocab, 16, dtype=np.uint32)
    lg = om.forward(prompt, st)
    # time the head separately: logits of a 0-layer model are not available, so time full steps and the head GEMV alone
    n = 0; t0 = time.perf_counter(); tok = np.array([orc.argmax(lg)], dtype=np.uint32)
    while True:
        lg = om.forward(tok, st); tok = np.array([orc.argmax(lg)], dtype=np.uint32); n += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or n >= 64:
            break
    step4 = dt / n
    ty, rows, cols, raw = hw.globals_[mg.G_OUT]
    x = np.ones((1, cols), np.float32)
    orc.matmul(ty, raw, rows, cols, x, threads=threads)
    t0 = time.perf_counter(); k = 0
    while k < 5:
        orc.matmul(ty, raw, rows, cols, x, threads=threads); k += 1
    head = (time.perf_counter() - t0) / k
    full = (step4 - head) * (cfg.n_layers / 4.0) + head
    return {"value": round(1.0 / full, 3), "unit": "tok/s", "cores": threads, "kind": "port",
            "sample": "oracle (C++ restatement of the reference's host f32 path, not the pyre executable): %d greedy steps of a 4-layer slice "
                      "(3 DeltaNet + 1 attention, 512 experts each) at context %d took %.3f s/step incl. the %.3f s vocabulary head; "
                      "scaled to %d layers: (step - head) * %d + head" % (n, len(st), step4, head, cfg.n_layers, cfg.n_layers // 4)}


def kv_bytes_per_token(cfg, n):
    """Bytes of KV cache one decode step reads at context n (packed region 0.625 B/value incl. scales, f32 recent)."""
    pb = ((n - cfg.kv_recent) // 64) * 64 if (cfg.kv_bits == 4 and n > cfg.kv_recent + 64) else 0
    per_layer = 2 * cfg.n_kv * cfg.hd * (pb * 0.625 + (n - pb) * 4.0)
    n_attn = cfg.n_layers // cfg.full_every
    return per_layer * n_attn


def bench_decode(args):
    from pyre_amd import lib, synth
    from pyre_amd import modelgen as mg
    ev = HipEvents()
    ctx = lib.Context(0)
    cfg = mg.a3b_config()
    if args.layers:
        cfg.n_layers = args.layers
    if args.indexer:             # variant: the reference's long-context mechanism (QSA sparse indexer, its GGUF defaults: 2048-token budget, blocks of 4)
        cfg.idx_nh, cfg.idx_hd, cfg.idx_ratio, cfg.idx_budget = args.indexer, 128, 4, 2048
    t0 = time.perf_counter()
    layers, globals_, raw = mg.build_device(ctx, cfg, seed=args.seed)
    ctx.sync()
    log("synthetic tensors on the device in %.1f s" % (time.perf_counter() - t0)); t0 = time.perf_counter()
    model = lib.Model(ctx, cfg, layers, globals_)
    for p in raw:
        ctx.free(p)
    log("model resident (re-laid-out) in %.1f s; weight bytes per token %.1f MB" % (time.perf_counter() - t0, model.weight_bytes_per_token / 1e6))
    n_ctx = args.ctx
    st = model.new_state(n_ctx + args.steps + args.warmup + 64 + args.spec_windows + 8 + args.host_steps + 1 + args.spec_loop_tokens + 16 + 256)
    g = np.random.Generator(np.random.PCG64(args.seed + 1))
    prompt = g.integers(0, cfg.vocab, n_ctx, dtype=np.uint32)
    t0 = time.perf_counter()
    done = 0
    while done < n_ctx:                      # prefill in pieces so a long prompt keeps printing progress
        piece = prompt[done:done + 2048]
        last = done + piece.size >= n_ctx
        lg = model.forward(piece, st, want_logits=last)
        done += piece.size
        if done % 8192 == 0 or last:
            log("prefill %d / %d tokens (%.1f s)" % (done, n_ctx, time.perf_counter() - t0))
    ctx.sync(); prefill_s = time.perf_counter() - t0
    first = int(np.argmax(lg))
    toks = model.decode_greedy_dev(st, first, args.warmup) if args.warmup else np.array([first], dtype=np.uint32)
    nxt = int(toks[-1])
    ctx.sync()
    e0, e1 = ev.event(), ev.event()
    n0 = len(st)
    ev.record(e0, ctx.stream)
    model.decode_greedy_dev(st, nxt, args.steps, fetch=False)
    ev.record(e1, ctx.stream)
    ms = ev.elapsed_ms(e0, e1)
    ctx.sync()
    per = ms / args.steps
    tok_s = 1e3 / per
    wbytes = model.weight_bytes_per_token
    n_mid = n0 + args.steps // 2
    kvb = kv_bytes_per_token(cfg, n_mid)
    n_lin = cfg.n_layers - cfg.n_layers // cfg.full_every
    state_b = n_lin * (2 * cfg.lin_nv * cfg.lin_dk * cfg.lin_dv * 4 + 2 * (cfg.conv_k - 1) * cfg.ch * 4)
    all_b = wbytes + kvb + state_b
    # the 4-token-draft speculative-verify variant: windows of [pending, 4 drafts] through pyre_forward_multi (logits of all
    # five tokens back on the host) + pyre_spec_keep.  Random drafts are all rejected, so each window yields one token;
    # with every draft accepted the same window would yield five.
    spec = None
    if args.spec_windows > 0:
        dr = g.integers(0, cfg.vocab, (args.spec_windows, 4), dtype=np.uint32)
        pend = nxt
        model.forward_multi(np.concatenate([[pend], dr[0]]).astype(np.uint32), st); model.spec_keep(st, 5, 1)      # untimed
        ctx.sync(); t0 = time.perf_counter()
        for i in range(args.spec_windows):
            ls = model.forward_multi(np.concatenate([[pend], dr[i]]).astype(np.uint32), st)
            pend = int(np.argmax(ls[0])); model.spec_keep(st, 5, 1)
        win_ms = (time.perf_counter() - t0) * 1e3 / args.spec_windows
        spec = {"window_tokens": 5, "ms_per_window": round(win_ms, 3), "tok_s_if_all_drafts_accepted": round(5e3 / win_ms, 1), "tok_s_if_none_accepted": round(1e3 / win_ms, 1),
                "note": "host-facing verify window incl. 5 x %d logits device->host and the host argmax; %d windows" % (cfg.vocab, args.spec_windows)}
    # the variant end to end through the library's own loop (spec::generate's greedy rounds, picks formed on the device):
    # fixed 4-token drafts that are the plain greedy run's own tokens (every draft accepted), then wrong ones (every
    # window rolled back to one token); both from the same snapshot, both must reproduce the plain stream
    spec_loop = None
    if args.spec_loop_tokens > 0:
        n_sl = args.spec_loop_tokens
        snap = st.snapshot()
        plain = model.decode_greedy_dev(st, nxt, n_sl)                  # tokens that follow nxt
        stream = np.concatenate([[nxt], plain]).astype(np.uint32)       # what generate emits when its first pick is nxt
        fl = np.zeros(cfg.vocab, dtype=np.float32); fl[nxt] = 1.0
        res = {}
        for name, ds in (("all_accepted", stream), ("none_accepted", (stream + 1) % cfg.vocab)):
            st.restore(snap)
            dsp = np.concatenate([ds, np.zeros(16, np.uint32)]).astype(np.uint32)
            ctx.sync(); t0 = time.perf_counter()
            out_t, rounds = model.generate_greedy(st, fl, n_sl + 1, n_draft=4, draft_stream=dsp)
            ctx.sync(); dt = time.perf_counter() - t0
            if not np.array_equal(out_t, stream):
                raise SystemExit("drafted generation diverged from plain greedy decoding")
            res[name] = {"tok_s": round(n_sl / dt, 1), "rounds": rounds}
        st.restore(snap)
        spec_loop = {"tokens": n_sl, "drafts_per_round": 4, **res,
                     "note": "pyre_generate_greedy with a fixed draft stream from the same snapshot; output checked against the plain greedy stream"}
    # the reference's own loop shape (Model::forward -> Vec<f32> logits -> sampler::argmax on the host): every step
    # carries 151936 logits over PCIe and a host argmax; reported beside `value`, never as it
    host_loop = None
    if args.host_steps > 0:
        tok = nxt
        lg = model.forward(np.array([tok], dtype=np.uint32), st); tok = int(np.argmax(lg))      # untimed
        ctx.sync(); t0 = time.perf_counter()
        for i in range(args.host_steps):
            lg = model.forward(np.array([tok], dtype=np.uint32), st); tok = int(np.argmax(lg))
        hms = (time.perf_counter() - t0) * 1e3 / args.host_steps
        host_loop = {"tok_s": round(1e3 / hms, 1), "ms_per_step": round(hms, 3), "steps": args.host_steps,
                     "note": "pyre_forward per token: ids from the host, %d f32 logits back over PCIe, argmax on the host" % cfg.vocab}
    # second pass: per-kernel-class durations from event pairs around every launch
    ctx.prof_reset(); ctx.prof_enable(True)
    pn = min(16, args.steps)
    model.decode_greedy_dev(st, nxt, pn, fetch=False)
    prof = ctx.prof_report(); ctx.prof_enable(False)
    classes = sorted(prof.items(), key=lambda kv: -kv[1][1])
    tot_ms = sum(v[1] for v in prof.values())
    breakdown = [{"kernel": k, "launches_per_token": round(v[0] / pn, 2), "us_per_token": round(v[1] / pn * 1e3, 2),
                  "avg_launch_us": round(v[1] / v[0] * 1e3, 3), "GBps": round(v[2] / (v[1] * 1e-3) / 1e9, 1) if v[1] > 0 else None} for k, v in classes]
    dom_k, dom = classes[0]
    dom_gbs = dom[2] / (dom[1] * 1e-3) / 1e9
    # HBM bytes per launch of the dominant class and its kernel-trace duration: not measured by this run but read from
    # the committed counter summaries (FETCH_SIZE / WRITE_SIZE on a three-layer slice of this step; --kernel-trace of this
    # command).  A summary whose kernel classes are not the classes this run reports is stale and is not quoted.
    traffic = None; traffic_source = None; trace_us = None
    def prof_fields(name):
        f = {}
        try:
            for line in open(os.path.join(ROOT, "profiles", name)):
                if ":" in line and not line.startswith(" "):
                    k_, v_ = line.split(":", 1); f[k_.strip()] = v_.strip()
        except OSError:
            pass
        return f
    mine = set(prof.keys())
    if cfg.n_layers == 48 and not args.indexer:
        f = prof_fields("decode_deltanet_slice_hbm_traffic.txt")
        theirs = set(x.strip() for x in f.get("profiled_kernel_classes", "").split(",") if x.strip())
        if theirs and theirs <= mine and ("traffic_bytes_per_launch_%s" % dom_k) in f:
            traffic = int(f["traffic_bytes_per_launch_%s" % dom_k])
            traffic_source = ("profiles/decode_deltanet_slice_hbm_traffic.txt: rocprofv3 FETCH_SIZE + WRITE_SIZE on a three-layer DeltaNet slice of this step launched kernel by kernel, not this run; "
                              "the attention layers' launches of the class and the traffic under graph replay are not measured")
        f = prof_fields("decode_a3b_ctx%d_kernel_stats.txt" % n_ctx)
        theirs = set(x.strip() for x in f.get("profiled_kernel_classes", "").split(",") if x.strip())
        if theirs and theirs <= mine and ("kernel_trace_avg_us_%s" % dom_k) in f:
            trace_us = float(f["kernel_trace_avg_us_%s" % dom_k])
    # the MTP drafter beside the model (synthetic weights of the main layers' geometry, draft head of the reference's
    # default draft vocabulary size): cost of a draft call and of a drafted round.  Random weights draft tokens the model
    # does not pick, so the acceptance seen here says nothing; tok/s at a given acceptance follows from the two costs.
    mtp = None
    if args.mtp_draft > 0:
        kd = args.mtp_draft
        mt, mraw = mg.build_mtp_device(ctx, cfg, cfg.n_exp, cfg.ff_exp, args.mtp_vocab, seed=args.seed + 5)
        dr_ = lib.Mtp(model, cfg.n_exp, cfg.top_k, cfg.ff_exp, 128, mt, np.arange(args.mtp_vocab, dtype=np.uint32) * (cfg.vocab // args.mtp_vocab))
        for p in mraw:
            ctx.free(p)
        n_g = 33
        snap = st.snapshot()
        plain_all = model.decode_greedy_dev(st, nxt, 136 + n_g + 16)    # the plain greedy stream the drafted loops must reproduce
        st.restore(snap)
        dr_.attach(st)
        def warm():
            tail = model.decode_greedy_dev(st, nxt, 136)                # fills the residual ring over a full window
            p_ = int(tail[-1])
            dr_.draft(st, p_, kd)                                       # untimed: the catch-up over the window's cells
            return p_
        pend = warm()
        ctx.sync(); t0 = time.perf_counter()
        for i in range(8):
            dr_.draft(st, pend, kd)
        d_ms = (time.perf_counter() - t0) * 1e3 / 8
        fl = np.zeros(cfg.vocab, dtype=np.float32); fl[pend] = 1.0
        # (1) every draft accepted: the drafter runs, then its ids are replaced by the plain stream's (the accepted path end to end)
        forced = np.concatenate([plain_all[135:], np.zeros(16, np.uint32)]).astype(np.uint32)
        ctx.sync(); t0 = time.perf_counter()
        out_a, rounds_a, drafted_a, accepted_a = dr_.generate_greedy_forced(st, fl, n_g, forced, k=kd)
        ctx.sync(); a_dt = time.perf_counter() - t0
        if not np.array_equal(out_a, plain_all[135:135 + n_g]):
            raise SystemExit("drafted generation (forced drafts) diverged from plain greedy decoding")
        # (2) the synthetic drafter's own drafts (random weights: the model picks none of them): the rejected path
        st.restore(snap); pend = warm()
        ctx.sync(); t0 = time.perf_counter()
        out_t, rounds, drafted, accepted = dr_.generate_greedy(st, fl, n_g, k=kd)
        ctx.sync(); g_dt = time.perf_counter() - t0
        if not np.array_equal(out_t, plain_all[135:135 + n_g]):
            raise SystemExit("drafted generation diverged from plain greedy decoding")
        r_acc, r_rej = a_dt * 1e3 / max(rounds_a, 1), g_dt * 1e3 / max(rounds, 1)
        def implied(a):          # per-draft acceptance a, kd drafts a round: 1 + a + .. + a^kd tokens per round; a round costs between the two measured ones
            toks = (1.0 - a ** (kd + 1)) / (1.0 - a) if a < 1.0 else kd + 1.0
            full = a ** kd                                              # rounds whose drafts are all kept take the accepted-path cost
            return round(toks / ((full * r_acc + (1.0 - full) * r_rej) * 1e-3), 1)
        mtp = {"drafts_per_call": kd, "draft_vocab": args.mtp_vocab, "window": 128, "ms_per_draft_call": round(d_ms, 3), "ms_per_draft_step": round(d_ms / kd, 3),
               "drafted_round_ms": {"all_drafts_accepted": round(r_acc, 3), "no_draft_accepted": round(r_rej, 3),
                                    "rounds": [rounds_a, rounds], "drafted": [drafted_a, drafted], "accepted": [accepted_a, accepted]},
               "accepted_path_tok_s": round((n_g - 1) / a_dt, 1),
               "implied_tok_s_at_acceptance": {"0.68": implied(0.68), "0.8": implied(0.8), "0.87": implied(0.87)},
               "plain_decode_tok_s": round(tok_s, 1),
               "note": "synthetic drafter (512 experts top-10 of width 512 like a main layer, random weights): its own drafts are never the model's pick, so the rate a trained drafter "
                       "would give is not measured; measured are the cost of a draft call (catch-up of the newly committed cells + k draft steps + one readback) and of a drafted round "
                       "with every draft accepted (the drafter's ids replaced by the plain stream's after it ran) and with none; implied = expected tokens per round at the "
                       "reference's per-draft acceptance range / the round cost"}
        dr_.close()
        st.restore(snap)
    out = {
        "metric": "decode tok/s batch-1 (A3B hybrid IQ3_S)", "value": round(tok_s, 2), "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(per, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[4]: Qwen-Next-style A3B hybrid, %d layers (3 Gated DeltaNet + 1 gated attention per group), 512 experts top-10 + shared, "
                               "IQ3_S weights (bf16 router), 4 hyper-connection streams (their synthetic matrices' block scales divided by hc_d_div = %g so that the streams stay bounded over 48 layers), "
                               "4-bit KV, greedy decode after a %d-token random prompt%s" % (
                                   cfg.n_layers, cfg.hc_d_div, n_ctx, (", QSA indexer with %d heads (budget 2048, blocks of 4): variant, not the configuration of the metric" % args.indexer) if args.indexer else ""),
                   "context": n_ctx, "layers": cfg.n_layers, "hc_d_div": cfg.hc_d_div},
        "roofline": {"bound": "hbm", "achieved": round(dom_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(dom_gbs / HBM_PEAK_GBS, 4),
                     "frac_is": "algorithmic bytes / this run's event-pair duration of the class (launches of a few microseconds read 3 to 4 us longer between two events than in the kernel trace)",
                     "frac_kernel_trace": round(dom[2] / dom[0] / (trace_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4) if trace_us else None, "kernel_trace_avg_us": trace_us,
                     "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": dom_k, "algorithmic_bytes_per_launch": round(dom[2] / dom[0]), "avg_launch_us": round(dom[1] / dom[0] * 1e3, 3),
                     "share_of_kernel_time": round(dom[1] / tot_ms, 3)},
        "token_roofline": {"weight_bytes_per_token": wbytes, "kv_bytes_per_token": round(kvb), "state_bytes_per_token": state_b,
                           "weights_only": {"GBps": round(wbytes / (per * 1e-3) / 1e9, 1), "frac": round(wbytes / (per * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
                           "all_bytes": {"GBps": round(all_b / (per * 1e-3) / 1e9, 1), "frac": round(all_b / (per * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
                           "kernel_time_us_per_token": round(tot_ms / pn * 1e3, 1),
                           "hyper_connection_share_of_kernel_time": round(sum(v[1] for k, v in prof.items() if k.startswith("hc_")) / tot_ms, 3)},
        "kernels": breakdown,
    }
    out["prompt"] = {"tokens": n_ctx, "seconds": round(prefill_s, 2), "tok_s": round(n_ctx / prefill_s, 1),
                     "note": "pyre_forward over the prompt in calls of 2048 tokens (windows of 8 tokens, three in flight, taken in blocks of up to 1024 tokens layer by layer, two blocks at a time, each block's FFN grouped by expert on the matrix cores beside the other block's windows), logits of the last token only; untimed part of the step metric"}
    if spec:
        out["spec_verify"] = spec
    if host_loop:
        out["host_loop"] = host_loop
    if spec_loop:
        out["spec_loop"] = spec_loop
    if mtp:
        out["mtp_drafter"] = mtp
    if not args.no_cpu:
        del model, st
        out["cpu_baseline"] = cpu_baseline_decode(cfg, args.seed)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--workload", default="decode", choices=["decode", "gemv", "gemv0", "sweep", "moe", "gdn", "attn"])
    ap.add_argument("--ctx", type=int, default=32768, help="prompt length for the decode workload")
    ap.add_argument("--layers", type=int, default=0, help="debug: fewer layers than the 48 of the configuration")
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--indexer", type=int, default=0, metavar="HEADS", help="decode workload variant: attention layers with a QSA sparse indexer of this many heads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--spec-windows", type=int, default=8, help="decode workload: verify windows of 5 tokens to time after the greedy run (0 = skip)")
    ap.add_argument("--spec-loop-tokens", type=int, default=64, help="decode workload: tokens to generate through the drafted loop (4 fixed drafts per round, all accepted / none accepted; 0 = skip)")
    ap.add_argument("--mtp-draft", type=int, default=3, metavar="K", help="decode workload: also time the MTP drafter (K drafts per call, 1..7; 0 = skip)")
    ap.add_argument("--mtp-vocab", type=int, default=40525, help="decode workload: rows of the drafter's head (the reference's default draft vocabulary has 40525 ids)")
    ap.add_argument("--host-steps", type=int, default=32, help="decode workload: steps of the host-facing loop (pyre_forward + host argmax) to time beside the device loop (0 = skip)")
    ap.add_argument("--t", type=int, default=1, help="gemv workload: tokens per launch (1..8)")
    ap.add_argument("--fmt", default="iq3_s", help="gemv workload: GGUF block type of the matrix (iq3_s, iq2_xs, q4_k, q8_0, q4_0, q5_0, q6_k, iq2_xxs, iq2_s, iq3_xxs, iq4_nl, iq4_xs, q3_k, q5_k, q2_0)")
    ap.add_argument("--calib-copy", type=int, default=0, metavar="MiB", help="gemv workload: also run 4 plain device copies of this size (counter calibration under rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the reference path is single-GPU, single-process); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    out = {"gemv": bench_gemv, "decode": bench_decode, "gemv0": bench_gemv0, "sweep": bench_sweep, "moe": bench_moe, "gdn": bench_gdn, "attn": bench_attn}[args.workload](args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
