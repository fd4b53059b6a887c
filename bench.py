#!/usr/bin/env python3
"""Benchmark driver.  `python bench.py --gpus 1 --steps K --warmup W` prints ONE JSON line.

Workloads (synthetic weights and inputs, resident in HBM before the timed region):
  decode  (default) batch-1 greedy decode of the Qwen-Next-style A3B hybrid of BASELINE.json configs[4]: 48 layers
          (3 Gated DeltaNet + 1 gated attention per group), 512 routed experts top-10 + 1 shared per layer, vocab
          151936, everything IQ3_S except the bf16 router, 4-bit KV cache behind a --ctx token prompt of random ids.
          One step = one generated token; the whole loop runs on the device without host round trips.
  gemv    one IQ3_S dequant-GEMV of the vocabulary-head shape (151936 x 2048, t = 1) per step, rotating over enough
          distinct weight buffers (> 512 MB) that nothing is served from the 256 MB Infinity Cache.
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
    run = (lambda m: m.matmul_mfma_dev(x, t, y)) if args.mfma else (lambda m: m.matmul_dev(x, t, y))
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
    traffic = None          # HBM bytes per launch from the committed FETCH_SIZE / WRITE_SIZE counter summary, when present
    try:
        prof_file = "gemv_iq3s_vocab_head_kernel_stats.txt" if os.environ.get("PYRE_QMATMUL_F32") == "1" else "gemv_i8_iq3s_vocab_head_kernel_stats.txt"
        for line in open(os.path.join(ROOT, "profiles", prof_file)):
            if t == 1 and ty == lib.IQ3_S and line.startswith("traffic_bytes_per_launch:"):
                traffic = int(line.split(":")[1])
    except OSError:
        pass
    gbs = alg_bytes / (per * 1e-3) / 1e9                 # whole step (every launch of the operator call)
    kgbs = alg_bytes / (dom_us * 1e-6) / 1e9             # the dominant kernel alone
    out = {
        "metric": "%s dequant-GEMV achieved HBM GB/s (vocab head 151936x2048, t=%d%s)" % (FN, t, ", matrix cores" if args.mfma else ""), "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(per, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: %s GEMV 2048->151936, batch %d, rotating over %d weight buffers (%.0f MB)" % (FN, t, nbuf, nbuf * mats[0].gguf_bytes / 1e6)},
        "roofline": {"bound": "hbm", "achieved": round(kgbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(kgbs / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "kernel": kernels[0]["kernel"] if kernels else None, "device_bytes_per_launch": mats[0].dev_bytes, "algorithmic_bytes_per_launch": alg_bytes, "avg_launch_us": dom_us},
        "kernels": kernels,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_gemv(ty, rows, cols, 9000)
    return out


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
    st = model.new_state(n_ctx + args.steps + args.warmup + 64 + args.spec_windows + 8 + args.host_steps + 1 + args.spec_loop_tokens + 16)
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
    traffic = None          # HBM bytes per launch of the dominant class from the committed FETCH_SIZE / WRITE_SIZE summary, when it covers it
    if cfg.n_layers == 48 and not args.indexer:
        try:
            for line in open(os.path.join(ROOT, "profiles", "decode_deltanet_slice_hbm_traffic.txt")):
                if line.startswith("traffic_bytes_per_launch_%s:" % dom_k):
                    traffic = int(line.split(":")[1])
        except OSError:
            pass
    out = {
        "metric": "decode tok/s batch-1 (A3B hybrid IQ3_S)", "value": round(tok_s, 2), "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(per, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[4]: Qwen-Next-style A3B hybrid, %d layers (3 Gated DeltaNet + 1 gated attention per group), 512 experts top-10 + shared, "
                               "IQ3_S weights (bf16 router), 4 hyper-connection streams, 4-bit KV, greedy decode after a %d-token random prompt%s" % (
                                   cfg.n_layers, n_ctx, (", QSA indexer with %d heads (budget 2048, blocks of 4): variant, not the configuration of the metric" % args.indexer) if args.indexer else ""),
                   "context": n_ctx, "layers": cfg.n_layers},
        "roofline": {"bound": "hbm", "achieved": round(dom_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(dom_gbs / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "kernel": dom_k, "algorithmic_bytes_per_launch": round(dom[2] / dom[0]), "avg_launch_us": round(dom[1] / dom[0] * 1e3, 3),
                     "share_of_kernel_time": round(dom[1] / tot_ms, 3)},
        "token_roofline": {"weight_bytes_per_token": wbytes, "kv_bytes_per_token": round(kvb), "state_bytes_per_token": state_b,
                           "weights_only": {"GBps": round(wbytes / (per * 1e-3) / 1e9, 1), "frac": round(wbytes / (per * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
                           "all_bytes": {"GBps": round(all_b / (per * 1e-3) / 1e9, 1), "frac": round(all_b / (per * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
                           "kernel_time_us_per_token": round(tot_ms / pn * 1e3, 1)},
        "kernels": breakdown,
    }
    if spec:
        out["spec_verify"] = spec
    if host_loop:
        out["host_loop"] = host_loop
    if spec_loop:
        out["spec_loop"] = spec_loop
    if not args.no_cpu:
        del model, st
        out["cpu_baseline"] = cpu_baseline_decode(cfg, args.seed)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--workload", default="decode", choices=["decode", "gemv"])
    ap.add_argument("--ctx", type=int, default=32768, help="prompt length for the decode workload")
    ap.add_argument("--layers", type=int, default=0, help="debug: fewer layers than the 48 of the configuration")
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--indexer", type=int, default=0, metavar="HEADS", help="decode workload variant: attention layers with a QSA sparse indexer of this many heads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--spec-windows", type=int, default=8, help="decode workload: verify windows of 5 tokens to time after the greedy run (0 = skip)")
    ap.add_argument("--spec-loop-tokens", type=int, default=64, help="decode workload: tokens to generate through the drafted loop (4 fixed drafts per round, all accepted / none accepted; 0 = skip)")
    ap.add_argument("--host-steps", type=int, default=32, help="decode workload: steps of the host-facing loop (pyre_forward + host argmax) to time beside the device loop (0 = skip)")
    ap.add_argument("--t", type=int, default=1, help="gemv workload: tokens per launch (1..8)")
    ap.add_argument("--fmt", default="iq3_s", help="gemv workload: GGUF block type of the matrix (iq3_s, iq2_xs, q4_k, q8_0, q4_0, q5_0, q6_k, iq2_xxs, iq2_s, iq3_xxs, iq4_nl, iq4_xs, q3_k, q5_k, q2_0)")
    ap.add_argument("--mfma", action="store_true", help="gemv workload, t >= 2: the matrix-core verify GEMM instead of the T-accumulator GEMV")
    ap.add_argument("--calib-copy", type=int, default=0, metavar="MiB", help="gemv workload: also run 4 plain device copies of this size (counter calibration under rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the reference path is single-GPU, single-process); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    out = {"gemv": bench_gemv, "decode": bench_decode}[args.workload](args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
