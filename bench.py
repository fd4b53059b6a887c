#!/usr/bin/env python3
"""Benchmark driver.  `python bench.py --gpus 1 --steps K --warmup W` prints ONE JSON line.

Workloads (all synthetic, inputs resident in HBM before the timed region):
  gemv    one IQ3_S dequant-GEMV of the vocabulary-head shape (151936 x 2048, t = 1) per step, rotating over enough
          distinct weight buffers (> 512 MB) that nothing is served from the 256 MB Infinity Cache.
The timed region is bracketed by HIP events recorded on the library's own stream.
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


def cpu_baseline_gemv(ty, rows, cols, seed, budget_s=12.0):
    """The oracle's QMat::matmul restatement (row dequant + f32 dot, rows over all host threads) on a bounded row
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
    rows_per_s = n * sample_rows / dt
    gb_s = rows_per_s * (cols // el * bs) / 1e9
    return {"value": round(gb_s, 3), "unit": "GB/s of GGUF weight bytes", "cores": threads, "kind": "port",
            "sample": "%d launches of the oracle matmul over the first %d rows x %d cols (IQ3_S), t=1" % (n, sample_rows, cols)}


def bench_gemv(args):
    from pyre_amd import lib, synth
    ev = HipEvents()
    ctx = lib.Context(0)
    ty, rows, cols = lib.IQ3_S, 151936, 2048
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
    for i in range(args.warmup):
        mats[i % nbuf].matmul_dev(x, 1, y)
    ctx.sync()
    e0, e1 = ev.event(), ev.event()
    t0 = time.perf_counter()
    ev.record(e0, ctx.stream)
    for i in range(args.steps):
        mats[i % nbuf].matmul_dev(x, 1, y)
    ev.record(e1, ctx.stream)
    ms = ev.elapsed_ms(e0, e1)
    ctx.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    per = ms / args.steps
    alg_bytes = mats[0].gguf_bytes + 4 * cols + 4 * rows
    gbs = alg_bytes / (per * 1e-3) / 1e9
    out = {
        "metric": "IQ3_S dequant-GEMV achieved HBM GB/s (vocab head 151936x2048, t=1)", "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(per, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: IQ3_S GEMV 2048->151936, batch 1, rotating over %d weight buffers (%.0f MB)" % (nbuf, nbuf * mats[0].gguf_bytes / 1e6)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "k_gemv<IQ3_S,1>", "algorithmic_bytes_per_launch": alg_bytes, "avg_launch_us": round(per * 1e3, 3)},
        "wall_ms_per_step": round(wall_ms / args.steps, 5),
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_gemv(ty, rows, cols, 9000)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="gemv")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the reference path is single-GPU, single-process); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    out = {"gemv": bench_gemv}[args.workload](args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
