#!/usr/bin/env python3
"""Benchmark of the quantized decode hot path on one MI355X.

`python bench.py --gpus 1 --steps K --warmup W` prints ONE JSON line.

Headline workload (config.workload = "cfg0"): Q4_K GEMV, rows=4096 cols=4096,
batch 1, f32 activations in and out.  One step = one GEMV launch.  The K
timed launches cycle through `--copies` distinct copies of the weight matrix
(64 x 9.4 MB = 604 MB, more than the 256 MB last-level cache plus L2), so every
launch streams its weights from HBM; inputs are resident in HBM before the
timed region.  The launches are captured in one HIP graph and timed with HIP
events recorded on the stream the graph runs on.

value            algorithmic GB/s = (W + x + y bytes) * K / elapsed
roofline         the same figure against MI355X's 8 TB/s HBM peak
cpu_baseline     the CPU checker's dequant+dot (the reference's CPU path
                 restated in C) on the same matrix, on this machine's host cores
also             secondary workloads measured in the same run (hot-cache GEMV,
                 Q6_K LM head, FFN-sized GEMVs, and further configs as they land)
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


class HipEvents:
    """hipEvent timing on a given stream (torch's events only see torch's stream)."""

    def __init__(self):
        self.rt = C.CDLL("libamdhip64.so")
        self.rt.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.rt.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.rt.hipEventSynchronize.argtypes = [C.c_void_p]
        self.rt.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.a, self.b = C.c_void_p(), C.c_void_p()
        assert self.rt.hipEventCreate(C.byref(self.a)) == 0 and self.rt.hipEventCreate(C.byref(self.b)) == 0

    def start(self, stream):
        assert self.rt.hipEventRecord(self.a, stream) == 0

    def stop_ms(self, stream) -> float:
        assert self.rt.hipEventRecord(self.b, stream) == 0
        assert self.rt.hipEventSynchronize(self.b) == 0
        ms = C.c_float()
        assert self.rt.hipEventElapsedTime(C.byref(ms), self.a, self.b) == 0
        return float(ms.value)


def timed_graph(ctx, ev, encode_one, n_launches: int, warmup: int) -> float:
    """Captures `n_launches` calls of encode_one(i) into a graph, runs `warmup`
    launches eagerly first, then times one replay.  Returns ms for the replay."""
    for i in range(warmup):
        encode_one(i)
    ctx.synchronize()
    ctx.graph_begin()
    for i in range(n_launches):
        encode_one(i)
    g = ctx.graph_end()
    ctx.synchronize()
    ev.start(ctx.stream)
    ctx.graph_launch(g)
    ms = ev.stop_ms(ctx.stream)
    ctx.synchronize()
    ctx.graph_destroy(g)
    return ms


def bench_matvec(ctx, eng, ev, dtype, rows, cols, w_host, x_host, copies, steps, warmup, sched=None):
    from ksearch_amd import hip

    wbytes = w_host.size
    big = ctx.buffer_bytes(np.tile(w_host, copies)) if copies > 1 else ctx.buffer_bytes(w_host)
    bx, by = ctx.buffer_f32(x_host), ctx.buffer_empty_f32(rows)
    k = ctx.compile(hip.make_desc(hip.Kind.MATVEC, (rows, cols), (dtype, hip.DType.F32), (), sched))

    def one(i):
        ctx.encode_offsets_multi(k, [big, bx], [(i % copies) * wbytes, 0], [by], [0])

    ms = timed_graph(ctx, ev, one, steps, warmup)
    alg = wbytes + cols * 4 + rows * 4
    big.release()
    return dict(kernel=k.name, us_per_launch=ms * 1e3 / steps, gbps=alg * steps / (ms * 1e-3) / 1e9,
                alg_bytes=alg, ms=ms)


def cpu_baseline_matvec(w, x, rows, cols, budget_s=1.5):
    """The CPU checker (oracle/) timed on this machine: all cores, then one."""
    import oracle

    out = {}
    for label, threads in (("all", 0), ("one", 1)):
        oracle.matvec(oracle.Q4K, w, rows, cols, x, threads)        # warm-up
        reps, t0 = 0, time.perf_counter()
        times = []
        while time.perf_counter() - t0 < budget_s or reps < 5:
            t1 = time.perf_counter()
            oracle.matvec(oracle.Q4K, w, rows, cols, x, threads)
            times.append(time.perf_counter() - t1)
            reps += 1
        out[label] = (float(np.median(times)), reps)
    return out, oracle.max_threads()


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1024)
    ap.add_argument("--warmup", type=int, default=128)
    ap.add_argument("--copies", type=int, default=64)
    ap.add_argument("--no-extras", action="store_true", help="headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the hot path is a single-GPU kernel path); "
              "--gpus must be 1", file=sys.stderr)
        return 2

    from ksearch_amd import hip, synth
    from ksearch_amd.hip import DType

    ctx, eng, ev = hip.Context(), hip.Eng(), HipEvents()
    rows = cols = 4096
    w, x = synth.cfg0_q4k_matvec()
    head = bench_matvec(ctx, eng, ev, DType.Q4K, rows, cols, w, x, args.copies, args.steps, args.warmup)

    also = {}
    if not args.no_extras:
        hot = bench_matvec(ctx, eng, ev, DType.Q4K, rows, cols, w, x, 1, args.steps, args.warmup)
        also["cfg0_hot_cache"] = dict(us_per_launch=round(hot["us_per_launch"], 3), gbps=round(hot["gbps"], 1))
        w1, x1 = synth.cfg1_q6k_lm_head()
        r1 = bench_matvec(ctx, eng, ev, DType.Q6K, 262144, 2048, w1, x1, 1, 50, 5)
        also["cfg1_q6k_lm_head"] = dict(kernel=r1["kernel"], us_per_launch=round(r1["us_per_launch"], 2),
                                        gbps=round(r1["gbps"], 1), frac_hbm=round(r1["gbps"] / HBM_PEAK_GBPS, 4))
        del w1

    cpu = None
    if not args.no_cpu:
        t, cores = cpu_baseline_matvec(w, x, rows, cols)
        alg = head["alg_bytes"]
        cpu = dict(value=round(alg / t["all"][0] / 1e9, 3), unit="GB/s", cores=cores, kind="port",
                   sample=f"cfg0 full matrix, {t['all'][1]} repetitions, median; "
                          f"1 thread: {alg / t['one'][0] / 1e9:.3f} GB/s")

    line = {
        "metric": "q4k_matvec_GBps", "value": round(head["gbps"], 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms"] / args.steps,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "cfg0: Q4_K GEMV rows=4096 cols=4096 batch=1, f32 x/y, weights streamed from HBM "
                               f"({args.copies} rotating copies)", "kernel": head["kernel"]},
        "roofline": {"bound": "hbm", "achieved": round(head["gbps"], 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(head["gbps"] / HBM_PEAK_GBPS, 4), "traffic": None},
        "cpu_baseline": cpu,
        "also": also,
    }
    ctx.close()
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
