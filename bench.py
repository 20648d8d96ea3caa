#!/usr/bin/env python3
"""Benchmark of the quantized decode hot path on one MI355X.

`python bench.py --gpus 1 --steps K --warmup W` prints ONE JSON line.

Headline workload (config.workload = "cfg0"): Q4_K GEMV, rows=4096 cols=4096,
batch 1, f32 activations in and out.  One step = one GEMV launch.  The K
timed launches cycle through `--copies` distinct copies of the weight matrix
(64 x 9.4 MB = 604 MB, more than the 256 MB last-level cache plus L2), so every
launch streams its weights from HBM; inputs are resident in HBM before the
timed region.  The launches are captured in one HIP graph and timed with HIP
events recorded on the stream the graph runs on; the figure is the median of
five replays of that graph, each of exactly K launches.

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

# kernels are chosen by the library's defaults, never by a plan file an earlier search left in the user's cache
if "KSEARCH_BEAM_CACHE" not in os.environ:
    import tempfile

    os.environ["KSEARCH_BEAM_CACHE"] = tempfile.mkdtemp(prefix="ksearch_bench_plans_")


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


def timed_graph(ctx, ev, encode_one, n_launches: int, warmup: int, replays: int = 1) -> float:
    """Captures `n_launches` calls of encode_one(i) into a graph, runs `warmup`
    launches eagerly first and (when there is a warm-up at all) one untimed replay,
    then times `replays` replays, each of exactly `n_launches` launches between a
    synchronisation and an event pair of its own, and returns the median replay's ms
    (a short graph's time is its launches plus the ~10 us it takes to get the graph
    going, and that part jitters from replay to replay)."""
    for i in range(warmup):
        encode_one(i)
    ctx.synchronize()
    ctx.graph_begin()
    for i in range(n_launches):
        encode_one(i)
    g = ctx.graph_end()
    if warmup:
        ctx.graph_launch(g)      # the first replay of a new executable graph also uploads it: part of the warm-up
    times = []
    for _ in range(max(1, replays)):
        ctx.synchronize()
        ev.start(ctx.stream)
        ctx.graph_launch(g)
        times.append(ev.stop_ms(ctx.stream))
    ctx.synchronize()
    ctx.graph_destroy(g)
    return float(np.median(times))


def bench_matvec(ctx, eng, ev, dtype, rows, cols, w_host, x_host, copies, steps, warmup, sched=None, replays=1):
    from ksearch_amd import hip

    wbytes = w_host.size
    big = ctx.buffer_bytes(np.tile(w_host, copies)) if copies > 1 else ctx.buffer_bytes(w_host)
    bx, by = ctx.buffer_f32(x_host), ctx.buffer_empty_f32(rows)
    k = ctx.compile(hip.make_desc(hip.Kind.MATVEC, (rows, cols), (dtype, hip.DType.F32), (), sched))

    def one(i):
        ctx.encode_offsets_multi(k, [big, bx], [(i % copies) * wbytes, 0], [by], [0])

    ms = timed_graph(ctx, ev, one, steps, warmup, replays)
    alg = wbytes + cols * 4 + rows * 4
    big.release()
    return dict(kernel=k.name, us_per_launch=ms * 1e3 / steps, gbps=alg * steps / (ms * 1e-3) / 1e9,
                alg_bytes=alg, ms=ms)


def bench_floor(ctx, eng, ev, copies, steps, warmup):
    """The memory-only floors of the headline launch, under the headline's protocol (one HIP graph of `steps`
    dependent launches over `copies` rotating weight copies, HIP events on the stream): the same grid / workgroup /
    LDS doing nothing, issuing only the GEMV's weight loads, and reading the same bytes with flat 128-bit loads;
    then the GEMV itself for comparison."""
    from ksearch_amd import hip, synth

    rows = cols = 4096
    w, x = synth.cfg0_q4k_matvec()
    wbytes = w.size
    big, sink = ctx.buffer_bytes(np.tile(w, copies)), ctx.buffer_empty_f32(1)
    out = {"protocol": f"graph of {steps} launches, {copies} rotating copies of the 9.4 MB matrix, hipEvents; best of 5 replays"}
    for mode, name in ((0, "empty_launch"), (1, "gemv_load_pattern_only"), (2, "flat_128bit_loads_only")):
        k = ctx.compile(hip.make_desc(hip.Kind.READ_FLOOR, (rows, cols, mode), (hip.DType.Q4K,)))

        def one(i, k=k):
            ctx.encode_offsets_multi(k, [big], [(i % copies) * wbytes], [sink], [0])

        us = min(timed_graph(ctx, ev, one, steps, warmup) for _ in range(5)) * 1e3 / steps
        out[name] = dict(kernel=k.name, us_per_launch=round(us, 3), tbps=round(wbytes / us / 1e6, 2) if mode else None)
    # what an empty launch costs in other shapes: workgroups x threads, with and without the LDS reservation, and with an
    # argument block of the GEMV's size
    shapes = {}
    for wgs in (256, 512, 1024):
        for thr in (64, 128, 256, 512):
            row = []
            for no_lds, big_args in ((0, 0), (1, 0), (0, 1)):
                k = ctx.compile(hip.make_desc(hip.Kind.READ_FLOOR, (rows, cols, 0, wgs, thr, no_lds, big_args), (hip.DType.Q4K,)))

                def one(i, k=k):
                    ctx.encode_offsets_multi(k, [big], [(i % copies) * wbytes], [sink], [0])

                row.append(round(min(timed_graph(ctx, ev, one, steps, warmup) for _ in range(3)) * 1e3 / steps, 3))
            shapes[f"{wgs}x{thr}"] = dict(us_with_lds=row[0], us_without_lds=row[1], us_with_gemv_sized_arguments=row[2])
    out["empty_launch_by_shape"] = shapes
    big.release()
    g = min((bench_matvec(ctx, eng, ev, hip.DType.Q4K, rows, cols, w, x, copies, steps, warmup) for _ in range(5)),
            key=lambda r: r["us_per_launch"])
    out["gemv"] = dict(kernel=g["kernel"], us_per_launch=round(g["us_per_launch"], 3), tbps=round(g["gbps"] / 1e3, 2))
    return out


def bench_lm_head(ctx, eng, ev):
    """cfg1: the Q6_K LM head, 262144 x 2048, on the weights as the decode loop keeps them in HBM (each row's
    fields grouped at load time, KSH_REPACK_ROWS: the same 210 bytes per 256 weights) and on the GGUF byte order."""
    from ksearch_amd import hip, synth
    from ksearch_amd.hip import DType

    rows, cols = 262144, 2048
    w1, x1 = synth.cfg1_q6k_lm_head()
    gguf = bench_matvec(ctx, eng, ev, DType.Q6K, rows, cols, w1, x1, 1, 50, 5)
    src, dst = ctx.buffer_bytes(w1), ctx.buffer_empty_bytes(w1.size)
    eng.repack_rows(ctx, rows, cols, src, dst)
    grouped = ctx.read_bytes(dst, w1.size)
    src.release()
    dst.release()
    r = bench_matvec(ctx, eng, ev, DType.Q6K_ROWS, rows, cols, grouped, x1, 1, 50, 5)
    return dict(kernel=r["kernel"], us_per_launch=round(r["us_per_launch"], 2), gbps=round(r["gbps"], 1),
                frac_hbm=round(r["gbps"] / HBM_PEAK_GBPS, 4),
                weights="rows regrouped by field when loaded (lossless, same bytes); 440 MB streamed from HBM per launch",
                gguf_byte_order=dict(kernel=gguf["kernel"], us_per_launch=round(gguf["us_per_launch"], 2),
                                     gbps=round(gguf["gbps"], 1), frac_hbm=round(gguf["gbps"] / HBM_PEAK_GBPS, 4)))


def bench_prefill(ctx):
    """cfg2: 512 bf16 tokens x Q4_K [8192 x 2048] -> f32, hipEvent average of 50 launches; the same shape over
    Q6_K weights beside it."""
    from ksearch_amd import hip, synth

    tokens, rows, cols = 512, 8192, 2048
    w, _, xb = synth.cfg2_q4k_prefill()
    out = {}
    for dt, wq in ((hip.DType.Q4K, w), (hip.DType.Q6K, synth.q6k_blocks(rows * cols // 256, seed=1012))):
        bw, bx, by = ctx.buffer_bytes(wq), ctx.buffer_bytes(xb), ctx.buffer_empty_f32(tokens * rows)
        k = ctx.compile(hip.make_desc(hip.Kind.MATVEC_BATCH, (rows, cols, tokens), (dt, hip.DType.BF16, hip.DType.F32)))
        ctx.run(k, [bw, bx], [by], iters=5)
        ms = ctx.run(k, [bw, bx], [by], iters=50)
        tf = 2.0 * tokens * rows * cols / (ms * 1e-3) / 1e12
        for b in (bw, bx, by):
            b.release()
        r = dict(kernel=k.name, us_per_launch=round(ms * 1e3, 2), tflops=round(tf, 1), frac_mfma_f16=round(tf / 2500.0, 4))
        if dt == hip.DType.Q4K:
            out = r
        else:
            out["q6k_weights"] = r
    return out


def bench_attention(ctx, ev, copies=16, sched=None):
    """cfg3: 4 slots, 8 q / 1 kv heads of 256, Q4_0 KV, lengths ~U{1024..16384}, one launch pair.  Timed twice: with
    the 7 MB of rows resident in cache between launches, and cold, cycling through `copies` copies of the K / V
    pools (16 x 18.9 MB = 302 MB, more than the 256 MB last-level cache) inside one HIP graph."""
    from ksearch_amd import hip, synth

    n_slots, n_q, n_kv, hd, max_t = 4, 8, 1, 256, 16384
    lens, kk, vv, q = synth.cfg3_q40_attention()
    meta = np.zeros((n_slots, 4), dtype=np.float32)
    meta[:, 0] = lens
    k = ctx.compile(hip.make_desc(hip.Kind.SDPA_SLOTS, (n_q, n_kv, hd, max_t, n_slots, 0),
                                  (hip.DType.Q40, hip.DType.F32), (1.0 / 16.0,), sched))
    nwg = k.info.sched.k_split
    ins = [ctx.buffer_f32(q), ctx.buffer_bytes(kk), ctx.buffer_bytes(vv), ctx.buffer_f32(meta)]
    outs = [ctx.buffer_empty_f32(n_slots * n_q * nwg * (hd + 2)), ctx.buffer_empty_f32(n_slots * n_q * hd)]
    ctx.run(k, ins, outs, iters=5)
    ms = ctx.run(k, ins, outs, iters=50)
    alg = int(sum(288 * int(t) + 16384 for t in lens))
    bk, bv = ctx.buffer_bytes(np.tile(kk.reshape(-1), copies)), ctx.buffer_bytes(np.tile(vv.reshape(-1), copies))

    def one(i):
        c = i % copies
        ctx.encode_offsets_multi(k, [ins[0], bk, bv, ins[3]], [0, c * kk.size, c * vv.size, 0], outs, [0, 0])

    cold_ms = min(timed_graph(ctx, ev, one, 64, 8) for _ in range(3)) / 64
    for b in ins + outs + [bk, bv]:
        b.release()

    def rec(t_ms):
        return dict(us_per_launch=round(t_ms * 1e3, 2), gbps=round(alg / (t_ms * 1e-3) / 1e9, 1),
                    frac_hbm=round(alg / (t_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4))

    return dict(kernel=k.name, lens=[int(t) for t in lens], alg_bytes=alg, **rec(cold_ms),
                protocol=f"cold: graph of 64 launch pairs over {copies} rotating copies of the K / V pools ({copies * (kk.size + vv.size) >> 20} MiB)",
                hot_cache=rec(ms))


def bench_decode(ctx, eng, use_graph=True):
    """cfg4: synthetic Gemma-4-E2B-shaped greedy decode, 64-token prompt then 256 tokens, HIP-graph replay."""
    from ksearch_amd import hip, synth

    cfg = synth.GEMMA_E2B_SYNTH
    q4k, q6k = hip.device_quantizers(ctx, eng)
    w = synth.gemma_weights(cfg, 4000, q4k, q6k)
    m = hip.Gemma(ctx, cfg, w)
    prompt = [int(t) for t in np.random.default_rng(4001).integers(0, cfg["vocab"], 64)]
    m.generate(prompt, 8, use_graph=use_graph)     # warm-up: binds kernels, captures the graphs
    m.reset()
    _, serial_pre_ms, _ = m.generate(prompt, 1, use_graph=use_graph, serial_prefill=True)
    m.reset()
    _, pre_ms, dec_ms = m.generate(prompt, 256, use_graph=use_graph)
    h, f, hd = cfg["hidden"], cfg["ffn"], cfg["hd"]
    layer = (cfg["n_q"] * hd * h + 2 * cfg["n_kv"] * hd * h + h * cfg["n_q"] * hd + 3 * f * h) // 256 * 144
    per_tok = cfg["n_layers"] * layer + cfg["vocab"] * h // 256 * 210
    # a long prompt: 1024 tokens are one chunk of the batched pass
    long_prompt = [int(t) for t in np.random.default_rng(4002).integers(0, cfg["vocab"], 1025)]
    long_ms, mid_ms = [], []
    for _ in range(2):
        m.reset()
        long_ms.append(m.generate(long_prompt, 1, use_graph=use_graph)[1])
        m.reset()
        mid_ms.append(m.generate(long_prompt[:257], 1, use_graph=use_graph)[1])
    m.reset()
    out = dict(tok_per_s=round(256 / dec_ms * 1e3, 1), ms_per_token=round(dec_ms / 256, 4),
               launches_per_token=m.launches_per_token, weight_gbps=round(per_tok * 256 / (dec_ms * 1e-3) / 1e9, 1),
               frac_hbm=round(per_tok * 256 / (dec_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
               prompt_tokens=64, new_tokens=256, graph=bool(use_graph),
               prefill_ms=round(pre_ms, 3), prefill_tok_per_s=round(63 / pre_ms * 1e3, 1),
               prefill_ms_token_by_token=round(serial_pre_ms, 3),
               prefill_256_tokens_ms=round(min(mid_ms), 2), prefill_256_tok_per_s=round(256 / min(mid_ms) * 1e3, 1),
               prefill_1024_tokens_ms=round(min(long_ms), 2), prefill_1024_tok_per_s=round(1024 / min(long_ms) * 1e3, 1))
    m.close()
    return out


def bench_prompt_pass(ctx, eng):
    """Prompt passes of cfg4's model alone (eager launches, for kernel traces): prompts of 256, 1024 and 4000 tokens
    from an empty cache, each timed on its second run."""
    from ksearch_amd import hip, synth

    cfg = synth.GEMMA_E2B_SYNTH
    q4k, q6k = hip.device_quantizers(ctx, eng)
    m = hip.Gemma(ctx, cfg, synth.gemma_weights(cfg, 4000, q4k, q6k))
    rng = np.random.default_rng(4002)
    out = {}
    for n in (256, 1024, 4000):
        prompt = [int(t) for t in rng.integers(0, cfg["vocab"], n + 1)]
        for _ in range(2):
            m.reset()
            ms = m.generate(prompt, 1, use_graph=False)[1]
        out[f"prompt_{n}"] = dict(ms=round(ms, 2), tok_per_s=round(n / ms * 1e3, 1))
    m.close()
    return out


def bench_decode_gemma4_layout(ctx, eng, use_graph=True):
    """Greedy decode at the layer layout of the real Gemma-4 E2B checkpoints (synthetic weights): 35 layers of
    hidden 1536, four sliding-window layers (head dim 256, window 512) per full-attention layer (head dim 512),
    the last 20 layers reading earlier layers' KV caches with a double-wide feed-forward, per-layer embeddings
    (a Q5_K table of 35 x 256 per token), Q6_K tied LM head.  Not the headline configuration (that one has none
    of these features): a second point, for the loop that takes GGUF files."""
    from ksearch_amd import hip, synth

    n, shared = 35, 20
    cfg = dict(n_layers=n, hidden=1536, n_q=8, n_kv=1, vocab=262144, max_seq=4096, hd_swa=256, hd_full=512, sliding_window=512,
               shared_kv_layers=shared, ple_dim=256, eps=1e-6, softcap=30.0, rope_theta_swa=1e4, rope_theta_full=1e6, partial_rotary=0.25,
               attn_scale=1.0)
    ffn = [6144 if i < n - shared else 12288 for i in range(n)]
    q4k, q6k = hip.device_quantizers(ctx, eng)
    w = synth.gemma4_weights(cfg, 1005, q4k, lambda x: q6k([x]), ffn=ffn)
    model = hip.Gemma4(ctx, cfg, w)
    prompt = [int(t) for t in np.random.default_rng(1005).integers(0, cfg["vocab"], 64)]
    ms, pre = [], []
    for _ in range(3):
        model.reset()
        ids, prefill_ms, decode_ms = model.generate(prompt, 256, use_graph=use_graph)
        ms.append(decode_ms)
        pre.append(prefill_ms)
    # bytes a token streams: every packed matrix once (the per-layer table contributes one row)
    wbytes = sum(b.nbytes for lw in w["layers"] for b in lw.values() if isinstance(b, hip.Buffer))
    wbytes += w["globals"]["token_embd"].nbytes + w["globals"]["ple_model_proj"].nbytes
    r = {"tok_s": round(256 / min(ms) * 1e3, 1), "ms_per_token": round(min(ms) / 256, 4), "launches_per_token": model.launches_per_token,
         "weight_GB_per_token": round(wbytes / 1e9, 3), "GB_s": round(wbytes / (min(ms) / 256 * 1e-3) / 1e9, 1),
         "prefill_ms": round(min(pre), 3), "prefill_tok_per_s": round(63 / min(pre) * 1e3, 1),
         "layout": "35 layers, hidden 1536, 4 SWA(256, window 512) : 1 full(512), 20 shared-KV layers, PLE 256, ffn 6144/12288"}
    # the same model under the slot scheduler: requests of 64 + 128 tokens from as many KV slots, the decoding ones
    # taking each step together as one pass over the weights (one by one, as the reference's serving loop does it,
    # for comparison); one host read-back per round
    pool = hip.KvPool(ctx, 16, cfg["max_seq"], n - shared, 512, 1)
    served = {}
    for n_req, batched in ((2, 0), (2, 2), (3, 2), (4, 0), (4, 2), (8, 2), (16, 2)):
        sv = hip.Serve(model, pool, slots=n_req, eos=(0xFFFFFFFF, 0xFFFFFFFE), use_graph=use_graph, batched_decode=batched)
        best = 1e9
        for rep in range(2):
            for i in range(n_req):
                sv.submit(prompt[i:] + prompt[:i], 128)
            sv.tick()                                   # admission + prefill of the prompts
            ctx.synchronize()
            t0 = time.perf_counter()
            n_tok = sum(1 for e in sv.run() if e[0] == "token")
            best = min(best, (time.perf_counter() - t0) / n_tok)
        served[f"{n_req}_slots" + ("" if batched else "_one_by_one")] = round(1.0 / best, 1)
        sv.close()
    r["served_tok_s"] = served
    model.bind_slot(None, 0)
    pool.close()
    model.close()
    return r


def bench_timeline(ctx, eng, tokens=24):
    """Where a decode step's launches spend their time, from inside: the timeline build of the library
    (ksearch_amd/lib/libksearch_hip_stamps.so: the same sources with -DKSH_STAMPS) has lane 0 of every wave write the
    chip-wide 100 MHz counter between its phases.  cfg4's model decodes `tokens` tokens from position 64 through the
    captured graph; after each token the records of the last launch of every shape are read -- the last layer's
    QKV, attention step, o-projection, gate || up, down, and the LM head, which follow one another, so their records
    share one time axis.  Per launch: when its waves enter, and the median / slowest wave at each phase boundary,
    in microseconds from the launch's first wave; `gap_before_us` is the time from the previous launch's last
    acknowledged store to this launch's first wave.  The timestamps themselves cost a little (one counter read and
    one store per wave): the timeline build decodes a few per cent slower than the product build."""
    from ksearch_amd import hip, synth

    L = hip.lib()
    S, W, T = 8, 4096, 8          # slots per record, records per tag, tags (ksh_device.hpp)
    readers = {}
    for name in ("ksh_stamps_matvec_q4k", "ksh_stamps_sdpa_lanes", "ksh_stamps_matvec_q6k"):
        fn = getattr(L, name)
        fn.restype, fn.argtypes = C.c_int, [C.POINTER(C.c_ulonglong), C.c_size_t]
        readers[name] = fn

    def read(name):
        buf = (C.c_ulonglong * (T * W * S))()
        assert readers[name](buf, T * W * S) == 0
        return np.frombuffer(buf, dtype=np.uint64).reshape(T, W, S).astype(np.int64)

    cfg = synth.GEMMA_E2B_SYNTH
    q4k, q6k = hip.device_quantizers(ctx, eng)
    m = hip.Gemma(ctx, cfg, synth.gemma_weights(cfg, 4000, q4k, q6k))
    prompt = [int(t) for t in np.random.default_rng(4001).integers(0, cfg["vocab"], 64)]
    out, _, _ = m.generate(prompt, 4, use_graph=True)
    tok = out[-1]
    for r in readers:
        read(r)                    # clears what the warm-up left
    # (kernel, reader, tag, names of the phase boundaries 1..6)
    gemv = ["loads issued", "vector staged", "barrier passed", "products done", "stores issued", "stores acknowledged"]
    launches = [
        ("qkv (add + norm prologue, 2.9 MB)", "ksh_stamps_matvec_q4k", 4, gemv),
        ("attention step (norm, rope, append, <= 8 partitions)", "ksh_stamps_sdpa_lanes", 1,
         ["front loads issued", "length and position in", "q and new row ready", "rows done", "row groups folded", "records acknowledged"]),
        ("o-projection (merges the partitions, 2.4 MB)", "ksh_stamps_matvec_q4k", 6, gemv),
        ("gate || up + GELU (add + norm prologue, 18.9 MB)", "ksh_stamps_matvec_q4k", 5, gemv),
        ("down (9.4 MB)", "ksh_stamps_matvec_q4k", 0, gemv),
        ("LM head (add + norm prologue, 440 MB; every 4th workgroup)", "ksh_stamps_matvec_q6k", 0,
         ["loads issued", "vector staged", "barrier passed", "first row done", "last row stored", "stores acknowledged"]),
    ]
    acc = {name: [] for name, *_ in launches}
    for _ in range(tokens):
        tok = m.forward_token(tok, use_graph=True)
        bufs = {r: read(r) for r in readers}
        prev_end = None
        for name, reader, tag, phases in launches:
            a = bufs[reader][tag]
            a = a[a[:, 0] > 0]
            if not len(a):
                raise SystemExit(f"bench.py: the timeline build left no records for {name!r}")
            t0 = a[:, 0].min()
            row = dict(waves=len(a), gap=None if prev_end is None else (t0 - prev_end) * 0.01,
                       entry_p50=(np.median(a[:, 0]) - t0) * 0.01, entry_max=(a[:, 0].max() - t0) * 0.01)
            for i in range(1, 7):
                v = a[:, i][a[:, i] > 0]
                row[f"p50_{i}"] = (np.median(v) - t0) * 0.01 if len(v) else None
                row[f"max_{i}"] = (v.max() - t0) * 0.01 if len(v) else None
            prev_end = max(int(a[:, i][a[:, i] > 0].max()) for i in range(1, 7) if (a[:, i] > 0).any())
            row["span"] = (prev_end - t0) * 0.01
            acc[name].append(row)
    m.close()
    res = {"tokens": tokens, "unit": "us from the launch's first wave; median over the tokens of (p50 over waves | slowest wave)"}
    for name, reader, tag, phases in launches:
        rows = acc[name]

        def med(k):
            v = [r[k] for r in rows if r[k] is not None]
            return round(float(np.median(v)), 2) if v else None

        rec = {"waves": rows[0]["waves"], "gap_before_us": med("gap"), "entry_p50": med("entry_p50"), "entry_last": med("entry_max"),
               "first_wave_to_last_ack_us": med("span")}
        for i, ph in enumerate(phases, 1):
            rec[ph] = [med(f"p50_{i}"), med(f"max_{i}")]
        res[name] = rec

    # cfg3's row kernel (the matrix-core form whose waves share P.V by V block), hot: the same statistics over twelve launches
    n_slots, n_q, n_kv, hd, max_t = 4, 8, 1, 256, 16384
    lens, kk, vv, q = synth.cfg3_q40_attention()
    meta = np.zeros((n_slots, 4), dtype=np.float32)
    meta[:, 0] = lens
    k = ctx.compile(hip.make_desc(hip.Kind.SDPA_SLOTS, (n_q, n_kv, hd, max_t, n_slots, 0), (hip.DType.Q40, hip.DType.F32), (1.0 / 16.0,)))
    nwg = k.info.sched.k_split
    ins = [ctx.buffer_f32(q), ctx.buffer_bytes(kk), ctx.buffer_bytes(vv), ctx.buffer_f32(meta)]
    outs = [ctx.buffer_empty_f32(n_slots * n_q * nwg * (hd + 2)), ctx.buffer_empty_f32(n_slots * n_q * hd)]
    ctx.run(k, ins, outs, iters=3)
    read("ksh_stamps_sdpa_lanes")
    phases = ["the deal is known", "q operands shared", "tile and scale tables in LDS", "probabilities written", "products done", "stores acknowledged"]
    rows = []
    for _ in range(12):
        ctx.run(k, ins, outs, iters=1)
        a = read("ksh_stamps_sdpa_lanes")[2]
        a = a[a[:, 6] > 0]
        if not len(a):
            raise SystemExit("bench.py: the timeline build left no records for cfg3's row kernel")
        t0 = a[:, 0].min()
        row = dict(waves=len(a), entry_p50=(np.median(a[:, 0]) - t0) * 0.01, entry_max=(a[:, 0].max() - t0) * 0.01)
        for i in range(1, 7):
            row[f"p50_{i}"], row[f"max_{i}"] = (np.median(a[:, i]) - t0) * 0.01, (a[:, i].max() - t0) * 0.01
        rows.append(row)
    rec = {"waves": rows[0]["waves"], "kernel": k.name, "gap_before_us": None,
           "entry_p50": round(float(np.median([r["entry_p50"] for r in rows])), 2), "entry_last": round(float(np.median([r["entry_max"] for r in rows])), 2),
           "first_wave_to_last_ack_us": round(float(np.median([r["max_6"] for r in rows])), 2)}
    for i, ph in enumerate(phases, 1):
        rec[ph] = [round(float(np.median([r[f"p50_{i}"] for r in rows])), 2), round(float(np.median([r[f"max_{i}"] for r in rows])), 2)]
    res["cfg3 attention, row kernel (waves with rows)"] = rec
    return res


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


# HBM bytes per launch of the headline kernel, from the FETCH_SIZE / WRITE_SIZE counter runs summarised in
# profiles/q4k_gemv_cfg0_cold.txt (2.00 x 4705.5 KiB fetched + 16.0 KiB written).  Counters cannot be read from
# inside this script, so the figure is carried here for the kernel it was taken on; a headline kernel that is not in
# the table is an error (the counters have to be taken again for it), never a silent null.
MEASURED_TRAFFIC_BYTES = {"matvec_q4k_r2_w8_v3": 9653248}


def measured_traffic(kernel: str) -> int:
    if kernel not in MEASURED_TRAFFIC_BYTES:
        raise SystemExit(f"bench.py: no FETCH_SIZE / WRITE_SIZE figures for the headline kernel {kernel!r}: take the two "
                         f"counter runs on it (profiles/q4k_gemv_cfg0_cold.txt holds the commands) and add it to MEASURED_TRAFFIC_BYTES")
    return MEASURED_TRAFFIC_BYTES[kernel]


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1024)
    ap.add_argument("--warmup", type=int, default=128)
    ap.add_argument("--copies", type=int, default=64)
    ap.add_argument("--no-extras", action="store_true", help="headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--eager", action="store_true", help="cfg4 without HIP-graph replay (kernel-trace profiling)")
    ap.add_argument("--attn-form", choices=["default", "lanes", "mfma"], default="default",
                    help="cfg3: the split-KV row phase as the register (lanes) or the matrix-core (mfma) kernel instead of "
                         "the library's choice for the shape")
    ap.add_argument("--only", choices=["cfg1", "cfg2", "cfg3", "cfg4", "gemma4", "prefill", "copy", "floor", "timeline"],
                    help="run one secondary workload and print its record (for profiling runs); 'copy' is a plain "
                         "64 MiB device copy, the known-size kernel that calibrates the FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the hot path is a single-GPU kernel path); "
              "--gpus must be 1", file=sys.stderr)
        return 2

    from ksearch_amd import hip, synth
    from ksearch_amd.hip import DType

    if args.only == "timeline":
        # the timeline build of the library (phase timestamps compiled in); nothing else in this script uses it
        from ksearch_amd import _build

        hip.LIB_PATH = _build.STAMPS_LIB_PATH
        os.environ["KSEARCH_SKIP_BEAM"] = "1"      # the library's default schedules
        ctx, eng = hip.Context(), hip.Eng()
        r = bench_timeline(ctx, eng)
        ctx.close()
        print(json.dumps({"timeline": r}))
        for name, rec in r.items():
            if isinstance(rec, dict):
                print(f"{name}: waves {rec['waves']}, gap before {rec['gap_before_us']}, entries p50 {rec['entry_p50']} last {rec['entry_last']}, "
                      f"first wave -> last ack {rec['first_wave_to_last_ack_us']}", file=sys.stderr)
                for k, v in rec.items():
                    if isinstance(v, list):
                        print(f"    {k:28s} p50 {v[0]}   slowest {v[1]}", file=sys.stderr)
        return 0
    ctx, eng, ev = hip.Context(), hip.Eng(), HipEvents()
    if args.only == "copy":
        n = 16 << 20
        src, dst = ctx.buffer_f32(np.ones(n, dtype=np.float32)), ctx.buffer_empty_f32(n)
        k = ctx.compile(hip.make_desc(hip.Kind.COPY_SLICE, (n,)))
        ms = ctx.run(k, [src], [dst], iters=8)
        ctx.close()
        print(json.dumps({"copy": {"bytes_read": n * 4, "bytes_written": n * 4, "us_per_launch": round(ms * 1e3, 2)}}))
        return 0
    if args.only:
        if args.only == "cfg1":
            r = bench_lm_head(ctx, eng, ev)
        elif args.only == "floor":
            r = bench_floor(ctx, eng, ev, args.copies, args.steps, args.warmup)
        else:
            r = {"cfg2": lambda: bench_prefill(ctx), "cfg3": lambda: bench_attention(ctx, ev, sched={"lanes": dict(vec=3), "mfma": dict(vec=2)}.get(args.attn_form)),
                 "cfg4": lambda: bench_decode(ctx, eng, not args.eager),
                 "prefill": lambda: bench_prompt_pass(ctx, eng),
                 "gemma4": lambda: bench_decode_gemma4_layout(ctx, eng, not args.eager)}[args.only]()
        ctx.close()
        print(json.dumps({args.only: r}))
        return 0
    rows = cols = 4096
    w, x = synth.cfg0_q4k_matvec()
    head = bench_matvec(ctx, eng, ev, DType.Q4K, rows, cols, w, x, args.copies, args.steps, args.warmup, replays=5)
    traffic = measured_traffic(head["kernel"])      # before the minutes of secondary workloads, not after

    also = {}
    if not args.no_extras:
        hot = bench_matvec(ctx, eng, ev, DType.Q4K, rows, cols, w, x, 1, args.steps, args.warmup)
        also["cfg0_hot_cache"] = dict(us_per_launch=round(hot["us_per_launch"], 3), gbps=round(hot["gbps"], 1))
        also["cfg1_q6k_lm_head"] = bench_lm_head(ctx, eng, ev)
        also["cfg2_q4k_prefill_gemm"] = bench_prefill(ctx)
        also["cfg3_q40_attention"] = bench_attention(ctx, ev)
        also["cfg4_gemma_decode"] = bench_decode(ctx, eng)
        also["gemma4_e2b_layer_layout_decode"] = bench_decode_gemma4_layout(ctx, eng)

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
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "i8+f32", "data": "synthetic",
        "config": {"workload": "cfg0: Q4_K GEMV rows=4096 cols=4096 batch=1, f32 x/y, weights streamed from HBM "
                               f"({args.copies} rotating copies)", "kernel": head["kernel"]},
        "roofline": {"bound": "hbm", "achieved": round(head["gbps"], 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(head["gbps"] / HBM_PEAK_GBPS, 4),
                     "traffic": traffic},
        "cpu_baseline": cpu,
        "also": also,
    }
    ctx.close()
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
