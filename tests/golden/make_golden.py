#!/usr/bin/env python3
"""Writes the committed fixtures under tests/golden/ from the CPU oracle.

    python tests/golden/make_golden.py            # small.npz (seconds)
    python tests/golden/make_golden.py --cfg4     # + cfg4_tokens.json (minutes: full-size CPU decode)
    python tests/golden/make_golden.py --gemma4   # gemma4_small.npz only (seconds)

The reference ships no golden vectors for this path (its kernel checks only
print statistics), so these are the oracle's outputs on seeded inputs, kept as
data: inputs and expected outputs only.  They guard the oracle against
regressions and give the HIP path fixed vectors to be compared with.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from ksearch_amd import synth  # noqa: E402


def small():
    out = {}
    edge4 = np.zeros((3, 144), dtype=np.uint8)
    edge4[1, 4:] = 0xFF
    edge4[1, 0:4] = np.array([2.0, 0.5], dtype=np.float16).view(np.uint8)
    edge4[2] = np.arange(144, dtype=np.uint8)
    q4 = np.concatenate([edge4.reshape(-1), synth.q4k_blocks(5, 9001)])
    q6 = synth.q6k_blocks(6, 9002)
    q0 = synth.q40_blocks(24, 9003)
    out["q4k_blocks"], out["q4k_deq"] = q4, oracle.dequant(oracle.Q4K, q4, 8 * 256)
    out["q6k_blocks"], out["q6k_deq"] = q6, oracle.dequant(oracle.Q6K, q6, 6 * 256)
    out["q40_blocks"], out["q40_deq"] = q0, oracle.dequant(oracle.Q40, q0, 24 * 32)
    x = synth.normal_f32(512, 9004)
    w4, w6 = synth.q4k_blocks(8 * 2, 9005), synth.q6k_blocks(8 * 2, 9006)
    out["gemv_x"] = x
    out["gemv_q4k_w"], out["gemv_q4k_y"] = w4, oracle.matvec(oracle.Q4K, w4, 8, 512, x)
    out["gemv_q6k_w"], out["gemv_q6k_y"] = w6, oracle.matvec(oracle.Q6K, w6, 8, 512, x)
    n_q, hd, nt = 2, 64, 40
    k, v = synth.q40_blocks(nt * hd // 32, 9007), synth.q40_blocks(nt * hd // 32, 9008)
    q = synth.normal_f32(n_q * hd, 9009)
    out["attn_q"], out["attn_k"], out["attn_v"] = q, k, v
    out["attn_out"] = oracle.sdpa(q, k, v, n_q, 1, hd, nt, 0, 0.125)
    out["rope_row_pos7_hd64"] = oracle.rope_table(8, 64, 10000.0)[7]
    pk = synth.normal_f32(32 * 6, 9010)
    out["pack_src"], out["pack_q40"] = pk, oracle.pack_q40(pk)
    qz = synth.normal_f32(512, 9011, std=0.02)
    out["quant_src"], out["quant_q4k"], out["quant_q6k"] = qz, oracle.quantize_q4k(qz), oracle.quantize_q6k(qz)
    out["argmax_x"] = synth.normal_f32(1000, 9012)
    out["argmax_idx"] = np.array([oracle.softcap_argmax(out["argmax_x"], 30.0)], dtype=np.int64)
    np.savez_compressed(os.path.join(HERE, "small.npz"), **out)
    print("wrote small.npz", {k_: v_.shape for k_, v_ in out.items()})


G4_PATTERN = [1, 1, 0, 1, 1, 1, 0, 1]
G4_FFN = [1024, 1024, 2048, 1024, 1024, 1024, 2048, 1024]
G4_Q6K = ((1, "wv"), (2, "wdown"), (4, "wgate"))


def gemma4_tiny_weights():
    return synth.gemma4_weights(dict(synth.GEMMA4_TINY), 9100, oracle.quantize_q4k, oracle.quantize_q6k, ffn=G4_FFN,
                                swa_pattern=G4_PATTERN, q6k_tensors=set(G4_Q6K), std=0.05)


def gemma4():
    """gemma4_small.npz: the ops and the loop that the real checkpoints add (Q5_K, per-head norm + RoPE,
    gelu(Wx)*ctx, the tiny 8-layer model with both layer kinds, shared caches and per-layer embeddings)."""
    out = {}
    q5 = synth.q5k_blocks(6, 9101, 1e-3, 1e-2)
    out["q5k_blocks"], out["q5k_deq"] = q5, oracle.dequant(oracle.Q5K, q5, 6 * 256)
    x, w = synth.normal_f32(3 * 128, 9102), 1.0 + 0.2 * synth.normal_f32(128, 9103)
    rope = oracle.rope_table(6, 128, 10000.0, 16)[5]
    out["ph_x"], out["ph_w"], out["ph_rope"] = x, w, rope
    out["ph_norm"], out["ph_rope_out"] = oracle.rmsnorm_per_head(x, w, 3, 128, 1e-6), oracle.rmsnorm_per_head(x, w, 3, 128, 1e-6, rope)
    wg, xg, cg = synth.q4k_blocks(16 * 2, 9104), synth.normal_f32(512, 9105), synth.normal_f32(16, 9106)
    out["gm_w"], out["gm_x"], out["gm_ctx"], out["gm_y"] = wg, xg, cg, oracle.matvec_gelu_mul(oracle.Q4K, wg, 16, 512, xg, cg)
    cfg = dict(synth.GEMMA4_TINY)
    m = oracle.Gemma4(cfg, gemma4_tiny_weights())
    # teacher-forced on random ids (the free-running model settles on one token): 20 positions, past the window of 8
    prompt = [int(t) for t in np.random.default_rng(9107).integers(0, cfg["vocab"], 20)]
    toks, top, margin = [], [], []
    for t in prompt:
        tok, lg = m.forward(t, return_logits=True)
        s2 = np.sort(lg)[-2:]
        toks.append(tok)
        top.append(float(s2[1]))
        margin.append(float((s2[1] - s2[0]) / max(abs(s2[1]), 1e-6)))
    out["g4_prompt"], out["g4_tokens"] = np.array(prompt, np.int64), np.array(toks, np.int64)
    out["g4_top_logit"], out["g4_margin"] = np.array(top, np.float32), np.array(margin, np.float32)
    out["g4_hidden"] = m.hidden()
    out["g4_kv_source"] = np.array([m.kv_source(l) for l in range(cfg["n_layers"])], np.int64)
    np.savez_compressed(os.path.join(HERE, "gemma4_small.npz"), **out)
    print("wrote gemma4_small.npz", {k_: v_.shape for k_, v_ in out.items()})


CFG4_SEED, PROMPT_SEED, N_PROMPT, N_NEW, KV_STEPS = 4000, 4001, 64, 256, 40


def cfg4(n_new=N_NEW):
    cfg = synth.GEMMA_E2B_SYNTH
    t0 = time.time()
    w = synth.gemma_weights(cfg, CFG4_SEED, oracle.quantize_q4k, synth.chunked(oracle.quantize_q6k))
    print(f"weights packed in {time.time() - t0:.0f}s", flush=True)
    prompt = [int(t) for t in np.random.default_rng(PROMPT_SEED).integers(0, cfg["vocab"], N_PROMPT)]
    m = oracle.Gemma(cfg, w)

    def record(lg, rec):
        idx = np.argpartition(lg, -8)[-8:]
        idx = idx[np.argsort(-lg[idx], kind="stable")]
        rec["top8_idx"].append([int(i) for i in idx])
        rec["top8_val"].append([float(lg[i]) for i in idx])
        rec["rms"].append(float(np.sqrt(np.mean(lg.astype(np.float64) ** 2))))

    # teacher-forced part: the random prompt, with logits at every position
    forced = dict(argmax=[], top8_idx=[], top8_val=[], rms=[])
    row = cfg["n_kv"] * cfg["hd"] // 32 * 18
    kv_rows = np.zeros((KV_STEPS, cfg["n_layers"], 2, row), dtype=np.uint8)
    for i, t in enumerate(prompt[:-1]):
        nxt, lg = m.forward(t, return_logits=True)
        forced["argmax"].append(int(nxt))
        record(lg, forced)
        if i < KV_STEPS:      # the Q4_0 rows this step appended, every layer, K and V
            for l in range(cfg["n_layers"]):
                for which in (0, 1):
                    kv_rows[i, l, which] = m.kv(l, which, (i + 1) * row)[i * row:]
    np.savez_compressed(os.path.join(HERE, "cfg4_kv.npz"), kv_rows=kv_rows)
    toks, margins, top = [], [], []
    free = dict(top8_idx=[], top8_val=[], rms=[])
    t = prompt[-1]
    for i in range(n_new):
        t, lg = m.forward(t, return_logits=True)
        s = np.partition(lg, -2)[-2:]
        margins.append(float(abs(s[1] - s[0])))
        top.append(float(lg.max()))
        toks.append(int(t))
        if i < 32:
            record(lg, free)
        if i % 16 == 0:
            print(f"token {i}: {t} margin {margins[-1]:.3e} ({time.time() - t0:.0f}s)", flush=True)
    json.dump(dict(config=cfg, weight_seed=CFG4_SEED, prompt_seed=PROMPT_SEED, prompt=prompt, tokens=toks,
                   top2_margin=margins, top_logit=top, forced=forced, free=free), open(os.path.join(HERE, "cfg4_tokens.json"), "w"))
    print("wrote cfg4_tokens.json")


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--cfg4", action="store_true")
    ap.add_argument("--gemma4", action="store_true")
    ap.add_argument("--n-new", type=int, default=N_NEW)
    a = ap.parse_args()
    if a.gemma4:
        gemma4()
    else:
        small()
        if a.cfg4:
            cfg4(a.n_new)
