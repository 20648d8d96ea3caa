"""Seeded synthetic inputs for the benchmark configurations.

Every generator takes an explicit seed and returns plain numpy arrays, so the
HIP path and the CPU checker consume byte-identical inputs.  The block layouts
are GGML's: Q4_K 256 elems / 144 B, Q6_K 256 / 210 B, Q4_0 32 / 18 B
(crates/ksearch_ir/src/lib.rs:52-74 in the ksearch tree).
"""
from __future__ import annotations

import numpy as np

Q4K_BYTES, Q6K_BYTES, Q40_BYTES = 144, 210, 18


def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def _f16_uniform(rng, n, lo, hi) -> np.ndarray:
    """n half-precision values ~U(lo, hi), as raw uint16 bit patterns."""
    return rng.uniform(lo, hi, size=n).astype(np.float32).astype(np.float16).view(np.uint16)


def q4k_blocks(n_blocks: int, seed: int) -> np.ndarray:
    """Random Q4_K superblocks: d, dmin = f16(U(1e-3,1e-2)); 12 scale bytes and
    128 quant bytes uniform over all byte values (every 6-bit field and every
    nibble is then uniform)."""
    rng = _rng(seed)
    blk = np.empty((n_blocks, Q4K_BYTES), dtype=np.uint8)
    blk[:, 0:2] = _f16_uniform(rng, n_blocks, 1e-3, 1e-2).view(np.uint8).reshape(n_blocks, 2)
    blk[:, 2:4] = _f16_uniform(rng, n_blocks, 1e-3, 1e-2).view(np.uint8).reshape(n_blocks, 2)
    blk[:, 4:] = rng.integers(0, 256, size=(n_blocks, Q4K_BYTES - 4), dtype=np.uint8)
    return blk.reshape(-1)


def q6k_blocks(n_blocks: int, seed: int) -> np.ndarray:
    """Random Q6_K superblocks: ql/qh random bytes, 16 int8 scales ~U{-32..31},
    d = f16(U(1e-3,1e-2))."""
    rng = _rng(seed)
    blk = np.empty((n_blocks, Q6K_BYTES), dtype=np.uint8)
    blk[:, :192] = rng.integers(0, 256, size=(n_blocks, 192), dtype=np.uint8)
    blk[:, 192:208] = rng.integers(-32, 32, size=(n_blocks, 16), dtype=np.int8).view(np.uint8)
    blk[:, 208:210] = _f16_uniform(rng, n_blocks, 1e-3, 1e-2).view(np.uint8).reshape(n_blocks, 2)
    return blk.reshape(-1)


def q40_blocks(n_blocks: int, seed: int) -> np.ndarray:
    """Random Q4_0 blocks: scale f16(U(0.01,0.1)) + 16 B of uniform nibbles."""
    rng = _rng(seed)
    blk = np.empty((n_blocks, Q40_BYTES), dtype=np.uint8)
    blk[:, 0:2] = _f16_uniform(rng, n_blocks, 0.01, 0.1).view(np.uint8).reshape(n_blocks, 2)
    blk[:, 2:] = rng.integers(0, 256, size=(n_blocks, 16), dtype=np.uint8)
    return blk.reshape(-1)


def normal_f32(n, seed: int, std: float = 1.0) -> np.ndarray:
    return (_rng(seed).standard_normal(size=n) * std).astype(np.float32)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """f32 -> nearest-even bf16, returned as f32 values and raw uint16 bits."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return (r.astype(np.uint32) << 16).view(np.float32), r


# -- the five benchmark configurations --------------------------------------

def cfg0_q4k_matvec(rows=4096, cols=4096, seed=1000):
    w = q4k_blocks(rows * cols // 256, seed)
    x = normal_f32(cols, seed + 1)
    return w, x


def cfg1_q6k_lm_head(rows=262144, cols=2048, seed=1001):
    w = q6k_blocks(rows * cols // 256, seed)
    x = normal_f32(cols, seed + 1)
    return w, x


def cfg2_q4k_prefill(tokens=512, rows=8192, cols=2048, seed=1002):
    w = q4k_blocks(rows * cols // 256, seed)
    xf, xb = bf16_round(normal_f32(tokens * cols, seed + 1))
    return w, xf.reshape(tokens, cols), xb.reshape(tokens, cols)


def cfg3_q40_attention(n_slots=4, n_q=8, n_kv=1, hd=256, max_t=16384, lo=1024, seed=1003):
    rng = _rng(seed)
    lens = rng.integers(lo, max_t + 1, size=n_slots).astype(np.int32)
    nblk = n_slots * max_t * n_kv * hd // 32
    k = q40_blocks(nblk, seed + 1).reshape(n_slots, -1)
    v = q40_blocks(nblk, seed + 2).reshape(n_slots, -1)
    q = normal_f32(n_slots * n_q * hd, seed + 3).reshape(n_slots, n_q * hd)
    return lens, k, v, q


GEMMA_E2B_SYNTH = dict(n_layers=30, hidden=2048, ffn=8192, n_q=8, n_kv=1, hd=256,
                       vocab=262144, max_seq=4096, eps=1e-6, softcap=30.0,
                       rope_theta=10000.0, attn_scale=1.0 / 16.0)


def chunked(quantize):
    """Lifts a host quantizer (one f32 array -> packed bytes) to the list-of-row-
    chunks form gemma_weights hands the embedding table over in."""
    return lambda parts: np.concatenate([quantize(p) for p in parts])


def gemma_weights(cfg: dict, seed: int, quantize_q4k, quantize_q6k, std: float = 0.02, threads: int = 0) -> dict:
    """N(0, std) weights packed to Q4_K (attention/FFN) and Q6_K (tied
    embedding / LM head); norm weights are 1.  The two quantizers are passed
    in by the caller (host arrays in, anything out: packed host arrays from a
    CPU routine, device buffers from the device kernels), so this module does
    not depend on where they live.  Every tensor has its own seed, so the
    result does not depend on `threads` (float generation runs in a thread
    pool; the quantizers are called from the calling thread, in order)."""
    import concurrent.futures as cf
    import os

    h, f, hd = cfg["hidden"], cfg["ffn"], cfg["hd"]
    nq, nkv = cfg["n_q"] * hd, cfg["n_kv"] * hd
    shapes = (("wq", (nq, h)), ("wk", (nkv, h)), ("wv", (nkv, h)), ("wo", (h, nq)),
              ("wgate", (f, h)), ("wup", (f, h)), ("wdown", (h, f)))
    layers = []
    s = seed
    with cf.ThreadPoolExecutor(max_workers=threads or min(16, os.cpu_count() or 1)) as ex:
        for _ in range(cfg["n_layers"]):
            futs = {}
            for name, (r, c) in shapes:
                s += 1
                futs[name] = ex.submit(normal_f32, r * c, s, std)
            lw = {name: quantize_q4k(futs[name].result()) for name, _ in shapes}
            for name, n in (("attn_norm", h), ("q_norm", hd), ("k_norm", hd),
                            ("post_attn_norm", h), ("ffn_norm", h), ("post_ffw_norm", h)):
                lw[name] = np.ones(n, dtype=np.float32)
            layers.append(lw)
        # the embedding table in row chunks, so that no single float array exceeds ~0.5 GB
        rows, chunk = cfg["vocab"], max(1, min(cfg["vocab"], (1 << 27) // h))
        futs = []
        for r0 in range(0, rows, chunk):
            s += 1
            futs.append(ex.submit(normal_f32, min(chunk, rows - r0) * h, s, std))
        embd = quantize_q6k([fu.result() for fu in futs])
    return dict(layers=layers, token_embd=embd, output_norm=np.ones(h, dtype=np.float32))


def q5k_blocks(n_blocks: int, seed: int, d_lo: float = 1e-4, d_hi: float = 1e-3) -> np.ndarray:
    """Random Q5_K superblocks (176 B): d, dmin = f16(U(d_lo, d_hi)); scales, high bits and nibbles uniform."""
    rng = _rng(seed)
    blk = np.empty((n_blocks, 176), dtype=np.uint8)
    blk[:, 0:2] = _f16_uniform(rng, n_blocks, d_lo, d_hi).view(np.uint8).reshape(n_blocks, 2)
    blk[:, 2:4] = _f16_uniform(rng, n_blocks, d_lo, d_hi).view(np.uint8).reshape(n_blocks, 2)
    blk[:, 4:] = rng.integers(0, 256, size=(n_blocks, 172), dtype=np.uint8)
    return blk.reshape(-1)


# dtype codes shared by the C ABI and the CPU checker
_Q4K, _Q5K, _Q6K = 2, 3, 4

# a small model with every layer feature of the real checkpoints: five sliding-window layers per full-attention
# layer, the last three layers reusing earlier caches, per-layer embeddings, a window shorter than the test runs
GEMMA4_TINY = dict(n_layers=8, hidden=512, n_q=4, n_kv=1, vocab=1024, max_seq=64, hd_swa=128, hd_full=256,
                   sliding_window=8, shared_kv_layers=3, ple_dim=256, eps=1e-6, softcap=30.0,
                   rope_theta_swa=10000.0, rope_theta_full=1000000.0, partial_rotary=0.25, attn_scale=1.0)


def gemma4_weights(cfg: dict, seed: int, quantize_q4k, quantize_q6k, ffn=None, swa_pattern=None, q6k_tensors=(),
                   std: float = 0.02) -> dict:
    """Weights for the Gemma-4 decode loop: N(0, std) matrices packed to Q4_K (or Q6_K for the (layer, name)
    pairs in `q6k_tensors`), the tied embedding / LM head in Q6_K, a random Q5_K per-layer-embedding table, norm
    vectors 1 + 0.1 N(0,1), layer scales in [0.5, 1.5].  `ffn` is one width or a list per layer; `swa_pattern`
    defaults to the reference's (every sixth layer attends everything, crates/ksearch_gemma/src/lib.rs:93-96)."""
    n, h, pd = cfg["n_layers"], cfg["hidden"], cfg["ple_dim"]
    ffn = [ffn or 4 * h] * n if not isinstance(ffn, (list, tuple)) else list(ffn)
    swa = list(swa_pattern) if swa_pattern is not None else [(i + 1) % 6 != 0 for i in range(n)]
    owners = n - cfg["shared_kv_layers"]
    rng = _rng(seed)
    s = seed * 1000

    def norm(k):
        return (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)

    layers = []
    for i in range(n):
        hd = cfg["hd_swa"] if swa[i] else cfg["hd_full"]
        qd, kvd = cfg["n_q"] * hd, cfg["n_kv"] * hd
        shapes = [("wq", "dt_q", qd, h), ("wo", "dt_o", h, qd), ("wgate", "dt_gate", ffn[i], h),
                  ("wup", "dt_up", ffn[i], h), ("wdown", "dt_down", h, ffn[i])]
        if i < owners:
            shapes += [("wk", "dt_k", kvd, h), ("wv", "dt_v", kvd, h)]
        if pd:
            shapes += [("inp_gate", "dt_inp_gate", pd, h), ("proj", "dt_proj", h, pd)]
        lw = dict(is_swa=int(swa[i]), ffn=ffn[i], layer_scale=float(rng.uniform(0.5, 1.5)))
        for name, dt, r, c in shapes:
            s += 1
            x = normal_f32(r * c, s, std)
            six = (i, name) in q6k_tensors
            lw[name] = quantize_q6k(x) if six else quantize_q4k(x)
            lw[dt] = _Q6K if six else _Q4K
        for name, k in (("attn_norm", h), ("q_norm", hd), ("k_norm", hd), ("post_attn_norm", h), ("ffn_norm", h),
                        ("post_ffw_norm", h), ("post_norm", h)):
            lw[name] = norm(k)
        layers.append(lw)
    g = dict(token_embd=quantize_q6k(normal_f32(cfg["vocab"] * h, s + 1, std)), dt_embd=_Q6K, output_norm=norm(h))
    if pd:
        pt = n * pd
        g.update(ple_embd=q5k_blocks(cfg["vocab"] * pt // 256, s + 2), dt_ple=_Q5K,
                 ple_model_proj=quantize_q4k(normal_f32(pt * h, s + 3, std)), dt_ple_proj=_Q4K, ple_proj_norm=norm(pd))
    return dict(layers=layers, globals=g)
