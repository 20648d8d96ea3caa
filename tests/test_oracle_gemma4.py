"""Pins the oracle's restatement of the ops and layer rules that the real Gemma-4 checkpoints add to the decode
step: Q5_K dequant, per-head RMSNorm (+RoPE), add_scale, the gelu(.)*ctx GEMV, kv_source, and the whole-model loop
(against the already-pinned loop for the synthetic shape, which it must reduce to when the extras are off)."""
import numpy as np

import oracle
from ksearch_amd import synth
from tests.gpu_util import assert_close
from tests.refforms import half_bits_to_f64, scale_min_k4_bitfield


def q5k_elementwise(blk: np.ndarray) -> np.ndarray:
    """The per-element formulation the reference's GPU helper uses (crates/ksearch_codegen/src/render.rs:695-724),
    restated independently of the block loop the oracle follows: group g = j/64, low nibbles for j%64 < 32, the
    fifth bit of element (g, low/high) is bit 2g / 2g+1 of qh[j%32]."""
    d, dmin = (np.float32(v) for v in half_bits_to_f64(blk[:4].view(np.uint16)))
    sc, mn = scale_min_k4_bitfield(blk[4:16])
    qh, qs = blk[16:48], blk[48:176]
    out = np.empty(256, np.float32)
    for j in range(256):
        g, jl = j // 64, j % 64
        l, hi_half = jl % 32, jl >= 32
        sub = 2 * g + int(hi_half)
        nib = (int(qs[32 * g + l]) >> 4) if hi_half else (int(qs[32 * g + l]) & 15)
        bit = 16.0 if (int(qh[l]) >> sub) & 1 else 0.0
        out[j] = np.float32(d * np.float32(sc[sub])) * np.float32(np.float32(nib) + np.float32(bit)) - np.float32(dmin * np.float32(mn[sub]))
    return out


def test_q5k_dequant_two_formulations_bit_exact():
    blocks = synth.q5k_blocks(24, 11, 1e-3, 1e-2).reshape(24, 176)
    got = oracle.dequant(oracle.Q5K, blocks.reshape(-1), 24 * 256).reshape(24, 256)
    for b in range(24):
        assert np.array_equal(got[b], q5k_elementwise(blocks[b])), b


def test_q5k_special_cases():
    """With every fifth bit clear a Q5_K block is the Q4_K block of the same header, scales and nibbles; with
    every fifth bit set each element gains exactly 16*d*sc of its sub-block."""
    rng = np.random.default_rng(12)
    q4 = synth.q4k_blocks(6, 13).reshape(6, 144)
    q5 = np.zeros((6, 176), np.uint8)
    q5[:, :16], q5[:, 48:] = q4[:, :16], q4[:, 16:]
    base = oracle.dequant(oracle.Q4K, q4.reshape(-1), 6 * 256)
    assert np.array_equal(oracle.dequant(oracle.Q5K, q5.reshape(-1), 6 * 256), base)
    q5[:, 16:48] = 0xFF
    full = oracle.dequant(oracle.Q5K, q5.reshape(-1), 6 * 256).reshape(6, 8, 32)
    for b in range(6):
        d = float(half_bits_to_f64(q4[b, :2].view(np.uint16))[0])
        dmin = float(half_bits_to_f64(q4[b, 2:4].view(np.uint16))[0])
        sc, mn = scale_min_k4_bitfield(q4[b, 4:16])
        for sub in range(8):
            g, hi = sub // 2, sub % 2
            nib = (q4[b, 16 + 32 * g:48 + 32 * g] >> 4) if hi else (q4[b, 16 + 32 * g:48 + 32 * g] & 15)
            want = d * sc[sub] * (nib.astype(np.float64) + 16.0) - dmin * mn[sub]
            assert np.abs(full[b, sub] - want).max() <= 1e-6 * max(1.0, np.abs(want).max())
    # a single set bit moves one element only
    q5[:, 16:48] = 0
    q5[0, 16 + 5] = 1 << 3          # element l=5 of sub-block 3 (group 1, high nibbles)
    one = oracle.dequant(oracle.Q5K, q5.reshape(-1), 6 * 256)
    changed = np.nonzero(one != base)[0]
    assert list(changed) == [3 * 32 + 5]
    del rng


def test_rmsnorm_per_head_closed_forms():
    rng = np.random.default_rng(14)
    for n_heads, hd in ((3, 64), (8, 256), (2, 512)):
        x = rng.standard_normal(n_heads * hd).astype(np.float32) * 3
        w = (1 + 0.2 * rng.standard_normal(hd)).astype(np.float32)
        eps = 1e-6
        x64 = x.astype(np.float64).reshape(n_heads, hd)
        want = x64 / np.sqrt((x64 ** 2).mean(1, keepdims=True) + eps) * w
        assert_close(oracle.rmsnorm_per_head(x, w, n_heads, hd, eps), want, 1e-6, "norm")
        # RoPE: position 0 is the identity; any row is a rotation of the pairs (i, i + hd/2)
        tab = oracle.rope_table(5, hd, 10000.0)
        assert np.array_equal(oracle.rmsnorm_per_head(x, w, n_heads, hd, eps, tab[0]), oracle.rmsnorm_per_head(x, w, n_heads, hd, eps))
        got = oracle.rmsnorm_per_head(x, w, n_heads, hd, eps, tab[3]).astype(np.float64).reshape(n_heads, hd)
        half = hd // 2
        c, s = tab[3, :half].astype(np.float64), tab[3, half:].astype(np.float64)
        rot = np.concatenate([want[:, :half] * c - want[:, half:] * s, want[:, :half] * s + want[:, half:] * c], axis=1)
        assert_close(got, rot, 1e-5, "rope")
        assert_close((got ** 2).sum(1), (want ** 2).sum(1), 1e-5, "rotation keeps the norm")
        # the query half of the pinned QKV op is the same function
        q_ref, _, _ = oracle.rmsnorm_per_head_qkv_q40(x, w, tab[3], x[:hd], w, x[:hd], n_heads, 1, hd, eps)
        assert np.array_equal(q_ref, got.astype(np.float32).ravel())


def test_add_scale_and_gelu_mul_gemv():
    rng = np.random.default_rng(15)
    a, b = rng.standard_normal(1000).astype(np.float32), rng.standard_normal(1000).astype(np.float32)
    assert np.array_equal(oracle.add_scale(a, b, 0.5), np.float32(0.5) * (a + b))
    rows, cols = 64, 512
    w = synth.q4k_blocks(rows * cols // 256, 16)
    x, ctx = rng.standard_normal(cols).astype(np.float32), rng.standard_normal(rows).astype(np.float32)
    dot = oracle.matvec_f64(oracle.Q4K, w, rows, cols, x)
    ax = np.clip(dot, -20, 20)
    want = 0.5 * ax * (1 + np.tanh(np.sqrt(2 / np.pi) * (ax + 0.044715 * ax ** 3))) * ctx
    assert_close(oracle.matvec_gelu_mul(oracle.Q4K, w, rows, cols, x, ctx), want, 1e-4, "gelu(Wx)*ctx")
    # ctx = 1 and a tiny dot: gelu(z) ~ z/2
    tiny = oracle.matvec_gelu_mul(oracle.Q4K, w, rows, cols, x * np.float32(1e-6), np.ones(rows, np.float32))
    assert_close(tiny, 0.5 * dot * 1e-6, 1e-3, "gelu near 0")


def kv_source_rule(n_layers, shared, swa, layer):
    """crates/ksearch_gemma/src/lib.rs:147-162 restated."""
    owns = lambda i: i < max(n_layers - shared, 0)
    if owns(layer):
        return layer
    for i in range(layer - 1, -1, -1):
        if owns(i) and swa[i] == swa[layer]:
            return i
    return 0


def tiny_weights(cfg, seed, **kw):
    return synth.gemma4_weights(cfg, seed, oracle.quantize_q4k, oracle.quantize_q6k, **kw)


def test_kv_source_follows_the_layer_rule():
    cfg = dict(synth.GEMMA4_TINY, n_layers=12, shared_kv_layers=5, ple_dim=0, vocab=256)
    w = tiny_weights(cfg, 17, ffn=256)
    m = oracle.Gemma4(cfg, w)
    swa = [bool(l["is_swa"]) for l in w["layers"]]
    assert swa == [True] * 5 + [False] + [True] * 5 + [False]
    assert [m.kv_source(l) for l in range(12)] == [kv_source_rule(12, 5, swa, l) for l in range(12)]
    assert [m.kv_source(l) for l in range(12)] == [0, 1, 2, 3, 4, 5, 6, 6, 6, 6, 6, 5]
    m.close()


def test_gemma4_loop_reduces_to_the_plain_loop():
    """No per-layer embeddings, no shared caches, every layer a sliding-window layer whose window covers the
    whole run: the same tokens, logits and caches as the loop for the synthetic shape."""
    base = dict(n_layers=3, hidden=512, ffn=1024, n_q=4, n_kv=1, hd=128, vocab=512, max_seq=160, eps=1e-6, softcap=30.0,
                rope_theta=10000.0, attn_scale=1.0 / np.sqrt(128.0))
    w = synth.gemma_weights(base, 18, oracle.quantize_q4k, synth.chunked(oracle.quantize_q6k), std=0.05)
    rng = np.random.default_rng(19)
    for lw in w["layers"]:
        for name in ("attn_norm", "q_norm", "k_norm", "post_attn_norm", "ffn_norm", "post_ffw_norm"):
            lw[name] = (1.0 + 0.2 * rng.standard_normal(lw[name].size)).astype(np.float32)
    cfg4 = dict(n_layers=3, hidden=512, n_q=4, n_kv=1, vocab=512, max_seq=160, hd_swa=128, hd_full=256, sliding_window=160,
                shared_kv_layers=0, ple_dim=0, eps=1e-6, softcap=30.0, rope_theta_swa=10000.0, rope_theta_full=1e6,
                partial_rotary=0.25, attn_scale=base["attn_scale"])
    w4 = dict(layers=[dict(lw, is_swa=1, ffn=1024, layer_scale=1.0) for lw in w["layers"]],
              globals=dict(token_embd=w["token_embd"], dt_embd=oracle.Q6K, output_norm=w["output_norm"]))
    a, b = oracle.Gemma(base, w), oracle.Gemma4(cfg4, w4)
    tok_a = tok_b = 5
    for step in range(140):       # crosses the 128-row switch to the split-KV form
        tok_a, la = a.forward(tok_a, return_logits=True)
        tok_b, lb = b.forward(tok_b, return_logits=True)
        assert tok_a == tok_b and np.array_equal(la, lb), step
    row = 128 // 32 * 18
    for l in range(3):
        for which in (0, 1):
            assert np.array_equal(a.kv(l, which, 140 * row), b.kv(l, which, 140 * row))
    a.close()
    b.close()


def test_gemma4_window_and_shared_cache_semantics():
    """A sliding-window layer sees exactly the last `window` rows: with the window at least as long as the run the
    model equals the same model with a huge window, and differs once the run outgrows it.  A layer that reuses a
    cache appends nothing of its own."""
    cfg = dict(synth.GEMMA4_TINY, vocab=256)
    pattern = [1, 1, 0, 1, 1, 1, 0, 1]
    w = tiny_weights(cfg, 20, ffn=512, swa_pattern=pattern)
    wide = oracle.Gemma4(dict(cfg, sliding_window=64), w)
    tight = oracle.Gemma4(cfg, w)
    assert [tight.kv_source(l) for l in range(8)] == [0, 1, 2, 3, 4, 4, 2, 4]
    same = []
    tok = 9
    for step in range(14):
        nxt, l1 = wide.forward(tok, return_logits=True)
        _, l2 = tight.forward(tok, return_logits=True)   # teacher-forced on the wide model's tokens
        same.append(np.array_equal(l1, l2))
        tok = nxt
    # identical while kv_len <= window (8 positions), different afterwards
    assert all(same[:8]) and not any(same[8:])
    wide.close()
    tight.close()
