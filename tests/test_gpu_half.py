"""Half-precision activations at the boundary (descriptor dtypes[1] = F16): the reference's runtime keeps activations,
norm weights and logits in half buffers (crates/ksearch_codegen/src/lower.rs:1134-1140,
crates/ksearch_gemma/src/gemma_prim.rs:164-182, 229-252) and its kernels compute in f32.

Two kinds of check, both through the C ABI:
  - against the oracle: inputs rounded to half, the oracle run on exactly those values, its result rounded to half
    (round to nearest even); the device's half output must be within the parity bar of 1e-3 plus half an ulp of
    half (2^-11: a result next to a rounding boundary may land on either side);
  - against the f32 handle of the same descriptor on the widened inputs: bit-identical after rounding, for every kind
    that takes half activations (what is not an activation -- packed weights and caches, rope table, meta record,
    token ids, split-KV partials, argmax index -- keeps its type)."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip, synth
from ksearch_amd.hip import DType, Kind
from tests.gpu_util import rel_err

pytestmark = pytest.mark.gpu
BAR = 1e-3 + 2.0 ** -11


@pytest.fixture(scope="module")
def ctx():
    c = hip.Context()
    yield c
    c.close()


def halfed(a):
    """f32 values that are exactly representable in half"""
    return np.asarray(a, np.float32).astype(np.float16).astype(np.float32)


def run(ctx, kind, dims, dtypes, params, ins, outs, half):
    """ins: (array, cls); outs: (n_elems or n_bytes, cls).  cls 'A' activation (f32 values; bound as half when `half`),
    'F' f32, 'W' bytes.  Returns the outputs ('A' and 'F' as f32 arrays, 'W' as bytes)."""
    dt = list(dtypes) + [0] * (4 - len(dtypes))
    dt[1] = DType.F16 if half else DType.F32
    if half and kind == Kind.MATVEC_BATCH:
        dt[2] = DType.F16
    k = ctx.compile(hip.make_desc(kind, dims, dt, params))
    bi = []
    for arr, cls in ins:
        if cls == "A" and half:
            bi.append(ctx.buffer_bytes(np.asarray(arr, np.float32).astype(np.float16).view(np.uint8)))
        elif cls == "W":
            bi.append(ctx.buffer_bytes(np.asarray(arr, np.uint8)))
        else:
            bi.append(ctx.buffer_f32(np.asarray(arr, np.float32)))
    bo = []
    for n, cls in outs:
        bo.append(ctx.buffer_empty_bytes(n * (2 if (cls == "A" and half) else 4 if cls != "W" else 1)))
    ctx.encode_multi(k, bi, bo)
    res = []
    for (n, cls), b in zip(outs, bo):
        if cls == "W":
            res.append(ctx.read_bytes(b, n))
        elif cls == "A" and half:
            res.append(ctx.read_bytes(b, 2 * n).view(np.float16).astype(np.float32))
        else:
            res.append(ctx.read_f32(b, n))
    return res, k


def both(ctx, kind, dims, dtypes, params, ins, outs):
    """The half handle against the f32 handle on the same (half-representable) values: equal after rounding."""
    h, kh = run(ctx, kind, dims, dtypes, params, ins, outs, True)
    f, _ = run(ctx, kind, dims, dtypes, params, ins, outs, False)
    assert kh.name.endswith("_f16")
    for i, ((n, cls), a, b) in enumerate(zip(outs, h, f)):
        if cls == "A":
            assert np.array_equal(a.view(np.uint32), b.astype(np.float16).astype(np.float32).view(np.uint32)), f"{kh.name}: output {i}"
        else:
            assert np.array_equal(a, b), f"{kh.name}: output {i} (not an activation) differs"
    return h


@pytest.mark.parametrize("wdt,rows,cols", [(DType.Q4K, 512, 4096), (DType.Q4K, 300, 2048), (DType.Q6K, 700, 2048)])
def test_matvec_half_against_oracle(ctx, wdt, rows, cols):
    w, x = (synth.cfg0_q4k_matvec if wdt == DType.Q4K else synth.cfg1_q6k_lm_head)(rows, cols, seed=71)
    x = halfed(x)
    (y,) = both(ctx, Kind.MATVEC, (rows, cols), (wdt,), (), [(w, "W"), (x, "A")], [(rows, "A")])
    want = oracle.matvec(oracle.Q4K if wdt == DType.Q4K else oracle.Q6K, w, rows, cols, x).astype(np.float16).astype(np.float32)
    assert rel_err(y, want).max() <= BAR


def test_norms_gelu_and_argmax_half_against_oracle(ctx):
    n, eps = 2048, 1e-6
    x, w, r, w2 = (halfed(synth.normal_f32(n, 720 + i)) for i in range(4))
    (y,) = both(ctx, Kind.RMSNORM, (n, 0, 0), (), (eps,), [(x, "A"), (w, "A")], [(n, "A")])
    assert rel_err(y, oracle.rmsnorm(x, w, eps).astype(np.float16).astype(np.float32)).max() <= BAR
    (y,) = both(ctx, Kind.RMSNORM, (n, 1, 1), (), (eps, 0.25), [(x, "A"), (w, "A"), (r, "A")], [(n, "A")])
    assert rel_err(y, oracle.rmsnorm(x, w, eps, res=r, scale=0.25).astype(np.float16).astype(np.float32)).max() <= BAR
    o1, o2 = both(ctx, Kind.RMSNORM_ADD_THEN_RMSNORM, (n,), (), (eps,), [(x, "A"), (w, "A"), (r, "A"), (w2, "A")], [(n, "A"), (n, "A")])
    w1, w2_ = oracle.rmsnorm_add_then_rmsnorm(x, w, r, w2, eps)
    assert rel_err(o1, w1.astype(np.float16).astype(np.float32)).max() <= BAR
    assert rel_err(o2, w2_.astype(np.float16).astype(np.float32)).max() <= BAR
    g, u = halfed(3 * synth.normal_f32(n, 725)), halfed(synth.normal_f32(n, 726))
    (y,) = both(ctx, Kind.GELU_MUL, (n,), (), (), [(g, "A"), (u, "A")], [(n, "A")])
    assert rel_err(y, oracle.gelu_mul(g, u).astype(np.float16).astype(np.float32)).max() <= BAR
    (y,) = both(ctx, Kind.ADD_SCALE, (n,), (), (0.5,), [(x, "A"), (r, "A")], [(n, "A")])
    assert rel_err(y, oracle.add_scale(x, r, 0.5).astype(np.float16).astype(np.float32)).max() <= BAR
    # logits in half, the index in f32 (the reference reads it with read_f32)
    logits = halfed(8 * synth.normal_f32(50001, 727))
    (idx,) = both(ctx, Kind.SOFTCAP_ARGMAX, (logits.size,), (), (30.0,), [(logits, "A")], [(1, "F")])
    assert int(idx[0]) == oracle.softcap_argmax(logits, 30.0)


def test_fused_norm_gemvs_half_against_oracle(ctx):
    hidden, ffn, qd, kvd, eps = 2048, 1024, 512, 256, 1e-6
    y, wn, wp, res = (halfed(synth.normal_f32(hidden, 730 + i)) for i in range(4))
    wq, _ = synth.cfg0_q4k_matvec(qd, hidden, seed=734)
    wk, _ = synth.cfg0_q4k_matvec(kvd, hidden, seed=735)
    wv, _ = synth.cfg0_q4k_matvec(kvd, hidden, seed=736)
    x_new, h = oracle.rmsnorm_add_then_rmsnorm(y, wp, res, wn, eps)
    q, k, v, xo = both(ctx, Kind.RMSNORM_MATVEC_QKV, (qd, kvd, hidden, 1), (DType.Q4K,), (eps,),
                       [(wq, "W"), (wk, "W"), (wv, "W"), (y, "A"), (wn, "A"), (wp, "A"), (res, "A")],
                       [(qd, "A"), (kvd, "A"), (kvd, "A"), (hidden, "A")])
    for got, wmat, rows in ((q, wq, qd), (k, wk, kvd), (v, wv, kvd)):
        want = oracle.matvec(oracle.Q4K, wmat, rows, hidden, h).astype(np.float16).astype(np.float32)
        assert rel_err(got, want).max() <= BAR
    assert rel_err(xo, x_new.astype(np.float16).astype(np.float32)).max() <= BAR
    wg, _ = synth.cfg0_q4k_matvec(ffn, hidden, seed=737)
    wu, _ = synth.cfg0_q4k_matvec(ffn, hidden, seed=738)
    hn = oracle.rmsnorm(y, wn, eps)
    (ff,) = both(ctx, Kind.RMSNORM_MATVEC_GATE_UP_GELU, (ffn, hidden, 0), (DType.Q4K,), (eps,),
                 [(wg, "W"), (wu, "W"), (y, "A"), (wn, "A")], [(ffn, "A")])
    want = oracle.gelu_mul(oracle.matvec(oracle.Q4K, wg, ffn, hidden, hn), oracle.matvec(oracle.Q4K, wu, ffn, hidden, hn))
    assert rel_err(ff, want.astype(np.float16).astype(np.float32)).max() <= BAR
    # the plain fused kinds and the LM-head form over Q6_K
    both(ctx, Kind.MATVEC_QKV, (qd, kvd, hidden), (DType.Q4K,), (), [(wq, "W"), (wk, "W"), (wv, "W"), (y, "A")], [(qd, "A"), (kvd, "A"), (kvd, "A")])
    both(ctx, Kind.MATVEC_GATE_UP_GELU, (ffn, hidden), (DType.Q4K,), (), [(wg, "W"), (wu, "W"), (y, "A")], [(ffn, "A")])
    w6, _ = synth.cfg1_q6k_lm_head(1024, hidden, seed=739)
    (lg,) = both(ctx, Kind.RMSNORM_MATVEC, (1024, hidden, 0), (DType.Q6K,), (eps,), [(w6, "W"), (y, "A"), (wn, "A")], [(1024, "A")])
    assert rel_err(lg, oracle.matvec(oracle.Q6K, w6, 1024, hidden, hn).astype(np.float16).astype(np.float32)).max() <= BAR


def kv_cache(rng, max_t, n_kv, hd):
    nb = max_t * n_kv * hd // 32
    blocks = np.zeros((nb, 18), np.uint8)
    blocks[:, :2] = rng.uniform(0.01, 0.1, nb).astype(np.float16).view(np.uint8).reshape(nb, 2)
    blocks[:, 2:] = rng.integers(0, 256, (nb, 16), dtype=np.uint8)
    return blocks.reshape(-1)


def test_attention_kinds_half_against_oracle(ctx):
    n_q, n_kv, hd, max_t, tlen, eps = 8, 1, 256, 512, 300, 1e-6
    rng = np.random.default_rng(740)
    kc, vc = kv_cache(rng, max_t, n_kv, hd), kv_cache(rng, max_t, n_kv, hd)
    q = halfed(synth.normal_f32(n_q * hd, 741))
    meta = np.array([tlen, 0, 0, tlen - 1], np.float32)
    want = oracle.sdpa(q, kc, vc, n_q, n_kv, hd, tlen, 0, 1.0 / 16).astype(np.float16).astype(np.float32)
    (o,) = both(ctx, Kind.SDPA_NAIVE, (n_q, n_kv, hd, max_t), (DType.Q40,), (1.0 / 16,), [(q, "A"), (kc, "W"), (vc, "W"), (meta, "F")], [(n_q * hd, "A")])
    assert rel_err(o, want).max() <= BAR
    nwg = 8
    tmp, o = both(ctx, Kind.SDPA_SLOTS, (n_q, n_kv, hd, max_t, 1, nwg), (DType.Q40,), (1.0 / 16,),
                  [(q, "A"), (kc, "W"), (vc, "W"), (meta, "F")], [(n_q * nwg * (hd + 2), "F"), (n_q * hd, "A")])
    assert rel_err(o, want).max() <= BAR
    # the reference's two passes: partials stay f32, the reduce's output is half
    (parts,) = both(ctx, Kind.SDPA_MWG_PART, (n_q, n_kv, hd, max_t, 16), (DType.Q40,), (1.0 / 16,),
                    [(q, "A"), (kc, "W"), (vc, "W"), (meta, "F")], [(n_q * 16 * (hd + 2), "F")])
    (o,) = both(ctx, Kind.SDPA_MWG_REDUCE, (n_q, hd, 16), (), (), [(parts, "F")], [(n_q * hd, "A")])
    assert rel_err(o, want).max() <= BAR
    # per-head norm + RoPE + Q4_0 append: q out in half, the packed rows are bytes as ever
    k, v = halfed(synth.normal_f32(n_kv * hd, 742)), halfed(synth.normal_f32(n_kv * hd, 743))
    qw, kw = halfed(1 + 0.2 * synth.normal_f32(hd, 744)), halfed(1 + 0.2 * synth.normal_f32(hd, 745))
    rope = oracle.rope_table(64, hd, 10000.0)
    row = n_kv * hd // 32 * 18
    qo, krow, vrow = both(ctx, Kind.RMSNORM_PER_HEAD_QKV_Q40, (n_q, n_kv, hd, 0), (), (eps,),
                          [(q, "A"), (qw, "A"), (rope[7], "F"), (k, "A"), (kw, "A"), (v, "A")], [(n_q * hd, "A"), (row, "W"), (row, "W")])
    wq_, wk_, wv_ = oracle.rmsnorm_per_head_qkv_q40(q, qw, rope[7], k, kw, v, n_q, n_kv, hd, eps)
    assert rel_err(qo, wq_.astype(np.float16).astype(np.float32)).max() <= BAR
    assert np.array_equal(krow, wk_) and np.array_equal(vrow, wv_)
    (y,) = both(ctx, Kind.RMSNORM_PER_HEAD, (n_q, hd, 1), (), (eps,), [(q, "A"), (qw, "A"), (rope[7], "F")], [(n_q * hd, "A")])
    assert rel_err(y, oracle.rmsnorm_per_head(q, qw, n_q, hd, eps, rope_row=rope[7]).astype(np.float16).astype(np.float32)).max() <= BAR


def test_decode_step_kinds_half_equal_f32_handles(ctx):
    """The library's fused decode-step kinds with half activations: equal to their f32 handles on the widened inputs."""
    n_q, n_kv, hd, max_seq, eps, pos = 8, 1, 256, 128, 1e-6, 40
    rng = np.random.default_rng(750)
    kc, vc = kv_cache(rng, max_seq, n_kv, hd), kv_cache(rng, max_seq, n_kv, hd)
    q, k, v = (halfed(synth.normal_f32(r * hd, 751 + i)) for i, r in enumerate((n_q, n_kv, n_kv)))
    qw, kw = halfed(1 + 0.2 * synth.normal_f32(hd, 754)), halfed(1 + 0.2 * synth.normal_f32(hd, 755))
    rope = oracle.rope_table(max_seq, hd, 10000.0)
    meta = np.array([pos + 1, 0, 0, pos], np.float32)
    row = n_kv * hd // 32 * 18
    nwg = 8
    ins = [(q, "A"), (qw, "A"), (rope[pos], "F"), (k, "A"), (kw, "A"), (v, "A"), (meta, "F")]
    # caches are in/out: hand both runs the same starting bytes by passing them as outputs that the test pre-fills
    for merged in (0, 1):
        dims = (n_q, n_kv, hd, max_seq, nwg, 0 if merged else 1, 1)
        res = {}
        for half in (True, False):
            dt = [DType.Q40, DType.F16 if half else DType.F32, 0, 0]
            kk = ctx.compile(hip.make_desc(Kind.ATTEND_DECODE, dims, dt, (eps, 1.0 / 16)))
            bi = [ctx.buffer_bytes(a.astype(np.float16).view(np.uint8)) if (c == "A" and half) else ctx.buffer_f32(a) for a, c in ins]
            bk, bv = ctx.buffer_bytes(kc), ctx.buffer_bytes(vc)
            parts_n = n_q * nwg * (hd + 2)
            outs = [bk, bv, ctx.buffer_empty_f32(parts_n)]
            if merged:
                outs.append(ctx.buffer_empty_bytes(n_q * hd * (2 if half else 4)))
            ctx.encode_multi(kk, bi, outs)
            got = [ctx.read_bytes(bk, kc.size), ctx.read_bytes(bv, vc.size)]
            if merged:
                o = ctx.read_bytes(outs[3], n_q * hd * 2).view(np.float16).astype(np.float32) if half else ctx.read_f32(outs[3], n_q * hd)
                got.append(o)
            else:
                got.append(ctx.read_f32(outs[2], n_q * nwg * hd + n_q * nwg * 2))
            res[half] = got
        assert np.array_equal(res[True][0], res[False][0]) and np.array_equal(res[True][1], res[False][1])
        if merged:
            assert np.array_equal(res[True][2], res[False][2].astype(np.float16).astype(np.float32))
        else:
            assert np.array_equal(res[True][2], res[False][2])
            # ... and the o-projection that merges those partitions: parts f32, y half
            wo, _ = synth.cfg0_q4k_matvec(512, n_q * hd, seed=756)
            both(ctx, Kind.ATTN_MERGE_MATVEC, (512, n_q, hd, nwg), (DType.Q4K,), (), [(wo, "W"), (res[False][2], "F")], [(512, "A")])
    # embedding gather: id f32, row out half; per-layer-embedding gate; the prefill GEMM on half rows
    emb, _ = synth.cfg1_q6k_lm_head(64, 2048, seed=757)
    (row_out,) = both(ctx, Kind.COPY_SCALE_INDEXED, (2048, 64), (DType.Q6K,), (45.25,), [(emb, "W"), (np.array([17], np.float32), "F")], [(2048, "A")])
    assert rel_err(row_out, oracle.copy_scale_indexed(oracle.Q6K, emb, 17, 2048, 45.25).astype(np.float16).astype(np.float32)).max() <= BAR
    wg, x = synth.cfg0_q4k_matvec(256, 2048, seed=758)
    c = halfed(synth.normal_f32(256, 759))
    both(ctx, Kind.MATVEC_GELU_MUL, (256, 2048, 0), (DType.Q4K,), (), [(wg, "W"), (halfed(x), "A"), (c, "A")], [(256, "A")])
    wm, _ = synth.cfg0_q4k_matvec(256, 2048, seed=760)
    xs = halfed(synth.normal_f32(32 * 2048, 761))
    (ym,) = both(ctx, Kind.MATVEC_BATCH, (256, 2048, 32), (DType.Q4K,), (), [(wm, "W"), (xs, "A")], [(32 * 256, "A")])
    want = oracle.matmul(oracle.Q4K, wm, 256, 2048, xs, 32).astype(np.float16).astype(np.float32)
    assert rel_err(ym, want).max() <= BAR


def test_half_boundary_sizes_and_refusals(ctx):
    k = ctx.compile(hip.make_desc(Kind.MATVEC, (512, 2048), (DType.Q4K, DType.F16)))
    w, x = synth.cfg0_q4k_matvec(512, 2048, seed=770)
    bw, bx32, by = ctx.buffer_bytes(w), ctx.buffer_f32(x), ctx.buffer_empty_bytes(512 * 2)
    ctx.encode_multi(k, [bw, bx32], [by])              # a larger buffer is fine: the first 2048 halves are read
    with pytest.raises(hip.KshError, match="needs 4096 bytes"):
        ctx.encode_multi(k, [bw, ctx.buffer_empty_bytes(2048)], [by])
    with pytest.raises(hip.KshError, match="needs 1024 bytes"):
        ctx.encode_multi(k, [bw, bx32], [ctx.buffer_empty_bytes(512)])
    # the prompt pass's own forms of the GEMM (producers inside the preparation) take f32 rows only
    with pytest.raises(hip.KshError):
        ctx.compile(hip.make_desc(Kind.MATVEC_BATCH, (256, 2048, 32, 0, 0, 1), (DType.Q4K, DType.F16), (1e-6,)))
