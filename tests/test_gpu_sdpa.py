"""HIP decode attention over a Q4_0 KV cache vs the CPU oracle (1e-3 relative),
plus the invariants the reference's own example checks: batch equals serial,
partition-count independence, the needle."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip, synth
from ksearch_amd.hip import DType
from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def ctx():
    c = hip.Context()
    yield c
    c.close()


@pytest.fixture(scope="module")
def eng():
    return hip.Eng()


def kv(max_t, n_kv, hd, seed):
    n = max_t * n_kv * hd // 32
    return synth.q40_blocks(n, seed), synth.q40_blocks(n, seed + 1)


@pytest.mark.parametrize("n_q,n_kv,hd,max_t,tlen,start,scale", [
    (8, 1, 256, 64, 1, 0, 1.0 / 16),          # a single row
    (8, 1, 256, 64, 33, 0, 1.0 / 16),         # one row past a tile
    (8, 1, 256, 300, 127, 50, 1.0 / 16),      # largest online case, non-zero start (sliding window)
    (8, 1, 256, 300, 128, 0, 1.0 / 16),       # first split-KV case
    (8, 1, 256, 2048, 2048, 0, 1.0 / 16),
    (8, 1, 256, 1000, 777, 200, 1.0),         # the reference's scale (none)
    (4, 2, 128, 500, 300, 100, 0.09),         # GQA with two kv heads
    (16, 1, 64, 200, 150, 3, 0.125),
    (8, 1, 512, 400, 260, 7, 1.0 / 16),       # full-attention head size
])
def test_sdpa_hybrid_vs_oracle(ctx, eng, n_q, n_kv, hd, max_t, tlen, start, scale):
    k, v = kv(max_t, n_kv, hd, 300 + hd)
    q = synth.normal_f32(n_q * hd, 310)
    bq, bk, bv = ctx.buffer_f32(q), ctx.buffer_bytes(k), ctx.buffer_bytes(v)
    meta = ctx.buffer_f32([tlen, start, 0, 0])                   # write_meta_win, gemma_prim.rs:636-644
    tmp = ctx.buffer_empty_f32(n_q * eng.SDPA_MWG_NWG * (hd + 2))
    out = ctx.buffer_empty_f32(n_q * hd)
    eng.sdpa_hybrid_kv(ctx, n_q, n_kv, hd, max_t, tlen, DType.Q40, bq, bk, bv, meta, tmp, out, scale)
    got = ctx.read_f32(out, n_q * hd)
    assert_close(got, oracle.sdpa_hybrid(q, k, v, n_q, n_kv, hd, tlen, start, scale), TOL, "vs oracle")
    assert_close(got, oracle.sdpa(q, k, v, n_q, n_kv, hd, tlen, start, scale, f64=True), TOL, "vs f64")


def test_sdpa_partition_count_independence(ctx, eng):
    n_q, n_kv, hd, max_t, tlen = 8, 1, 256, 1024, 1000
    k, v = kv(max_t, n_kv, hd, 320)
    q = synth.normal_f32(n_q * hd, 321)
    bq, bk, bv = ctx.buffer_f32(q), ctx.buffer_bytes(k), ctx.buffer_bytes(v)
    meta = ctx.buffer_f32([tlen, 0, 0, 0])
    out = ctx.buffer_empty_f32(n_q * hd)
    want = oracle.sdpa(q, k, v, n_q, n_kv, hd, tlen, 0, 0.0625, f64=True)
    for nwg in (1, 2, 16, 33, 1000, 1024):     # 1024 > tlen: trailing partitions are empty
        tmp = ctx.buffer_empty_f32(n_q * nwg * (hd + 2))
        eng.sdpa_mwg_kv(ctx, n_q, n_kv, hd, max_t, DType.Q40, bq, bk, bv, meta, tmp, out, 0.0625, nwg=nwg)
        assert_close(ctx.read_f32(out, n_q * hd), want, TOL, f"nwg={nwg}")


def test_sdpa_needle(ctx, eng):
    # check_mul_mm.rs:250-294: Q = 1, K[0] = 1, V[0] = 1, other rows 0; the
    # expectation comes from the brute-force oracle, not from "O ~ 1"
    n_q, hd = 8, 256
    for tlen in (64, 512):
        kf = np.zeros((tlen, hd), dtype=np.float32)
        vf = np.zeros((tlen, hd), dtype=np.float32)
        kf[0] = vf[0] = 1.0
        src = ctx.buffer_f32(kf)
        bk, bv = ctx.buffer_empty_bytes(tlen * hd // 32 * 18), ctx.buffer_empty_bytes(tlen * hd // 32 * 18)
        eng.quantize_q40(ctx, tlen * hd, src, bk)
        eng.quantize_q40(ctx, tlen * hd, ctx.buffer_f32(vf), bv)
        k, v = ctx.read_bytes(bk, tlen * hd // 32 * 18), ctx.read_bytes(bv, tlen * hd // 32 * 18)
        assert np.array_equal(k, oracle.pack_q40(kf))
        q = np.ones(n_q * hd, dtype=np.float32)
        meta, out = ctx.buffer_f32([tlen, 0, tlen, 0]), ctx.buffer_empty_f32(n_q * hd)
        tmp = ctx.buffer_empty_f32(n_q * eng.SDPA_MWG_NWG * (hd + 2))
        for scale in (1.0, 1.0 / 256):
            eng.sdpa_hybrid_kv(ctx, n_q, 1, hd, tlen, tlen, DType.Q40, ctx.buffer_f32(q), bk, bv, meta, tmp, out, scale)
            assert_close(ctx.read_f32(out, n_q * hd), oracle.sdpa(q, k, v, n_q, 1, hd, tlen, 0, scale, f64=True), TOL,
                         f"needle tlen={tlen} scale={scale}")


# the two forms of the row phase for heads of 256: the library's choice (matrix cores) and the vector form by name
FORMS = [pytest.param(None, id="default"), pytest.param(dict(vec=3), id="vector_form")]


@pytest.mark.parametrize("sched", FORMS)
@pytest.mark.parametrize("nwg", [0, 16, 64])
def test_sdpa_slots_batch_equals_serial(ctx, eng, nwg, sched):
    # cfg3 at reduced context, then at full size below
    n_slots, n_q, n_kv, hd, max_t = 4, 8, 1, 256, 2048
    lens, k, v, q = synth.cfg3_q40_attention(n_slots, n_q, n_kv, hd, max_t, lo=100, seed=330)
    lens[1] = 1           # one slot with a single row: every other partition of it is empty
    bq, bk, bv = ctx.buffer_f32(q), ctx.buffer_bytes(k), ctx.buffer_bytes(v)
    meta = np.zeros((n_slots, 4), dtype=np.float32)
    meta[:, 0] = lens
    bm = ctx.buffer_f32(meta)
    kk = ctx.compile(hip.make_desc(hip.Kind.SDPA_SLOTS, (n_q, n_kv, hd, max_t, n_slots, nwg), (DType.Q40, DType.F32), (0.0625,), sched))
    assert ("regs" if sched else "mfma") in kk.name
    real_nwg = kk.info.sched.k_split
    tmp = ctx.buffer_empty_f32(n_slots * n_q * real_nwg * (hd + 2))
    out = ctx.buffer_empty_f32(n_slots * n_q * hd)
    eng.sdpa_slots(ctx, n_q, n_kv, hd, max_t, n_slots, bq, bk, bv, bm, tmp, out, 0.0625, nwg, sched)
    got = ctx.read_f32(out, n_slots * n_q * hd).reshape(n_slots, -1)
    for s in range(n_slots):
        want = oracle.sdpa_hybrid(q[s], k[s], v[s], n_q, n_kv, hd, int(lens[s]), 0, 0.0625)
        assert_close(got[s], want, TOL, f"slot {s} len {lens[s]}")


@pytest.mark.parametrize("sched", FORMS)
def test_sdpa_cfg3_full_size(ctx, eng, sched):
    n_slots, n_q, n_kv, hd, max_t = 4, 8, 1, 256, 16384
    lens, k, v, q = synth.cfg3_q40_attention()
    bq, bk, bv = ctx.buffer_f32(q), ctx.buffer_bytes(k), ctx.buffer_bytes(v)
    meta = np.zeros((n_slots, 4), dtype=np.float32)
    meta[:, 0] = lens
    kk = ctx.compile(hip.make_desc(hip.Kind.SDPA_SLOTS, (n_q, n_kv, hd, max_t, n_slots, 0), (DType.Q40, DType.F32), (0.0625,), sched))
    tmp = ctx.buffer_empty_f32(n_slots * n_q * kk.info.sched.k_split * (hd + 2))
    out = ctx.buffer_empty_f32(n_slots * n_q * hd)
    eng.sdpa_slots(ctx, n_q, n_kv, hd, max_t, n_slots, bq, bk, bv, ctx.buffer_f32(meta), tmp, out, 0.0625, 0, sched)
    got = ctx.read_f32(out, n_slots * n_q * hd).reshape(n_slots, -1)
    for s in range(n_slots):
        assert_close(got[s], oracle.sdpa_hybrid(q[s], k[s], v[s], n_q, n_kv, hd, int(lens[s]), 0, 0.0625), TOL, f"slot {s}")
    # softmax weights sum to one: with V == const c every output equals c (size-independent property)
    vc = np.tile(np.concatenate([np.array([0.5], dtype=np.float16).view(np.uint8), np.full(16, 0xBB, np.uint8)]), k.size // 18)
    eng.sdpa_slots(ctx, n_q, n_kv, hd, max_t, n_slots, bq, bk, ctx.buffer_bytes(vc), ctx.buffer_f32(meta), tmp, out, 0.0625, 0, sched)
    assert np.allclose(ctx.read_f32(out, n_slots * n_q * hd), 1.5, rtol=1e-5)


@pytest.mark.parametrize("n_slots,nwg,lens", [
    (4, 2, [2048, 1, 1, 1]),            # nearly every partition goes to one slot
    (3, 8, [7, 5, 2048]),               # fewer rows than partitions in two slots
    (16, 4, None),                      # the most slots that share partitions by length
    (17, 4, None),                      # one more: every slot keeps its own nwg partitions
    (2, 16, [2048, 2048]),              # equal lengths
])
@pytest.mark.parametrize("sched", FORMS)
def test_sdpa_slots_partitions_dealt_by_length(ctx, eng, n_slots, nwg, lens, sched):
    """A launch's nwg * n_slots partitions are shared out by slot length (up to 16 slots); every slot's result is
    still the oracle's attention over its own rows, on two launches in a row (the arrival counters return to zero)."""
    n_q, n_kv, hd, max_t = 8, 1, 256, 2048
    rnd, k, v, q = synth.cfg3_q40_attention(n_slots, n_q, n_kv, hd, max_t, lo=1, seed=360 + n_slots)
    lens = [int(t) for t in (rnd if lens is None else lens)]
    meta = np.zeros((n_slots, 4), dtype=np.float32)
    meta[:, 0] = lens
    bq, bk, bv, bm = ctx.buffer_f32(q), ctx.buffer_bytes(k), ctx.buffer_bytes(v), ctx.buffer_f32(meta)
    tmp = ctx.buffer_empty_f32(n_slots * n_q * nwg * (hd + 2))
    out = ctx.buffer_empty_f32(n_slots * n_q * hd)
    for rep in range(2):
        eng.sdpa_slots(ctx, n_q, n_kv, hd, max_t, n_slots, bq, bk, bv, bm, tmp, out, 0.0625, nwg, sched)
        got = ctx.read_f32(out, n_slots * n_q * hd).reshape(n_slots, -1)
        for s in range(n_slots):
            want = oracle.sdpa(q[s], k[s], v[s], n_q, n_kv, hd, lens[s], 0, 0.0625, f64=True)
            assert_close(got[s], want, TOL, f"rep {rep} slot {s} len {lens[s]}")


def test_sdpa_errors(ctx):
    with pytest.raises(hip.KshError, match="multiple of 32"):
        ctx.compile(hip.make_desc(hip.Kind.SDPA_NAIVE, (8, 1, 100, 64), (DType.Q40, DType.F32), (1.0,)))
    with pytest.raises(hip.KshError, match="not built"):
        ctx.compile(hip.make_desc(hip.Kind.SDPA_NAIVE, (8, 1, 256, 64), (DType.F16, DType.F32), (1.0,)))
    with pytest.raises(hip.KshError, match="divide evenly"):
        ctx.compile(hip.make_desc(hip.Kind.SDPA_NAIVE, (8, 3, 256, 64), (DType.Q40, DType.F32), (1.0,)))


@pytest.mark.parametrize("n_q,n_kv,hd,max_seq,pos,nwg,start", [
    (8, 1, 256, 512, 0, 0, 0),        # the first token attends only itself
    (8, 1, 256, 512, 1, 4, 0),
    (8, 1, 256, 512, 200, 16, 0),     # row groups dealt round robin: some partitions get one more than others
    (8, 1, 256, 4096, 319, 0, 0),     # the decode loop's shape and default split
    (8, 1, 256, 4096, 1500, 16, 0),   # several rounds of row groups per partition
    (4, 1, 128, 256, 77, 3, 0),       # the small decode model
    (4, 2, 128, 300, 150, 5, 0),      # two kv heads
    (8, 1, 256, 512, 300, 4, 173),    # a window that has begun to slide: rows [173, 300]
    (4, 1, 128, 256, 255, 2, 250),    # ... ending at the last row of the cache
    (8, 1, 512, 512, 0, 0, 0),        # 512-wide heads (the full-attention layers of the real checkpoints): a row per wave
    (8, 1, 512, 1024, 700, 16, 0),
    (4, 2, 512, 300, 150, 5, 40),
])
def test_attend_decode_vs_unfused_oracle(ctx, eng, n_q, n_kv, hd, max_seq, pos, nwg, start):
    """AttendDecode = RmsNormPerHeadQkvQ40 at `pos` + attention over rows [0, pos] + merge.  The oracle runs the
    three reference ops one after the other; the cache rows the kernel appends are compared as codes (they may
    differ by one step where a value sits on a rounding boundary) and the attention output against the oracle's
    attention over the DEVICE's cache, so that such a step does not leak into the comparison."""
    eps, scale = 1e-6, 1.0 / float(np.sqrt(hd))
    row = n_kv * hd // 32 * 18
    k, v = kv(max_seq, n_kv, hd, 340 + pos)
    k[pos * row:] = 0
    v[pos * row:] = 0
    q, kr, vr = (synth.normal_f32(r * hd, 350 + i) for i, r in enumerate((n_q, n_kv, n_kv)))
    qw, kw = 1.0 + 0.2 * synth.normal_f32(hd, 353), 1.0 + 0.2 * synth.normal_f32(hd, 354)
    rope = oracle.rope_table(max_seq, hd, 10000.0)
    kc, vc = ctx.buffer_bytes(k), ctx.buffer_bytes(v)
    out = ctx.buffer_empty_f32(n_q * hd)
    tlen = pos + 1 - start
    meta = ctx.buffer_f32([tlen, start, tlen if start else 0, pos])
    kk = ctx.compile(hip.make_desc(hip.Kind.ATTEND_DECODE, (n_q, n_kv, hd, max_seq, nwg), (DType.Q40, DType.F32), (eps, scale)))
    tmp = ctx.buffer_empty_f32(n_q * kk.grid[0] * (hd + 2))
    for rep in range(2):                     # twice: the arrival counter must come back to zero
        ctx.encode_multi(kk, [ctx.buffer_f32(q), ctx.buffer_f32(qw), ctx.buffer_f32(rope), ctx.buffer_f32(kr), ctx.buffer_f32(kw),
                              ctx.buffer_f32(vr), meta], [kc, vc, tmp, out])
        got = ctx.read_f32(out, n_q * hd)
        wq, wk, wv = oracle.rmsnorm_per_head_qkv_q40(q, qw, rope[pos], kr, kw, vr, n_q, n_kv, hd, eps)
        gk, gv = ctx.read_bytes(kc, (pos + 1) * row), ctx.read_bytes(vc, (pos + 1) * row)
        assert np.array_equal(gk[:pos * row], k[:pos * row]) and np.array_equal(gv[:pos * row], v[:pos * row])
        for g, w_ in ((gk[pos * row:], wk), (gv[pos * row:], wv)):
            dg, dw = oracle.dequant(oracle.Q40, g, n_kv * hd), oracle.dequant(oracle.Q40, w_, n_kv * hd)
            assert np.abs(dg - dw).max() <= np.abs(dw).max() / 7.0 * 1.01
            assert (g != w_).mean() < 0.02
        want = oracle.sdpa(wq, gk, gv, n_q, n_kv, hd, tlen, start, scale, f64=True)
        assert_close(got, want, TOL, f"rep {rep}")
    # the same launch given the position's rope row instead of the table (dims[6] = 1): identical bits
    k2 = ctx.compile(hip.make_desc(hip.Kind.ATTEND_DECODE, (n_q, n_kv, hd, max_seq, nwg, 0, 1), (DType.Q40, DType.F32), (eps, scale)))
    kc2, vc2, out2 = ctx.buffer_bytes(k), ctx.buffer_bytes(v), ctx.buffer_empty_f32(n_q * hd)
    ctx.encode_multi(k2, [ctx.buffer_f32(q), ctx.buffer_f32(qw), ctx.buffer_f32(rope[pos]), ctx.buffer_f32(kr), ctx.buffer_f32(kw),
                          ctx.buffer_f32(vr), meta], [kc2, vc2, tmp, out2])
    assert np.array_equal(ctx.read_f32(out2, n_q * hd), got)
    assert np.array_equal(ctx.read_bytes(kc2, (pos + 1) * row), gk) and np.array_equal(ctx.read_bytes(vc2, (pos + 1) * row), gv)
    if pos + 1 < max_seq:
        assert not ctx.read_bytes(kc, row, (pos + 1) * row).any()


@pytest.mark.parametrize("n_q,n_kv,hd,max_seq,pos,nwg,start,parts", [
    (8, 1, 256, 1024, 0, 8, 0, True),       # one row, every partition but one empty
    (8, 1, 256, 1024, 600, 8, 89, True),    # the sliding-window layers that reuse a cache: 512 rows, unmerged
    (8, 1, 256, 1024, 300, 16, 0, False),
    (8, 1, 512, 1024, 700, 16, 0, False),   # the full-attention ones
    (8, 1, 512, 512, 3, 16, 0, False),      # fewer rows than partitions
    (4, 2, 128, 300, 150, 5, 40, False),
    (4, 1, 128, 256, 77, 1, 0, False),      # a single partition
])
def test_attend_decode_reading_another_layers_cache(ctx, eng, n_q, n_kv, hd, max_seq, pos, nwg, start, parts):
    """dims[7] = 1: q is normed and roped, nothing is appended, rows [start, pos] all come from the cache (which
    must come back untouched).  Against the oracle's per-head norm + RoPE and attention, merged or through the
    unmerged partitions."""
    eps, scale = 1e-6, 1.0 / float(np.sqrt(hd))
    row = n_kv * hd // 32 * 18
    k, v = kv(max_seq, n_kv, hd, 540 + pos)
    q = synth.normal_f32(n_q * hd, 550)
    qw = 1.0 + 0.2 * synth.normal_f32(hd, 553)
    rope = oracle.rope_table(max_seq, hd, 10000.0, hd // 4 if hd == 512 else None)
    kc, vc = ctx.buffer_bytes(k), ctx.buffer_bytes(v)
    tlen = pos + 1 - start
    meta = ctx.buffer_f32([tlen, start, tlen if start else 0, pos])
    kk = ctx.compile(hip.make_desc(hip.Kind.ATTEND_DECODE, (n_q, n_kv, hd, max_seq, nwg, int(parts), 1, 1), (DType.Q40, DType.F32), (eps, scale)))
    assert "reader" in kk.name and kk.info.n_inputs == 6 and kk.info.n_outputs == (1 if parts else 2)
    tmp, out = ctx.buffer_empty_f32(n_q * nwg * (hd + 2)), ctx.buffer_empty_f32(n_q * hd)
    ins = [ctx.buffer_f32(q), ctx.buffer_f32(qw), ctx.buffer_f32(rope[pos]), kc, vc, meta]
    want = oracle.sdpa(oracle.rmsnorm_per_head(q, qw, n_q, hd, eps, rope[pos]), k, v, n_q, n_kv, hd, tlen, start, scale, f64=True)
    for rep in range(2):
        ctx.encode_multi(kk, ins, [tmp] if parts else [tmp, out])
        if parts:
            t = ctx.read_f32(tmp, n_q * nwg * (hd + 2))
            o, ml = t[:n_q * nwg * hd].reshape(n_q, nwg, hd).astype(np.float64), t[n_q * nwg * hd:].reshape(n_q, nwg, 2).astype(np.float64)
            wt = np.exp(ml[:, :, 0] - ml[:, :, 0].max(1, keepdims=True))
            got = (wt[:, :, None] * o).sum(1) / (wt * ml[:, :, 1]).sum(1)[:, None]
        else:
            got = ctx.read_f32(out, n_q * hd)
        assert_close(got, want, TOL, f"rep {rep}")
    assert np.array_equal(ctx.read_bytes(kc, max_seq * row), k) and np.array_equal(ctx.read_bytes(vc, max_seq * row), v)


@pytest.mark.parametrize("n_q,n_kv,hd,max_seq,pos,nwg,start", [
    (8, 1, 256, 1024, 300, 8, 0),
    (8, 1, 256, 1024, 700, 16, 150),    # a window that has begun to slide
    (8, 1, 512, 1024, 300, 8, 0),       # 512-wide heads: at most four per workgroup
    (8, 2, 256, 512, 200, 4, 0),        # two kv heads of four q heads each
])
@pytest.mark.parametrize("parts", [False, True])
def test_attend_decode_every_head_split(ctx, eng, n_q, n_kv, hd, max_seq, pos, nwg, start, parts):
    """The decode step under every split of a kv head's q heads over workgroups (sched.unroll) and both workgroup sizes:
    eight, four, two heads per workgroup or one (the last two have kernel instances of their own at heads of 256 / 512),
    merged in the launch or left as partitions; each against the oracle's attention over the device's cache."""
    eps, scale = 1e-6, 1.0 / float(np.sqrt(hd))
    row = n_kv * hd // 32 * 18
    k, v = kv(max_seq, n_kv, hd, 740 + pos)
    k[pos * row:] = 0
    v[pos * row:] = 0
    q, kr, vr = (synth.normal_f32(r * hd, 750 + i) for i, r in enumerate((n_q, n_kv, n_kv)))
    qw, kw = 1.0 + 0.2 * synth.normal_f32(hd, 753), 1.0 + 0.2 * synth.normal_f32(hd, 754)
    rope = oracle.rope_table(max_seq, hd, 10000.0)
    tlen = pos + 1 - start
    meta = ctx.buffer_f32([tlen, start, tlen if start else 0, pos])
    groups, ran = n_q // n_kv, 0
    for unroll in (1, 2, 4, 8):
        if groups % unroll or (hd == 512 and groups // unroll > 4):
            continue
        for nsg in (4, 8):
            kk = ctx.compile(hip.make_desc(hip.Kind.ATTEND_DECODE, (n_q, n_kv, hd, max_seq, nwg, int(parts), 1), (DType.Q40, DType.F32), (eps, scale),
                                           dict(vec=3, unroll=unroll, nsg=nsg)))
            assert kk.info.sched.unroll == unroll and kk.info.sched.nsg == nsg
            kc, vc, tmp, out = ctx.buffer_bytes(k), ctx.buffer_bytes(v), ctx.buffer_empty_f32(n_q * nwg * (hd + 2)), ctx.buffer_empty_f32(n_q * hd)
            ins = [ctx.buffer_f32(a) for a in (q, qw, rope[pos], kr, kw, vr)] + [meta]
            for rep in range(2):                 # twice: the arrival counter of the merging form must come back to zero
                ctx.encode_multi(kk, ins, [kc, vc, tmp] if parts else [kc, vc, tmp, out])
            if parts:
                t = ctx.read_f32(tmp, n_q * nwg * (hd + 2))
                o, ml = t[:n_q * nwg * hd].reshape(n_q, nwg, hd).astype(np.float64), t[n_q * nwg * hd:].reshape(n_q, nwg, 2).astype(np.float64)
                wt = np.exp(ml[:, :, 0] - ml[:, :, 0].max(1, keepdims=True))
                got = ((wt[:, :, None] * o).sum(1) / (wt * ml[:, :, 1]).sum(1)[:, None]).reshape(-1)
            else:
                got = ctx.read_f32(out, n_q * hd)
            gk, gv = ctx.read_bytes(kc, max_seq * row), ctx.read_bytes(vc, max_seq * row)
            wq = oracle.rmsnorm_per_head_qkv_q40(q, qw, rope[pos], kr, kw, vr, n_q, n_kv, hd, eps)[0]
            want = oracle.sdpa(wq, gk, gv, n_q, n_kv, hd, tlen, start, scale, f64=True)
            assert_close(got, want, TOL, f"unroll {unroll}, {nsg} waves")
            ran += 1
    assert ran >= 4


@pytest.mark.parametrize("n_q,n_kv,hd,max_seq,pos,nwg,rows", [
    (8, 1, 256, 4096, 0, 8, 2048),      # one row: seven partitions are empty
    (8, 1, 256, 4096, 5, 8, 2048),      # fewer rows than partitions
    (8, 1, 256, 4096, 319, 8, 2048),    # the decode loop's shape
    (8, 1, 256, 512, 200, 3, 512),      # fewer partitions than the prologue holds
    (4, 1, 128, 256, 77, 4, 512),       # the small decode model: half of the threads hold no element
    (4, 2, 128, 300, 150, 1, 300),      # a single partition
])
def test_attn_merge_matvec_vs_merged_attention(ctx, eng, n_q, n_kv, hd, max_seq, pos, nwg, rows):
    """AttendDecode without its merge, then the o-projection that merges the partitions in its prologue, against
    (a) the oracle's attention over the device's cache followed by the oracle's Q4_K GEMV and (b) the merging
    AttendDecode followed by the plain GEMV."""
    eps, scale = 1e-6, 1.0 / float(np.sqrt(hd))
    row = n_kv * hd // 32 * 18
    k, v = kv(max_seq, n_kv, hd, 440 + pos)
    k[pos * row:] = 0
    v[pos * row:] = 0
    q, kr, vr = (synth.normal_f32(r * hd, 450 + i) for i, r in enumerate((n_q, n_kv, n_kv)))
    qw, kw = 1.0 + 0.2 * synth.normal_f32(hd, 453), 1.0 + 0.2 * synth.normal_f32(hd, 454)
    rope = oracle.rope_table(max_seq, hd, 10000.0)
    cols = n_q * hd
    w = synth.q4k_blocks(rows * cols // 256, seed=455)
    bw = ctx.buffer_bytes(w)
    ins = [ctx.buffer_f32(a) for a in (q, qw, rope, kr, kw, vr)] + [ctx.buffer_f32([pos + 1, 0, 0, pos])]
    # (b) merge inside the attention launch, plain GEMV
    kc, vc = ctx.buffer_bytes(k), ctx.buffer_bytes(v)
    out, y_ref = ctx.buffer_empty_f32(cols), ctx.buffer_empty_f32(rows)
    tmp = ctx.buffer_empty_f32(n_q * nwg * (hd + 2))
    eng.attend_decode(ctx, n_q, n_kv, hd, max_seq, eps, scale, *ins, kc, vc, tmp, out, nwg=nwg)
    eng.matvec_wd(ctx, rows, cols, DType.Q4K, bw, out, y_ref)
    want_b = ctx.read_f32(y_ref, rows)
    # the path under test, twice (nothing may depend on what the last call left in `parts`)
    kc2, vc2 = ctx.buffer_bytes(k), ctx.buffer_bytes(v)
    parts, y = ctx.buffer_f32(np.full(n_q * nwg * (hd + 2), np.nan, np.float32)), ctx.buffer_empty_f32(rows)
    for rep in range(2):
        eng.attend_decode_parts(ctx, n_q, n_kv, hd, max_seq, eps, scale, *ins, kc2, vc2, parts, nwg)
        kk = eng.attn_merge_matvec_wd(ctx, rows, n_q, hd, nwg, DType.Q4K, bw, parts, y)
        got = ctx.read_f32(y, rows)
        assert np.array_equal(ctx.read_bytes(kc2, (pos + 1) * row), ctx.read_bytes(kc, (pos + 1) * row))
        wq = oracle.rmsnorm_per_head_qkv_q40(q, qw, rope[pos], kr, kw, vr, n_q, n_kv, hd, eps)[0]
        att = oracle.sdpa(wq, ctx.read_bytes(kc2, (pos + 1) * row), ctx.read_bytes(vc2, (pos + 1) * row), n_q, n_kv, hd,
                          pos + 1, 0, scale, f64=True)
        want_a = oracle.matvec(oracle.Q4K, w, rows, cols, att.astype(np.float32))
        assert_close(got, want_a, TOL, f"vs oracle, rep {rep}")
        assert_close(got, want_b, 1e-4, f"vs merging launch, rep {rep}")
    assert "attn_merge" in kk.name


def test_attn_merge_matvec_errors(ctx):
    with pytest.raises(hip.KshError, match="at most 8"):
        ctx.compile(hip.make_desc(hip.Kind.ATTN_MERGE_MATVEC, (2048, 8, 256, 16), (DType.Q4K, DType.F32), ()))
    with pytest.raises(hip.KshError, match="power of two"):
        ctx.compile(hip.make_desc(hip.Kind.ATTN_MERGE_MATVEC, (2048, 8, 96, 4), (DType.Q4K, DType.F32), ()))
    with pytest.raises(hip.KshError, match="one float4 per thread"):
        ctx.compile(hip.make_desc(hip.Kind.ATTN_MERGE_MATVEC, (2048, 16, 256, 4), (DType.Q4K, DType.F32), ()))


def test_beam_search_attention_kinds(ctx, tmp_path, monkeypatch):
    """The schedule search over the attention kinds' knobs (K-split = partitions per sequence, waves per workgroup,
    workgroups per kv head for the fused decode step): every candidate is timed on the device, the winner is saved
    under KSEARCH_BEAM_CACHE keyed by kind, dims and chip, a second search is served from the file, a kernel
    requested with an all-zero schedule in a fresh context picks the plan up, and the result stays the oracle's."""
    monkeypatch.setenv("KSEARCH_BEAM_CACHE", str(tmp_path / "beam"))
    n_slots, n_q, n_kv, hd, max_t = 2, 8, 1, 256, 2048
    lens, kk, vv, q = synth.cfg3_q40_attention(n_slots=n_slots, max_t=max_t, lo=700, seed=1203)
    meta = np.zeros((n_slots, 4), np.float32)
    meta[:, 0] = lens
    desc = hip.make_desc(hip.Kind.SDPA_SLOTS, (n_q, n_kv, hd, max_t, n_slots, 0), (hip.DType.Q40, hip.DType.F32), (1.0 / 16.0,))
    cands = [c.as_dict() for c in hip.beam_candidates(desc)]
    assert len(cands) >= 6 and {c["k_split"] for c in cands} >= {8, 16, 32} and {c["nsg"] for c in cands} == {4, 8}
    ins = [ctx.buffer_f32(q), ctx.buffer_bytes(kk), ctx.buffer_bytes(vv), ctx.buffer_f32(meta)]
    outs = [ctx.buffer_empty_f32(n_slots * n_q * 64 * (hd + 2)), ctx.buffer_empty_f32(n_slots * n_q * hd)]
    best, ms, cached = ctx.beam_search(desc, ins, outs, iters=5, force=True)
    assert not cached and 0 < ms < 1.0 and best.k_split >= 1
    files = list((tmp_path / "beam").glob("sdpa_q40_*.txt"))
    assert len(files) == 1
    best2, _, cached2 = ctx.beam_search(desc, ins, outs, iters=5)
    assert cached2 and best2.as_dict() == best.as_dict()
    ctx2 = hip.Context()
    try:
        k = ctx2.compile(desc)
        assert k.info.sched.k_split == best.k_split and k.info.sched.nsg == best.nsg
        ins2 = [ctx2.buffer_f32(q), ctx2.buffer_bytes(kk), ctx2.buffer_bytes(vv), ctx2.buffer_f32(meta)]
        outs2 = [ctx2.buffer_empty_f32(n_slots * n_q * k.info.sched.k_split * (hd + 2)), ctx2.buffer_empty_f32(n_slots * n_q * hd)]
        ctx2.encode_multi(k, ins2, outs2)
        ctx2.synchronize()
        got = ctx2.read_f32(outs2[1], n_slots * n_q * hd).reshape(n_slots, -1)
        for s in range(n_slots):
            want = oracle.sdpa(q[s], kk[s], vv[s], n_q, n_kv, hd, int(lens[s]), 0, 1.0 / 16.0)
            assert_close(got[s], want, 1e-3, f"slot {s} under the planned schedule")
    finally:
        ctx2.close()
    # the fused decode step: K-split, waves and the head split are all open
    d2 = hip.make_desc(hip.Kind.ATTEND_DECODE, (n_q, n_kv, hd, max_t, 0, 0, 0), (hip.DType.Q40, hip.DType.F32), (1e-6, 1.0 / 16.0))
    c2 = [c.as_dict() for c in hip.beam_candidates(d2)]
    assert {c["unroll"] for c in c2} == {1, 2, 4, 8} and {c["k_split"] for c in c2} >= {8, 16, 32}
    rope = oracle.rope_table(max_t, hd, 10000.0)
    raw_q, raw_k, raw_v = synth.normal_f32(n_q * hd, 1210), synth.normal_f32(hd, 1211), synth.normal_f32(hd, 1212)
    m2 = np.array([601, 0, 0, 600], np.float32)
    ones = np.ones(hd, np.float32)
    ins3 = [ctx.buffer_f32(raw_q), ctx.buffer_f32(ones), ctx.buffer_f32(rope), ctx.buffer_f32(raw_k), ctx.buffer_f32(ones),
            ctx.buffer_f32(raw_v), ctx.buffer_f32(m2)]
    kc, vc = ctx.buffer_bytes(kk[0]), ctx.buffer_bytes(vv[0])
    outs3 = [kc, vc, ctx.buffer_empty_f32(n_q * 64 * (hd + 2)), ctx.buffer_empty_f32(n_q * hd)]
    best3, ms3, cached3 = ctx.beam_search(d2, ins3, outs3, iters=5, force=True)
    assert not cached3 and 0 < ms3 < 1.0
    assert len(list((tmp_path / "beam").glob("attend_decode_q40_*.txt"))) == 1
    # whichever candidate ran last left the oracle's result for that step
    q_o, k_row, v_row = oracle.rmsnorm_per_head_qkv_q40(raw_q, ones, rope[600], raw_k, ones, raw_v, n_q, n_kv, hd, 1e-6)
    kh, vh = kk[0].copy(), vv[0].copy()
    kh[600 * 144:601 * 144], vh[600 * 144:601 * 144] = k_row, v_row
    want = oracle.sdpa(q_o, kh, vh, n_q, n_kv, hd, 601, 0, 1.0 / 16.0)
    assert_close(ctx.read_f32(outs3[3], n_q * hd), want, 1e-3, "attend_decode after the search")


@pytest.mark.parametrize("n_q,n_kv,lens,max_t,nwg,start", [
    (8, 1, [5583, 3908, 9979, 4967], 16384, 0, 0),     # BASELINE config 3
    (8, 1, [1, 33, 127, 128, 129, 700], 1024, 8, 0),   # a single row, tile edges, the wave-tile boundary
    (8, 1, [2048], 2048, 16, 0),                       # one slot
    (8, 2, [300, 1500, 31], 2048, 8, 0),               # two kv heads of four q heads each
    (4, 1, [900, 64], 1024, 4, 100),                   # four q heads, a window that starts at row 100
    (8, 1, [16384, 1024], 16384, 64, 0),               # the longest sequence beside a short one
])
@pytest.mark.parametrize("tile", [32, 16])
def test_sdpa_slots_matrix_core_form(ctx, n_q, n_kv, lens, max_t, nwg, start, tile):
    """The matrix-core form of the row phase (schedule vec = 2: f16 MFMA on exact integer codes, q and p*dv split
    hi | lo; four waves with tiles of 32 rows or eight with tiles of 16) against the serial oracle per slot, 1e-3
    relative; and against the float64 brute force, where it is held to 1e-4 (the products are exact, only f32
    accumulation and exp remain)."""
    hd, n_slots = 256, len(lens)
    _, kk, vv, q = synth.cfg3_q40_attention(n_slots=n_slots, n_q=n_q, n_kv=n_kv, hd=hd, max_t=max_t, lo=1, seed=1303)
    meta = np.zeros((n_slots, 4), np.float32)
    meta[:, 0] = lens
    meta[:, 1] = start
    lens = [min(t, max_t - start) for t in lens]
    meta[:, 0] = lens
    scale = 1.0 / 16.0
    k = ctx.compile(hip.make_desc(hip.Kind.SDPA_SLOTS, (n_q, n_kv, hd, max_t, n_slots, nwg), (DType.Q40, DType.F32), (scale,), dict(vec=2, lds_tile=tile)))
    assert "mfma" in k.name and k.info.sched.lds_tile == tile and k.info.sched.nsg == 128 // tile
    parts = k.info.sched.k_split
    tmp, out = ctx.buffer_empty_f32(n_slots * n_q * parts * (hd + 2)), ctx.buffer_empty_f32(n_slots * n_q * hd)
    ins = [ctx.buffer_f32(q), ctx.buffer_bytes(kk.reshape(-1)), ctx.buffer_bytes(vv.reshape(-1)), ctx.buffer_f32(meta)]
    ctx.encode_multi(k, ins, [tmp, out])
    ctx.synchronize()
    got = ctx.read_f32(out, n_slots * n_q * hd).reshape(n_slots, -1)
    worst64 = 0.0
    for s in range(n_slots):
        want = oracle.sdpa(q[s], kk[s], vv[s], n_q, n_kv, hd, lens[s], start, scale)
        assert_close(got[s], want, TOL, f"{k.name} slot {s} ({lens[s]} rows)")
        if lens[s] <= 4096:
            w64 = oracle.sdpa(q[s], kk[s], vv[s], n_q, n_kv, hd, lens[s], start, scale, f64=True)
            worst64 = max(worst64, float(np.max(np.abs(got[s] - w64) / np.maximum(np.abs(w64), np.sqrt(np.mean(w64 ** 2))))))
    assert worst64 <= 1e-4, worst64
    # a second launch on the same buffers gives the same bits (fixed summation order)
    ctx.encode_multi(k, ins, [tmp, out])
    ctx.synchronize()
    assert np.array_equal(ctx.read_f32(out, n_slots * n_q * hd).reshape(n_slots, -1), got)
