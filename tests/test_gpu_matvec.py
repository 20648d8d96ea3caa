"""HIP GEMV family vs the CPU oracle, through the C ABI.  Bars: dequantized
weights bit-exact; GEMV outputs within 1e-3 relative of the oracle's
dequant + sequential-f32 dot (f32 accumulate on both sides)."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip, synth
from ksearch_amd.hip import DType
from tests.gpu_util import assert_close, q6k_rows

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


def test_device_name(ctx, monkeypatch):
    assert ctx.device_name() == "gfx950"
    monkeypatch.setenv("KSEARCH_CHIP", "my-chip")
    c2 = hip.Context()
    assert c2.device_name() == "my-chip"
    c2.close()


@pytest.mark.parametrize("dtype,gen,n_blocks", [
    (DType.Q4K, synth.q4k_blocks, 4099), (DType.Q6K, synth.q6k_blocks, 2051), (DType.Q40, synth.q40_blocks, 40003)])
def test_dequant_bit_exact(ctx, eng, dtype, gen, n_blocks):
    blocks = gen(n_blocks, seed=100 + int(dtype))
    n = n_blocks * (32 if dtype == DType.Q40 else 256)
    src, dst = ctx.buffer_bytes(blocks), ctx.buffer_empty_f32(n)
    eng.dequant(ctx, dtype, n, src, dst)
    got = ctx.read_f32(dst, n)
    want = oracle.dequant(int(dtype), blocks, n)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequant_edge_blocks(ctx, eng):
    # zero scales, saturated scales, subnormal and largest half d/dmin
    blk = np.zeros((6, 144), dtype=np.uint8)
    blk[1, 4:16] = 0xFF
    blk[1, 16:] = 0xFF
    blk[1, 0:4] = np.array([65504.0, 65504.0], dtype=np.float16).view(np.uint8)
    blk[2, 0:4] = np.array([6e-8, 6e-8], dtype=np.float16).view(np.uint8)
    blk[2, 4:] = 0xA5
    blk[3, 0:4] = np.array([-1.5, 0.25], dtype=np.float16).view(np.uint8)
    blk[3, 4:] = np.arange(140, dtype=np.uint8)
    blk[4:] = synth.q4k_blocks(2, 5).reshape(2, 144)
    src, dst = ctx.buffer_bytes(blk), ctx.buffer_empty_f32(6 * 256)
    eng.dequant(ctx, DType.Q4K, 6 * 256, src, dst)
    got, want = ctx.read_f32(dst, 6 * 256), oracle.dequant(oracle.Q4K, blk, 6 * 256)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


SCHEDS_Q4K = [None] + [dict(tg=64 * w, vec=v, unroll=1, nsg=w, nr0=r, k_split=1, lds_tile=0)
                       for v in (3, 1) for w, r in ((4, 4), (4, 1), (8, 2))]


@pytest.mark.parametrize("rows,cols", [(64, 256), (128, 256), (2048, 1536), (50, 2048), (37, 4096), (33, 8192), (512, 4096)])
@pytest.mark.parametrize("sched", SCHEDS_Q4K)
def test_matvec_q4k_small(ctx, eng, rows, cols, sched):
    w = synth.q4k_blocks(rows * cols // 256, seed=rows + cols)
    x = synth.normal_f32(cols, seed=7)
    bw, bx, by = ctx.buffer_bytes(w), ctx.buffer_f32(x), ctx.buffer_empty_f32(rows)
    eng.matvec_wd(ctx, rows, cols, DType.Q4K, bw, bx, by, sched)
    assert_close(ctx.read_f32(by, rows), oracle.matvec(oracle.Q4K, w, rows, cols, x), TOL, f"q4k {rows}x{cols} {sched}")


@pytest.mark.parametrize("sched", SCHEDS_Q4K)
def test_matvec_q4k_cfg0_full_size(ctx, eng, sched):
    rows = cols = 4096
    w, x = synth.cfg0_q4k_matvec()
    bw, bx, by = ctx.buffer_bytes(w), ctx.buffer_f32(x), ctx.buffer_empty_f32(rows)
    eng.matvec_wd(ctx, rows, cols, DType.Q4K, bw, bx, by, sched)
    got = ctx.read_f32(by, rows)
    want = oracle.matvec(oracle.Q4K, w, rows, cols, x)
    assert_close(got, want, TOL, f"cfg0 {sched}")
    # and it sits within 1e-5 of the f64 truth (closer than the sequential-f32 oracle itself does),
    # for the int8-digit inner product as much as for the f32 one
    assert_close(got, oracle.matvec_f64(oracle.Q4K, w, rows, cols, x), 1e-5, "cfg0 vs f64")


@pytest.mark.parametrize("rows,cols,nsg,nr0", [(4096, 4096, 8, 2), (2048, 2048, 8, 1), (2048, 1536, 8, 2), (512, 8192, 4, 1)])
def test_matvec_q4k_two_digit_planes(ctx, eng, rows, cols, nsg, nr0):
    # vec = 2: the activations as two int8 digits, 2^-16 of the sub-block's largest magnitude.  By request only (the
    # schedule search does not list it); held to the 1e-3 bar against the oracle and to 1e-4 of the f64 truth on
    # normal inputs, and bit-exact on unit vectors (one digit pair per sub-block is then exact)
    sched = dict(tg=64 * nsg, vec=2, unroll=1, nsg=nsg, nr0=nr0, k_split=1, lds_tile=0)
    w = synth.q4k_blocks(rows * cols // 256, seed=rows + cols)
    x = synth.normal_f32(cols, seed=11)
    bw, bx, by = ctx.buffer_bytes(w), ctx.buffer_f32(x), ctx.buffer_empty_f32(rows)
    eng.matvec_wd(ctx, rows, cols, DType.Q4K, bw, bx, by, sched)
    got = ctx.read_f32(by, rows)
    assert_close(got, oracle.matvec(oracle.Q4K, w, rows, cols, x), TOL, f"two planes {rows}x{cols}")
    assert_close(got, oracle.matvec_f64(oracle.Q4K, w, rows, cols, x), 1e-4, "two planes vs f64")
    wd = oracle.dequant(oracle.Q4K, w, rows * cols).reshape(rows, cols)
    for j in (0, 31, 32, cols - 1):
        e = np.zeros(cols, dtype=np.float32)
        e[j] = 1.0
        eng.matvec_wd(ctx, rows, cols, DType.Q4K, bw, ctx.buffer_f32(e), by, sched)
        assert np.allclose(ctx.read_f32(by, rows), wd[:, j], rtol=1e-6, atol=1e-9), j


def test_matvec_q4k_unit_vectors_recover_weights(ctx, eng):
    # y = W e_j is column j of the dequantized matrix: pins the lane -> element map
    rows, cols = 8, 4096
    w = synth.q4k_blocks(rows * cols // 256, seed=3)
    wd = oracle.dequant(oracle.Q4K, w, rows * cols).reshape(rows, cols)
    bw, by = ctx.buffer_bytes(w), ctx.buffer_empty_f32(rows)
    for j in [0, 1, 15, 16, 31, 32, 63, 64, 255, 256, 1000, 2047, 2048, 4095]:
        e = np.zeros(cols, dtype=np.float32)
        e[j] = 1.0
        eng.matvec_wd(ctx, rows, cols, DType.Q4K, bw, ctx.buffer_f32(e), by)
        assert np.allclose(ctx.read_f32(by, rows), wd[:, j], rtol=1e-6, atol=1e-9), j


def test_matvec_q4k_1536_columns_unit_vectors(ctx, eng):
    # rows of six superblocks go through the half-wave form with a quarter of the lanes masked
    rows, cols = 9, 1536
    w = synth.q4k_blocks(rows * cols // 256, seed=4)
    wd = oracle.dequant(oracle.Q4K, w, rows * cols).reshape(rows, cols)
    bw, by = ctx.buffer_bytes(w), ctx.buffer_empty_f32(rows)
    for j in [0, 31, 32, 63, 64, 255, 256, 1279, 1280, 1535]:
        e = np.zeros(cols, dtype=np.float32)
        e[j] = 1.0
        eng.matvec_wd(ctx, rows, cols, DType.Q4K, bw, ctx.buffer_f32(e), by)
        assert np.allclose(ctx.read_f32(by, rows), wd[:, j], rtol=1e-6, atol=1e-9), j


def test_matvec_offsets_and_errors(ctx, eng):
    rows, cols = 64, 512
    w = synth.q4k_blocks(rows * cols // 256, seed=9)
    xs = synth.normal_f32(3 * cols, seed=10)
    bw, bx, by = ctx.buffer_bytes(w), ctx.buffer_f32(xs), ctx.buffer_empty_f32(3 * rows)
    for t in range(3):
        eng.matvec_wd_at(ctx, rows, cols, DType.Q4K, bw, bx, t * cols, by, t * rows)
    got = ctx.read_f32(by, 3 * rows).reshape(3, rows)
    for t in range(3):
        assert_close(got[t], oracle.matvec(oracle.Q4K, w, rows, cols, xs[t * cols:(t + 1) * cols]), TOL)
    k = ctx.compile(hip.make_desc(hip.Kind.MATVEC, (rows, cols), (DType.Q4K, DType.F32)))
    with pytest.raises(hip.KshError, match="expected 2 inputs, got 1"):
        ctx.encode_offsets_multi(k, [bw], None, [by], None)
    with pytest.raises(hip.KshError, match="expected 1 outputs, got 2"):
        ctx.encode_offsets_multi(k, [bw, bx], None, [by, by], None)
    with pytest.raises(hip.KshError, match="needs"):
        ctx.encode_offsets_multi(k, [bw, bx], [0, 3 * cols * 4 - 16], [by], [0])
    with pytest.raises(hip.KshError, match="not built"):
        ctx.compile(hip.make_desc(hip.Kind.MATVEC, (rows, cols), (DType.Q5K, DType.F32)))
    with pytest.raises(hip.KshError, match="multiple of 256"):
        ctx.compile(hip.make_desc(hip.Kind.MATVEC, (rows, 300), (DType.Q4K, DType.F32)))


SCHEDS_Q6K = [None, dict(tg=256, vec=0, unroll=2, nsg=4, nr0=1, k_split=1, lds_tile=0),
              dict(tg=512, vec=0, unroll=8, nsg=8, nr0=4, k_split=1, lds_tile=0),
              dict(tg=128, vec=0, unroll=2, nsg=2, nr0=2, k_split=1, lds_tile=0)]


@pytest.mark.parametrize("rows,cols", [(8, 2048), (1000, 2048), (4099, 2048), (300, 4096), (70, 256), (33, 512), (65, 1536), (40, 8192)])
@pytest.mark.parametrize("sched", SCHEDS_Q6K)
def test_matvec_q6k(ctx, eng, rows, cols, sched):
    w = synth.q6k_blocks(rows * cols // 256, seed=rows)
    x = synth.normal_f32(cols, seed=11)
    bw, bx, by = ctx.buffer_bytes(w), ctx.buffer_f32(x), ctx.buffer_empty_f32(rows)
    eng.matvec_wd(ctx, rows, cols, DType.Q6K, bw, bx, by, sched)
    assert_close(ctx.read_f32(by, rows), oracle.matvec(oracle.Q6K, w, rows, cols, x), TOL, f"q6k {rows}x{cols} {sched}")


@pytest.mark.parametrize("rows,cols", [(8, 2048), (1000, 2048), (4099, 2048), (300, 4096), (1, 2048), (1000, 1536), (7, 1536)])
@pytest.mark.parametrize("sched", SCHEDS_Q6K)
def test_matvec_q6k_row_grouped(ctx, eng, rows, cols, sched):
    """The LM head's storage form: the device repack is the stated byte permutation, and the GEMV over it gives
    what the oracle gives for the original Q6_K bytes."""
    w = synth.q6k_blocks(rows * cols // 256, seed=rows + 1)
    x = synth.normal_f32(cols, seed=12)
    want_rows = q6k_rows(w, rows, cols)           # (1536-column rows are padded from 1260 to 1264 bytes)
    bw, br = ctx.buffer_bytes(w), ctx.buffer_empty_bytes(want_rows.size)
    eng.repack_rows(ctx, rows, cols, bw, br)
    assert np.array_equal(ctx.read_bytes(br, want_rows.size), want_rows)
    by = ctx.buffer_empty_f32(rows)
    eng.matvec_wd(ctx, rows, cols, DType.Q6K_ROWS, br, ctx.buffer_f32(x), by, sched)
    assert_close(ctx.read_f32(by, rows), oracle.matvec(oracle.Q6K, w, rows, cols, x), TOL, f"q6k rows {rows}x{cols} {sched}")
    assert_close(ctx.read_f32(by, rows), oracle.matvec_f64(oracle.Q6K, w, rows, cols, x), 1e-5, "vs f64")


def test_matvec_q6k_row_grouped_unit_vectors_and_errors(ctx, eng):
    rows, cols = 4, 2048
    w = synth.q6k_blocks(rows * cols // 256, seed=5)
    wd = oracle.dequant(oracle.Q6K, w, rows * cols).reshape(rows, cols)
    br, by = ctx.buffer_bytes(q6k_rows(w, rows, cols)), ctx.buffer_empty_f32(rows)
    for j in [0, 7, 8, 15, 16, 31, 32, 64, 96, 127, 128, 255, 256, 2047]:   # pins the position of every field
        e = np.zeros(cols, dtype=np.float32)
        e[j] = 1.0
        eng.matvec_wd(ctx, rows, cols, DType.Q6K_ROWS, br, ctx.buffer_f32(e), by)
        assert np.allclose(ctx.read_f32(by, rows), wd[:, j], rtol=1e-6, atol=1e-9), j
    with pytest.raises(hip.KshError, match="1536, 2048 and 4096"):
        ctx.compile(hip.make_desc(hip.Kind.MATVEC, (64, 1024), (DType.Q6K_ROWS, DType.F32)))
    with pytest.raises(hip.KshError, match="multiple of 256"):
        ctx.compile(hip.make_desc(hip.Kind.REPACK_ROWS, (64, 1000), (DType.Q6K, DType.Q6K_ROWS)))
    # 1536 columns: six of a step's eight superblock slots hold weights
    rows, cols = 3, 1536
    w = synth.q6k_blocks(rows * cols // 256, seed=6)
    wd = oracle.dequant(oracle.Q6K, w, rows * cols).reshape(rows, cols)
    br, by = ctx.buffer_bytes(q6k_rows(w, rows, cols)), ctx.buffer_empty_f32(rows)
    for j in [0, 127, 128, 255, 256, 1279, 1280, 1535]:
        e = np.zeros(cols, dtype=np.float32)
        e[j] = 1.0
        eng.matvec_wd(ctx, rows, cols, DType.Q6K_ROWS, br, ctx.buffer_f32(e), by)
        assert np.allclose(ctx.read_f32(by, rows), wd[:, j], rtol=1e-6, atol=1e-9), j
    with pytest.raises(hip.KshError, match="only Q6_K"):
        ctx.compile(hip.make_desc(hip.Kind.REPACK_ROWS, (64, 2048), (DType.Q4K, DType.Q6K_ROWS)))


def test_matvec_q6k_unit_vectors(ctx, eng):
    rows, cols = 4, 2048
    w = synth.q6k_blocks(rows * cols // 256, seed=4)
    wd = oracle.dequant(oracle.Q6K, w, rows * cols).reshape(rows, cols)
    bw, by = ctx.buffer_bytes(w), ctx.buffer_empty_f32(rows)
    for j in [0, 7, 8, 15, 16, 31, 32, 64, 96, 127, 128, 255, 256, 2047]:
        e = np.zeros(cols, dtype=np.float32)
        e[j] = 1.0
        eng.matvec_wd(ctx, rows, cols, DType.Q6K, bw, ctx.buffer_f32(e), by)
        assert np.allclose(ctx.read_f32(by, rows), wd[:, j], rtol=1e-6, atol=1e-9), j


def test_lm_head_cfg1_full_size_with_argmax(ctx, eng):
    rows, cols = 262144, 2048
    w, x = synth.cfg1_q6k_lm_head()
    bw, bx, by = ctx.buffer_bytes(w), ctx.buffer_f32(x), ctx.buffer_empty_f32(rows)
    bi = ctx.buffer_empty_f32(1)
    eng.matvec_wd(ctx, rows, cols, DType.Q6K, bw, bx, by)
    eng.softcap_argmax(ctx, rows, 30.0, by, bi)
    got = ctx.read_f32(by, rows)
    want = oracle.matvec(oracle.Q6K, w, rows, cols, x)
    assert_close(got, want, TOL, "cfg1 logits")
    # the GPU argmax of the GPU logits follows the oracle's rule on the same logits ...
    assert int(ctx.read_f32(bi, 1)[0]) == oracle.softcap_argmax(got, 30.0)
    # ... and equals the oracle's token whenever the oracle's top-2 margin exceeds the tolerance
    top2 = np.sort(want)[-2:]
    if top2[1] - top2[0] > 2 * TOL * abs(top2[1]):
        assert int(ctx.read_f32(bi, 1)[0]) == oracle.softcap_argmax(want, 30.0)


@pytest.mark.parametrize("q_rows,kv_rows,cols", [(2048, 256, 2048), (512, 256, 4096), (100, 36, 1024), (2048, 256, 1536), (77, 19, 1536)])
def test_matvec_qkv(ctx, eng, q_rows, kv_rows, cols):
    ws = [synth.q4k_blocks(r * cols // 256, seed=20 + i) for i, r in enumerate((q_rows, kv_rows, kv_rows))]
    x = synth.normal_f32(cols, seed=23)
    bws = [ctx.buffer_bytes(w) for w in ws]
    outs = [ctx.buffer_empty_f32(r) for r in (q_rows, kv_rows, kv_rows)]
    eng.matvec_qkv_wds(ctx, q_rows, kv_rows, cols, DType.Q4K, *bws, ctx.buffer_f32(x), *outs)
    for w, r, o in zip(ws, (q_rows, kv_rows, kv_rows), outs):
        assert_close(ctx.read_f32(o, r), oracle.matvec(oracle.Q4K, w, r, cols, x), TOL, f"qkv {r}")


@pytest.mark.parametrize("rows,cols", [(8192, 2048), (100, 4096), (64, 512), (6144, 1536), (12288, 1536), (45, 1536)])
def test_matvec_gate_up_gelu(ctx, eng, rows, cols):
    wg = synth.q4k_blocks(rows * cols // 256, seed=30)
    wu = synth.q4k_blocks(rows * cols // 256, seed=31)
    x = synth.normal_f32(cols, seed=32, std=0.05)      # keeps gate values inside GELU's curved range
    out = ctx.buffer_empty_f32(rows)
    eng.matvec_gate_up_gelu_wd(ctx, rows, cols, DType.Q4K, ctx.buffer_bytes(wg), ctx.buffer_bytes(wu), ctx.buffer_f32(x), out)
    g = oracle.matvec(oracle.Q4K, wg, rows, cols, x)
    u = oracle.matvec(oracle.Q4K, wu, rows, cols, x)
    assert_close(ctx.read_f32(out, rows), oracle.gelu_mul(g, u), TOL, "gate_up_gelu")


@pytest.mark.parametrize("sched", [None, dict(tg=256, vec=1, unroll=1, nsg=4, nr0=2, k_split=1, lds_tile=0)])
@pytest.mark.parametrize("has_res", [False, True])
def test_rmsnorm_matvec_prologues(ctx, eng, has_res, sched):
    """RmsNormMatvec / RmsNormMatvecQkv / RmsNormMatvecGateUpGelu, alone and with the previous block's
    residual add folded in, against the unfused oracle ops."""
    n, eps = 2048, 1e-6
    x, w_norm, w_post, res = (synth.normal_f32(n, 700 + i) for i in range(4))
    w_norm, w_post = 1.0 + 0.1 * w_norm, 1.0 + 0.1 * w_post
    if has_res:
        x_new, vec = oracle.rmsnorm_add_then_rmsnorm(x, w_post, res, w_norm, eps)
    else:
        x_new, vec = None, oracle.rmsnorm(x, w_norm, eps)
    bx, bwn, bwp, br = (ctx.buffer_f32(a) for a in (x, w_norm, w_post, res))
    extra = dict(w_post=bwp, res=br) if has_res else {}

    def check_xnew(b):
        if has_res:
            assert_close(ctx.read_f32(b, n), x_new, 1e-5, "x_new")
            assert np.array_equal(ctx.read_f32(br, n), res)          # the old residual stream is left alone

    # plain
    rows = 2048
    w = synth.q4k_blocks(rows * n // 256, seed=710)
    y, xn = ctx.buffer_empty_f32(rows), ctx.buffer_empty_f32(n)
    eng.rmsnorm_matvec_wd(ctx, rows, n, eps, DType.Q4K, bx, bwn, ctx.buffer_bytes(w), y, x_new=xn if has_res else None, sched=sched, **extra)
    assert_close(ctx.read_f32(y, rows), oracle.matvec(oracle.Q4K, w, rows, n, vec), TOL, "rms_matvec")
    check_xnew(xn)
    # qkv
    ws = [synth.q4k_blocks(r * n // 256, seed=711 + i) for i, r in enumerate((2048, 256, 256))]
    outs = [ctx.buffer_empty_f32(r) for r in (2048, 256, 256)]
    xn = ctx.buffer_empty_f32(n)
    eng.rmsnorm_matvec_qkv_w(ctx, 2048, 256, n, eps, DType.Q4K, bx, bwn, *[ctx.buffer_bytes(a) for a in ws], *outs,
                             x_new=xn if has_res else None, sched=sched, **extra)
    for a, r, o in zip(ws, (2048, 256, 256), outs):
        assert_close(ctx.read_f32(o, r), oracle.matvec(oracle.Q4K, a, r, n, vec), TOL, "rms_qkv")
    check_xnew(xn)
    # gate-up
    rows = 8192
    wg, wu = synth.q4k_blocks(rows * n // 256, seed=720), synth.q4k_blocks(rows * n // 256, seed=721)
    out, xn = ctx.buffer_empty_f32(rows), ctx.buffer_empty_f32(n)
    eng.rmsnorm_matvec_gate_up_gelu_w(ctx, rows, n, eps, DType.Q4K, bx, bwn, ctx.buffer_bytes(wg), ctx.buffer_bytes(wu), out,
                                      x_new=xn if has_res else None, sched=sched, **extra)
    v2 = vec * np.float32(0.05)
    g, u = oracle.matvec(oracle.Q4K, wg, rows, n, vec), oracle.matvec(oracle.Q4K, wu, rows, n, vec)
    assert_close(ctx.read_f32(out, rows), oracle.gelu_mul(g, u), TOL, "rms_gate_up")
    check_xnew(xn)


@pytest.mark.parametrize("has_res", [False, True])
def test_rmsnorm_matvec_q6k_lm_head_prologue(ctx, eng, has_res):
    """The LM head with the output norm (and the last layer's residual add) in its prologue."""
    n, rows, eps = 2048, 3000, 1e-6
    x, w_norm, w_post, res = (synth.normal_f32(n, 800 + i) for i in range(4))
    w_norm, w_post = 1.0 + 0.1 * w_norm, 1.0 + 0.1 * w_post
    if has_res:
        x_new, vec = oracle.rmsnorm_add_then_rmsnorm(x, w_post, res, w_norm, eps)
    else:
        x_new, vec = None, oracle.rmsnorm(x, w_norm, eps)
    w = synth.q6k_blocks(rows * n // 256, seed=810)
    bx, bwn, bwp, br = (ctx.buffer_f32(a) for a in (x, w_norm, w_post, res))
    y, xn = ctx.buffer_empty_f32(rows), ctx.buffer_empty_f32(n)
    extra = dict(w_post=bwp, res=br, x_new=xn) if has_res else {}
    for dt, wb in ((DType.Q6K, w), (DType.Q6K_ROWS, q6k_rows(w, rows, n))):
        eng.rmsnorm_matvec_wd(ctx, rows, n, eps, dt, bx, bwn, ctx.buffer_bytes(wb), y, **extra)
        assert_close(ctx.read_f32(y, rows), oracle.matvec(oracle.Q6K, w, rows, n, vec), TOL, f"rms_matvec_q6k {dt}")
        assert_close(ctx.read_f32(y, rows), oracle.matvec_f64(oracle.Q6K, w, rows, n, vec), 1e-5, f"rms_matvec_q6k vs f64 {dt}")
        if has_res:
            assert_close(ctx.read_f32(xn, n), x_new, 1e-5, "x_new")


def test_beam_search_on_device(ctx, eng, tmp_path, monkeypatch):
    """Eng::beam_matvec (ksearch_kernels/src/lib.rs:1985-2043): every candidate is timed on the device, the best one
    is saved as a plan under KSEARCH_BEAM_CACHE, a second search is served from the file, and a kernel compiled
    with an all-zero schedule then picks the plan up."""
    monkeypatch.setenv("KSEARCH_BEAM_CACHE", str(tmp_path / "beam"))
    monkeypatch.setenv("KSEARCH_CHIP", "gfx950-test")
    rows, cols = 1024, 2048
    w = synth.q4k_blocks(rows * cols // 256, seed=900)
    x = synth.normal_f32(cols, seed=901)
    bw, bx, by = ctx.buffer_bytes(w), ctx.buffer_f32(x), ctx.buffer_empty_f32(rows)
    best, ms, cached = eng.beam_matvec(ctx, rows, cols, DType.Q4K, bw, bx, by, iters=5, force=True)
    cands = [c.as_dict() for c in hip.beam_candidates(hip.make_desc(hip.Kind.MATVEC, (rows, cols), (DType.Q4K, DType.F32)))]
    assert not cached and 0 < ms < 1.0
    assert any(all(best.as_dict()[k] == c[k] for k in ("nsg", "nr0", "vec")) for c in cands)
    # the search leaves a correct result behind, whichever candidate ran last
    assert_close(ctx.read_f32(by, rows), oracle.matvec(oracle.Q4K, w, rows, cols, x), TOL, "after beam")
    files = list((tmp_path / "beam").glob("*.txt"))
    assert len(files) == 1 and files[0].name.startswith("matvec_q4k_1024x2048_")     # the chip name is in the hash
    best2, ms2, cached2 = eng.beam_matvec(ctx, rows, cols, DType.Q4K, bw, bx, by, iters=5)
    assert cached2 and best2.as_dict() == best.as_dict()


def test_beam_search_over_a_chain_of_layers(ctx, tmp_path, monkeypatch):
    """The search as a model load runs it (Eng::warm_matvec_plans, ksearch_kernels/src/lib.rs:2057-2080): each
    candidate is one graph of dependent launches, one per layer over that layer's weights; the winner is a member of
    the candidate list (or the library's default), it is saved, and the last set's output is that set's product."""
    monkeypatch.setenv("KSEARCH_BEAM_CACHE", str(tmp_path / "beam"))
    rows, cols, n_sets = 512, 1024, 5
    ws = [synth.q4k_blocks(rows * cols // 256, seed=910 + i) for i in range(n_sets)]
    x = synth.normal_f32(cols, seed=920)
    bx = ctx.buffer_f32(x)
    bws = [ctx.buffer_bytes(w) for w in ws]
    bys = [ctx.buffer_empty_f32(rows) for _ in range(n_sets)]
    desc = hip.make_desc(hip.Kind.MATVEC, (rows, cols), (DType.Q4K, DType.F32))
    best, ms, cached = ctx.beam_search_chain(desc, [[w, bx] for w in bws], [[y] for y in bys], iters=3, force=True)
    assert not cached and 0 < ms < 1.0
    for w, y in zip(ws, bys):
        assert_close(ctx.read_f32(y, rows), oracle.matvec(oracle.Q4K, w, rows, cols, x), TOL, "after chain search")
    files = list((tmp_path / "beam").glob("*.txt"))
    assert len(files) == 1 and files[0].name.startswith("matvec_q4k_512x1024_")
    best2, _, cached2 = ctx.beam_search_chain(desc, [[w, bx] for w in bws], [[y] for y in bys])
    assert cached2 and best2.as_dict() == best.as_dict()
    # bad arguments are errors, not crashes
    with pytest.raises(hip.KshError):
        ctx.beam_search_chain(hip.make_desc(hip.Kind.RMSNORM_ADD_THEN_RMSNORM, (64,), (), (1e-6,)), [[bx]], [[bys[0]]], force=True)
