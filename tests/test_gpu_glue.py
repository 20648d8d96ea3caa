"""HIP glue ops of a decode step vs the CPU oracle.  Integer outputs (Q4_0
codes, argmax index) are compared exactly; float outputs to 1e-5 relative."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip, synth
from ksearch_amd.hip import DType
from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = hip.Context()
    yield c
    c.close()


@pytest.fixture(scope="module")
def eng():
    return hip.Eng()


@pytest.mark.parametrize("n", [2048, 256, 1000, 8192])
def test_rmsnorm_family(ctx, eng, n):
    eps = 1e-6
    x, w, r, w2 = (synth.normal_f32(n, 200 + i) for i in range(4))
    bx, bw, br, bw2 = (ctx.buffer_f32(a) for a in (x, w, r, w2))
    o1, o2 = ctx.buffer_empty_f32(n), ctx.buffer_empty_f32(n)
    eng.rmsnorm(ctx, n, eps, bx, bw, o1)
    assert_close(ctx.read_f32(o1, n), oracle.rmsnorm(x, w, eps), 1e-5, "rmsnorm")
    eng.rmsnorm_add(ctx, n, eps, bx, bw, br, o1)
    assert_close(ctx.read_f32(o1, n), oracle.rmsnorm(x, w, eps, res=r), 1e-5, "rmsnorm_add")
    eng.rmsnorm_add_scale(ctx, n, eps, 0.25, bx, bw, br, o1)
    assert_close(ctx.read_f32(o1, n), oracle.rmsnorm(x, w, eps, res=r, scale=0.25), 1e-5, "rmsnorm_add_scale")
    eng.rmsnorm_add_then_rmsnorm(ctx, n, eps, bx, bw, br, bw2, o1, o2)
    wx, wx2 = oracle.rmsnorm_add_then_rmsnorm(x, w, r, w2, eps)
    assert_close(ctx.read_f32(o1, n), wx, 1e-5, "add_then x")
    assert_close(ctx.read_f32(o2, n), wx2, 1e-5, "add_then x2")
    # in place, as the decode loop uses it (out_x aliases the residual, out_x2 aliases y)
    by, bres = ctx.buffer_f32(x), ctx.buffer_f32(r)
    eng.rmsnorm_add_then_rmsnorm(ctx, n, eps, by, bw, bres, bw2, bres, by)
    assert_close(ctx.read_f32(bres, n), wx, 1e-5, "in-place x")
    assert_close(ctx.read_f32(by, n), wx2, 1e-5, "in-place x2")


def test_rmsnorm_add_then_rmsnorm_refuses_large_n(ctx):
    with pytest.raises(hip.KshError, match="LOCAL staging"):
        ctx.compile(hip.make_desc(hip.Kind.RMSNORM_ADD_THEN_RMSNORM, (16384,), (), (1e-6,)))


def test_quantize_q40_bit_exact(ctx, eng):
    n = 32 * 1001
    v = synth.normal_f32(n, 210)
    v[64:96] = 0.0                      # all-zero block: scale 1, codes 8
    v[96:128] = np.float32(3.0)         # constant block
    v[128] = 1e-7                       # below half's subnormal range
    v[160:192] *= 1e4                   # large magnitudes (still finite in half)
    src, dst = ctx.buffer_f32(v), ctx.buffer_empty_bytes(n // 32 * 18)
    eng.quantize_q40(ctx, n, src, dst)
    got, want = ctx.read_bytes(dst, n // 32 * 18), oracle.pack_q40(v)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("n_q,n_kv,hd", [(8, 1, 256), (4, 2, 128), (8, 1, 512)])
@pytest.mark.parametrize("pos", [0, 5, 1000])
def test_rmsnorm_per_head_qkv_q40(ctx, eng, n_q, n_kv, hd, pos):
    eps, max_seq = 1e-6, 1024 + 8
    q, k, v = (synth.normal_f32(r * hd, 220 + i) for i, r in enumerate((n_q, n_kv, n_kv)))
    qw, kw = synth.normal_f32(hd, 223), synth.normal_f32(hd, 224)
    rope = oracle.rope_table(max_seq, hd, 10000.0)
    row_bytes = n_kv * hd // 32 * 18
    bq, bk, bv = ctx.buffer_f32(q), ctx.buffer_f32(k), ctx.buffer_f32(v)
    kc, vc = ctx.buffer_empty_bytes(max_seq * row_bytes), ctx.buffer_empty_bytes(max_seq * row_bytes)
    # in place for Q, as forward_token does (gemma_prim.rs:983-990)
    eng.rmsnorm_per_head_qkv_q40_off(ctx, n_q, n_kv, hd, eps, bq, ctx.buffer_f32(qw), ctx.buffer_f32(rope), pos * hd,
                                     bk, ctx.buffer_f32(kw), bv, bq, kc, vc, pos * row_bytes)
    wq, wk, wv = oracle.rmsnorm_per_head_qkv_q40(q, qw, rope[pos], k, kw, v, n_q, n_kv, hd, eps)
    assert_close(ctx.read_f32(bq, n_q * hd), wq, 1e-5, "q")
    gk, gv = ctx.read_bytes(kc, row_bytes, pos * row_bytes), ctx.read_bytes(vc, row_bytes, pos * row_bytes)
    # Q4_0 codes are integer functions of f32 values that can differ in the last
    # bits between the two sides (reduction order of the RMS sum): compare the
    # dequantized rows to within one code step, and count exact byte agreement
    for got, want in ((gk, wk), (gv, wv)):
        dg, dw = oracle.dequant(oracle.Q40, got, n_kv * hd), oracle.dequant(oracle.Q40, want, n_kv * hd)
        step = np.abs(dw).max() / 7.0
        assert np.abs(dg - dw).max() <= step * 1.01
        assert (got != want).mean() < 0.02
    # untouched rows stay zero
    if pos:
        assert not ctx.read_bytes(kc, row_bytes, (pos - 1) * row_bytes).any()


def test_copy_scale_indexed_q6k_rows(ctx, eng):
    n, rows = 2048, 50
    E = synth.q6k_blocks(rows * n // 256, seed=230)
    be, out = ctx.buffer_bytes(E), ctx.buffer_empty_f32(n)
    scale = float(np.sqrt(np.float32(n)))
    for tok in (0, 7, 49):
        eng.copy_scale_indexed_wd(ctx, n, scale, DType.Q6K, be, ctx.buffer_f32([float(tok)]), out, rows)
        want = oracle.copy_scale_indexed(oracle.Q6K, E, tok, n, scale)
        assert np.array_equal(ctx.read_f32(out, n).view(np.uint32), want.view(np.uint32))
    E4 = synth.q4k_blocks(rows * n // 256, seed=231)
    eng.copy_scale_indexed_wd(ctx, n, scale, DType.Q4K, ctx.buffer_bytes(E4), ctx.buffer_f32([3.0]), out, rows)
    want = oracle.copy_scale_indexed(oracle.Q4K, E4, 3, n, scale)
    assert np.array_equal(ctx.read_f32(out, n).view(np.uint32), want.view(np.uint32))


def test_gelu_mul_and_copy_slice(ctx, eng):
    n = 8192
    g, u = synth.normal_f32(n, 240, std=3.0), synth.normal_f32(n, 241)
    g[:4] = [-30.0, 30.0, 0.0, -0.0]
    out = ctx.buffer_empty_f32(n)
    eng.gelu_mul(ctx, n, ctx.buffer_f32(g), ctx.buffer_f32(u), out)
    assert_close(ctx.read_f32(out, n), oracle.gelu_mul(g, u), 1e-5, "gelu_mul")
    dst = ctx.buffer_empty_f32(n)
    eng.copy_slice(ctx, 100, ctx.buffer_f32(g), 17, dst, 5)
    got = ctx.read_f32(dst, n)
    assert np.array_equal(got[5:105], g[17:117]) and not got[:5].any() and not got[105:].any()


def test_softcap_argmax(ctx, eng):
    out = ctx.buffer_empty_f32(1)

    def run(x, cap=30.0):
        x = np.asarray(x, dtype=np.float32)
        eng.softcap_argmax(ctx, x.size, cap, ctx.buffer_f32(x), out)
        return int(ctx.read_f32(out, 1)[0])

    assert run([1.0, 9.0, 3.0]) == 1                       # sample.rs:92-96
    assert run([5.0, 7.0, 7.0, 2.0]) == 1                  # ties: lowest index
    assert run([1000.0, 2000.0, -5.0]) == 0                # both saturate to cap
    x = synth.normal_f32(262144, 250)
    assert run(x) == oracle.softcap_argmax(x, 30.0) == int(np.argmax(x))
    x[1234] = x[200000] = 50.0                             # a tie far apart, across workgroups
    assert run(x) == 1234
    x = synth.normal_f32(1000, 251)
    assert run(x) == oracle.softcap_argmax(x, 30.0)
    assert run(x, cap=0.0) == int(np.argmax(x))


def test_fill_zero_and_transfers(ctx):
    for n in (1, 15, 16, 17, 4096 + 3):
        b = ctx.buffer_bytes(np.full(n, 0xAB, dtype=np.uint8))
        ctx.fill_zero(b)
        assert not ctx.read_bytes(b, n).any()
    b = ctx.buffer_empty_f32(8)
    assert ctx.has_gpu_work() is False
    ctx.write_buffer_nosync(b, [1, 2, 3], off=8)
    assert np.array_equal(ctx.read_f32(b, 8), [0, 0, 1, 2, 3, 0, 0, 0])
    with pytest.raises(hip.KshError, match="exceeds"):
        ctx.write_buffer(b, np.zeros(9))
    with pytest.raises(hip.KshError, match="exceeds"):
        ctx.read_f32(b, 4, off=20)


def test_flush_wait_and_graph_replay(ctx, eng):
    rows, cols = 256, 2048
    w = synth.q4k_blocks(rows * cols // 256, seed=260)
    bw, by = ctx.buffer_bytes(w), ctx.buffer_empty_f32(rows)
    bx = ctx.buffer_empty_f32(cols)
    eng.matvec_wd(ctx, rows, cols, DType.Q4K, bw, bx, by)       # bind outside the capture
    ctx.synchronize()
    assert not ctx.has_gpu_work()
    eng.matvec_wd(ctx, rows, cols, DType.Q4K, bw, bx, by)
    assert ctx.has_gpu_work()
    ctx.flush_async()
    ctx.flush_async()                                           # nothing pending: no second event
    ctx.wait_inflight_at_most(0)
    assert not ctx.has_gpu_work()
    ctx.graph_begin()
    eng.matvec_wd(ctx, rows, cols, DType.Q4K, bw, bx, by)
    with pytest.raises(hip.KshError, match="captured"):
        ctx.synchronize()
    g = ctx.graph_end()
    # replay several times with fresh inputs and eager work in between
    for i in range(4):
        x = synth.normal_f32(cols, seed=270 + i)
        ctx.write_buffer(bx, x)
        ctx.graph_launch(g)
        got = ctx.read_f32(by, rows)
        assert_close(got, oracle.matvec(oracle.Q4K, w, rows, cols, x), 1e-3, f"replay {i}")
        ctx.fill_zero(by)
        ctx.synchronize()
    ctx.graph_destroy(g)
