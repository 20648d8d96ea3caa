"""The decode round's GEMMs (KSH_ROUND_PREP + KSH_MATVEC_ROUND: up to 16 f32 rows against Q4_K matrices on the matrix
cores, several matrices or a gate | up pair per launch) vs the CPU oracle's dequant + sequential f32 dot per row,
1e-3 relative; against the float64 product where the claim is the GEMV's accuracy; one-hot rows recover the
dequantized columns."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip, synth
from ksearch_amd.hip import DType, Kind
from tests.gpu_util import assert_close, q6k_rows

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = hip.Context()
    yield c
    c.close()


def prepared(ctx, x, batch, cols):
    kp = ctx.compile(hip.make_desc(Kind.ROUND_PREP, (cols, batch), (DType.F32,)))
    xp = ctx.buffer_empty_bytes(64 * cols + 2048 * (cols // 256))
    ctx.encode_multi(kp, [ctx.buffer_f32(x.reshape(-1))], [xp])
    return xp


def round_mm(ctx, ws, rows, cols, x, batch, pair=False):
    xp = prepared(ctx, x, batch, cols)
    r = list(rows) + [0] * (3 - len(rows))
    k = ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (r[0], cols, batch, 0 if pair else r[1], r[2], int(pair)), (DType.Q4K,)))
    bw = [ctx.buffer_bytes(w) for w in ws]
    outs = [ctx.buffer_empty_f32(batch * rows[0])] if pair else [ctx.buffer_empty_f32(batch * n) for n in rows]
    ctx.encode_multi(k, [bw[0], xp] + bw[1:], outs)
    ctx.synchronize()
    return k, [ctx.read_f32(o, batch * n).reshape(batch, n) for o, n in zip(outs, rows)]


@pytest.mark.parametrize("rows,cols,batch", [
    ((2048,), 1536, 16),            # q of the real checkpoints' layout
    ((2048, 256, 256), 1536, 16),   # q | k | v in one launch
    ((2048, 256), 2048, 5),         # two matrices, every wave busy
    ((100,), 256, 1),               # one row of input, a ragged tile, one superblock
    ((1536,), 6144, 16),            # down: columns split over three workgroups per tile
    ((1536,), 12288, 7),            # the double-wide feed-forward: six slices
    ((33, 1, 31), 512, 3),          # tiles that end inside a matrix
])
def test_matvec_round_vs_oracle(ctx, rows, cols, batch):
    ws = [synth.q4k_blocks(n * cols // 256, seed=900 + i + n) for i, n in enumerate(rows)]
    x = synth.normal_f32(batch * cols, 901).reshape(batch, cols)
    k, got = round_mm(ctx, ws, rows, cols, x, batch)
    assert ("ksplit" in k.name) == (cols > 2048)
    for w, n, g in zip(ws, rows, got):
        want = oracle.matmul(oracle.Q4K, w, n, cols, x, batch)
        assert_close(g, want, 1e-3, f"round {n}x{cols} b{batch}")
        for t in (0, batch - 1):   # the GEMV's accuracy: f32 activations keep 22 bits
            w64 = oracle.matvec_f64(oracle.Q4K, w, n, cols, x[t])
            err = np.max(np.abs(g[t] - w64) / np.maximum(np.abs(w64), np.sqrt(np.mean(w64 ** 2))))
            assert err < 2e-5, err


@pytest.mark.parametrize("rows,cols,batch", [(6144, 1536, 16), (12288, 1536, 3), (96, 2048, 9)])
def test_matvec_round_gate_up_gelu(ctx, rows, cols, batch):
    wg, wu = synth.q4k_blocks(rows * cols // 256, seed=910), synth.q4k_blocks(rows * cols // 256, seed=911)
    x = synth.normal_f32(batch * cols, 912).reshape(batch, cols) * 0.25
    k, (got,) = round_mm(ctx, [wg, wu], (rows,), cols, x, batch, pair=True)
    assert "gate_up_gelu" in k.name
    g, u = oracle.matmul(oracle.Q4K, wg, rows, cols, x, batch), oracle.matmul(oracle.Q4K, wu, rows, cols, x, batch)
    assert_close(got, oracle.gelu_mul(g.reshape(-1), u.reshape(-1)).reshape(batch, rows), 1e-3, f"gate|up {rows}x{cols} b{batch}")


@pytest.mark.parametrize("batch", [16, 3])
def test_matvec_round_result_as_prepared_operand(ctx, batch):
    """dims[6] = 1: a launch's result leaves as the next GEMM's prepared operand (here gate | up -> down, and the
    per-layer-embedding gate with its multiplier -> projection); the values it holds are the f32 results' to 2^-20."""
    rows, cols = 512, 1536
    wg, wu = synth.q4k_blocks(rows * cols // 256, seed=970), synth.q4k_blocks(rows * cols // 256, seed=971)
    x = synth.normal_f32(batch * cols, 972).reshape(batch, cols) * 0.25
    _, (plain,) = round_mm(ctx, [wg, wu], (rows,), cols, x, batch, pair=True)
    xp = prepared(ctx, x, batch, cols)
    out = ctx.buffer_empty_bytes(64 * rows + 2048 * (rows // 256))
    k = ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (rows, cols, batch, 0, 0, 1, 1), (DType.Q4K,)))
    assert k.name.endswith("_prepared")
    ctx.encode_multi(k, [ctx.buffer_bytes(wg), xp, ctx.buffer_bytes(wu)], [out])
    vals, sums = xp_values(ctx, out, rows)
    want = np.zeros((16, rows))
    want[:batch] = plain
    assert np.max(np.abs(vals - want) / np.maximum(np.abs(want), 2.0 ** -10 * np.abs(want).max())) < 2.0 ** -20
    assert np.allclose(sums, want.reshape(16, -1, 32).sum(axis=2), rtol=0, atol=2e-3 * np.abs(want).max())
    # the gate with its multiplier: gelu(W x) * ctx[t, r], ctx rows `stride` apart
    stride = 3 * rows
    ctxv = synth.normal_f32(batch * stride, 973).reshape(batch, stride)
    k2 = ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (rows, cols, batch, 0, 0, 0, 0, stride), (DType.Q4K,)))
    y = ctx.buffer_empty_f32(batch * rows)
    ctx.encode_offsets_multi(k2, [ctx.buffer_bytes(wg), xp, ctx.buffer_f32(ctxv.reshape(-1))], [0, 0, rows * 4], [y], [0])
    g = oracle.matmul(oracle.Q4K, wg, rows, cols, x, batch)
    want2 = oracle.gelu_mul(g.reshape(-1), ctxv[:, rows:2 * rows].reshape(-1)).reshape(batch, rows)
    assert_close(ctx.read_f32(y, batch * rows).reshape(batch, rows), want2, 1e-3, "gelu(W x) * ctx")
    k3 = ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (rows, cols, batch, 0, 0, 0, 1, stride), (DType.Q4K,)))
    ctx.encode_offsets_multi(k3, [ctx.buffer_bytes(wg), xp, ctx.buffer_f32(ctxv.reshape(-1))], [0, 0, rows * 4], [out], [0])
    vals, _ = xp_values(ctx, out, rows)
    assert np.allclose(vals[:batch], ctx.read_f32(y, batch * rows).reshape(batch, rows), rtol=2.0 ** -19, atol=1e-6)


def test_matvec_round_partial_sums_into_the_closing_norm(ctx):
    """dims[6] = 2 leaves a split GEMM's column slices unadded, and KSH_ROUND_PREP with dims[3] = slices adds them
    on its way into the norm: the same x_new and operand as the folded GEMM followed by the plain norm kinds."""
    rows, cols, batch, eps = 1536, 6144, 9, 1e-6
    w = synth.q4k_blocks(rows * cols // 256, seed=980)
    x = synth.normal_f32(batch * cols, 981).reshape(batch, cols) * 0.1
    res, wn = synth.normal_f32(batch * rows, 982), (1.0 + 0.05 * synth.normal_f32(rows, 983)).astype(np.float32)
    _, (y,) = round_mm(ctx, [w], (rows,), cols, x, batch)
    xp = prepared(ctx, x, batch, cols)
    k = ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (rows, cols, batch, 0, 0, 0, 2), (DType.Q4K,)))
    slices = k.info.sched.k_split
    assert slices == 3
    parts = ctx.buffer_empty_f32(slices * batch * rows)
    ctx.encode_multi(k, [ctx.buffer_bytes(w), xp], [parts])
    p = ctx.read_f32(parts, slices * batch * rows).reshape(slices, batch, rows)
    assert np.array_equal((p[0] + p[1] + p[2]).view(np.uint32), y.view(np.uint32))      # slice after slice, as the fold adds them
    n_xp = 64 * rows + 2048 * (rows // 256)
    got, want = ctx.buffer_empty_bytes(n_xp), ctx.buffer_empty_bytes(n_xp)
    xn_got, xn_want = ctx.buffer_empty_f32(batch * rows), ctx.buffer_empty_f32(batch * rows)
    bres, bwn = ctx.buffer_f32(res), ctx.buffer_f32(wn)
    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.ROUND_PREP, (rows, batch, 3, slices), (DType.F32,), (eps,))), [parts, bwn, bres], [got, xn_got])
    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.ROUND_PREP, (rows, batch, 3), (DType.F32,), (eps,))), [ctx.buffer_f32(y.reshape(-1)), bwn, bres], [want, xn_want])
    assert np.array_equal(ctx.read_f32(xn_got, batch * rows).view(np.uint32), ctx.read_f32(xn_want, batch * rows).view(np.uint32))
    assert np.array_equal(ctx.read_bytes(got, n_xp), ctx.read_bytes(want, n_xp))


@pytest.mark.parametrize("hd,sched", [(256, None), (256, dict(vec=3)), (512, None)])
def test_sdpa_slots_result_as_prepared_operand(ctx, hd, sched):
    """KSH_SDPA_SLOTS with params[1] = 1: the merge writes the prepared operand of the o projection; its values are the
    f32 rows' of the plain launch to 2^-20."""
    n_slots, n_q, n_kv, max_t, nwg = 5, 8, 1, 1024, 8
    lens, kk, vv, q = synth.cfg3_q40_attention(n_slots, n_q, n_kv, hd, max_t, lo=1, seed=990)
    meta = np.zeros((n_slots, 4), np.float32)
    meta[:, 0] = lens
    ins = [ctx.buffer_f32(q), ctx.buffer_bytes(kk.reshape(-1)), ctx.buffer_bytes(vv.reshape(-1)), ctx.buffer_f32(meta)]
    cols = n_q * hd
    outs = {}
    for flag in (0.0, 1.0):
        k = ctx.compile(hip.make_desc(Kind.SDPA_SLOTS, (n_q, n_kv, hd, max_t, n_slots, nwg), (DType.Q40, DType.F32), (0.0625, flag), sched))
        tmp = ctx.buffer_empty_f32(n_slots * n_q * k.info.sched.k_split * (hd + 2))
        out = ctx.buffer_empty_bytes(64 * cols + 2048 * (cols // 256)) if flag else ctx.buffer_empty_f32(n_slots * cols)
        ctx.encode_multi(k, ins, [tmp, out])
        outs[flag] = out
    want = np.zeros((16, cols))
    want[:n_slots] = ctx.read_f32(outs[0.0], n_slots * cols).reshape(n_slots, cols)
    vals, sums = xp_values(ctx, outs[1.0], cols)
    err = np.abs(vals[:n_slots] - want[:n_slots]) / np.maximum(np.abs(want[:n_slots]), 2.0 ** -10 * np.abs(want).max())
    assert err.max() < 2.0 ** -20, err.max()
    assert np.allclose(sums[:n_slots], want[:n_slots].reshape(n_slots, -1, 32).sum(axis=2), rtol=0, atol=2e-3 * np.abs(want).max())


def test_matvec_round_unit_rows_recover_weights(ctx):
    # X = one-hot rows: Y[t] is column k_t of the dequantized matrix (pins the K order and the hi | lo tile end to end)
    rows, cols = 64, 4096
    w = synth.q4k_blocks(rows * cols // 256, seed=920)
    wd = oracle.dequant(oracle.Q4K, w, rows * cols).reshape(rows, cols)
    ks = [0, 1, 2, 3, 15, 16, 31, 32, 33, 63, 64, 255, 256, 2047, 2048, 4095]
    x = np.zeros((len(ks), cols), dtype=np.float32)
    for t, kk in enumerate(ks):
        x[t, kk] = 1.0 + 2.0 ** -13      # a value whose lo part is not zero
    _, (got,) = round_mm(ctx, [w], (rows,), cols, x, len(ks))
    for t, kk in enumerate(ks):
        want = wd[:, kk].astype(np.float64) * (1.0 + 2.0 ** -13)
        assert np.allclose(got[t], want, rtol=1e-5, atol=1e-5 * np.abs(wd).max()), kk


def xp_values(ctx, xp, cols):
    """A prepared operand back as numbers: x[16, cols] = hi + 2^-11 lo from the fragments (lane = row + 32 * ((k / 8) % 2)
    per 16 columns, rows 0..15 hi parts and 16..31 lo parts, k stored in the order (0, 2, 1, 3) within every 4), and the
    per-sub-block sums [16, cols / 32] (hi + lo of the f16 pairs, hi part + 2^-11 lo part)."""
    nsb = cols // 256
    raw = ctx.read_bytes(xp, 64 * cols + 2048 * nsb).view(np.float16).astype(np.float64)
    frag = raw[:32 * cols].reshape(cols // 16, 2, 32, 8)        # [slice][k half][row][position]
    perm = [0, 2, 1, 3, 4, 6, 5, 7]                              # position kperm(i) holds k = i
    x = np.empty((32, cols))
    for i in range(8):
        x[:, i::16] = frag[:, 0, :, perm[i]].T
        x[:, 8 + i::16] = frag[:, 1, :, perm[i]].T
    sums = raw[32 * cols:].reshape(2, 16, nsb, 32)
    parts = sums[..., 0:8] + sums[..., 16:24]                   # [part][token][superblock][sub-block]
    return x[:16] + x[16:] / 2048.0, (parts[0] + parts[1] / 2048.0).reshape(16, -1)


@pytest.mark.parametrize("cols,batch", [(1536, 16), (256, 3), (8192, 5)])
def test_round_prep_norm_forms_equal_norm_then_prep(ctx, cols, batch):
    """Modes 1 and 2 of KSH_ROUND_PREP prepare what the rows norms would have written as f32 rows (to the last bit or
    two of f32: the operand keeps 22 bits), mode 2's x_new is the add-then-norm kernel's, and the operand of mode 0
    holds its input to 2^-21."""
    rng = np.random.default_rng(950 + cols)
    x, res = synth.normal_f32(batch * cols, 951), synth.normal_f32(batch * cols, 952)
    w1, w2 = (1.0 + 0.1 * rng.standard_normal(cols)).astype(np.float32), (1.0 + 0.1 * rng.standard_normal(cols)).astype(np.float32)
    eps = 1e-6
    n_xp = 64 * cols + 2048 * (cols // 256)
    bx, br, bw1, bw2 = ctx.buffer_f32(x), ctx.buffer_f32(res), ctx.buffer_f32(w1), ctx.buffer_f32(w2)
    got = ctx.buffer_empty_bytes(n_xp)

    def check(want_rows, what, tol=2.0 ** -20, floor=2.0 ** -10):
        vals, sums = xp_values(ctx, got, cols)
        want = np.zeros((16, cols))
        want[:batch] = want_rows.astype(np.float64).reshape(batch, cols)
        err = np.abs(vals - want) / np.maximum(np.abs(want), floor * np.abs(want).max())
        assert err.max() < tol, (what, err.max(), np.unravel_index(err.argmax(), err.shape))
        assert np.allclose(sums.reshape(16, -1), want.reshape(16, -1, 32).sum(axis=2), rtol=0, atol=2e-3 * np.abs(want).max()), what

    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.ROUND_PREP, (cols, batch), (DType.F32,))), [bx], [got])
    check(x, "mode 0")
    y = ctx.buffer_empty_f32(batch * cols)
    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.RMSNORM, (cols, 0, 0, batch), (), (eps,))), [bx, bw1], [y])
    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.ROUND_PREP, (cols, batch, 1), (DType.F32,), (eps,))), [bx, bw1], [got])
    check(ctx.read_f32(y, batch * cols), "mode 1")
    xn_want, x2 = ctx.buffer_empty_f32(batch * cols), ctx.buffer_empty_f32(batch * cols)
    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.RMSNORM_ADD_THEN_RMSNORM, (cols, batch), (), (eps,))), [bx, bw1, br, bw2], [xn_want, x2])
    xn_got = ctx.buffer_empty_f32(batch * cols)
    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.ROUND_PREP, (cols, batch, 2), (DType.F32,), (eps,))), [bx, bw1, br, bw2], [got, xn_got])
    assert np.allclose(ctx.read_f32(xn_got, batch * cols), ctx.read_f32(xn_want, batch * cols), rtol=1e-6, atol=1e-6)   # (a sum that may cancel)
    # (x_new is a sum that may cancel: the two kernels' last bits of it differ, and the second norm carries that along)
    check(ctx.read_f32(x2, batch * cols), "mode 2", tol=1e-5, floor=0.1)
    # mode 2 with a scale on x_new (rmsnorm_add_scale rows, then the next norm), mode 3 (rmsnorm_add rows, prepared as it is)
    scale = 0.375
    xs = ctx.buffer_empty_f32(batch * cols)
    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.RMSNORM, (cols, 1, 1, batch), (), (eps, scale))), [bx, bw1, br], [xs])
    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.RMSNORM, (cols, 0, 0, batch), (), (eps,))), [xs, bw2], [x2])
    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.ROUND_PREP, (cols, batch, 2), (DType.F32,), (eps, scale))), [bx, bw1, br, bw2], [got, xn_got])
    assert np.allclose(ctx.read_f32(xn_got, batch * cols), ctx.read_f32(xs, batch * cols), rtol=1e-6, atol=1e-6)
    check(ctx.read_f32(x2, batch * cols), "mode 2 with a scale", tol=1e-5, floor=0.1)
    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.RMSNORM, (cols, 1, 0, batch), (), (eps,))), [bx, bw1, br], [xs])
    ctx.encode_multi(ctx.compile(hip.make_desc(Kind.ROUND_PREP, (cols, batch, 3), (DType.F32,), (eps,))), [bx, bw1, br], [got, xn_got])
    assert np.allclose(ctx.read_f32(xn_got, batch * cols), ctx.read_f32(xs, batch * cols), rtol=1e-6, atol=1e-6)
    check(ctx.read_f32(xn_got, batch * cols), "mode 3")


def q6k_blocks_full_scales(n_blocks, seed):
    """Q6_K blocks whose int8 scales use the whole range (sc * q up to 127 * 32: what an f16 operand would round)."""
    w = synth.q6k_blocks(n_blocks, seed=seed).reshape(n_blocks, 210).copy()
    w[:, 192:208] = np.random.default_rng(seed + 1).integers(-128, 128, (n_blocks, 16)).astype(np.int8).view(np.uint8)
    return w.reshape(-1)


@pytest.mark.parametrize("rows,cols,batch,full", [(8192, 1536, 16, False), (4096, 2048, 7, True), (100, 1536, 1, True), (20000, 2048, 16, False)])
def test_matvec_round_q6k_rows(ctx, rows, cols, batch, full):
    """The LM head of a round: row-grouped Q6_K, the scale applied in f32 to the matrix instruction's result, so the
    GEMV's accuracy also holds where |sc * q| passes 2048."""
    nb = rows * cols // 256
    w = q6k_blocks_full_scales(nb, 930) if full else synth.q6k_blocks(nb, seed=930)
    x = synth.normal_f32(batch * cols, 931).reshape(batch, cols)
    xp = prepared(ctx, x, batch, cols)
    k = ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (rows, cols, batch, 0, 0, 0), (DType.Q6K_ROWS,)))
    y = ctx.buffer_empty_f32(batch * rows)
    ctx.encode_multi(k, [ctx.buffer_bytes(q6k_rows(w, rows, cols)), xp], [y])
    got = ctx.read_f32(y, batch * rows).reshape(batch, rows)
    assert_close(got, oracle.matmul(oracle.Q6K, w, rows, cols, x, batch), 1e-3, f"round q6k rows {rows}x{cols} b{batch}")
    for t in (0, batch - 1):
        w64 = oracle.matvec_f64(oracle.Q6K, w, rows, cols, x[t])
        err = np.max(np.abs(got[t] - w64) / np.maximum(np.abs(w64), np.sqrt(np.mean(w64 ** 2))))
        assert err < 2e-5, err


def test_matvec_round_q6k_rows_unit_rows_recover_weights(ctx):
    rows, cols = 64, 2048
    w = q6k_blocks_full_scales(rows * cols // 256, 940)
    wd = oracle.dequant(oracle.Q6K, w, rows * cols).reshape(rows, cols)
    ks = [0, 1, 7, 8, 15, 16, 31, 32, 63, 64, 127, 128, 255, 256, 1000, 2047]
    x = np.zeros((len(ks), cols), dtype=np.float32)
    for t, kk in enumerate(ks):
        x[t, kk] = 1.0
    xp = prepared(ctx, x, len(ks), cols)
    k = ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (rows, cols, len(ks), 0, 0, 0), (DType.Q6K_ROWS,)))
    y = ctx.buffer_empty_f32(len(ks) * rows)
    ctx.encode_multi(k, [ctx.buffer_bytes(q6k_rows(w, rows, cols)), xp], [y])
    got = ctx.read_f32(y, len(ks) * rows).reshape(len(ks), rows)
    for t, kk in enumerate(ks):
        assert np.array_equal(got[t], wd[:, kk]), kk      # d * sc * (q - 32): exact in f32


@pytest.mark.parametrize("n,rows", [(1000, 5), (262144, 16), (7, 2)])
def test_softcap_argmax_rows(ctx, n, rows):
    """The argmax of every row of a round in one launch pair: per row the single-vector kernel's index (lowest index
    wins ties, soft cap applied before comparing)."""
    x = synth.normal_f32(rows * n, 960).reshape(rows, n) * 8.0
    x[0, n // 2] = x[0, n - 1] = 1e9          # a tie after the cap: the lower index
    x[rows - 1, :] = -3.0                     # all equal: index 0
    k = ctx.compile(hip.make_desc(Kind.SOFTCAP_ARGMAX, (n, rows), (), (30.0,)))
    out = ctx.buffer_empty_f32(rows)
    ctx.encode_multi(k, [ctx.buffer_f32(x.reshape(-1))], [out])
    got = ctx.read_f32(out, rows).astype(np.int64)
    assert list(got) == [oracle.softcap_argmax(x[r], 30.0) for r in range(rows)]
    assert got[0] == n // 2 and got[rows - 1] == 0


def test_matvec_round_errors(ctx):
    with pytest.raises(hip.KshError, match="1 to 16"):
        ctx.compile(hip.make_desc(Kind.ROUND_PREP, (1536, 17), (DType.F32,)))
    with pytest.raises(hip.KshError, match="1 to 16"):
        ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (64, 1536, 0, 0, 0, 0), (DType.Q4K,)))
    with pytest.raises(hip.KshError, match="multiple of 256"):
        ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (64, 100, 4, 0, 0, 0), (DType.Q4K,)))
    with pytest.raises(hip.KshError, match="not built"):
        ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (64, 1536, 4, 0, 0, 0), (DType.Q6K,)))
    with pytest.raises(hip.KshError, match="up to 2048 columns"):
        ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (64, 4096, 4, 0, 0, 0), (DType.Q6K_ROWS,)))
    with pytest.raises(hip.KshError, match="one matrix per launch"):
        ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (64, 4096, 4, 64, 0, 0), (DType.Q4K,)))
    with pytest.raises(hip.KshError, match="multiple of 256"):
        ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (96, 1536, 4, 0, 0, 0, 1), (DType.Q4K,)))
    with pytest.raises(hip.KshError, match="one row count"):
        ctx.compile(hip.make_desc(Kind.MATVEC_ROUND, (64, 1536, 4, 64, 0, 1), (DType.Q4K,)))
