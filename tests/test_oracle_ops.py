"""Pins the oracle's GEMV/GEMM, attention, argmax and glue ops against brute
force in float64, closed forms and invariants."""
import numpy as np
import pytest

import oracle
from ksearch_amd import synth
from tests import refforms as rf


def check_mul_mm_inputs(rows, cols, batch):
    """The integer-formula inputs of crates/ksearch_kernels/examples/check_mul_mm.rs:50-59."""
    r = np.arange(rows)[:, None]
    c = np.arange(cols)[None, :]
    w = (((r * 17 + c * 13) % 200).astype(np.float32) - np.float32(100.0)) * np.float32(0.02)
    t = np.arange(batch)[:, None]
    x = (((t * 11 + c * 7) % 50).astype(np.float32) - np.float32(25.0)) * np.float32(0.04)
    return w.astype(np.float32), x.astype(np.float32)


@pytest.mark.parametrize("rows,cols,batch", [(64, 256, 16), (128, 256, 9)])
def test_matmul_check_mul_mm_shapes(rows, cols, batch):
    w, x = check_mul_mm_inputs(rows, cols, batch)
    wq = oracle.quantize_q4k(w)
    wd = oracle.dequant(oracle.Q4K, wq, rows * cols).reshape(rows, cols)
    # the quantizer reproduces this signal to Q4_K accuracy
    assert np.abs(wd - w).max() < 0.15
    got = oracle.matmul(oracle.Q4K, wq, rows, cols, x, batch)
    want = x.astype(np.float64) @ wd.astype(np.float64).T
    mag = np.abs(x.astype(np.float64)) @ np.abs(wd.astype(np.float64)).T
    assert np.all(np.abs(got - want) <= 3e-6 * mag + 1e-12)
    # batch row t equals the GEMV on x[t]
    for t in (0, batch - 1):
        assert np.array_equal(oracle.matvec(oracle.Q4K, wq, rows, cols, x[t]), got[t])


@pytest.mark.parametrize("rows,cols,batch", [(64, 256, 16), (33, 1536, 5)])
def test_matmul_q6k_brute_force(rows, cols, batch):
    # the checker of the Q6_K prefill GEMM: float64 brute force on the dequantized matrix, batch row = GEMV
    w, x = check_mul_mm_inputs(rows, cols, batch)
    wq = oracle.quantize_q6k(w)
    wd = oracle.dequant(oracle.Q6K, wq, rows * cols).reshape(rows, cols)
    assert np.abs(wd - w).max() < 0.05
    got = oracle.matmul(oracle.Q6K, wq, rows, cols, x, batch)
    want = x.astype(np.float64) @ wd.astype(np.float64).T
    mag = np.abs(x.astype(np.float64)) @ np.abs(wd.astype(np.float64)).T
    assert np.all(np.abs(got - want) <= 3e-6 * mag + 1e-12)
    for t in (0, batch - 1):
        assert np.array_equal(oracle.matvec(oracle.Q6K, wq, rows, cols, x[t]), got[t])


@pytest.mark.parametrize("dtype,gen,bpb", [(oracle.Q4K, synth.q4k_blocks, 144), (oracle.Q6K, synth.q6k_blocks, 210)])
def test_matvec_sequential_f32_order(dtype, gen, bpb):
    rows, cols = 6, 512
    w = gen(rows * cols // 256, seed=41)
    x = synth.normal_f32(cols, 42)
    wd = oracle.dequant(dtype, w, rows * cols).reshape(rows, cols)
    got = oracle.matvec(dtype, w, rows, cols, x, threads=1)
    for r in range(rows):
        s = np.float32(0.0)
        for c in range(cols):          # s += w*x, c ascending, two roundings
            s = np.float32(s + np.float32(wd[r, c] * x[c]))
        assert s == got[r]
    got64 = oracle.matvec_f64(dtype, w, rows, cols, x)
    assert np.allclose(got64, wd.astype(np.float64) @ x.astype(np.float64), rtol=1e-13, atol=1e-15)
    # thread count does not change a bit
    assert np.array_equal(got, oracle.matvec(dtype, w, rows, cols, x, threads=0))


def test_matvec_linearity_and_unit_vectors():
    rows, cols = 16, 256
    w = synth.q4k_blocks(rows, seed=43)
    wd = oracle.dequant(oracle.Q4K, w, rows * cols).reshape(rows, cols)
    for j in (0, 31, 32, 100, 255):
        e = np.zeros(cols, dtype=np.float32)
        e[j] = 1.0
        assert np.array_equal(oracle.matvec(oracle.Q4K, w, rows, cols, e), wd[:, j])
    x = synth.normal_f32(cols, 44)
    a = oracle.matvec(oracle.Q4K, w, rows, cols, x)
    b = oracle.matvec(oracle.Q4K, w, rows, cols, 2.0 * x)
    assert np.array_equal(b, 2.0 * a)


def _kv(n_tok, n_kv, hd, seed):
    k = synth.q40_blocks(n_tok * n_kv * hd // 32, seed)
    v = synth.q40_blocks(n_tok * n_kv * hd // 32, seed + 1)
    kd = oracle.dequant(oracle.Q40, k, n_tok * n_kv * hd).reshape(n_tok, n_kv, hd)
    vd = oracle.dequant(oracle.Q40, v, n_tok * n_kv * hd).reshape(n_tok, n_kv, hd)
    return k, v, kd, vd


@pytest.mark.parametrize("n_q,n_kv,hd,max_t,tlen,start,scale", [
    (2, 1, 64, 40, 40, 0, 1.0),
    (8, 1, 256, 300, 257, 13, 1.0 / 16.0),
    (4, 2, 128, 200, 130, 70, 0.125),
    (8, 1, 256, 64, 1, 0, 1.0 / 16.0),
])
def test_sdpa_vs_f64_brute_force(n_q, n_kv, hd, max_t, tlen, start, scale):
    k, v, kd, vd = _kv(max_t, n_kv, hd, 51)
    q = synth.normal_f32(n_q * hd, 53)
    want = rf.sdpa_f64(q, kd, vd, n_q, n_kv, hd, tlen, start, scale)
    got64 = oracle.sdpa(q, k, v, n_q, n_kv, hd, tlen, start, scale, f64=True)
    assert np.allclose(got64, want, rtol=1e-11, atol=1e-13)
    online = oracle.sdpa(q, k, v, n_q, n_kv, hd, tlen, start, scale)
    assert np.allclose(online, want, rtol=2e-5, atol=2e-6)
    # partition-count independence (nwg=1 is the online form bit for bit)
    assert np.array_equal(oracle.sdpa(q, k, v, n_q, n_kv, hd, tlen, start, scale, nwg=1), online)
    for nwg in (2, 16, 33):
        part = oracle.sdpa(q, k, v, n_q, n_kv, hd, tlen, start, scale, nwg=nwg)
        assert np.allclose(part, want, rtol=2e-5, atol=2e-6), nwg


def test_sdpa_needle():
    # check_mul_mm.rs:250-294: Q = 1, K[0] = 1, V[0] = 1, every other row 0.
    # q.k[0] = hd, q.k[t>0] = 0, so out = e^hd / (e^hd + tlen-1) per element
    # (Q4_0 reproduces 1.0 as 7 * half(1/7) up to half rounding).
    n_q, hd, tlen = 8, 256, 64
    kf = np.zeros((tlen, hd), dtype=np.float32)
    vf = np.zeros((tlen, hd), dtype=np.float32)
    kf[0] = 1.0
    vf[0] = 1.0
    k, v = oracle.pack_q40(kf), oracle.pack_q40(vf)
    one = oracle.dequant(oracle.Q40, k, hd)[0]
    assert abs(one - 1.0) < 1e-3
    out = oracle.sdpa_hybrid(np.ones(n_q * hd, dtype=np.float32), k, v, n_q, 1, hd, tlen)
    assert np.allclose(out, one, rtol=1e-6)      # weight of row 0 is 1 - 63*e^-256 = 1
    # with a small scale the needle no longer dominates: closed form
    s = np.float32(1.0 / 256.0)
    out = oracle.sdpa_hybrid(np.ones(n_q * hd, dtype=np.float32), k, v, n_q, 1, hd, tlen, scale=float(s))
    w0 = np.exp(np.float64(s) * hd * one) / (np.exp(np.float64(s) * hd * one) + tlen - 1)
    assert np.allclose(out, w0 * one, rtol=1e-5)


def test_softcap_argmax():
    assert oracle.softcap_argmax([1.0, 9.0, 3.0], 30.0) == 1      # sample.rs:92-96
    assert oracle.softcap_argmax([5.0, 7.0, 7.0, 2.0], 30.0) == 1   # ties: lowest index
    assert oracle.softcap_argmax([1000.0, 2000.0, -5.0], 30.0) == 0  # both saturate to cap
    assert oracle.softcap_argmax([1.0, 9.0, 3.0], 0.0) == 1
    x = synth.normal_f32(5000, 61)
    assert oracle.softcap_argmax(x, 30.0) == int(np.argmax(x))


def test_rmsnorm_family():
    n, eps = 512, 1e-6
    x, w, r = synth.normal_f32(n, 71), synth.normal_f32(n, 72), synth.normal_f32(n, 73)
    inv = 1.0 / np.sqrt((x.astype(np.float64) ** 2).mean() + eps)
    assert np.allclose(oracle.rmsnorm(x, w, eps), x * inv * w, rtol=2e-6, atol=1e-7)
    assert np.allclose(oracle.rmsnorm(x, w, eps, res=r), x * inv * w + r, rtol=2e-6, atol=1e-6)
    assert np.allclose(oracle.rmsnorm(x, w, eps, res=r, scale=0.5), 0.5 * (x * inv * w + r), rtol=2e-6, atol=1e-6)
    w2 = synth.normal_f32(n, 74)
    ox, ox2 = oracle.rmsnorm_add_then_rmsnorm(x, w, r, w2, eps)
    mid = r + x * inv * w
    inv2 = 1.0 / np.sqrt((mid ** 2).mean() + eps)
    assert np.allclose(ox, mid, rtol=2e-6, atol=1e-6)
    assert np.allclose(ox2, mid * inv2 * w2, rtol=4e-6, atol=1e-6)
    # eps is inside the square root: all-zero input stays finite and zero
    assert np.all(oracle.rmsnorm(np.zeros(n), w, eps) == 0.0)


def test_rope_table_and_per_head_qkv():
    hd, theta = 64, 10000.0
    tab = oracle.rope_table(8, hd, theta)
    assert np.all(tab[0, :hd // 2] == 1.0) and np.all(tab[0, hd // 2:] == 0.0)
    i = np.arange(hd // 2)
    freq = (1.0 / theta ** (2.0 * i / hd)).astype(np.float32)
    ang = (np.float32(5.0) * freq).astype(np.float32)
    assert np.allclose(tab[5, :hd // 2], np.cos(ang.astype(np.float64)), atol=1e-6)
    assert np.allclose(tab[5, hd // 2:], np.sin(ang.astype(np.float64)), atol=1e-6)
    # fewer angles than hd/2: identity tail
    tab2 = oracle.rope_table(4, hd, theta, rope_angles=8)
    assert np.all(tab2[3, 8:hd // 2] == 1.0) and np.all(tab2[3, hd // 2 + 8:] == 0.0)

    n_q, n_kv, eps = 4, 1, 1e-6
    q, k, v = synth.normal_f32(n_q * hd, 81), synth.normal_f32(n_kv * hd, 82), synth.normal_f32(n_kv * hd, 83)
    qw, kw = synth.normal_f32(hd, 84), synth.normal_f32(hd, 85)
    # pos 0 rotates by nothing: Q is the plain per-head RMS norm times weight
    qo, ko, vo = oracle.rmsnorm_per_head_qkv_q40(q, qw, tab[0], k, kw, v, n_q, n_kv, hd, eps)
    for h in range(n_q):
        seg = q[h * hd:(h + 1) * hd].astype(np.float64)
        assert np.allclose(qo[h * hd:(h + 1) * hd], seg / np.sqrt((seg ** 2).mean() + eps) * qw, rtol=3e-6, atol=1e-6)
    kn = k.astype(np.float64) / np.sqrt((k.astype(np.float64) ** 2).mean() + eps) * kw
    assert np.array_equal(ko, oracle.pack_q40(kn.astype(np.float32)))
    vn = v.astype(np.float64) / np.sqrt((v.astype(np.float64) ** 2).mean() + eps)
    kd = oracle.dequant(oracle.Q40, vo, hd)
    assert np.abs(kd - vn).max() <= np.abs(vn).max() / 7.0 * 0.51
    # a rotation preserves each (i, i+hd/2) pair's norm
    qo5, _, _ = oracle.rmsnorm_per_head_qkv_q40(q, qw, tab[5], k, kw, v, n_q, n_kv, hd, eps)
    a0 = qo[:hd // 2] ** 2 + qo[hd // 2:hd] ** 2
    a5 = qo5[:hd // 2] ** 2 + qo5[hd // 2:hd] ** 2
    assert np.allclose(a0, a5, rtol=1e-5, atol=1e-7)
    # and by the table's angle: out[i] = u cos - v sin
    u, vv = qo[:hd // 2].astype(np.float64), qo[hd // 2:hd].astype(np.float64)
    assert np.allclose(qo5[:hd // 2], u * tab[5, :hd // 2] - vv * tab[5, hd // 2:], rtol=1e-5, atol=1e-6)
    assert np.allclose(qo5[hd // 2:hd], u * tab[5, hd // 2:] + vv * tab[5, :hd // 2], rtol=1e-5, atol=1e-6)


def test_gelu_mul_and_embed():
    g = np.array([-30.0, -3.0, -0.5, 0.0, 0.5, 3.0, 30.0], dtype=np.float32)
    u = np.full_like(g, 2.0)
    ax = np.clip(g.astype(np.float64), -20, 20)
    want = 0.5 * ax * (1 + np.tanh(0.79788456 * (ax + 0.044715 * ax ** 3))) * 2.0
    assert np.allclose(oracle.gelu_mul(g, u), want, rtol=1e-6, atol=1e-7)
    E = synth.q6k_blocks(5 * 2, seed=91)          # 5 rows of 512
    row = oracle.copy_scale_indexed(oracle.Q6K, E, 3, 512, float(np.sqrt(np.float32(512))))
    want = np.sqrt(np.float32(512)) * oracle.dequant(oracle.Q6K, E, 5 * 512).reshape(5, 512)[3]
    assert np.array_equal(row, want.astype(np.float32))
