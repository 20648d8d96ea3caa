"""Pins the CPU oracle's number formats and block dequantizers against
independent evidence: numpy's IEEE half, bit-field readings of the GGML
layouts, float64 closed forms, and the other formulations the reference
itself holds for the same blocks (tests/refforms.py)."""
import numpy as np
import pytest

import oracle
from ksearch_amd import synth
from tests import refforms as rf


def test_f16_to_f32_all_65536():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oracle.f16_to_f32(bits)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_matches_ieee_off_ties():
    rng = np.random.default_rng(1)
    v = np.concatenate([rng.standard_normal(20000) * 10.0 ** rng.integers(-6, 5, 20000),
                        [0.0, -0.0, 65504.0, 1e-8, 6.1e-5, 5.96e-8, 70000.0, -70000.0]]).astype(np.float32)
    want = v.astype(np.float16).view(np.uint16)
    # drop exact ties (13 dropped bits == 0x1000) and the band the reference flushes
    u = v.view(np.uint32)
    tie = (u & 0x1FFF) == 0x1000
    sub = np.abs(v) < 6.2e-5
    keep = ~tie & ~sub
    assert np.array_equal(oracle.f32_to_f16(v[keep]), want[keep])
    assert np.array_equal(oracle.f32_to_f16(v, rne=True), want)


def test_f32_to_f16_reference_tie_rule():
    # 1 + 2^-11 is exactly half way between 1.0 and 1 + 2^-10: the reference
    # adds 0x1000 and truncates (rounds up), IEEE ties-to-even rounds down.
    tie = np.float32(1.0 + 2.0 ** -11)
    assert oracle.f32_to_f16([tie])[0] == 0x3C01
    assert oracle.f32_to_f16([tie], rne=True)[0] == 0x3C00
    # odd neighbour: both round up
    tie2 = np.float32(1.0 + 3 * 2.0 ** -11)
    assert oracle.f32_to_f16([tie2])[0] == 0x3C02 == oracle.f32_to_f16([tie2], rne=True)[0]
    # mantissa carry into the exponent
    assert oracle.f32_to_f16([np.float32(2.0 - 2.0 ** -12)])[0] == 0x4000
    # [2^-25, 2^-24) is flushed to zero by the reference, rounded up by IEEE
    x = np.float32(1.5 * 2.0 ** -25)
    assert oracle.f32_to_f16([x])[0] == 0 and oracle.f32_to_f16([x], rne=True)[0] == 1
    # subnormal halves round half up as well
    assert oracle.f32_to_f16([np.float32(2.5 * 2.0 ** -24)])[0] == 3
    assert oracle.f32_to_f16([np.float32(2.5 * 2.0 ** -24)], rne=True)[0] == 2
    assert oracle.f32_to_f16([np.float32(np.inf)])[0] == 0x7C00
    assert oracle.f32_to_f16([np.float32(-1e6)])[0] == 0xFC00


def test_f32_to_f16_rne_exhaustive_halves_roundtrip():
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float32)
    ok = ~np.isnan(vals)
    assert np.array_equal(oracle.f32_to_f16(vals[ok], rne=True), bits[ok])
    assert np.array_equal(oracle.f32_to_f16(vals[ok]), bits[ok])


def test_bf16():
    L = oracle.lib()
    assert L.ko_bf16_to_f32(0x3F80) == 1.0
    assert L.ko_f32_to_bf16(1.0) == 0x3F80
    # add 0x8000 then shift: 1 + 2^-8 is a tie and goes up
    assert L.ko_f32_to_bf16(float(np.float32(1.0 + 2.0 ** -8))) == 0x3F81


def test_scale_min_k4_three_readings_agree():
    rng = np.random.default_rng(2)
    for _ in range(300):
        s12 = rng.integers(0, 256, 12, dtype=np.uint8)
        sc_b, mn_b = rf.scale_min_k4_bitfield(s12)
        sc_k, mn_k = rf.scale_min_k4_kmask(s12)
        got = [oracle.get_scale_min_k4(j, s12) for j in range(8)]
        assert [g[0] for g in got] == sc_b == sc_k
        assert [g[1] for g in got] == mn_b == mn_k


def test_scale_min_k4_inverts_reference_packer():
    # the packing half of quantize_f32_to_q4k (gguf_impl.rs:971-984)
    rng = np.random.default_rng(3)
    for _ in range(100):
        ls = rng.integers(0, 64, 8)
        lm = rng.integers(0, 64, 8)
        sc = np.zeros(12, dtype=np.uint8)
        for j in range(8):
            if j < 4:
                sc[j] = ls[j]
                sc[j + 4] = lm[j]
            else:
                sc[j + 4] = (ls[j] & 0xF) | ((lm[j] & 0xF) << 4)
                sc[j - 4] |= (ls[j] >> 4) << 6
                sc[j] |= (lm[j] >> 4) << 6
        for j in range(8):
            assert oracle.get_scale_min_k4(j, sc) == (ls[j], lm[j])


def test_q4k_dequant_four_formulations_bit_exact():
    blocks = synth.q4k_blocks(24, seed=11)
    got = oracle.dequant(oracle.Q4K, blocks, 24 * 256)
    for name, fn in (("closed", rf.q4k_closed_form), ("scalar", rf.q4k_scalar_gpu), ("mulmm16", rf.q4k_mulmm16)):
        want = fn(blocks)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), name


def test_q4k_coop_form_recovers_elements():
    # dotting the coop fragment with a unit vector recovers element j exactly
    blocks = synth.q4k_blocks(2, seed=12).reshape(2, 144)
    deq = oracle.dequant(oracle.Q4K, blocks, 512).reshape(2, 256)
    for b in range(2):
        for j in list(range(0, 256, 7)) + [31, 32, 63, 64, 255]:
            e = np.zeros(256, dtype=np.float32)
            e[j] = 1.0
            assert np.float32(rf.q4k_coop_dot(blocks[b], e)) == deq[b, j], (b, j)
    # and on a dense x it equals the dequant+dot up to reassociation
    x = synth.normal_f32(256, 13)
    ref = float(np.dot(deq[0].astype(np.float64), x.astype(np.float64)))
    assert abs(rf.q4k_coop_dot(blocks[0], x) - ref) <= 1e-5 * np.abs(deq[0] * x).sum()


def test_q4k_special_cases():
    blk = np.zeros(144, dtype=np.uint8)
    blk[0:2] = np.array([1.0], dtype=np.float16).view(np.uint8)   # d = 1
    blk[2:4] = np.array([0.5], dtype=np.float16).view(np.uint8)   # dmin = .5
    blk[4:8] = 1          # sc[0..3] = 1
    blk[8:12] = 3         # m[0..3] = 3
    blk[12:16] = 0x21     # j>=4: sc = 1, m = 2 (no high bits)
    out = oracle.dequant(oracle.Q4K, blk, 256)
    assert np.all(out[:128] == -1.5) and np.all(out[128:] == -1.0)   # qs=0 -> -dmin*m
    blk[2:4] = 0
    blk[16:] = np.arange(128, dtype=np.uint8)
    out = oracle.dequant(oracle.Q4K, blk, 256)                    # dmin=0, sc=1, d=1 -> the nibble
    qs = blk[16:]
    want = np.concatenate([np.concatenate([qs[32 * g:32 * g + 32] & 0xF, qs[32 * g:32 * g + 32] >> 4]) for g in range(4)])
    assert np.array_equal(out, want.astype(np.float32))
    # scales j>=4 take their two high bits from bytes 0..7
    blk[4] = 0xC0 | 1     # -> sc[4] high bits = 3
    blk[12] = 0x05        # low nibble 5
    assert oracle.get_scale_min_k4(4, blk[4:16])[0] == 5 + 48
    blk[8] = 0x80 | 3     # -> m[4] high bits = 2
    assert oracle.get_scale_min_k4(4, blk[4:16])[1] == 0 + 32


def test_q4k_reference_roundtrip_unit_test():
    # crates/ksearch_gguf/src/gguf_impl.rs:1022-1059 restated
    i = np.arange(1024, dtype=np.float32)
    elems = (np.sin(i * np.float32(0.017) + np.float32(0.3)) * np.float32(1.7)
             + np.cos(i * np.float32(0.041)) * np.float32(0.4) - np.float32(0.15)).astype(np.float32)
    elems[256:512] = 0.0
    elems[512:768] = -0.25
    q = oracle.quantize_q4k(elems)
    assert q.size == 1024 // 256 * 144
    back = oracle.dequant(oracle.Q4K, q, 1024)
    e = np.abs(elems - back)
    assert float((e.astype(np.float64) ** 2).mean()) < 0.01
    assert float(e.max()) < 0.35
    assert np.all(back[256:512] == 0.0)
    # constant block: reproduced to quantization accuracy
    assert np.abs(back[512:768] + 0.25).max() < 0.01


def test_q6k_dequant_three_formulations_bit_exact():
    blocks = synth.q6k_blocks(16, seed=21)
    got = oracle.dequant(oracle.Q6K, blocks, 16 * 256)
    for name, fn in (("closed", rf.q6k_closed_form), ("scalar", rf.q6k_scalar_gpu)):
        assert np.array_equal(got.view(np.uint32), fn(blocks).view(np.uint32)), name
    blocks = blocks.reshape(16, 210)
    deq = got.reshape(16, 256)
    for j in list(range(0, 256, 5)) + [15, 16, 31, 32, 127, 128, 255]:
        e = np.zeros(256, dtype=np.float32)
        e[j] = 1.0
        assert np.float32(rf.q6k_coop_dot(blocks[3], e)) == deq[3, j], j


def test_q6k_special_cases():
    blk = np.zeros(210, dtype=np.uint8)
    blk[208:210] = np.array([1.0], dtype=np.float16).view(np.uint8)
    blk[192:208] = 1
    out = oracle.dequant(oracle.Q6K, blk, 256)
    assert np.all(out == -32.0)                   # q bits 0 -> -32
    blk[:128] = 0xFF
    blk[128:192] = 0xFF
    assert np.all(oracle.dequant(oracle.Q6K, blk, 256) == 31.0)
    blk[192:208] = np.arange(-8, 8, dtype=np.int8).view(np.uint8)
    out = oracle.dequant(oracle.Q6K, blk, 256).reshape(16, 16)
    assert np.array_equal(out[:, 0], 31.0 * np.arange(-8, 8))   # one scale per 16 elements, in order


def test_q6k_quantizer_roundtrip():
    x = synth.normal_f32(4096, 22, std=0.02)
    q = oracle.quantize_q6k(x)
    back = oracle.dequant(oracle.Q6K, q, 4096)
    assert np.abs(back - x).max() < 0.02 * 4.5 / 32 * 1.1 + 1e-4
    assert np.all(oracle.dequant(oracle.Q6K, oracle.quantize_q6k(np.zeros(256)), 256) == 0.0)


def test_q40_dequant_and_pack():
    blocks = synth.q40_blocks(64, seed=31)
    got = oracle.dequant(oracle.Q40, blocks, 64 * 32)
    assert np.array_equal(got.view(np.uint32), rf.q40_closed_form(blocks).view(np.uint32))
    assert np.array_equal(got.view(np.uint32), rf.q40_scalar_gpu(blocks).view(np.uint32))
    v = synth.normal_f32(32 * 50, 32)
    v[64:96] = 0.0
    p = oracle.pack_q40(v)
    d = oracle.dequant(oracle.Q40, p, v.size).reshape(-1, 32)
    vv = v.astype(np.float16).astype(np.float32).reshape(-1, 32)
    scale = np.abs(vv).max(axis=1) / 7.0
    scale[scale == 0] = 1.0
    hs = p.reshape(-1, 18)[:, :2].copy().view(np.float16).astype(np.float32).reshape(-1)
    assert np.array_equal(hs, scale.astype(np.float32).astype(np.float16).astype(np.float32))
    # every element within half a step (+ the half rounding of the stored scale)
    assert np.all(np.abs(d - vv) <= (0.5 * scale + 7 * np.abs(hs - scale))[:, None] * 1.0001 + 1e-12)
    # the largest magnitude maps to +-7 (code 15 or 1); zeros block -> code 8, scale 1
    codes = np.concatenate([p.reshape(-1, 18)[:, 2:] & 0xF, p.reshape(-1, 18)[:, 2:] >> 4], axis=1).astype(int) - 8
    assert np.all(np.abs(codes).max(axis=1)[scale != 1.0] == 7)
    assert np.all(codes[2] == 0) and hs[2] == 1.0
    # round() is half away from zero: 2.5 steps -> 3
    blk = np.zeros(32, dtype=np.float32)
    blk[0], blk[1], blk[2] = 7.0, 2.5, -2.5
    c = oracle.pack_q40(blk)
    assert (c[2] & 0xF, c[3] & 0xF, c[4] & 0xF) == (15, 11, 5)


def test_row_bytes():
    assert oracle.row_bytes(oracle.Q4K, 4096) == 16 * 144
    assert oracle.row_bytes(oracle.Q6K, 2048) == 8 * 210
    assert oracle.row_bytes(oracle.Q40, 256) == 144
    assert oracle.row_bytes(oracle.Q4K, 100) == 0
