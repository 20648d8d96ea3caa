"""Independent numpy restatements of the OTHER formulations the reference
holds for the same block formats (its generated-GPU helper bodies in
crates/ksearch_codegen/src/render.rs) plus float64 closed forms.  The oracle
(which follows the CPU loop in crates/ksearch_gguf/src/gguf_impl.rs) must
agree with all of them; a dropped term, wrong nibble, wrong scale index or
transposed half fails at least one.
"""
import numpy as np

f32 = np.float32


def half_bits_to_f64(bits) -> np.ndarray:
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float64)


# ---- Q4_K ------------------------------------------------------------------

def scale_min_k4_bitfield(scales12: np.ndarray):
    """GGML block_q4_K scale layout read as a bit field: 8 six-bit scales and 8
    six-bit mins.  j<4: low 6 bits of byte j / j+4.  j>=4: low/high nibble of
    byte j+4 plus the top two bits of byte j-4 / j."""
    s = [int(b) for b in scales12]
    sc, mn = [], []
    for j in range(8):
        if j < 4:
            sc.append(s[j] % 64)
            mn.append(s[j + 4] % 64)
        else:
            sc.append((s[j + 4] % 16) + 16 * (s[j - 4] // 64))
            mn.append((s[j + 4] // 16) + 16 * (s[j] // 64))
    return sc, mn


def scale_min_k4_kmask(scales12: np.ndarray):
    """The 16-bit mask form the coop GEMV uses (render.rs:486-489), for both
    iq halves; returns the same (sc[8], mn[8])."""
    u16 = np.frombuffer(np.asarray(scales12, dtype=np.uint8).tobytes(), dtype="<u2").astype(np.uint32)
    sc, mn = [0] * 8, [0] * 8
    for iq in range(2):
        s = u16[iq:]
        sc16 = [s[0] & 0x3F3F, s[2] & 0x3F3F,
                ((s[4] >> 0) & 0x0F0F) | ((s[0] & 0xC0C0) >> 2),
                ((s[4] >> 4) & 0x0F0F) | ((s[2] & 0xC0C0) >> 2)]
        sc8 = np.array(sc16, dtype="<u2").view(np.uint8)
        # sc8[0],sc8[1]: scales of sub-blocks 2iq, 2iq+1; sc8[2],sc8[3]: their mins;
        # sc8[4],sc8[5]: scales of sub-blocks 4+2iq, 5+2iq; sc8[6],sc8[7]: their mins.
        sc[2 * iq], sc[2 * iq + 1] = int(sc8[0]), int(sc8[1])
        mn[2 * iq], mn[2 * iq + 1] = int(sc8[2]), int(sc8[3])
        sc[4 + 2 * iq], sc[5 + 2 * iq] = int(sc8[4]), int(sc8[5])
        mn[4 + 2 * iq], mn[5 + 2 * iq] = int(sc8[6]), int(sc8[7])
    return sc, mn


def q4k_closed_form(blocks: np.ndarray) -> np.ndarray:
    """value = d*sc*n - dmin*m evaluated in float64 (both products are exact
    there), rounded once to f32."""
    blocks = np.asarray(blocks, dtype=np.uint8).reshape(-1, 144)
    out = np.empty((blocks.shape[0], 256), dtype=np.float32)
    for b, blk in enumerate(blocks):
        d = half_bits_to_f64(blk[0:2].view("<u2"))[0]
        dmin = half_bits_to_f64(blk[2:4].view("<u2"))[0]
        sc, mn = scale_min_k4_bitfield(blk[4:16])
        qs = blk[16:]
        for j in range(256):
            sub = j // 32
            byte = qs[(j // 64) * 32 + (j % 32)]
            n = (byte >> 4) if (j % 64) >= 32 else (byte & 0xF)
            out[b, j] = np.float32(d * sc[sub] * float(n) - dmin * mn[sub])
    return out.reshape(-1)


def q4k_scalar_gpu(blocks: np.ndarray) -> np.ndarray:
    """ksearch_q4k_at (render.rs:12-26) in f32: d*float(sc)*float(q) - dmin*float(mn)."""
    blocks = np.asarray(blocks, dtype=np.uint8).reshape(-1, 144)
    out = np.empty((blocks.shape[0], 256), dtype=np.float32)
    for b, blk in enumerate(blocks):
        d = f32(blk[0:2].view("<u2").view(np.float16)[0])
        dmin = f32(blk[2:4].view("<u2").view(np.float16)[0])
        sc, mn = scale_min_k4_bitfield(blk[4:16])
        qs = blk[16:]
        for j in range(256):
            is_ = (j // 64) * 2
            qoff = (j // 64) * 32
            jl = j % 64
            if jl < 32:
                out[b, j] = d * f32(sc[is_]) * f32(qs[qoff + jl] & 0x0F) - dmin * f32(mn[is_])
            else:
                out[b, j] = d * f32(sc[is_ + 1]) * f32(qs[qoff + jl - 32] >> 4) - dmin * f32(mn[is_ + 1])
    return out.reshape(-1)


def q4k_mulmm16(blocks: np.ndarray) -> np.ndarray:
    """ksearch_q4k_dequant16 (render.rs:1075-1096) before its final half()
    cast: 16 chunks of 16; high nibbles use d/16 with mask 0xF0."""
    blocks = np.asarray(blocks, dtype=np.uint8).reshape(-1, 144)
    out = np.empty((blocks.shape[0], 256), dtype=np.float32)
    for b, blk in enumerate(blocks):
        dd = f32(blk[0:2].view("<u2").view(np.float16)[0])
        dm = f32(blk[2:4].view("<u2").view(np.float16)[0])
        sq = blk[4:16]
        for il_full in range(16):
            il = il_full
            q = 16 + (il // 4) * 32 + 16 * (il & 1)
            is_ = (il // 4) * 2
            il &= 3
            k = il // 2
            j = is_
            if j < 4:
                s0, s1 = sq[j + k] & 63, sq[j + 4 + k] & 63
            else:
                s0 = (sq[j + 4 + k] & 0xF) | ((sq[j - 4 + k] & 0xC0) >> 2)
                s1 = (sq[j + 4 + k] >> 4) | ((sq[j + k] & 0xC0) >> 2)
            d = dd if il < 2 else dd / f32(16.0)
            ml = dm * f32(s1)
            dl = d * f32(s0)
            mask = 0x0F if il < 2 else 0xF0
            for i in range(16):
                out[b, il_full * 16 + i] = dl * f32(int(blk[q + i]) & mask) - ml
    return out.reshape(-1)


def q4k_coop_dot(block: np.ndarray, x: np.ndarray) -> float:
    """One superblock of the coop GEMV (render.rs:459-517): eight lanes
    (it=0..7), masks 0x000F/0x0F00/0x00F0/0xF000 with 1/256 and 1/16 folded
    in, d*(...) - dmin*(...).  x: 256 f32.  Returns the f32 sum over lanes."""
    blk = np.asarray(block, dtype=np.uint8)
    x = np.asarray(x, dtype=np.float32)
    dd0 = f32(blk[0:2].view("<u2").view(np.float16)[0])
    dd1 = f32(blk[2:4].view("<u2").view(np.float16)[0])
    u16 = np.frombuffer(blk.tobytes(), dtype="<u2").astype(np.uint32)
    total = f32(0)
    for it in range(8):
        iq, ir = it // 4, it % 4
        y4 = 64 * iq + 8 * ir
        yl = np.zeros(16, dtype=np.float32)
        yh = np.zeros(16, dtype=np.float32)
        sumy = np.zeros(4, dtype=np.float32)
        for i in range(8):
            yl[i] = x[y4 + i];        sumy[0] += yl[i]
            yl[i + 8] = x[y4 + i + 32];   sumy[1] += yl[i + 8]
            yh[i] = x[y4 + i + 128];  sumy[2] += yh[i]
            yh[i + 8] = x[y4 + i + 160];  sumy[3] += yh[i + 8]
        sc = u16[2 + iq:]
        q1 = u16[8 + 16 * iq + 4 * ir:]
        q2 = q1[32:]
        sc16 = [sc[0] & 0x3F3F, sc[2] & 0x3F3F,
                ((sc[4] >> 0) & 0x0F0F) | ((sc[0] & 0xC0C0) >> 2),
                ((sc[4] >> 4) & 0x0F0F) | ((sc[2] & 0xC0C0) >> 2)]
        sc8 = np.array(sc16, dtype="<u2").view(np.uint8)
        a1 = np.zeros(4, dtype=np.float32)
        a2 = np.zeros(4, dtype=np.float32)
        for i in range(4):
            a1[0] += yl[2 * i + 0] * f32(q1[i] & 0x000F)
            a1[1] += yl[2 * i + 1] * f32(q1[i] & 0x0F00)
            a1[2] += yl[2 * i + 8] * f32(q1[i] & 0x00F0)
            a1[3] += yl[2 * i + 9] * f32(q1[i] & 0xF000)
            a2[0] += yh[2 * i + 0] * f32(q2[i] & 0x000F)
            a2[1] += yh[2 * i + 1] * f32(q2[i] & 0x0F00)
            a2[2] += yh[2 * i + 8] * f32(q2[i] & 0x00F0)
            a2[3] += yh[2 * i + 9] * f32(q2[i] & 0xF000)
        k256, k16 = f32(1.0 / 256.0), f32(1.0 / 16.0)
        total += dd0 * ((a1[0] + k256 * a1[1]) * f32(sc8[0]) +
                        (a1[2] + k256 * a1[3]) * f32(sc8[1]) * k16 +
                        (a2[0] + k256 * a2[1]) * f32(sc8[4]) +
                        (a2[2] + k256 * a2[3]) * f32(sc8[5]) * k16) - \
            dd1 * (sumy[0] * f32(sc8[2]) + sumy[1] * f32(sc8[3]) +
                   sumy[2] * f32(sc8[6]) + sumy[3] * f32(sc8[7]))
    return float(total)


# ---- Q6_K ------------------------------------------------------------------

def q6k_closed_form(blocks: np.ndarray) -> np.ndarray:
    """GGML block_q6_K read as a bit field, value = d*sc*(q-32) in float64."""
    blocks = np.asarray(blocks, dtype=np.uint8).reshape(-1, 210)
    out = np.empty((blocks.shape[0], 256), dtype=np.float32)
    for b, blk in enumerate(blocks):
        ql, qh = blk[:128], blk[128:192]
        sc = blk[192:208].view(np.int8)
        d = half_bits_to_f64(blk[208:210].view("<u2"))[0]
        for j in range(256):
            half, jl = j // 128, j % 128
            quad, l = jl // 32, jl % 32
            lo_byte = ql[64 * half + l + (32 if quad in (1, 3) else 0)]
            lo = (lo_byte >> 4) if quad >= 2 else (lo_byte & 0xF)
            hi = (qh[32 * half + l] >> (2 * quad)) & 3
            q = int(lo | (hi << 4)) - 32
            out[b, j] = np.float32(d * float(sc[8 * half + 2 * quad + l // 16]) * q)
    return out.reshape(-1)


def q6k_scalar_gpu(blocks: np.ndarray) -> np.ndarray:
    """ksearch_load_q6k (render.rs:729-756) in f32."""
    blocks = np.asarray(blocks, dtype=np.uint8).reshape(-1, 210)
    out = np.empty((blocks.shape[0], 256), dtype=np.float32)
    for b, blk in enumerate(blocks):
        d = f32(blk[208:210].view("<u2").view(np.float16)[0])
        for j in range(256):
            hpart, jl = j // 128, j % 128
            ql = blk[hpart * 64:]
            qh = blk[128 + hpart * 32:]
            sc = blk[192 + hpart * 8:].view(np.int8)
            l = jl % 32
            is_ = l // 16
            if jl < 32:
                q = int((ql[l] & 0x0F) | (((qh[l] >> 0) & 3) << 4)) - 32
                out[b, j] = d * f32(sc[is_]) * f32(q)
            elif jl < 64:
                q = int((ql[l + 32] & 0x0F) | (((qh[l] >> 2) & 3) << 4)) - 32
                out[b, j] = d * f32(sc[is_ + 2]) * f32(q)
            elif jl < 96:
                q = int((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32
                out[b, j] = d * f32(sc[is_ + 4]) * f32(q)
            else:
                q = int((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32
                out[b, j] = d * f32(sc[is_ + 6]) * f32(q)
    return out.reshape(-1)


def q6k_coop_dot(block: np.ndarray, x: np.ndarray) -> float:
    """One superblock of the Q6_K coop GEMV (render.rs:886-930): sixteen lanes
    (tid=0..15), kmask 0x03/0x0C/0x30/0xC0, d*(sum sums[k]*sc[2k])."""
    blk = np.asarray(block, dtype=np.uint8)
    x = np.asarray(x, dtype=np.float32)
    d = f32(blk[208:210].view("<u2").view(np.float16)[0])
    total = f32(0)
    for tid in range(16):
        ip, il = tid // 8, tid % 8
        l0 = 4 * il
        is_ = 8 * ip + l0 // 16
        y = x[128 * ip + l0:]
        q1 = blk[64 * ip + l0:]
        q2 = q1[32:]
        qh = blk[128 + 32 * ip + l0:]
        sc = blk[192 + is_:].view(np.int8)
        sums = np.zeros(4, dtype=np.float32)
        for l in range(4):
            sums[0] += y[l + 0] * f32(np.int8((q1[l] & 0x0F) | ((qh[l] & 0x03) << 4)) - 32)
            sums[1] += y[l + 32] * f32(np.int8((q2[l] & 0x0F) | ((qh[l] & 0x0C) << 2)) - 32)
            sums[2] += y[l + 64] * f32(np.int8((q1[l] >> 4) | ((qh[l] & 0x30) << 0)) - 32)
            sums[3] += y[l + 96] * f32(np.int8((q2[l] >> 4) | ((qh[l] & 0xC0) >> 2)) - 32)
        total += d * (sums[0] * f32(sc[0]) + sums[1] * f32(sc[2]) + sums[2] * f32(sc[4]) + sums[3] * f32(sc[6]))
    return float(total)


# ---- Q4_0 ------------------------------------------------------------------

def q40_closed_form(blocks: np.ndarray) -> np.ndarray:
    blocks = np.asarray(blocks, dtype=np.uint8).reshape(-1, 18)
    d = half_bits_to_f64(blocks[:, 0:2].copy().view("<u2").reshape(-1))
    qs = blocks[:, 2:].astype(np.int32)
    out = np.empty((blocks.shape[0], 32), dtype=np.float64)
    out[:, :16] = ((qs & 0xF) - 8) * d[:, None]
    out[:, 16:] = ((qs >> 4) - 8) * d[:, None]
    return out.astype(np.float32).reshape(-1)


def q40_scalar_gpu(blocks: np.ndarray) -> np.ndarray:
    """ksearch_q40_at (render.rs:999-1003)."""
    blocks = np.asarray(blocks, dtype=np.uint8).reshape(-1, 18)
    out = np.empty((blocks.shape[0], 32), dtype=np.float32)
    for b, blk in enumerate(blocks):
        d = f32(blk[0:2].view("<u2").view(np.float16)[0])
        for j in range(32):
            q = blk[2 + (j & 15)]
            qv = int(q & 0x0F) - 8 if j < 16 else int(q >> 4) - 8
            out[b, j] = f32(qv) * d
    return out.reshape(-1)


# ---- attention -------------------------------------------------------------

def sdpa_f64(q, kd, vd, n_q, n_kv, hd, tlen, start, scale):
    """softmax(scale * q K^T) V in float64 over dequantized K/V arrays of
    shape [max_t, n_kv, hd]."""
    q = np.asarray(q, dtype=np.float64).reshape(n_q, hd)
    out = np.empty((n_q, hd))
    g = n_q // n_kv
    for h in range(n_q):
        K = kd[start:start + tlen, h // g, :].astype(np.float64)
        V = vd[start:start + tlen, h // g, :].astype(np.float64)
        s = (K @ q[h]) * scale
        p = np.exp(s - s.max())
        out[h] = (p @ V) / p.sum()
    return out.reshape(-1)
