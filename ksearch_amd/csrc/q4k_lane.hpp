// What one lane of the Q4_K GEMV kernels does with one (row, superblock, 64-element group): the three 16-byte loads,
// the group's activations as registers (padded f32, or three int8 digit planes), and the f32 contribution to y[row].
// Shared by the kernels of the GEMV family (matvec_q4k.hip).
//
// Arithmetic per (row, superblock, group), all f32:
//   acc += d*sc_lo * sum(n_lo*x) + d*sc_hi * sum(n_hi*x) - dmin*(m_lo*Sx_lo + m_hi*Sx_hi)
// which is the reference's coop form (crates/ksearch_codegen/src/render.rs:506-511).
#pragma once
#include "gemv_prologue.hpp"

namespace ksh {
namespace {

constexpr int kQ4kBytes = 144;

struct Q4kLane {
    uint4 hdr;   // d | dmin<<16, then the 12 scale bytes
    uint4 qa;    // quant bytes 0..15 of the lane's group
    uint4 qb;    // quant bytes 16..31
};

__device__ __forceinline__ Q4kLane q4k_load(const uint8_t *blk, int g)
{
    Q4kLane r;
    r.hdr = ldg_u4(blk, 0);
    r.qa = ldg_u4(blk, 1 + 2 * g);
    r.qb = ldg_u4(blk, 2 + 2 * g);
    return r;
}

// The activations of one lane's 64-element group, as registers, in the format
// its inner product wants.
template <int XF>
struct XGroup;

template <>
struct XGroup<kXF32> {
    float xr[64], sx_lo, sx_hi;
    __device__ __forceinline__ void load(const uint8_t *lds, int cols, int b, int g)
    {
        (void)cols;
        const float *xg = reinterpret_cast<const float *>(lds) + xs_f32_index(b * 256 + g * 64);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float4 v = *reinterpret_cast<const float4 *>(xg + 4 * i);
            xr[4 * i] = v.x; xr[4 * i + 1] = v.y; xr[4 * i + 2] = v.z; xr[4 * i + 3] = v.w;
        }
        float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
#pragma unroll
        for (int i = 0; i < 32; i += 2) { a0 += xr[i]; a1 += xr[i + 1]; b0 += xr[32 + i]; b1 += xr[33 + i]; }
        sx_lo = a0 + a1;
        sx_hi = b0 + b1;
    }
    // sum(n_lo*x) and 16*sum(n_hi*x): the high nibbles stay in place, the 1/16 is folded into the scale
    __device__ __forceinline__ void dot(const Q4kLane &L, float &lo, float &hi) const
    {
        float lo0 = 0.f, lo1 = 0.f, hi0 = 0.f, hi1 = 0.f;
        const uint32_t q[8] = {L.qa.x, L.qa.y, L.qa.z, L.qa.w, L.qb.x, L.qb.y, L.qb.z, L.qb.w};
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const uint32_t t = q[k] & 0x0F0F0F0Fu, u = q[k] & 0xF0F0F0F0u;
            const float *xl = xr + 4 * k, *xh = xr + 32 + 4 * k;
            float &a = (k & 1) ? lo1 : lo0, &c = (k & 1) ? hi1 : hi0;
            a = fmaf(ubyte_f32<0>(t), xl[0], a); c = fmaf(ubyte_f32<0>(u), xh[0], c);
            a = fmaf(ubyte_f32<1>(t), xl[1], a); c = fmaf(ubyte_f32<1>(u), xh[1], c);
            a = fmaf(ubyte_f32<2>(t), xl[2], a); c = fmaf(ubyte_f32<2>(u), xh[2], c);
            a = fmaf(ubyte_f32<3>(t), xl[3], a); c = fmaf(ubyte_f32<3>(u), xh[3], c);
        }
        lo = lo0 + lo1;
        hi = (hi0 + hi1) * 0.0625f;
    }
};

template <>
struct XGroup<kXI8> {
    uint32_t H[16], M[16], Lo[16];   // digit planes: dwords 0..7 low sub-block, 8..15 high sub-block
    float s_lo, s_hi, sx_lo, sx_hi;
    __device__ __forceinline__ void load(const uint8_t *lds, int cols, int b, int g)
    {
        const int c = b * 4 + g;
        const uint4 *p = reinterpret_cast<const uint4 *>(lds + c * 208);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint4 h = p[i], m = p[4 + i], l = p[8 + i];
            H[4 * i] = h.x; H[4 * i + 1] = h.y; H[4 * i + 2] = h.z; H[4 * i + 3] = h.w;
            M[4 * i] = m.x; M[4 * i + 1] = m.y; M[4 * i + 2] = m.z; M[4 * i + 3] = m.w;
            Lo[4 * i] = l.x; Lo[4 * i + 1] = l.y; Lo[4 * i + 2] = l.z; Lo[4 * i + 3] = l.w;
        }
        const float4 sc = *reinterpret_cast<const float4 *>(lds + (cols >> 6) * 208 + c * 16);
        s_lo = sc.x; sx_lo = sc.y; s_hi = sc.z; sx_hi = sc.w;
    }
    __device__ __forceinline__ void dot(const Q4kLane &L, float &lo, float &hi) const
    {
        int hl = 0, ml = 0, ll = 0, hh = 0, mh = 0, lh = 0;
        const uint32_t q[8] = {L.qa.x, L.qa.y, L.qa.z, L.qa.w, L.qb.x, L.qb.y, L.qb.z, L.qb.w};
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int a = (int)(q[k] & 0x0F0F0F0Fu), c = (int)((q[k] >> 4) & 0x0F0F0F0Fu);
            hl = __builtin_amdgcn_sdot4(a, (int)H[k], hl, false);
            ml = __builtin_amdgcn_sdot4(a, (int)M[k], ml, false);
            ll = __builtin_amdgcn_sdot4(a, (int)Lo[k], ll, false);
            hh = __builtin_amdgcn_sdot4(c, (int)H[8 + k], hh, false);
            mh = __builtin_amdgcn_sdot4(c, (int)M[8 + k], mh, false);
            lh = __builtin_amdgcn_sdot4(c, (int)Lo[8 + k], lh, false);
        }
        lo = s_lo * (float)((hl << 14) + (ml << 7) + ll);
        hi = s_hi * (float)((hh << 14) + (mh << 7) + lh);
    }
};

template <>
struct XGroup<kXI2> {
    uint32_t M[16], Lo[16];   // two digit planes (signed high bytes, unsigned low bytes): dwords 0..7 low sub-block, 8..15 high sub-block
    float s_lo, s_hi, sx_lo, sx_hi;
    __device__ __forceinline__ void load(const uint8_t *lds, int cols, int b, int g)
    {
        const int c = b * 4 + g;
        const uint4 *p = reinterpret_cast<const uint4 *>(lds + c * 144);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint4 m = p[i], l = p[4 + i];
            M[4 * i] = m.x; M[4 * i + 1] = m.y; M[4 * i + 2] = m.z; M[4 * i + 3] = m.w;
            Lo[4 * i] = l.x; Lo[4 * i + 1] = l.y; Lo[4 * i + 2] = l.z; Lo[4 * i + 3] = l.w;
        }
        const float4 sc = *reinterpret_cast<const float4 *>(lds + (cols >> 6) * 144 + c * 16);
        s_lo = sc.x; sx_lo = sc.y; s_hi = sc.z; sx_hi = sc.w;
    }
    __device__ __forceinline__ void dot(const Q4kLane &L, float &lo, float &hi) const
    {
        int ml = 0, ll = 0, mh = 0, lh = 0;
        const uint32_t q[8] = {L.qa.x, L.qa.y, L.qa.z, L.qa.w, L.qb.x, L.qb.y, L.qb.z, L.qb.w};
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int a = (int)(q[k] & 0x0F0F0F0Fu), c = (int)((q[k] >> 4) & 0x0F0F0F0Fu);
            ml = __builtin_amdgcn_sdot4(a, (int)M[k], ml, false);
            ll = (int)__builtin_amdgcn_udot4((uint32_t)a, Lo[k], (uint32_t)ll, false);
            mh = __builtin_amdgcn_sdot4(c, (int)M[8 + k], mh, false);
            lh = (int)__builtin_amdgcn_udot4((uint32_t)c, Lo[8 + k], (uint32_t)lh, false);
        }
        // |256 ml + ll| <= 32 * 15 * 32767 < 2^24: the conversion is exact
        lo = s_lo * (float)((ml << 8) + ll);
        hi = s_hi * (float)((mh << 8) + lh);
    }
};

// one (row, superblock, group): the f32 contribution to y[row]
template <int XF>
__device__ __forceinline__ float q4k_group_dot(const Q4kLane &L, int g, const XGroup<XF> &X)
{
    float lo, hi;
    X.dot(L, lo, hi);
    const float d = half_bits_to_f32(L.hdr.x & 0xFFFFu), dmin = half_bits_to_f32(L.hdr.x >> 16);
    const uint4 s = q4k_group_scales(L.hdr.y, L.hdr.z, L.hdr.w, g);
    const float pos = fmaf((float)s.x, lo, (float)s.z * hi);
    const float neg = fmaf((float)s.y, X.sx_lo, (float)s.w * X.sx_hi);
    return fmaf(d, pos, -(dmin * neg));
}

__device__ __forceinline__ float gelu_mul_f32(float g, float u)
{
    // lower.rs:2926-2955: clamp, tanh-GELU on the f32 accumulator, times up
    const float ax = fminf(20.0f, fmaxf(-20.0f, g));
    const float t = 0.79788456f * (ax + 0.044715f * ((ax * ax) * ax));
    return (0.5f * ax) * (1.0f + tanhf(t)) * u;
}

}  // namespace
}  // namespace ksh
