// Q4_0 packing of values held in registers, shared by the standalone
// quantize / per-head kernels and the fused decode attention.
#pragma once

#include "ksh_device.hpp"

namespace ksh {

// ksearch_pack_q40_th for one 32-value block held by 32 consecutive lanes of
// a wave (lane l of the group holds element l).  Values pass through a half
// round trip first; scale = max|v|/7 (1 if all zero); code = clamp(round(v/scale)+8).
// `group_base` is the first lane of the group.  Lanes 0..15 of the group store.
__device__ __forceinline__ void pack_q40_group(float v, int l, uint8_t *blk, bool store)
{
    v = half_bits_to_f32(f32_to_half_bits(v));
    float m = fabsf(v);
    // max over the 32 lanes of the group: row of 16 via DPP, then the neighbour row
    m = fmaxf(m, dpp_f32<0xB1>(m));
    m = fmaxf(m, dpp_f32<0x4E>(m));
    m = fmaxf(m, dpp_f32<0x141>(m));
    m = fmaxf(m, dpp_f32<0x140>(m));
    m = fmaxf(m, __shfl_xor(m, 16, 64));
    const float scale = m > 0.0f ? m / 7.0f : 1.0f;
    const float inv = 1.0f / scale;
    int q = (int)roundf(v * inv) + 8;
    q = min(15, max(0, q));
    const int qhi = __shfl_down(q, 16, 64);    // element l+16's code, for l < 16
    if (!store) return;
    if (l == 0) {
        const uint32_t h = f32_to_half_bits(scale);
        blk[0] = (uint8_t)(h & 0xFF);
        blk[1] = (uint8_t)(h >> 8);
    }
    if (l < 16) blk[2 + l] = (uint8_t)(q | (qhi << 4));
}

}  // namespace ksh
