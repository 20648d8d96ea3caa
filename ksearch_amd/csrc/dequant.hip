// Packed block -> f32 dequantization on the device, bit-exact with the CPU
// loops of crates/ksearch_gguf/src/gguf_impl.rs:618-633 (Q4_0), :690-721
// (Q4_K), :722-760 (Q5_K) and :761-791 (Q6_K).  Built with -ffp-contract=off: the reference
// rounds `d1*q` and `- mn1` separately.
//
// One thread per 16-byte-aligned unit of packed input is not possible for
// Q6_K / Q4_0 (blocks are 2-byte aligned), so the mapping is by OUTPUT: a
// thread produces 4 consecutive f32 (one float4 store) and reads the few bytes
// it needs with byte loads; the packed input is tiny next to the f32 output it
// expands to (x7 for Q4_K), so the store stream is what bounds this kernel.
#include "ksh_device.hpp"
#include "ksh_internal.hpp"

namespace ksh {
namespace {

__device__ __forceinline__ uint32_t ld16(const uint8_t *p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8); }

// get_scale_min_k4, gguf_impl.rs:563-573
__device__ __forceinline__ void scale_min_k4(int j, const uint8_t *q, uint32_t &d, uint32_t &m)
{
    if (j < 4) {
        d = q[j] & 63u;
        m = q[j + 4] & 63u;
    } else {
        d = (q[j + 4] & 0x0Fu) | ((uint32_t)(q[j - 4] >> 6) << 4);
        m = (uint32_t)(q[j + 4] >> 4) | ((uint32_t)(q[j] >> 6) << 4);
    }
}

__global__ void dequant_q4k_kernel(const uint8_t *__restrict__ src, float *__restrict__ dst, size_t n4)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    const size_t e = i * 4, b = e >> 8;
    const int j = (int)(e & 255);
    const uint8_t *blk = src + b * 144;
    const float d = half_bits_to_f32(ld16(blk)), dmin = half_bits_to_f32(ld16(blk + 2));
    const int sub = j >> 5;                 // 32-wide sub-block
    uint32_t sc, mn;
    scale_min_k4(sub, blk + 4, sc, mn);
    const float d1 = d * (float)sc, mn1 = dmin * (float)mn;
    const uint8_t *qs = blk + 16 + (j >> 6) * 32 + (j & 31);
    const bool hi = (j & 32) != 0;
    float4 o;
    o.x = d1 * (float)(hi ? (qs[0] >> 4) : (qs[0] & 0x0F)) - mn1;
    o.y = d1 * (float)(hi ? (qs[1] >> 4) : (qs[1] & 0x0F)) - mn1;
    o.z = d1 * (float)(hi ? (qs[2] >> 4) : (qs[2] & 0x0F)) - mn1;
    o.w = d1 * (float)(hi ? (qs[3] >> 4) : (qs[3] & 0x0F)) - mn1;
    reinterpret_cast<float4 *>(dst)[i] = o;
}

// Q5_K: the Q4_K layout with a fifth bit per weight (qh[l] bit 2g for the low nibbles of group g, bit 2g+1 for
// the high ones): d1*(nibble + 16*bit) - mn1
__global__ void dequant_q5k_kernel(const uint8_t *__restrict__ src, float *__restrict__ dst, size_t n4)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    const size_t e = i * 4, b = e >> 8;
    const int j = (int)(e & 255);
    const uint8_t *blk = src + b * 176;
    const float d = half_bits_to_f32(ld16(blk)), dmin = half_bits_to_f32(ld16(blk + 2));
    const int sub = j >> 5;
    uint32_t sc, mn;
    scale_min_k4(sub, blk + 4, sc, mn);
    const float d1 = d * (float)sc, mn1 = dmin * (float)mn;
    const uint8_t *qh = blk + 16 + (j & 31);
    const uint8_t *qs = blk + 48 + (j >> 6) * 32 + (j & 31);
    const bool hi = (j & 32) != 0;
    float o[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const float nib = (float)(hi ? (qs[t] >> 4) : (qs[t] & 0x0F));
        const float bit = ((qh[t] >> sub) & 1) ? 16.0f : 0.0f;
        o[t] = d1 * (nib + bit) - mn1;
    }
    reinterpret_cast<float4 *>(dst)[i] = make_float4(o[0], o[1], o[2], o[3]);
}

__global__ void dequant_q6k_kernel(const uint8_t *__restrict__ src, float *__restrict__ dst, size_t n4)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    const size_t e = i * 4, b = e >> 8;
    const int j = (int)(e & 255);
    const uint8_t *blk = src + b * 210;
    const int half = j >> 7, jl = j & 127, quad = jl >> 5, l = jl & 31;
    const uint8_t *ql = blk + 64 * half + l + ((quad & 1) ? 32 : 0);
    const uint8_t *qh = blk + 128 + 32 * half + l;
    const int8_t sc = (int8_t)blk[192 + 8 * half + 2 * quad + (l >> 4)];
    const float d = half_bits_to_f32(ld16(blk + 208));
    const float ds = d * (float)sc;
    float o[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const uint32_t lo = quad >= 2 ? (uint32_t)(ql[t] >> 4) : (uint32_t)(ql[t] & 0x0F);
        const uint32_t hi2 = ((uint32_t)qh[t] >> (2 * quad)) & 3u;
        const int q = (int)(lo | (hi2 << 4)) - 32;
        o[t] = ds * (float)q;
    }
    reinterpret_cast<float4 *>(dst)[i] = make_float4(o[0], o[1], o[2], o[3]);
}

__global__ void dequant_q40_kernel(const uint8_t *__restrict__ src, float *__restrict__ dst, size_t n4)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    const size_t e = i * 4, b = e >> 5;
    const int j = (int)(e & 31);
    const uint8_t *blk = src + b * 18;
    const float d = half_bits_to_f32(ld16(blk));
    const uint8_t *qs = blk + 2 + (j & 15);
    const bool hi = j >= 16;
    float o[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const int q = (int)(hi ? (qs[t] >> 4) : (qs[t] & 0x0F)) - 8;
        o[t] = (float)q * d;
    }
    reinterpret_cast<float4 *>(dst)[i] = make_float4(o[0], o[1], o[2], o[3]);
}

int launch_dequant(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const size_t n4 = (size_t)k.desc.dims[0] / 4;
    const unsigned grid = (unsigned)((n4 + 255) / 256);
    const uint8_t *src = (const uint8_t *)a.in[0];
    float *dst = (float *)a.out[0];
    switch (k.desc.dtypes[0]) {
    case KSH_Q4K: hipLaunchKernelGGL(dequant_q4k_kernel, dim3(grid), dim3(256), 0, st, src, dst, n4); break;
    case KSH_Q5K: hipLaunchKernelGGL(dequant_q5k_kernel, dim3(grid), dim3(256), 0, st, src, dst, n4); break;
    case KSH_Q6K: hipLaunchKernelGGL(dequant_q6k_kernel, dim3(grid), dim3(256), 0, st, src, dst, n4); break;
    case KSH_Q40: hipLaunchKernelGGL(dequant_q40_kernel, dim3(grid), dim3(256), 0, st, src, dst, n4); break;
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "dequant launch");
}

// Q6_K -> Q6K_ROWS: one workgroup per weight row, one thread per output dword.  Row of bpr superblocks:
// ql [bpr][128] | qh [bpr][64] | sc [bpr][16] | d [bpr][2], then zero padding to a multiple of 16 bytes.
__global__ __launch_bounds__(256) void repack_q6k_rows_kernel(const uint8_t *src, uint8_t *dst, int bpr)
{
    const size_t row = blockIdx.x, rb = (size_t)bpr * 210, stride = (rb + 15) / 16 * 16;
    const uint16_t *s = reinterpret_cast<const uint16_t *>(src + row * rb);   // blocks are 2-byte aligned
    uint16_t *d = reinterpret_cast<uint16_t *>(dst + row * stride);
    for (int o = (int)(rb / 2) + threadIdx.x; o < (int)(stride / 2); o += 256) d[o] = 0;
    const int nql = bpr * 64, nqh = bpr * 32, nsc = bpr * 8;                   // in 16-bit units
    for (int o = threadIdx.x; o < (int)(rb / 2); o += 256) {
        int b, i;
        if (o < nql) { b = o / 64; i = o % 64; }
        else if (o < nql + nqh) { b = (o - nql) / 32; i = 64 + (o - nql) % 32; }
        else if (o < nql + nqh + nsc) { b = (o - nql - nqh) / 8; i = 96 + (o - nql - nqh) % 8; }
        else { b = o - nql - nqh - nsc; i = 104; }
        d[o] = s[b * 105 + i];
    }
}

int launch_repack_rows(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    hipLaunchKernelGGL(repack_q6k_rows_kernel, dim3((unsigned)k.desc.dims[0]), dim3(256), 0, st, (const uint8_t *)a.in[0],
                       (uint8_t *)a.out[0], (int)(k.desc.dims[1] / 256));
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "repack launch");
}

}  // namespace

int bind_repack_rows(ksh_kernel &k)
{
    const int64_t rows = k.desc.dims[0], cols = k.desc.dims[1];
    if (k.desc.dtypes[0] != KSH_Q6K || k.desc.dtypes[1] != KSH_Q6K_ROWS)
        return set_error("repack_rows: only Q6_K -> Q6K_ROWS is built (got %d -> %d)", k.desc.dtypes[0], k.desc.dtypes[1]);
    if (rows <= 0 || rows > 0x7FFFFFFF || cols <= 0 || cols % 256 || cols > (1 << 20))
        return set_error("repack_rows: rows=%lld cols=%lld (cols must be a positive multiple of 256)", (long long)rows, (long long)cols);
    k.info.n_inputs = 1;
    k.info.n_outputs = 1;
    k.in_bytes[0] = (size_t)rows * (cols / 256) * 210;
    k.out_bytes[0] = (size_t)rows * (((size_t)(cols / 256) * 210 + 15) / 16 * 16);   // rows padded to 16 bytes
    k.in_align[0] = 2;
    k.out_align[0] = 16;
    set_launch(k, (uint32_t)rows, 1, 1, 256, 0);
    set_name(k, "repack_q6k_rows");
    k.launch = launch_repack_rows;
    return 0;
}

int bind_dequant(ksh_kernel &k)
{
    const int dt = k.desc.dtypes[0];
    const int64_t n = k.desc.dims[0];
    if (dt != KSH_Q4K && dt != KSH_Q5K && dt != KSH_Q6K && dt != KSH_Q40) return set_error("dequant: dtype %d is not built", dt);
    const size_t pb = n > 0 ? packed_bytes(dt, (size_t)n) : 0;
    if (!pb || (uint64_t)n / 4 / 256 > 0x7FFFFFFFull) return set_error("dequant: n=%lld is not a valid element count", (long long)n);
    k.info.n_inputs = 1;
    k.info.n_outputs = 1;
    k.in_bytes[0] = pb;
    k.out_bytes[0] = (size_t)n * 4;
    k.in_align[0] = 2;
    k.out_align[0] = 16;
    set_launch(k, (uint32_t)(((size_t)n / 4 + 255) / 256), 1, 1, 256, 0);
    set_name(k, "dequant_%s", dt == KSH_Q4K ? "q4k" : dt == KSH_Q5K ? "q5k" : dt == KSH_Q6K ? "q6k" : "q40");
    k.launch = launch_dequant;
    return 0;
}

}  // namespace ksh
