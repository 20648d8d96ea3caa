// f32 -> Q4_K / Q6_K packers as device kernels: what a loader needs to turn
// float weights into the packed layouts the GEMVs stream.
//
// Q4_K follows quantize_f32_to_q4k / make_qkx2_quants
// (crates/ksearch_gguf/src/gguf_impl.rs:803-1016) operation for operation, one
// thread per 32-element sub-block and eight neighbouring lanes per superblock,
// so that the bytes equal the host routine's; built with -ffp-contract=off for
// that reason.  Q6_K has no
// counterpart in the reference (it carries no Q6_K quantizer): per 16-element
// group the largest-magnitude value maps to -32, and the 16 group scales are
// stored as int8 multiples of one f16 super-scale.
#include "ksh_device.hpp"
#include "ksh_internal.hpp"

namespace ksh {
namespace {

__device__ __forceinline__ int nearest_int(float fval)
{
    // magic-float rounding, gguf_impl.rs:803-808
    const float val = fval + 12582912.0f;
    return (int)(as_u32(val) & 0x007fffffu) - 0x00400000;
}

__device__ __forceinline__ int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// f32 -> half bits with the host routine's rule: add 0x1000 and truncate
// (crates/ksearch_gguf/src/lib.rs:39-75), which differs from RNE on exact ties
__device__ uint32_t f32_to_f16_ref(float value)
{
    const uint32_t bits = as_u32(value);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    int e = (int)((bits >> 23) & 0xFF);
    uint32_t mant = bits & 0x7FFFFFu;
    if (e == 255) return mant == 0 ? (sign | 0x7C00u) : (sign | 0x7C00u | (mant >> 13));
    e -= 127;
    if (e > 15) return sign | 0x7C00u;
    if (e < -14) {
        if (e < -24) return sign;
        mant |= 0x800000u;
        const uint32_t shift = (uint32_t)(-14 - e) + 13;
        return sign | ((mant + (1u << (shift - 1))) >> shift);
    }
    const uint32_t half_exp = (uint32_t)(e + 15);
    const uint32_t half_mant = mant + 0x1000u;
    if (half_mant & 0x800000u) return sign | ((half_exp + 1) << 10);
    return sign | (half_exp << 10) | (half_mant >> 13);
}

// gguf_impl.rs:811-901 with nmax=15, rmin=-1, rdelta=0.1, nstep=20, squared error.  One thread runs one 32-element
// sub-block with every array in registers (the loops over the elements are unrolled; the sums run in the host
// routine's order, element after element, so every rounding is the host's).  L: the 32 codes, one per byte.
__device__ __forceinline__ float make_qkx2_quants(const float (&x)[32], const float (&weights)[32], uint32_t (&L)[8], float *the_min)
{
    constexpr int n = 32, nmax = 15, nstep = 20;
    const float rmin = -1.0f, rdelta = 0.1f;
    float mn = x[0], mx = x[0], sum_w = weights[0], sum_x = sum_w * x[0];
#pragma unroll
    for (int i = 1; i < n; i++) {
        if (x[i] < mn) mn = x[i];
        if (x[i] > mx) mx = x[i];
        const float w = weights[i];
        sum_w += w;
        sum_x += w * x[i];
    }
    if (mn > 0.0f) mn = 0.0f;
    if (mx == mn) {
#pragma unroll
        for (int i = 0; i < 8; i++) L[i] = 0;
        *the_min = -mn;
        return 0.0f;
    }
    float iscale = (float)nmax / (mx - mn);
    float scale = 1.0f / iscale;
    float best_error = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) L[i] = 0;
#pragma unroll
    for (int i = 0; i < n; i++) {
        const int l = clampi(nearest_int(iscale * (x[i] - mn)), 0, nmax);
        L[i >> 2] |= (uint32_t)l << (8 * (i & 3));
        float diff = scale * (float)l + mn - x[i];
        diff = diff * diff;
        best_error += weights[i] * diff;
    }
    // (as in the host loop, a candidate's grid is laid out from the minimum as the previous accepted candidate left it)
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * (float)is + (float)nmax) / (mx - mn);
        float sum_l = 0.0f, sum_l2 = 0.0f, sum_xl = 0.0f;
        uint32_t Laux[8];
#pragma unroll
        for (int i = 0; i < 8; i++) Laux[i] = 0;
#pragma unroll
        for (int i = 0; i < n; i++) {
            const int l = clampi(nearest_int(iscale * (x[i] - mn)), 0, nmax);
            Laux[i >> 2] |= (uint32_t)l << (8 * (i & 3));
            const float w = weights[i], lf = (float)l;
            sum_l += w * lf;
            sum_l2 += w * lf * lf;
            sum_xl += w * lf * x[i];
        }
        const float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0.0f) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0.0f) {
                this_min = 0.0f;
                this_scale = sum_xl / sum_l2;
            }
            float cur_error = 0.0f;
#pragma unroll
            for (int i = 0; i < n; i++) {
                float diff = this_scale * (float)((Laux[i >> 2] >> (8 * (i & 3))) & 0xFFu) + this_min - x[i];
                diff = diff * diff;
                cur_error += weights[i] * diff;
            }
            if (cur_error < best_error) {
#pragma unroll
                for (int i = 0; i < 8; i++) L[i] = Laux[i];
                best_error = cur_error;
                scale = this_scale;
                mn = this_min;
            }
        }
    }
    *the_min = -mn;
    return scale;
}

// value of lane `j` of the caller's group of 8 consecutive lanes
__device__ __forceinline__ float oct_get(float v, int j) { return __shfl(v, j, 8); }
__device__ __forceinline__ uint32_t oct_get(uint32_t v, int j) { return (uint32_t)__shfl((int)v, j, 8); }

// quantize_f32_to_q4k, gguf_impl.rs:903-1016: eight consecutive lanes share a superblock, lane j runs sub-block j
// (the search over its scale, then its final codes); what the host routine combines across the sub-blocks -- the
// largest scale and minimum, the 12 packed scale bytes, the nibble pairs of two neighbouring sub-blocks -- crosses
// the lanes with shuffles.  Maxima are order-free, so the bytes are the host's.
__global__ __launch_bounds__(64) void quantize_q4k_kernel(const float *__restrict__ src, uint8_t *dst, size_t nb)
{
    const size_t t = (size_t)blockIdx.x * 64 + threadIdx.x;
    const int j = (int)(threadIdx.x & 7);
    // (whole groups of 8 lanes are in or out: nb counts superblocks; lanes past the end redo the last superblock and store nothing)
    const size_t b_real = t >> 3, b = b_real < nb ? b_real : nb - 1;
    const float *xp = src + b * 256 + 32 * j;
    float x[32], weights[32];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float4 v = ldg_f4(xp, i);
        x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
    }
    float sum_x2 = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) sum_x2 += x[i] * x[i];
    const float av_x = sqrtf(sum_x2 / 32.0f);
#pragma unroll
    for (int i = 0; i < 32; i++) weights[i] = av_x + fabsf(x[i]);
    uint32_t L[8];
    float mymin;
    const float myscale = make_qkx2_quants(x, weights, L, &mymin);
    float max_scale = 0.0f, max_min = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const float sk = oct_get(myscale, k), mk = oct_get(mymin, k);
        if (sk > max_scale) max_scale = sk;
        if (mk > max_min) max_min = mk;
    }
    const float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    const float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    const uint32_t db = f32_to_f16_ref(max_scale / 63.0f), mb = f32_to_f16_ref(max_min / 63.0f);
    uint32_t ls = (uint32_t)(uint8_t)nearest_int(inv_scale * myscale), lm = (uint32_t)(uint8_t)nearest_int(inv_min * mymin);
    if (ls > 63) ls = 63;
    if (lm > 63) lm = 63;
    // the sub-block's final codes against the scale and minimum as they will be unpacked (get_scale_min_k4 returns ls, lm)
    const float d = half_bits_to_f32(db), dmin = half_bits_to_f32(mb);
    const float dj = d * (float)ls;
    if (dj != 0.0f) {
        const float dm = dmin * (float)lm;
#pragma unroll
        for (int i = 0; i < 8; i++) L[i] = 0;
#pragma unroll
        for (int i = 0; i < 32; i++) L[i >> 2] |= (uint32_t)clampi(nearest_int((x[i] + dm) / dj), 0, 15) << (8 * (i & 3));
    }
    // quant bytes: sub-block 2g in the low nibbles, 2g+1 in the high ones; the even lane stores bytes 0..15 of the
    // pair's 32, the odd lane bytes 16..31
    uint32_t q[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t mine = (j & 1) ? L[i] << 4 : L[i];
        q[i] = mine | (uint32_t)__shfl_xor((int)mine, 1, 8);
    }
    uint8_t *blk = dst + b * 144;
    if (b_real < nb) {
        const int h = j & 1;
        *reinterpret_cast<uint4 *>(blk + 16 + 32 * (j >> 1) + 16 * h) = make_uint4(q[4 * h], q[4 * h + 1], q[4 * h + 2], q[4 * h + 3]);
    }
    // header: d, dmin and the 12 scale bytes, by lane 0 (every lane takes part in the shuffles)
    uint32_t lsv[8], lmv[8];
#pragma unroll
    for (int k = 0; k < 8; k++) { lsv[k] = oct_get(ls, k); lmv[k] = oct_get(lm, k); }
    if (j == 0 && b_real < nb) {
        uint32_t sc[12];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            sc[k] = lsv[k] | ((lsv[k + 4] >> 4) << 6);
            sc[k + 4] = lmv[k] | ((lmv[k + 4] >> 4) << 6);
            sc[k + 8] = (lsv[k + 4] & 0x0F) | ((lmv[k + 4] & 0x0F) << 4);
        }
        uint4 hdr;
        hdr.x = db | (mb << 16);
        hdr.y = sc[0] | (sc[1] << 8) | (sc[2] << 16) | (sc[3] << 24);
        hdr.z = sc[4] | (sc[5] << 8) | (sc[6] << 16) | (sc[7] << 24);
        hdr.w = sc[8] | (sc[9] << 8) | (sc[10] << 16) | (sc[11] << 24);
        *reinterpret_cast<uint4 *>(blk) = hdr;
    }
}

__global__ __launch_bounds__(64) void quantize_q6k_kernel(const float *__restrict__ src, uint8_t *dst, size_t nb)
{
    const size_t b = (size_t)blockIdx.x * 64 + threadIdx.x;
    if (b >= nb) return;
    const float *x = src + b * 256;
    uint8_t *blk = dst + b * 210;
    float gs[16], max_abs_scale = 0.0f, max_scale = 0.0f;
    for (int g = 0; g < 16; g++) {
        float amax = 0.0f, mx = 0.0f;
        for (int i = 0; i < 16; i++) {
            const float a = fabsf(x[16 * g + i]);
            if (a > amax) { amax = a; mx = x[16 * g + i]; }
        }
        gs[g] = amax > 0.0f ? mx / -32.0f : 0.0f;
        if (fabsf(gs[g]) > max_abs_scale) { max_abs_scale = fabsf(gs[g]); max_scale = gs[g]; }
    }
    if (max_abs_scale == 0.0f) {
        for (int i = 0; i < 210; i++) blk[i] = 0;
        return;
    }
    const float iscale = -128.0f / max_scale;
    const uint32_t db = f32_to_half_bits(1.0f / iscale);
    const float d = half_bits_to_f32(db);
    uint8_t L[256];
    for (int g = 0; g < 16; g++) {
        const int s = clampi(nearest_int(iscale * gs[g]), -128, 127);
        blk[192 + g] = (uint8_t)(int8_t)s;
        const float dg = d * (float)s;
        for (int i = 0; i < 16; i++) {
            const int l = dg != 0.0f ? clampi(nearest_int(x[16 * g + i] / dg), -32, 31) : 0;
            L[16 * g + i] = (uint8_t)(l + 32);
        }
    }
    for (int half = 0; half < 2; half++) {
        const uint8_t *Lh = L + 128 * half;
        for (int l = 0; l < 32; l++) {
            const uint8_t q1 = Lh[l], q2 = Lh[l + 32], q3 = Lh[l + 64], q4 = Lh[l + 96];
            blk[64 * half + l] = (uint8_t)((q1 & 0x0F) | ((q3 & 0x0F) << 4));
            blk[64 * half + l + 32] = (uint8_t)((q2 & 0x0F) | ((q4 & 0x0F) << 4));
            blk[128 + 32 * half + l] = (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
        }
    }
    blk[208] = (uint8_t)(db & 0xFF);
    blk[209] = (uint8_t)(db >> 8);
}

int launch_quantize_k(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const size_t nb = (size_t)k.desc.dims[0] / 256;
    const unsigned grid = (unsigned)((nb + 63) / 64);
    if (k.desc.dtypes[0] == KSH_Q4K)   // eight lanes per superblock
        hipLaunchKernelGGL(quantize_q4k_kernel, dim3((unsigned)((nb + 7) / 8)), dim3(64), 0, st, (const float *)a.in[0], (uint8_t *)a.out[0], nb);
    else
        hipLaunchKernelGGL(quantize_q6k_kernel, dim3(grid), dim3(64), 0, st, (const float *)a.in[0], (uint8_t *)a.out[0], nb);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "quantize_k launch");
}

}  // namespace

int bind_quantize_k(ksh_kernel &k)
{
    const int dt = k.desc.dtypes[0];
    const int64_t n = k.desc.dims[0];
    if (dt != KSH_Q4K && dt != KSH_Q6K) return set_error("quantize_k: dtype %d is not built (Q4_K and Q6_K are)", dt);
    if (n <= 0 || n % 256) return set_error("quantize_k: n=%lld is not a positive multiple of 256", (long long)n);
    k.info.n_inputs = 1;
    k.info.n_outputs = 1;
    k.in_bytes[0] = (size_t)n * 4; k.in_align[0] = 4;
    k.out_bytes[0] = packed_bytes(dt, (size_t)n); k.out_align[0] = dt == KSH_Q4K ? 16 : 2;
    set_launch(k, (uint32_t)(dt == KSH_Q4K ? ((size_t)n / 256 + 7) / 8 : ((size_t)n / 256 + 63) / 64), 1, 1, 64, 0);
    set_name(k, "quantize_%s", dt == KSH_Q4K ? "q4k" : "q6k");
    k.launch = launch_quantize_k;
    return 0;
}

}  // namespace ksh
