// Small ops between the GEMVs of a decode step: the RMSNorm family, per-head
// RMS + RoPE + Q4_0 KV append, embedding row gather, GELU*up, slice copy,
// Q4_0 packing, soft-capped argmax and a fill kernel.
//
// They take the place of lower_rmsnorm / lower_rmsnorm_add_then_rmsnorm
// (crates/ksearch_codegen/src/lower.rs:4079-4162, 3926-4077),
// lower_rmsnorm_per_head_qkv_q40 (:4619-4702), CopyScaleIndexed (:3899-3921),
// gelu_mul (:4775-4838), copy_slice (:3831), lower_quantize_q40 (:4886-4895),
// lower_softcap_argmax (:6090-6156) and ksearch_pack_q40_th
// (crates/ksearch_codegen/src/render.rs:1040-1059).
//
// Built with -ffp-contract=off so that `u*cos - v*sin` and `(x*inv)*w + res`
// round exactly like the unfused expressions they restate; the Q4_0 codes that
// come out of the pack are integer functions of those values.
#include <atomic>

#include "ksh_device.hpp"
#include "q40_pack.hpp"
#include "ksh_internal.hpp"

namespace ksh {
namespace {

constexpr int kNormThreads = 256;

// block-wide sum for 256 threads (4 waves): DPP inside the wave, LDS across
__device__ __forceinline__ float block_sum_256(float v, float *red)
{
    const float w = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();   // `red` may still be read from a previous call
    if (lane == 0) red[wave] = w;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

__global__ void fill_zero_kernel(uint4 *p, size_t n16, uint8_t *tail, size_t ntail)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t j = i; j < n16; j += stride) p[j] = make_uint4(0, 0, 0, 0);
    if (i < ntail) tail[i] = 0;
}

// y = (x * rsqrt(mean(x^2) + eps)) * w  (+ residual)  (* scale)
__global__ __launch_bounds__(kNormThreads) void rmsnorm_kernel(const float *__restrict__ x,
                                                               const float *__restrict__ w,
                                                               const float *res, float *y, int n, float eps,
                                                               int has_res, int has_scale, float scale)
{
    __shared__ float red[4];
    // rows form (rmsnorm_rows / rmsnorm_add_rows / rmsnorm_add_scale_rows, crates/ksearch_kernels/src/lib.rs:1478-1560):
    // one workgroup per row of a [rows, n] matrix, the weight shared
    x += (size_t)blockIdx.x * n;
    y += (size_t)blockIdx.x * n;
    if (has_res) res += (size_t)blockIdx.x * n;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += kNormThreads) ss += x[i] * x[i];
    ss = block_sum_256(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += kNormThreads) {
        float v = x[i] * inv * w[i];
        if (has_res) v = v + res[i];
        if (has_scale) v = scale * v;
        y[i] = v;
    }
}

// out_x = res + (y*inv)*w_post;  out_x2 = (out_x*inv2)*w_ffn   (n <= 8192)
__global__ __launch_bounds__(kNormThreads) void rmsnorm_add_then_rmsnorm_kernel(
    const float *__restrict__ y, const float *__restrict__ w_post, const float *res,
    const float *__restrict__ w_ffn, float *out_x, float *out_x2, int n, float eps)
{
    __shared__ float red[4];
    extern __shared__ float mid[];
    // rows form (rmsnorm_add_then_rmsnorm_rows): one workgroup per row
    y += (size_t)blockIdx.x * n;
    res += (size_t)blockIdx.x * n;
    out_x += (size_t)blockIdx.x * n;
    out_x2 += (size_t)blockIdx.x * n;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += kNormThreads) ss += y[i] * y[i];
    ss = block_sum_256(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    float ss2 = 0.f;
    for (int i = threadIdx.x; i < n; i += kNormThreads) {
        const float v = res[i] + y[i] * inv * w_post[i];
        mid[i] = v;
        out_x[i] = v;
        ss2 += v * v;
    }
    ss2 = block_sum_256(ss2, red);
    const float inv2 = 1.0f / sqrtf(ss2 / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += kNormThreads) out_x2[i] = mid[i] * inv2 * w_ffn[i];
}

// QuantizeQ40: one 32-lane group per block of 32 source values
__global__ __launch_bounds__(256) void quantize_q40_kernel(const float *__restrict__ src, uint8_t *dst, int nblk)
{
    const int gidx = (blockIdx.x * 256 + threadIdx.x) >> 5, l = threadIdx.x & 31;
    const bool ok = gidx < nblk;
    const float v = ok ? src[(size_t)gidx * 32 + l] : 0.f;
    // every lane takes part in the cross-lane steps; only valid groups store
    pack_q40_group(v, l, dst + (size_t)(ok ? gidx : 0) * 18, ok);
}

// RmsNormPerHeadQkvQ40, n_tok = 1.  One wave per head; blocks 0..n_q-1 do Q
// (rms*w, RoPE, f32 out); blocks n_q..n_q+n_kv-1 do K (rms*w, RoPE, Q4_0) and
// V (rms without weight, Q4_0) of one kv head.  RoPE pairs (i, i+hd/2) with
// the row cos[0..hd/2) || sin[0..hd/2).  hd is 128, 256 or 512.
template <int HD>
__global__ __launch_bounds__(64) void per_head_qkv_q40_kernel(
    const float *q, const float *__restrict__ qw, const float *__restrict__ rope,
    const float *__restrict__ k, const float *__restrict__ kw, const float *__restrict__ v,
    float *q_out, uint8_t *k_out, uint8_t *v_out, int n_q, int n_kv, float eps, const float *meta,
    int max_seq, const float *slot_ids, size_t slot_stride)
{
    constexpr int HALF = HD / 2, PER = HD / 64;   // elements per lane
    const int lane = threadIdx.x;
    // batch form (rmsnorm_per_head_qkv_q40_batch, crates/ksearch_kernels/src/lib.rs:1750): blockIdx.y is the token
    // of a chunk of consecutive positions; its q / k / v rows, rope row and cache rows follow the first token's
    const int tok = blockIdx.y;
    q += (size_t)tok * n_q * HD;
    k += (size_t)tok * n_kv * HD;
    v += (size_t)tok * n_kv * HD;
    q_out += (size_t)tok * n_q * HD;
    if (slot_ids) {
        // tokens of different sequences (one decode step for several KV slots): token i has its own record
        // meta[4 i .. ] with its position in [3], and appends to slot slot_ids[i] of caches laid out
        // [slot][max_seq, n_kv, hd]
        const size_t pos = (size_t)min(max((int)meta[4 * tok + 3], 0), max_seq - 1);
        const size_t slot_bytes = slot_stride ? slot_stride : (size_t)max_seq * n_kv * (HD / 32) * 18;
        const size_t slot = (size_t)max((int)slot_ids[tok], 0);
        rope += pos * HD;
        k_out += slot * slot_bytes + pos * (size_t)n_kv * (HD / 32) * 18;
        v_out += slot * slot_bytes + pos * (size_t)n_kv * (HD / 32) * 18;
    } else if (meta) {
        // position kept on the device (meta[3]): the rope input is the whole
        // table and the K/V outputs are the cache bases, so that one captured
        // graph serves every token
        // clamped: a position at or past max_seq must never write outside the cache
        const size_t pos = (size_t)min(max((int)meta[3] + tok, 0), max_seq - 1);
        rope += pos * HD;
        k_out += pos * (size_t)n_kv * (HD / 32) * 18;
        v_out += pos * (size_t)n_kv * (HD / 32) * 18;
    } else {
        rope += (size_t)tok * HD;
        k_out += (size_t)tok * n_kv * (HD / 32) * 18;
        v_out += (size_t)tok * n_kv * (HD / 32) * 18;
    }
    const int head = blockIdx.x;
    const bool is_q = head < n_q;
    const int h = is_q ? head : head - n_q;
    const float *x = (is_q ? q : k) + (size_t)h * HD;
    const float *w = is_q ? qw : kw;

    // lane owns elements lane + 64*j: consecutive lanes hold consecutive
    // elements, so every 32-lane half of the wave holds one Q4_0 block per j
    float xv[PER];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        xv[j] = x[lane + 64 * j];
        ss += xv[j] * xv[j];
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)HD + eps);
    float nv[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) nv[j] = xv[j] * inv * w[lane + 64 * j];
    // RoPE: element e < HALF pairs with e + HALF, i.e. register j with j + PER/2
    float ro[PER];
#pragma unroll
    for (int j = 0; j < PER / 2; j++) {
        const int e = lane + 64 * j;
        const float c = rope[e], s = rope[HALF + e];
        const float u = nv[j], vv = nv[j + PER / 2];
        ro[j] = u * c - vv * s;
        ro[j + PER / 2] = u * s + vv * c;
    }
    if (is_q) {
#pragma unroll
        for (int j = 0; j < PER; j++) q_out[(size_t)h * HD + lane + 64 * j] = ro[j];
        return;
    }
    uint8_t *krow = k_out + (size_t)h * (HD / 32) * 18;
    uint8_t *vrow = v_out + (size_t)h * (HD / 32) * 18;
#pragma unroll
    for (int j = 0; j < PER; j++) pack_q40_group(ro[j], lane & 31, krow + (size_t)(2 * j + (lane >> 5)) * 18, true);

    const float *vx = v + (size_t)h * HD;
    float vs = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        xv[j] = vx[lane + 64 * j];
        vs += xv[j] * xv[j];
    }
    vs = wave_sum(vs);
    const float vinv = 1.0f / sqrtf(vs / (float)HD + eps);
#pragma unroll
    for (int j = 0; j < PER; j++)
        pack_q40_group(xv[j] * vinv, lane & 31, vrow + (size_t)(2 * j + (lane >> 5)) * 18, true);
}

// ---- embedding gather: out[i] = scale * deq(src[id*n + i]) -------------------
__device__ __forceinline__ float deq_q6k_at(const uint8_t *blk, int j)
{
    // ksearch_load_q6k, render.rs:729-756 / gguf_impl.rs:761-791: (d*sc)*q
    const int half = j >> 7, jl = j & 127, quad = jl >> 5, l = jl & 31;
    const uint8_t qlb = blk[64 * half + l + ((quad & 1) ? 32 : 0)];
    const uint32_t lo = quad >= 2 ? (uint32_t)(qlb >> 4) : (uint32_t)(qlb & 0x0F);
    const uint32_t hi = ((uint32_t)blk[128 + 32 * half + l] >> (2 * quad)) & 3u;
    const int q = (int)(lo | (hi << 4)) - 32;
    const float d = half_bits_to_f32((uint32_t)blk[208] | ((uint32_t)blk[209] << 8));
    const float sc = (float)(int8_t)blk[192 + 8 * half + 2 * quad + (l >> 4)];
    return d * sc * (float)q;
}

__device__ __forceinline__ float deq_q4k_at(const uint8_t *blk, int j)
{
    // ksearch_q4k_at, render.rs:12-26 / gguf_impl.rs:690-721
    const float d = half_bits_to_f32((uint32_t)blk[0] | ((uint32_t)blk[1] << 8));
    const float dmin = half_bits_to_f32((uint32_t)blk[2] | ((uint32_t)blk[3] << 8));
    const uint8_t *sq = blk + 4;
    const int sub = j >> 5;
    uint32_t sc, mn;
    if (sub < 4) {
        sc = sq[sub] & 63u;
        mn = sq[sub + 4] & 63u;
    } else {
        sc = (sq[sub + 4] & 0x0Fu) | ((uint32_t)(sq[sub - 4] >> 6) << 4);
        mn = (uint32_t)(sq[sub + 4] >> 4) | ((uint32_t)(sq[sub] >> 6) << 4);
    }
    const uint8_t qb = blk[16 + (j >> 6) * 32 + (j & 31)];
    const uint32_t n = (j & 32) ? (uint32_t)(qb >> 4) : (uint32_t)(qb & 0x0F);
    return d * (float)sc * (float)n - dmin * (float)mn;
}

__device__ __forceinline__ float deq_q5k_at(const uint8_t *blk, int j)
{
    // ksearch_load_q5k, render.rs:695-724 / gguf_impl.rs:722-760
    const float d = half_bits_to_f32((uint32_t)blk[0] | ((uint32_t)blk[1] << 8));
    const float dmin = half_bits_to_f32((uint32_t)blk[2] | ((uint32_t)blk[3] << 8));
    const uint8_t *sq = blk + 4;
    const int sub = j >> 5;
    uint32_t sc, mn;
    if (sub < 4) {
        sc = sq[sub] & 63u;
        mn = sq[sub + 4] & 63u;
    } else {
        sc = (sq[sub + 4] & 0x0Fu) | ((uint32_t)(sq[sub - 4] >> 6) << 4);
        mn = (uint32_t)(sq[sub + 4] >> 4) | ((uint32_t)(sq[sub] >> 6) << 4);
    }
    const uint8_t qb = blk[48 + (j >> 6) * 32 + (j & 31)];
    const float n = (float)((j & 32) ? (uint32_t)(qb >> 4) : (uint32_t)(qb & 0x0F));
    const float hi = ((blk[16 + (j & 31)] >> sub) & 1) ? 16.0f : 0.0f;
    return d * (float)sc * (n + hi) - dmin * (float)mn;
}

__global__ void copy_scale_indexed_kernel(const uint8_t *__restrict__ src, const float *__restrict__ idx,
                                          float *out, int n, float scale, int dtype, int64_t n_rows)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    // batch form (copy_scale_indexed_batch_wd): blockIdx.y is the token, its id at idx[token], its row of `out`
    out += (size_t)blockIdx.y * n;
    int64_t id = (int64_t)idx[blockIdx.y];
    id = id < 0 ? 0 : (id >= n_rows ? n_rows - 1 : id);    // never read outside the table
    float v;
    if (dtype == KSH_Q6K) {
        const uint8_t *row = src + (size_t)id * (size_t)(n / 256) * 210;
        v = deq_q6k_at(row + (size_t)(i >> 8) * 210, i & 255);
    } else if (dtype == KSH_Q4K) {
        const uint8_t *row = src + (size_t)id * (size_t)(n / 256) * 144;
        v = deq_q4k_at(row + (size_t)(i >> 8) * 144, i & 255);
    } else if (dtype == KSH_Q5K) {
        const uint8_t *row = src + (size_t)id * (size_t)(n / 256) * 176;
        v = deq_q5k_at(row + (size_t)(i >> 8) * 176, i & 255);
    } else if (dtype == KSH_F16) {
        v = half_bits_to_f32(reinterpret_cast<const uint16_t *>(src)[(size_t)id * n + i]);
    } else {
        v = reinterpret_cast<const float *>(src)[(size_t)id * n + i];
    }
    out[i] = scale * v;
}

// inner > 0 (gelu_mul_strided, gemma_prim.rs:1566-1576): g and out are [n / inner, inner], row r of u starts at
// r * stride (one layer's slice of every token's per-layer context)
__global__ void gelu_mul_kernel(const float *__restrict__ g, const float *__restrict__ u, float *out, int n, int inner, int stride)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    if (inner > 0) u += (size_t)(i / inner) * stride - (size_t)(i / inner) * inner;
    // lower.rs:4775-4838, same expression tree as the fused epilogue (:2926-2955)
    const float ax = fminf(20.0f, fmaxf(-20.0f, g[i]));
    const float t = 0.79788456f * (ax + 0.044715f * ((ax * ax) * ax));
    out[i] = (0.5f * ax) * (1.0f + tanhf(t)) * u[i];
}

__global__ void copy_slice_kernel(const float *__restrict__ src, float *dst, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

// argmax_i cap*tanh(x_i/cap); lowest index wins ties.  Pass 1: one partial
// (value, index) per workgroup; pass 2: one workgroup folds the partials.
constexpr int kArgThreads = 256;

__device__ __forceinline__ void argmax_fold(float &bv, uint32_t &bi, float v, uint32_t i)
{
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
}

__device__ __forceinline__ void argmax_block(float &bv, uint32_t &bi, float *sv, uint32_t *si)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const uint32_t oi = (uint32_t)__shfl_xor((int)bi, off, 64);
        argmax_fold(bv, bi, ov, oi);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0)
        for (int w = 1; w < kArgThreads / 64; w++) argmax_fold(bv, bi, sv[w], si[w]);
}

__global__ __launch_bounds__(kArgThreads) void softcap_argmax_part_kernel(const float *__restrict__ x, int n,
                                                                         float cap, float *pv, uint32_t *pi)
{
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    float bv = -INFINITY;
    uint32_t bi = 0xFFFFFFFFu;
    // several rows of n values (blockIdx.y): each with its own partial results, gridDim.x of them
    x += (size_t)blockIdx.y * n;
    pv += (size_t)blockIdx.y * gridDim.x;
    pi += (size_t)blockIdx.y * gridDim.x;
    for (int i = blockIdx.x * kArgThreads + threadIdx.x; i < n; i += gridDim.x * kArgThreads) {
        const float y = cap > 0.0f ? cap * tanhf(x[i] / cap) : x[i];
        argmax_fold(bv, bi, y, (uint32_t)i);
    }
    argmax_block(bv, bi, sv, si);
    if (threadIdx.x == 0) { pv[blockIdx.x] = bv; pi[blockIdx.x] = bi; }
}

__global__ __launch_bounds__(kArgThreads) void softcap_argmax_final_kernel(const float *pv, const uint32_t *pi,
                                                                          int nparts, float *out)
{
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    float bv = -INFINITY;
    uint32_t bi = 0xFFFFFFFFu;
    pv += (size_t)blockIdx.x * nparts;     // one workgroup per row
    pi += (size_t)blockIdx.x * nparts;
    for (int i = threadIdx.x; i < nparts; i += kArgThreads) argmax_fold(bv, bi, pv[i], pi[i]);
    argmax_block(bv, bi, sv, si);
    // the reference carries the index as f32 (exact below 2^24), lower.rs:6126
    if (threadIdx.x == 0) out[blockIdx.x] = (float)(bi == 0xFFFFFFFFu ? 0u : bi);
}

// The end of a decode step as one launch behind the argmax's first pass: fold the partial maxima (the token id), then
// what were two more launches and the next step's first -- remember the id, advance the position / attended length /
// current rope row (gemma_prim.rs:1236-1275), and gather the new token's embedding row into the residual stream
// (copy_scale_indexed, gemma_prim.rs:683), so that the next step starts with its first GEMV.
__global__ __launch_bounds__(kArgThreads) void decode_tail_kernel(DecodeTail t)
{
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    __shared__ uint32_t s_id;
    float bv = -INFINITY;
    uint32_t bi = 0xFFFFFFFFu;
    for (int i = threadIdx.x; i < t.nparts; i += kArgThreads) argmax_fold(bv, bi, t.pv[i], t.pi[i]);
    argmax_block(bv, bi, sv, si);
    const int pos = (int)t.meta[3];
    if (threadIdx.x == 0) {
        const uint32_t id = bi == 0xFFFFFFFFu ? 0u : bi;
        s_id = id;
        t.tok[0] = (float)id;   // the reference carries the index as f32 (exact below 2^24), lower.rs:6126
        if (t.history && pos < t.max_hist) t.history[pos] = (float)id;
    }
    __syncthreads();   // the id is known; every thread has read the position before thread 0 moves it
    if (pos + 1 < t.max_hist)
        for (int i = threadIdx.x; i < t.hd; i += kArgThreads) t.rope_cur[i] = t.rope[(size_t)(pos + 1) * t.hd + i];
    if (threadIdx.x == 0) {
        t.meta[3] = (float)(pos + 1);
        t.meta[0] = (float)(pos + 2);   // the next token attends rows [0, pos+1]
    }
    int64_t id = (int64_t)s_id;
    id = id >= t.n_rows ? t.n_rows - 1 : id;    // never read outside the table
    for (int i = threadIdx.x; i < t.n; i += kArgThreads) {
        float v;
        if (t.dtype == KSH_Q6K) v = deq_q6k_at(t.embd + (size_t)id * (size_t)(t.n / 256) * 210 + (size_t)(i >> 8) * 210, i & 255);
        else v = deq_q4k_at(t.embd + (size_t)id * (size_t)(t.n / 256) * 144 + (size_t)(i >> 8) * 144, i & 255);
        t.x_out[i] = t.scale * v;
    }
}

int done(const char *what)
{
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, what);
}

int launch_rmsnorm(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int n = (int)k.desc.dims[0], has_res = (int)k.desc.dims[1], has_scale = (int)k.desc.dims[2];
    hipLaunchKernelGGL(rmsnorm_kernel, dim3((unsigned)max((int64_t)1, k.desc.dims[3])), dim3(kNormThreads), 0, st, (const float *)a.in[0],
                       (const float *)a.in[1], has_res ? (const float *)a.in[2] : nullptr, (float *)a.out[0], n,
                       k.desc.params[0], has_res, has_scale, k.desc.params[1]);
    return done("rmsnorm launch");
}

int launch_rmsnorm_add_then(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int n = (int)k.desc.dims[0];
    hipLaunchKernelGGL(rmsnorm_add_then_rmsnorm_kernel, dim3((unsigned)max((int64_t)1, k.desc.dims[1])), dim3(kNormThreads), (size_t)n * 4, st,
                       (const float *)a.in[0], (const float *)a.in[1], (const float *)a.in[2],
                       (const float *)a.in[3], (float *)a.out[0], (float *)a.out[1], n, k.desc.params[0]);
    return done("rmsnorm_add_then_rmsnorm launch");
}

int launch_per_head(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int n_q = (int)k.desc.dims[0], n_kv = (int)k.desc.dims[1], hd = (int)k.desc.dims[2];
    const dim3 grid(n_q + n_kv, (unsigned)max((int64_t)1, k.desc.dims[4])), block(64);
#define KSH_PH(HD)                                                                                           \
    hipLaunchKernelGGL((per_head_qkv_q40_kernel<HD>), grid, block, 0, st, (const float *)a.in[0],            \
                       (const float *)a.in[1], (const float *)a.in[2], (const float *)a.in[3],               \
                       (const float *)a.in[4], (const float *)a.in[5], (float *)a.out[0], (uint8_t *)a.out[1], \
                       (uint8_t *)a.out[2], n_q, n_kv, k.desc.params[0],                                      \
                       k.desc.dims[3] ? (const float *)a.in[6] : nullptr, (int)k.desc.dims[3],                \
                       k.desc.dims[5] ? (const float *)a.in[7] : nullptr, (size_t)k.desc.dims[6])
    switch (hd) {
    case 128: KSH_PH(128); break;
    case 256: KSH_PH(256); break;
    case 512: KSH_PH(512); break;
    }
#undef KSH_PH
    return done("rmsnorm_per_head_qkv_q40 launch");
}

int launch_quantize_q40(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int nblk = (int)(k.desc.dims[0] / 32);
    hipLaunchKernelGGL(quantize_q40_kernel, dim3((nblk + 7) / 8), dim3(256), 0, st, (const float *)a.in[0],
                       (uint8_t *)a.out[0], nblk);
    return done("quantize_q40 launch");
}

int launch_copy_scale_indexed(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int n = (int)k.desc.dims[0];
    hipLaunchKernelGGL(copy_scale_indexed_kernel, dim3((n + 255) / 256, (unsigned)max((int64_t)1, k.desc.dims[2])), dim3(256), 0, st,
                       (const uint8_t *)a.in[0], (const float *)a.in[1], (float *)a.out[0], n, k.desc.params[0],
                       k.desc.dtypes[0], k.desc.dims[1]);
    return done("copy_scale_indexed launch");
}

int launch_gelu_mul(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int n = (int)k.desc.dims[0];
    hipLaunchKernelGGL(gelu_mul_kernel, dim3((n + 255) / 256), dim3(256), 0, st, (const float *)a.in[0],
                       (const float *)a.in[1], (float *)a.out[0], n, (int)k.desc.dims[1], (int)k.desc.dims[2]);
    return done("gelu_mul launch");
}

int launch_copy_slice(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int n = (int)k.desc.dims[0];
    hipLaunchKernelGGL(copy_slice_kernel, dim3((n + 255) / 256), dim3(256), 0, st, (const float *)a.in[0],
                       (float *)a.out[0], n);
    return done("copy_slice launch");
}

constexpr int kArgParts = 256;

int launch_softcap_argmax(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    // k.scratch holds kArgParts (value, index) pairs per row: all values, then all indices
    const int n = (int)k.desc.dims[0], rows = (int)max((int64_t)1, k.desc.dims[1]);
    const int parts = min(kArgParts, (n + kArgThreads - 1) / kArgThreads);
    float *pv = (float *)k.scratch;
    uint32_t *pi = (uint32_t *)(pv + (size_t)kArgParts * rows);
    hipLaunchKernelGGL(softcap_argmax_part_kernel, dim3(parts, rows), dim3(kArgThreads), 0, st, (const float *)a.in[0], n,
                       k.desc.params[0], pv, pi);
    hipLaunchKernelGGL(softcap_argmax_final_kernel, dim3(rows), dim3(kArgThreads), 0, st, pv, pi, parts,
                       (float *)a.out[0]);
    return done("softcap_argmax launch");
}

// ---- ksh_softcap_argmax_static: the same two kernels over a fixed array in the device image ----
// kArgParts (value, index) pairs.  In host code the array's name is only a handle for hipGetSymbolAddress; the
// kernels get the per-device address that call returns.
static __device__ __align__(256) unsigned char scratch[kArgParts * 8];
constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];   // per device: every GPU holds its own copy of the array (set once, by whichever thread comes first)

}  // namespace

// the soft-capped argmax's first pass over `logits` with the handle's partial-result buffer, then decode_tail_kernel
int launch_decode_tail(const ksh_kernel &k_argmax, const float *logits, DecodeTail t, hipStream_t st)
{
    const int n = (int)k_argmax.desc.dims[0];
    const int parts = min(kArgParts, (n + kArgThreads - 1) / kArgThreads);
    float *pv = (float *)k_argmax.scratch;
    uint32_t *pi = (uint32_t *)(pv + kArgParts);
    if (t.dtype != KSH_Q6K && t.dtype != KSH_Q4K) return set_error("decode tail: embedding dtype %d", t.dtype);
    hipLaunchKernelGGL(softcap_argmax_part_kernel, dim3(parts), dim3(kArgThreads), 0, st, logits, n, k_argmax.desc.params[0], pv, pi);
    t.pv = pv; t.pi = pi; t.nparts = parts;
    hipLaunchKernelGGL(decode_tail_kernel, dim3(1), dim3(kArgThreads), 0, st, t);
    return done("decode tail launch");
}

int argmax_static_setup()
{
    int dev = -1;
    KSH_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return set_error("softcap_argmax_static: device ordinal %d", dev);
    if (g_scratch_ptr[dev].load(std::memory_order_acquire)) return 0;
    void *p = nullptr;
    KSH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return set_error("softcap_argmax_static: the partial-result array has no device address");
    g_scratch_ptr[dev].store(p, std::memory_order_release);   // (two threads racing here store the same address)
    return 0;
}

}  // namespace ksh

extern "C" int ksh_softcap_argmax_static(ksh_ctx *ctx, ksh_buf *x, uint64_t x_off, int64_t n, float cap, ksh_buf *out,
                                         uint64_t out_off)
{
    using namespace ksh;
    if (!ctx || !x || !out) return set_error("ksh_softcap_argmax_static: bad arguments");
    if (n < 1 || n > KSH_ARGMAX_STATIC_MAX_N)
        return set_error("ksh_softcap_argmax_static: n=%lld is outside [1, %d] (the f32 index is exact below 2^24 only)",
                         (long long)n, KSH_ARGMAX_STATIC_MAX_N);
    if (x_off % 4 || x_off > x->bytes || (uint64_t)n * 4 > x->bytes - x_off)
        return set_error("ksh_softcap_argmax_static: x needs %lld bytes from 4-byte-aligned offset %llu, buffer has %zu",
                         (long long)n * 4, (unsigned long long)x_off, x->bytes);
    if (out_off % 4 || out_off > out->bytes || 4 > out->bytes - out_off)
        return set_error("ksh_softcap_argmax_static: out needs 4 bytes from 4-byte-aligned offset %llu, buffer has %zu",
                         (unsigned long long)out_off, out->bytes);
    // the array of the device the context's stream runs on, whatever device the calling thread has current
    const int dev = ctx_device(ctx);
    if (dev < 0 || dev >= kMaxDevices) return set_error("ksh_softcap_argmax_static: device ordinal %d", dev);
    float *pv = (float *)g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!pv) return set_error("ksh_softcap_argmax_static: the context's device %d has no resolved array (ksh_ctx_create resolves it)", dev);
    uint32_t *pi = (uint32_t *)(pv + kArgParts);
    const int parts = (int)min((int64_t)kArgParts, (n + kArgThreads - 1) / kArgThreads);
    hipStream_t st = ctx_stream(ctx);
    hipLaunchKernelGGL(softcap_argmax_part_kernel, dim3(parts), dim3(kArgThreads), 0, st,
                       (const float *)((const char *)x->ptr + x_off), (int)n, cap, pv, pi);
    hipLaunchKernelGGL(softcap_argmax_final_kernel, dim3(1), dim3(kArgThreads), 0, st, pv, pi, parts,
                       (float *)((char *)out->ptr + out_off));
    if (done("softcap_argmax_static launch")) return 1;
    ctx_mark_pending(ctx);
    return 0;
}

namespace ksh {

int bind_rmsnorm(ksh_kernel &k)
{
    const int64_t n = k.desc.dims[0];
    if (n <= 0 || n > (1 << 24)) return set_error("rmsnorm: n=%lld", (long long)n);
    if (k.desc.kind == KSH_RMSNORM) {
        const bool has_res = k.desc.dims[1] != 0;
        const int64_t rows = k.desc.dims[3] ? k.desc.dims[3] : 1;
        if (rows < 0 || rows > 65535) return set_error("rmsnorm: rows=%lld", (long long)rows);
        k.info.n_inputs = has_res ? 3 : 2;
        k.info.n_outputs = 1;
        for (int i = 0; i < k.info.n_inputs; i++) { k.in_bytes[i] = (size_t)n * 4 * (i == 1 ? 1 : rows); k.in_align[i] = 4; }
        k.out_bytes[0] = (size_t)n * 4 * rows;
        k.out_align[0] = 4;
        set_launch(k, (uint32_t)rows, 1, 1, kNormThreads, 16);
        set_name(k, "rmsnorm%s%s%s", has_res ? "_add" : "", k.desc.dims[2] ? "_scale" : "", rows > 1 ? "_rows" : "");
        k.launch = launch_rmsnorm;
        return 0;
    }
    // the reference stages the residual stream in threadgroup memory and
    // refuses sizes that do not fit (lower.rs:3934-3938)
    if (n > 8192) return set_error("rmsnorm_add_then_rmsnorm requires LOCAL staging of residual stream (n=%lld > 8192)", (long long)n);
    const int64_t rows = k.desc.dims[1] ? k.desc.dims[1] : 1;
    if (rows < 0 || rows > 65535) return set_error("rmsnorm_add_then_rmsnorm: rows=%lld", (long long)rows);
    k.info.n_inputs = 4;
    k.info.n_outputs = 2;
    for (int i = 0; i < 4; i++) { k.in_bytes[i] = (size_t)n * 4 * ((i & 1) ? 1 : rows); k.in_align[i] = 4; }   // y, w_post, res, w_ffn
    for (int i = 0; i < 2; i++) { k.out_bytes[i] = (size_t)n * 4 * rows; k.out_align[i] = 4; }
    set_launch(k, (uint32_t)rows, 1, 1, kNormThreads, (uint32_t)n * 4 + 16);
    set_name(k, "rmsnorm_add_then_rmsnorm%s", rows > 1 ? "_rows" : "");
    k.launch = launch_rmsnorm_add_then;
    return 0;
}

int bind_per_head_qkv_q40(ksh_kernel &k)
{
    const int64_t n_q = k.desc.dims[0], n_kv = k.desc.dims[1], hd = k.desc.dims[2];
    if (n_q <= 0 || n_kv <= 0 || n_q > 4096 || n_kv > n_q) return set_error("rmsnorm_per_head_qkv_q40: n_q=%lld n_kv=%lld", (long long)n_q, (long long)n_kv);
    if (hd != 128 && hd != 256 && hd != 512)
        return set_error("rmsnorm_per_head_qkv_q40: hd=%lld is not built (128, 256, 512 are)", (long long)hd);
    // dims[3] = max_seq when the position comes from a device-side meta buffer
    // (7th input, f32[4] with the position in [3]); 0 for the host-offset form
    const int64_t max_seq = k.desc.dims[3];
    if (max_seq < 0 || max_seq > (1 << 24)) return set_error("rmsnorm_per_head_qkv_q40: max_seq=%lld", (long long)max_seq);
    // dims[4] = tokens of a chunk of consecutive positions (0 or 1: a single token)
    const int64_t n_tok = k.desc.dims[4] ? k.desc.dims[4] : 1;
    if (n_tok < 0 || n_tok > 65535) return set_error("rmsnorm_per_head_qkv_q40: n_tok=%lld", (long long)n_tok);
    const size_t rows = max_seq ? (size_t)max_seq : (size_t)n_tok;
    // dims[5] = KV slots when the tokens belong to different sequences: meta is then f32[n_tok][4] (token i's position
    // in [4 i + 3]), an 8th input f32[n_tok] names each token's slot, and the outputs are caches of dims[5] slots
    const int64_t n_slots = k.desc.dims[5];
    if (n_slots < 0 || n_slots > 4096 || (n_slots && !max_seq)) return set_error("rmsnorm_per_head_qkv_q40: slots=%lld", (long long)n_slots);
    k.info.n_inputs = n_slots ? 8 : max_seq ? 7 : 6;
    k.info.n_outputs = 3;
    // dims[6] = bytes from one slot of the caches to the next (0: max_seq rows)
    const size_t one = (size_t)n_kv * (hd / 32) * 18 * rows;
    const int64_t slot_stride = k.desc.dims[6];
    if (slot_stride < 0 || (slot_stride && (!n_slots || (size_t)slot_stride < one || slot_stride % 2)))
        return set_error("rmsnorm_per_head_qkv_q40: slot stride %lld", (long long)slot_stride);
    const size_t kvb = n_slots ? (size_t)(n_slots - 1) * (slot_stride ? (size_t)slot_stride : one) + one : one;
    const size_t ib[8] = {(size_t)n_q * hd * 4 * n_tok, (size_t)hd * 4, (size_t)hd * 4 * rows, (size_t)n_kv * hd * 4 * n_tok, (size_t)hd * 4,
                          (size_t)n_kv * hd * 4 * n_tok, n_slots ? (size_t)16 * n_tok : 16, (size_t)4 * n_tok};
    for (int i = 0; i < k.info.n_inputs; i++) { k.in_bytes[i] = ib[i]; k.in_align[i] = 4; }
    k.out_bytes[0] = (size_t)n_q * hd * 4 * n_tok; k.out_align[0] = 4;
    k.out_bytes[1] = k.out_bytes[2] = kvb; k.out_align[1] = k.out_align[2] = 2;
    set_launch(k, (uint32_t)(n_q + n_kv), (uint32_t)n_tok, 1, 64, 0);
    set_name(k, "rmsnorm_per_head_qkv_q40_hd%d%s", (int)hd, n_slots ? "_slots" : n_tok > 1 ? "_batch" : "");
    k.launch = launch_per_head;
    return 0;
}

int bind_quantize_q40(ksh_kernel &k)
{
    const int64_t n = k.desc.dims[0];
    if (n <= 0 || n % 32 || n > (1ll << 31) - 64) return set_error("quantize_q40: n=%lld is not a positive multiple of 32", (long long)n);
    k.info.n_inputs = 1;
    k.info.n_outputs = 1;
    k.in_bytes[0] = (size_t)n * 4; k.in_align[0] = 4;
    k.out_bytes[0] = (size_t)n / 32 * 18; k.out_align[0] = 2;
    set_launch(k, (uint32_t)((n / 32 + 7) / 8), 1, 1, 256, 0);
    set_name(k, "quantize_q40");
    k.launch = launch_quantize_q40;
    return 0;
}

int bind_glue(ksh_kernel &k)
{
    const int64_t n = k.desc.dims[0];
    if (n <= 0 || n > (1ll << 30)) return set_error("kernel kind %d: n=%lld", k.desc.kind, (long long)n);
    set_launch(k, (uint32_t)((n + 255) / 256), 1, 1, 256, 0);
    switch (k.desc.kind) {
    case KSH_COPY_SCALE_INDEXED: {
        const int dt = k.desc.dtypes[0];
        const int64_t n_rows = k.desc.dims[1];
        if (dt != KSH_Q6K && dt != KSH_Q5K && dt != KSH_Q4K && dt != KSH_F16 && dt != KSH_F32)
            return set_error("copy_scale_indexed: source dtype %d is not built", dt);
        if (n_rows <= 0) return set_error("copy_scale_indexed: dims[1] (rows in the table) must be positive");
        const size_t rb = dt == KSH_F32 ? (size_t)n * 4 : packed_bytes(dt, (size_t)n);
        if (!rb) return set_error("copy_scale_indexed: n=%lld is not a whole number of blocks", (long long)n);
        k.info.n_inputs = 2;
        k.info.n_outputs = 1;
        k.in_bytes[0] = rb * (size_t)n_rows; k.in_align[0] = dt == KSH_F32 ? 4 : 2;
        // dims[2] = tokens (0 or 1: a single id)
        const int64_t n_tok = k.desc.dims[2] ? k.desc.dims[2] : 1;
        if (n_tok < 0 || n_tok > 65535) return set_error("copy_scale_indexed: n_tok=%lld", (long long)n_tok);
        k.in_bytes[1] = 4 * (size_t)n_tok; k.in_align[1] = 4;
        k.out_bytes[0] = (size_t)n * 4 * n_tok; k.out_align[0] = 4;
        k.info.grid[1] = (uint32_t)n_tok;
        set_name(k, "copy_scale_indexed_%d%s", dt, n_tok > 1 ? "_batch" : "");
        k.launch = launch_copy_scale_indexed;
        return 0;
    }
    case KSH_GELU_MUL: {
        // dims[1] = inner, dims[2] = stride: the second operand's rows of `inner` values are `stride` floats apart
        const int64_t inner = k.desc.dims[1], stride = k.desc.dims[2];
        if (inner < 0 || stride < 0 || (inner && (n % inner || stride < inner))) return set_error("gelu_mul: inner=%lld stride=%lld", (long long)inner, (long long)stride);
        k.info.n_inputs = 2;
        k.info.n_outputs = 1;
        k.in_bytes[0] = k.in_bytes[1] = k.out_bytes[0] = (size_t)n * 4;
        if (inner) k.in_bytes[1] = ((size_t)(n / inner - 1) * stride + inner) * 4;
        k.in_align[0] = k.in_align[1] = k.out_align[0] = 4;
        set_name(k, "gelu_mul%s", inner ? "_strided" : "");
        k.launch = launch_gelu_mul;
        return 0;
    }
    case KSH_COPY_SLICE:
        k.info.n_inputs = 1;
        k.info.n_outputs = 1;
        k.in_bytes[0] = k.out_bytes[0] = (size_t)n * 4;
        k.in_align[0] = k.out_align[0] = 4;
        set_name(k, "copy_slice");
        k.launch = launch_copy_slice;
        return 0;
    }
    return set_error("bind_glue: kind %d", k.desc.kind);
}

int bind_softcap_argmax(ksh_kernel &k)
{
    const int64_t n = k.desc.dims[0], rows = std::max<int64_t>(1, k.desc.dims[1]);
    if (n <= 0 || n >= (1 << 24)) return set_error("softcap_argmax: n=%lld (the f32 index is exact below 2^24 only)", (long long)n);
    if (k.desc.dims[1] < 0 || rows > 4096) return set_error("softcap_argmax: %lld rows (up to 4096)", (long long)k.desc.dims[1]);
    k.info.n_inputs = 1;
    k.info.n_outputs = 1;
    k.in_bytes[0] = (size_t)rows * n * 4; k.in_align[0] = 4;
    k.out_bytes[0] = (size_t)rows * 4; k.out_align[0] = 4;
    k.scratch_bytes = (size_t)kArgParts * 8 * rows;
    set_launch(k, (uint32_t)min((int64_t)kArgParts, (n + kArgThreads - 1) / kArgThreads), 1, 1, kArgThreads, 32);
    set_name(k, "softcap_argmax");
    k.launch = launch_softcap_argmax;
    return 0;
}

}  // namespace ksh

extern "C" int ksh_fill_zero_launch(void *ptr, size_t bytes, hipStream_t st)
{
    using namespace ksh;
    const size_t n16 = bytes / 16, tail = bytes % 16;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (uint4 *)ptr, n16,
                       (uint8_t *)ptr + n16 * 16, tail);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "fill_zero launch");
}
