// The ops that the real Gemma-4 checkpoints add to a decode step on top of the
// synthetic shape's: per-head RMSNorm with and without RoPE (query heads of the
// layers that reuse another layer's KV cache; the per-layer-embedding prepass),
// y = scale*(a+b), and the per-layer-embedding gate GEMV with its gelu(.)*ctx
// epilogue.
//
// They take the place of lower_rmsnorm_per_head / lower_rmsnorm_per_head_rope_at
// (crates/ksearch_codegen/src/lower.rs:4164-4228, 4356-4435), Eng::add_scale
// (crates/ksearch_kernels/src/lib.rs:918-937) and KernelKind::MatvecGeluMul
// (lower.rs:622-643).
//
// Built with -ffp-contract=off: `u*cos - v*sin` and `(x*inv)*w` round like the
// unfused expressions they restate.
#include "ksh_device.hpp"
#include "ksh_internal.hpp"

namespace ksh {
namespace {

int done(const char *what)
{
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, what);
}

// One wave per head; lane owns elements lane + 64*j.  rope == nullptr: norm
// only.  meta != nullptr: `rope` is the whole table and the row is the
// position kept on the device (meta[3]), clamped to the table.
template <int HD>
__global__ __launch_bounds__(64) void per_head_kernel(const float *x, const float *__restrict__ w,
                                                      const float *__restrict__ rope, const float *__restrict__ meta,
                                                      float *y, float eps, int max_seq, int heads_per_token, int per_token_meta)
{
    constexpr int HALF = HD / 2, PER = HD / 64;
    const int lane = threadIdx.x;
    const size_t base = (size_t)blockIdx.x * HD;
    // heads_per_token > 0 (rmsnorm_per_head_rope_batch, gemma_prim.rs:1411-1424): the heads of a chunk of consecutive
    // positions, token after token; token i takes the rope row of (first position + i)
    const int tok = heads_per_token > 0 ? blockIdx.x / heads_per_token : 0;
    // per_token_meta: the tokens belong to different sequences, token i's position is meta[4 i + 3]
    if (meta) rope += (size_t)min(max(per_token_meta ? (int)meta[4 * tok + 3] : (int)meta[3] + tok, 0), max_seq - 1) * HD;
    float xv[PER], nv[PER];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        xv[j] = x[base + lane + 64 * j];
        ss += xv[j] * xv[j];
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)HD + eps);
#pragma unroll
    for (int j = 0; j < PER; j++) nv[j] = xv[j] * inv * w[lane + 64 * j];
    if (!rope) {
#pragma unroll
        for (int j = 0; j < PER; j++) y[base + lane + 64 * j] = nv[j];
        return;
    }
    if (PER >= 2) {
        // element e < HALF pairs with e + HALF: register j with j + PER/2
#pragma unroll
        for (int j = 0; j < PER / 2; j++) {
            const int e = lane + 64 * j;
            const float c = rope[e], s = rope[HALF + e];
            const float u = nv[j], vv = nv[j + PER / 2];
            y[base + e] = u * c - vv * s;
            y[base + HALF + e] = u * s + vv * c;
        }
    } else {
        // 64 elements: the partner of lane e < 32 is lane e + 32
        const float other = __shfl_xor(nv[0], 32, 64);
        const int e = lane & 31;
        const float c = rope[e], s = rope[HALF + e];
        y[base + lane] = lane < 32 ? nv[0] * c - other * s : other * s + nv[0] * c;
    }
}

__global__ void add_scale_kernel(const float *__restrict__ a, const float *__restrict__ b, float *out, int n, float scale)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = scale * (a[i] + b[i]);
}

__device__ __forceinline__ float gelu_mul_f32(float g, float u)
{
    // lower.rs:2926-2955: clamp, tanh-GELU on the f32 accumulator, times the context
    const float ax = fminf(20.0f, fmaxf(-20.0f, g));
    const float t = 0.79788456f * (ax + 0.044715f * ((ax * ax) * ax));
    return (0.5f * ax) * (1.0f + tanhf(t)) * u;
}

// y[r] = gelu(W[r].x) * ctx[r], W Q4_K.  A few hundred rows of a few thousand
// columns: one wave per row, four lanes per superblock (one 64-element group
// each).  The vector is staged in LDS once per workgroup; with HAS_RES the
// workgroup first closes the feed-forward block itself,
//   x = res + rms(y) * w_post      (RmsNormAdd, gemma_prim.rs:1150-1160)
// and workgroup 0 writes the new residual stream out.  The first superblock's
// weight loads are issued ahead of the staging.
constexpr int kGmWaves = 4;

template <bool HAS_RES>
__global__ __launch_bounds__(kGmWaves * 64) void q4k_gemv_gelu_mul_kernel(const uint8_t *__restrict__ W,
                                                                         const float *__restrict__ x,
                                                                         const float *__restrict__ ctx, float *y,
                                                                         int rows, int bpr, const float *__restrict__ w_post,
                                                                         const float *__restrict__ res, float *x_out, float eps)
{
    extern __shared__ __attribute__((aligned(16))) float xs[];
    __shared__ float red[kGmWaves];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = min(blockIdx.x * kGmWaves + wave, rows - 1);   // (a wave past the end repeats the last row: same barriers)
    const int g = lane & 3, cols = bpr * 256;
    const uint8_t *wr = W + (size_t)row * bpr * 144;
    const int b0 = min(lane >> 2, bpr - 1);
    const uint8_t *blk0 = wr + (size_t)b0 * 144;
    uint4 hdr = ldg_u4(blk0, 0), q0 = ldg_u4(blk0 + 16 + 32 * g, 0), q1 = ldg_u4(blk0 + 16 + 32 * g, 1);
    const float cr = ctx[row];   // fetched now: at the end it would be a cold round trip on the critical path

    // all of the vector's loads go out before anything is used (cols <= 8192: at most 8 float4 per thread and array)
    constexpr int KMAX = 8192 / 4 / (kGmWaves * 64);
    const int n4 = cols / 4;
    float4 xv[KMAX], wv[HAS_RES ? KMAX : 1], rv[HAS_RES ? KMAX : 1];
#pragma unroll
    for (int k = 0; k < KMAX; k++) {
        const int i = min(tid + k * kGmWaves * 64, n4 - 1);
        xv[k] = ldg_f4(x, i);
        if (HAS_RES) { wv[k] = ldg_f4(w_post, i); rv[k] = ldg_f4(res, i); }
    }
    float inv = 0.f;
    if (HAS_RES) {
        float ss = 0.f;
#pragma unroll
        for (int k = 0; k < KMAX; k++)
            if (tid + k * kGmWaves * 64 < n4) ss += (xv[k].x * xv[k].x + xv[k].y * xv[k].y) + (xv[k].z * xv[k].z + xv[k].w * xv[k].w);
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        inv = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)cols + eps);
    }
#pragma unroll
    for (int k = 0; k < KMAX; k++) {
        const int i = tid + k * kGmWaves * 64;
        if (i >= n4) continue;
        float4 o = xv[k];
        if (HAS_RES) {
            o = make_float4(rv[k].x + o.x * inv * wv[k].x, rv[k].y + o.y * inv * wv[k].y, rv[k].z + o.z * inv * wv[k].z, rv[k].w + o.w * inv * wv[k].w);
            if (blockIdx.x == 0) stg_f4(x_out, i, o);
        }
        *reinterpret_cast<float4 *>(xs + 4 * i + (i >> 4) * 4) = o;   // four floats of padding per 64: the groups of a wave land on distinct banks
    }
    __syncthreads();

    float acc = 0.f;
    for (int b = lane >> 2; b < bpr; b += 16) {
        if (b != b0) {
            const uint8_t *blk = wr + (size_t)b * 144;
            hdr = ldg_u4(blk, 0);
            q0 = ldg_u4(blk + 16 + 32 * g, 0);
            q1 = ldg_u4(blk + 16 + 32 * g, 1);
        }
        const uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        const float4 *xg = reinterpret_cast<const float4 *>(xs + (size_t)b * 256 + 64 * g + (4 * b + g) * 4);
        float lo = 0.f, hi = 0.f, sl = 0.f, sh = 0.f;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float4 a = xg[k], c = xg[8 + k];
            const uint32_t v = qw[k];
            lo += (float)(v & 15u) * a.x + (float)((v >> 8) & 15u) * a.y + (float)((v >> 16) & 15u) * a.z +
                  (float)((v >> 24) & 15u) * a.w;
            hi += (float)((v >> 4) & 15u) * c.x + (float)((v >> 12) & 15u) * c.y + (float)((v >> 20) & 15u) * c.z +
                  (float)(v >> 28) * c.w;
            sl += (a.x + a.y) + (a.z + a.w);
            sh += (c.x + c.y) + (c.z + c.w);
        }
        const float d = half_bits_to_f32(hdr.x & 0xFFFFu), dmin = half_bits_to_f32(hdr.x >> 16);
        const uint4 s = q4k_group_scales(hdr.y, hdr.z, hdr.w, g);
        acc += d * ((float)s.x * lo + (float)s.z * hi) - dmin * ((float)s.y * sl + (float)s.w * sh);
    }
    acc = wave_sum(acc);
    if (lane == 0 && blockIdx.x * kGmWaves + wave < rows) y[row] = gelu_mul_f32(acc, cr);
}

int launch_per_head(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int n_heads = (int)k.desc.dims[0], hd = (int)k.desc.dims[1], mode = (int)k.desc.dims[2];
    const float *rope = mode ? (const float *)a.in[2] : nullptr;
    const float *meta = mode == 2 ? (const float *)a.in[3] : nullptr;
#define KSH_PH(HD)                                                                                                  \
    hipLaunchKernelGGL((per_head_kernel<HD>), dim3(n_heads), dim3(64), 0, st, (const float *)a.in[0],               \
                       (const float *)a.in[1], rope, meta, (float *)a.out[0], k.desc.params[0], (int)k.desc.dims[3], (int)k.desc.dims[4], (int)k.desc.dims[5])
    switch (hd) {
    case 64: KSH_PH(64); break;
    case 128: KSH_PH(128); break;
    case 256: KSH_PH(256); break;
    case 512: KSH_PH(512); break;
    }
#undef KSH_PH
    return done("rmsnorm_per_head launch");
}

int launch_add_scale(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int n = (int)k.desc.dims[0];
    hipLaunchKernelGGL(add_scale_kernel, dim3((n + 255) / 256), dim3(256), 0, st, (const float *)a.in[0],
                       (const float *)a.in[1], (float *)a.out[0], n, k.desc.params[0]);
    return done("add_scale launch");
}

int launch_gelu_mul_gemv(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int rows = (int)k.desc.dims[0], bpr = (int)(k.desc.dims[1] / 256);
    const dim3 grid((rows + kGmWaves - 1) / kGmWaves), block(kGmWaves * 64);
    const size_t lds = (size_t)(k.desc.dims[1] + k.desc.dims[1] / 64 * 4) * 4;
    if (k.desc.dims[2])
        hipLaunchKernelGGL(q4k_gemv_gelu_mul_kernel<true>, grid, block, lds, st, (const uint8_t *)a.in[0], (const float *)a.in[1],
                           (const float *)a.in[2], (float *)a.out[0], rows, bpr, (const float *)a.in[3], (const float *)a.in[4],
                           (float *)a.out[1], k.desc.params[0]);
    else
        hipLaunchKernelGGL(q4k_gemv_gelu_mul_kernel<false>, grid, block, lds, st, (const uint8_t *)a.in[0], (const float *)a.in[1],
                           (const float *)a.in[2], (float *)a.out[0], rows, bpr, nullptr, nullptr, nullptr, 0.f);
    return done("matvec_gelu_mul launch");
}

}  // namespace

int bind_ple_ops(ksh_kernel &k)
{
    const int64_t *d = k.desc.dims;
    switch (k.desc.kind) {
    case KSH_RMSNORM_PER_HEAD: {
        const int64_t n_heads = d[0], hd = d[1], mode = d[2], max_seq = d[3];
        if (n_heads <= 0 || n_heads > 65535) return set_error("rmsnorm_per_head: n_heads=%lld", (long long)n_heads);
        if (hd != 64 && hd != 128 && hd != 256 && hd != 512)
            return set_error("rmsnorm_per_head: hd=%lld is not built (64, 128, 256, 512 are)", (long long)hd);
        if (mode < 0 || mode > 2) return set_error("rmsnorm_per_head: dims[2]=%lld (0 norm only, 1 rope row, 2 rope table + meta)", (long long)mode);
        if (mode == 2 && (max_seq <= 0 || max_seq > (1 << 24))) return set_error("rmsnorm_per_head: max_seq=%lld", (long long)max_seq);
        // dims[4] = heads per token when the heads belong to a chunk of consecutive positions (rope = 2 only)
        if (d[4] < 0 || (d[4] && (mode != 2 || n_heads % d[4]))) return set_error("rmsnorm_per_head: heads per token %lld", (long long)d[4]);
        k.info.n_inputs = 2 + (int)mode;
        k.info.n_outputs = 1;
        k.in_bytes[0] = k.out_bytes[0] = (size_t)n_heads * hd * 4;
        k.in_bytes[1] = (size_t)hd * 4;
        k.in_bytes[2] = (size_t)hd * 4 * (mode == 2 ? (size_t)max_seq : 1);
        // dims[5] = 1: one meta record per token (tokens of different sequences; needs heads per token)
        if (d[5] < 0 || d[5] > 1 || (d[5] && !d[4])) return set_error("rmsnorm_per_head: dims[5]=%lld (per-token positions need heads per token)", (long long)d[5]);
        k.in_bytes[3] = d[5] ? (size_t)16 * (n_heads / d[4]) : 16;
        for (int i = 0; i < 4; i++) k.in_align[i] = 4;
        k.out_align[0] = 4;
        set_launch(k, (uint32_t)n_heads, 1, 1, 64, 0);
        set_name(k, "rmsnorm_per_head%s_hd%d", mode ? "_rope" : "", (int)hd);
        k.launch = launch_per_head;
        return 0;
    }
    case KSH_ADD_SCALE: {
        const int64_t n = d[0];
        if (n <= 0 || n > (1ll << 30)) return set_error("add_scale: n=%lld", (long long)n);
        k.info.n_inputs = 2;
        k.info.n_outputs = 1;
        k.in_bytes[0] = k.in_bytes[1] = k.out_bytes[0] = (size_t)n * 4;
        k.in_align[0] = k.in_align[1] = k.out_align[0] = 4;
        set_launch(k, (uint32_t)((n + 255) / 256), 1, 1, 256, 0);
        set_name(k, "add_scale");
        k.launch = launch_add_scale;
        return 0;
    }
    case KSH_MATVEC_GELU_MUL: {
        const int64_t rows = d[0], cols = d[1];
        if (k.desc.dtypes[0] != KSH_Q4K) return set_error("matvec_gelu_mul: weight dtype %d is not built (Q4_K is)", k.desc.dtypes[0]);
        if (k.desc.dtypes[1] != KSH_F32 && k.desc.dtypes[1] != 0)
            return set_error("matvec_gelu_mul: activation dtype %d is not built (f32 only)", k.desc.dtypes[1]);
        if (rows <= 0 || rows > (1 << 24)) return set_error("matvec_gelu_mul: rows=%lld", (long long)rows);
        if (cols <= 0 || cols % 256 || cols > 8192) return set_error("matvec_gelu_mul: cols=%lld is not a positive multiple of 256 up to 8192", (long long)cols);
        const bool has_res = d[2] != 0;
        k.info.n_inputs = has_res ? 5 : 3;
        k.info.n_outputs = has_res ? 2 : 1;
        k.in_bytes[3] = k.in_bytes[4] = k.out_bytes[1] = (size_t)cols * 4;
        k.in_align[3] = k.in_align[4] = k.out_align[1] = 16;
        k.in_bytes[0] = (size_t)rows * (cols / 256) * 144; k.in_align[0] = 16;
        k.in_bytes[1] = (size_t)cols * 4; k.in_align[1] = 16;
        k.in_bytes[2] = (size_t)rows * 4; k.in_align[2] = 4;
        k.out_bytes[0] = (size_t)rows * 4; k.out_align[0] = 4;
        set_launch(k, (uint32_t)((rows + kGmWaves - 1) / kGmWaves), 1, 1, kGmWaves * 64, (uint32_t)(cols + cols / 64 * 4) * 4);
        set_name(k, "%smatvec_gelu_mul_q4k", has_res ? "addrms_" : "");
        k.launch = launch_gelu_mul_gemv;
        return 0;
    }
    }
    return set_error("bind_ple_ops: kind %d", k.desc.kind);
}

}  // namespace ksh
