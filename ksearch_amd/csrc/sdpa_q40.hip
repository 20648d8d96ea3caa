// Decode attention over a Q4_0 KV cache for MQA/GQA on gfx950.
//
// Takes the place of lower_sdpa_online, lower_sdpa_mwg_part and
// lower_sdpa_mwg_reduce (crates/ksearch_codegen/src/lower.rs:4897-5359,
// 5367-5894, 5897-6087) and of the serial per-slot loop of the reference's
// scheduler (crates/ksearch_cli/src/scheduler.rs:163-187): one launch covers
// every (slot, kv head, partition).
//
// Semantics kept from the reference:
//   - K/V are Q4_0 [max_t, n_kv, hd]; rows [start, start+tlen) are attended;
//     meta = f32 {tlen, start, window} per slot (window is carried, the host
//     already folded it into start/tlen, gemma_prim.rs:1010-1017);
//   - q heads h map to kv head h / (n_q / n_kv);
//   - split-KV: partition p of nwg covers [p*chunk, min((p+1)*chunk, tlen)),
//     chunk = ceil(tlen / nwg); its partial is (m, l, O[hd]) with m = -1e30,
//     l = 0 when empty; the merge is the log-sum-exp fold of :5897-6087;
//   - `scale` multiplies q.k (1.0 reproduces the reference, which has none).
// The softmax runs tile-wise (max over a tile of KV rows, then one rescale)
// instead of row by row; that is the same function up to rounding.
//
// This file holds the f32 vector-ALU form: a workgroup stages a tile of KV
// rows in LDS, dequantized, then
//   scores   thread = (row, head subset): dot of the LDS row with q (broadcast)
//   softmax  wave = head pair, lane = row
//   P.V      thread = head-dim element, 8 heads in registers
#include "ksh_device.hpp"
#include "ksh_internal.hpp"

namespace ksh {
namespace {

constexpr int kThreads = 256;
constexpr int kTile = 32;          // KV rows per LDS tile
constexpr int kMaxGroups = 16;     // q heads per kv head

struct SdpaParams {
    const float *q;         // [n_slots][n_q*hd]
    const uint8_t *k, *v;   // [n_slots][max_t*n_kv*row_bytes]
    const float *meta;      // [n_slots][meta_stride]
    float *tmp;             // [n_slots][n_q][nwg][hd+2]
    float *out;             // [n_slots][n_q*hd]
    int n_q, n_kv, hd, max_t, nwg, meta_stride;
    float scale;
    int direct;             // 1: single partition, write normalised output, no tmp
    int kv_shared;          // every slot attends the same cache (a chunk of prompt tokens)
};

__device__ __forceinline__ int pad_stride(int hd) { return hd + 4; }

// grid = (nwg, n_kv, n_slots)
__global__ __launch_bounds__(kThreads) void sdpa_part_kernel(SdpaParams p)
{
    extern __shared__ float smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int part = blockIdx.x, kvh = blockIdx.y, slot = blockIdx.z;
    const int hd = p.hd, groups = p.n_q / p.n_kv, nblk = hd / 32, stride = pad_stride(hd);
    float *qs = smem;                         // [groups][hd]
    float *kt = qs + groups * hd;             // [kTile][stride]
    float *vt = kt + kTile * stride;          // [kTile][stride]
    float *sc = vt + kTile * stride;          // [groups][kTile] scores, then probabilities
    float *alpha_s = sc + kMaxGroups * kTile; // [groups]

    const float *meta = p.meta + (size_t)slot * p.meta_stride;
    const int tlen = (int)meta[0], start = (int)meta[1];
    const int chunk = (tlen + p.nwg - 1) / p.nwg;
    const int p0 = part * chunk, p1 = min(p0 + chunk, tlen);

    const size_t row_bytes = (size_t)nblk * 18;
    const size_t slot_bytes = p.kv_shared ? 0 : (size_t)p.max_t * p.n_kv * row_bytes;
    const uint8_t *kbase = p.k + (size_t)slot * slot_bytes;
    const uint8_t *vbase = p.v + (size_t)slot * slot_bytes;
    const float *qg = p.q + ((size_t)slot * p.n_q + (size_t)kvh * groups) * hd;

    for (int i = tid; i < groups * hd; i += kThreads) qs[i] = qg[i];

    // running state: wave w owns heads w, w+4, ... for the softmax bookkeeping;
    // every thread keeps O for its head-dim elements and all heads
    float m_run[kMaxGroups / 4], l_run[kMaxGroups / 4];
#pragma unroll
    for (int j = 0; j < kMaxGroups / 4; j++) { m_run[j] = -1.0e30f; l_run[j] = 0.f; }
    float O[kMaxGroups][2];
#pragma unroll
    for (int h = 0; h < kMaxGroups; h++) O[h][0] = O[h][1] = 0.f;

    for (int t0 = p0; t0 < p1; t0 += kTile) {
        const int nt = min(kTile, p1 - t0);
        __syncthreads();   // previous tile fully consumed (and qs written, first time round)
        // dequantize the K and V rows of this tile into LDS: one thread per Q4_0 block
        for (int i = tid; i < nt * nblk * 2; i += kThreads) {
            const int which = i / (nt * nblk), j = i % (nt * nblk), r = j / nblk, b = j % nblk;
            const uint8_t *blk = (which ? vbase : kbase) +
                                 ((size_t)(start + t0 + r) * p.n_kv + kvh) * row_bytes + (size_t)b * 18;
            float *dst = (which ? vt : kt) + r * stride + b * 32;
            const float d = half_bits_to_f32((uint32_t)blk[0] | ((uint32_t)blk[1] << 8));
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const uint32_t byte = blk[2 + e];
                dst[e] = (float)((int)(byte & 0x0F) - 8) * d;        // gguf_impl.rs:626-629
                dst[e + 16] = (float)((int)(byte >> 4) - 8) * d;
            }
        }
        __syncthreads();
        // scores: thread (row r = tid % kTile, head subset tid / kTile)
        {
            const int r = tid % kTile, hs = tid / kTile;
            if (r < nt) {
                const float4 *krow = reinterpret_cast<const float4 *>(kt + r * stride);
                for (int h = hs; h < groups; h += kThreads / kTile) {
                    const float4 *qh = reinterpret_cast<const float4 *>(qs + h * hd);
                    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
                    for (int d4 = 0; d4 < hd / 4; d4++) {
                        const float4 kk = krow[d4], qq = qh[d4];
                        a0 = fmaf(qq.x, kk.x, a0);
                        a1 = fmaf(qq.y, kk.y, a1);
                        a2 = fmaf(qq.z, kk.z, a2);
                        a3 = fmaf(qq.w, kk.w, a3);
                    }
                    sc[h * kTile + r] = ((a0 + a1) + (a2 + a3)) * p.scale;
                }
            }
        }
        __syncthreads();
        // softmax bookkeeping: wave w, heads w, w+4, ...; lanes 0..kTile-1 = rows
#pragma unroll
        for (int j = 0; j < kMaxGroups / 4; j++) {
            const int h = wave + 4 * j;
            if (h < groups) {
                const float s = lane < nt ? sc[h * kTile + lane] : -INFINITY;
                const float m2 = fmaxf(m_run[j], wave_max(s));
                const float e = lane < nt ? __expf(s - m2) : 0.f;
                const float a = __expf(m_run[j] - m2);
                l_run[j] = l_run[j] * a + wave_sum(e);
                m_run[j] = m2;
                if (lane < kTile) sc[h * kTile + lane] = e;
                if (lane == 0) alpha_s[h] = a;
            }
        }
        __syncthreads();
        // O = O*alpha + P.V: thread owns head-dim elements tid and tid+256
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int d = tid + c * kThreads;
            if (d < hd) {
#pragma unroll
                for (int h = 0; h < kMaxGroups; h++)
                    if (h < groups) O[h][c] *= alpha_s[h];
                for (int r = 0; r < nt; r++) {
                    const float vv = vt[r * stride + d];
#pragma unroll
                    for (int h = 0; h < kMaxGroups; h++)
                        if (h < groups) O[h][c] = fmaf(sc[h * kTile + r], vv, O[h][c]);
                }
            }
        }
    }

    // publish (m, l) of each head, then write the partial or the final output
    __syncthreads();
    float *ml = sc;   // [groups][2]
#pragma unroll
    for (int j = 0; j < kMaxGroups / 4; j++) {
        const int h = wave + 4 * j;
        if (h < groups && lane == 0) { ml[2 * h] = m_run[j]; ml[2 * h + 1] = l_run[j]; }
    }
    __syncthreads();
    for (int h = 0; h < groups; h++) {
        const int head = kvh * groups + h;
        if (p.direct) {
            const float inv_l = 1.0f / ml[2 * h + 1];
            float *o = p.out + ((size_t)slot * p.n_q + head) * hd;
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const int d = tid + c * kThreads;
                if (d < hd) o[d] = O[h][c] * inv_l;
            }
        } else {
            float *rec = p.tmp + (((size_t)slot * p.n_q + head) * p.nwg + part) * (size_t)(hd + 2);
            if (tid == 0) { rec[0] = ml[2 * h]; rec[1] = ml[2 * h + 1]; }
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const int d = tid + c * kThreads;
                if (d < hd) rec[2 + d] = O[h][c];
            }
        }
    }
}

// grid = (n_q, n_slots); lower.rs:5897-6087
__global__ __launch_bounds__(kThreads) void sdpa_reduce_kernel(const float *tmp, float *out, int n_q, int hd, int nwg)
{
    const int head = blockIdx.x, slot = blockIdx.y, tid = threadIdx.x;
    const float *base = tmp + ((size_t)slot * n_q + head) * nwg * (size_t)(hd + 2);
    float m = -1.0e30f, l = 0.f, O0 = 0.f, O1 = 0.f;
    for (int pt = 0; pt < nwg; pt++) {
        const float *rec = base + (size_t)pt * (hd + 2);
        const float mp = rec[0], lp = rec[1];
        const float m2 = fmaxf(m, mp);
        const float a = __expf(m - m2), b = __expf(mp - m2);
        l = l * a + lp * b;
        m = m2;
        if (tid < hd) O0 = O0 * a + rec[2 + tid] * b;
        if (tid + kThreads < hd) O1 = O1 * a + rec[2 + tid + kThreads] * b;
    }
    const float inv_l = 1.0f / l;
    float *o = out + ((size_t)slot * n_q + head) * hd;
    if (tid < hd) o[tid] = O0 * inv_l;
    if (tid + kThreads < hd) o[tid + kThreads] = O1 * inv_l;
}

size_t part_lds_bytes(int groups, int hd)
{
    return ((size_t)groups * hd + 2 * (size_t)kTile * (hd + 4) + (size_t)kMaxGroups * kTile + kMaxGroups) * sizeof(float);
}

int done(const char *what)
{
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, what);
}

void launch_part(const SdpaParams &p, int n_slots, hipStream_t st)
{
    hipLaunchKernelGGL(sdpa_part_kernel, dim3(p.nwg, p.n_kv, n_slots), dim3(kThreads),
                       part_lds_bytes(p.n_q / p.n_kv, p.hd), st, p);
}

SdpaParams base_params(const ksh_kernel &k)
{
    SdpaParams p{};
    p.n_q = (int)k.desc.dims[0];
    p.n_kv = (int)k.desc.dims[1];
    p.hd = (int)k.desc.dims[2];
    p.max_t = (int)k.desc.dims[3];
    p.scale = k.desc.params[0];
    p.meta_stride = 0;
    return p;
}

int launch_naive(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    SdpaParams p = base_params(k);
    p.q = (const float *)a.in[0]; p.k = (const uint8_t *)a.in[1]; p.v = (const uint8_t *)a.in[2];
    p.meta = (const float *)a.in[3];
    p.out = (float *)a.out[0];
    p.nwg = 1;
    p.direct = 1;
    launch_part(p, 1, st);
    return done("sdpa_naive launch");
}

int launch_mwg_part(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    SdpaParams p = base_params(k);
    p.q = (const float *)a.in[0]; p.k = (const uint8_t *)a.in[1]; p.v = (const uint8_t *)a.in[2];
    p.meta = (const float *)a.in[3];
    p.tmp = (float *)a.out[0];
    p.nwg = (int)k.desc.dims[4];
    launch_part(p, 1, st);
    return done("sdpa_mwg_part launch");
}

int launch_mwg_reduce(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int n_q = (int)k.desc.dims[0], hd = (int)k.desc.dims[1], nwg = (int)k.desc.dims[2];
    hipLaunchKernelGGL(sdpa_reduce_kernel, dim3(n_q, 1), dim3(kThreads), 0, st, (const float *)a.in[0],
                       (float *)a.out[0], n_q, hd, nwg);
    return done("sdpa_mwg_reduce launch");
}

int launch_slots(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    SdpaParams p = base_params(k);
    const int n_slots = (int)k.desc.dims[4];
    p.q = (const float *)a.in[0]; p.k = (const uint8_t *)a.in[1]; p.v = (const uint8_t *)a.in[2];
    p.meta = (const float *)a.in[3];
    p.meta_stride = 4;
    p.tmp = (float *)a.out[0];
    p.out = (float *)a.out[1];
    p.nwg = k.variant;
    launch_part(p, n_slots, st);
    if (done("sdpa_slots part launch")) return 1;
    hipLaunchKernelGGL(sdpa_reduce_kernel, dim3(p.n_q, n_slots), dim3(kThreads), 0, st, p.tmp, p.out, p.n_q, p.hd,
                       p.nwg);
    return done("sdpa_slots reduce launch");
}

// same per-token records as the register form writes (lower.rs:4961-4983)
__global__ void sdpa_batch_meta_tile_kernel(const float *meta, float *tok_meta, int n_tok)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_tok) return;
    const int abs_t = (int)meta[0] + i, win = (int)meta[2];
    const int tlen = min(abs_t, win);
    tok_meta[4 * i] = (float)tlen;
    tok_meta[4 * i + 1] = (float)(abs_t - tlen);
    tok_meta[4 * i + 2] = (float)win;
    tok_meta[4 * i + 3] = 0.f;
}

int launch_batch(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    SdpaParams p = base_params(k);
    const int n_tok = (int)k.desc.dims[4];
    float *tok_meta = (float *)k.scratch;
    hipLaunchKernelGGL(sdpa_batch_meta_tile_kernel, dim3((n_tok + 255) / 256), dim3(256), 0, st, (const float *)a.in[3], tok_meta, n_tok);
    p.q = (const float *)a.in[0]; p.k = (const uint8_t *)a.in[1]; p.v = (const uint8_t *)a.in[2];
    p.meta = tok_meta;
    p.meta_stride = 4;
    p.tmp = (float *)a.out[0];
    p.out = (float *)a.out[1];
    p.nwg = k.variant;
    p.kv_shared = 1;
    launch_part(p, n_tok, st);
    if (done("sdpa_batch part launch")) return 1;
    hipLaunchKernelGGL(sdpa_reduce_kernel, dim3(p.n_q, n_tok), dim3(kThreads), 0, st, p.tmp, p.out, p.n_q, p.hd, p.nwg);
    return done("sdpa_batch reduce launch");
}

int check_shape(const char *what, int64_t n_q, int64_t n_kv, int64_t hd, int64_t max_t)
{
    if (n_q <= 0 || n_kv <= 0 || n_q % n_kv || n_q / n_kv > kMaxGroups || n_q > 4096)
        return set_error("%s: n_q=%lld n_kv=%lld (q heads per kv head must divide evenly and be <= %d)", what,
                         (long long)n_q, (long long)n_kv, kMaxGroups);
    if (hd <= 0 || hd % 32 || hd > 512) return set_error("%s: sdpa hd must be multiple of 32, at most 512 (got %lld)", what, (long long)hd);
    if (max_t <= 0 || max_t > (1 << 24)) return set_error("%s: max_t=%lld", what, (long long)max_t);
    if (part_lds_bytes((int)(n_q / n_kv), (int)hd) > 160 * 1024) return set_error("%s: tile does not fit LDS", what);
    return 0;
}

}  // namespace

int bind_sdpa(ksh_kernel &k)
{
    const int64_t *d = k.desc.dims;
    if (k.desc.kind == KSH_SDPA_MWG_REDUCE) {
        const int64_t n_q = d[0], hd = d[1], nwg = d[2];
        if (n_q <= 0 || hd <= 0 || hd % 32 || hd > 512 || nwg <= 0 || nwg > 4096)
            return set_error("sdpa_mwg_reduce: n_q=%lld hd=%lld nwg=%lld", (long long)n_q, (long long)hd, (long long)nwg);
        k.info.n_inputs = 1;
        k.info.n_outputs = 1;
        k.in_bytes[0] = (size_t)n_q * nwg * (hd + 2) * 4; k.in_align[0] = 4;
        k.out_bytes[0] = (size_t)n_q * hd * 4; k.out_align[0] = 4;
        set_launch(k, (uint32_t)n_q, 1, 1, kThreads, 0);
        set_name(k, "sdpa_mwg_reduce_hd%d_nwg%d", (int)hd, (int)nwg);
        k.launch = launch_mwg_reduce;
        return 0;
    }
    if (k.desc.dtypes[0] != KSH_Q40) return set_error("sdpa: kv dtype %d is not built (Q4_0 is)", k.desc.dtypes[0]);
    const int64_t n_q = d[0], n_kv = d[1], hd = d[2], max_t = d[3];
    if (check_shape("sdpa", n_q, n_kv, hd, max_t)) return 1;
    const size_t kvb = (size_t)max_t * n_kv * (hd / 32) * 18;
    const uint32_t lds = (uint32_t)part_lds_bytes((int)(n_q / n_kv), (int)hd);
    // the register form takes the shapes it is built for; sched.vec = 1 asks for the tile form
    const bool lanes = sdpa_lanes_supports(n_q, n_kv, hd) && k.desc.sched.vec != 1;
    int lanes_nwg = 1, lanes_slots = 1;
    switch (k.desc.kind) {
    case KSH_SDPA_NAIVE:
        k.info.n_inputs = 4;
        k.info.n_outputs = 1;
        k.in_bytes[0] = (size_t)n_q * hd * 4; k.in_bytes[1] = k.in_bytes[2] = kvb; k.in_bytes[3] = 12;
        k.out_bytes[0] = (size_t)n_q * hd * 4;
        set_launch(k, 1, (uint32_t)n_kv, 1, kThreads, lds);
        set_name(k, "sdpa_naive_hd%d", (int)hd);
        k.launch = launch_naive;
        break;
    case KSH_SDPA_MWG_PART: {
        const int64_t nwg = d[4];
        if (nwg <= 0 || nwg > 4096) return set_error("sdpa_mwg_part: nwg=%lld", (long long)nwg);
        k.info.n_inputs = 4;
        k.info.n_outputs = 1;
        k.in_bytes[0] = (size_t)n_q * hd * 4; k.in_bytes[1] = k.in_bytes[2] = kvb; k.in_bytes[3] = 12;
        k.out_bytes[0] = (size_t)n_q * nwg * (hd + 2) * 4;
        set_launch(k, (uint32_t)nwg, (uint32_t)n_kv, 1, kThreads, lds);
        set_name(k, "sdpa_mwg_part_hd%d_nwg%d", (int)hd, (int)nwg);
        k.launch = launch_mwg_part;
        lanes_nwg = (int)nwg;
        break;
    }
    case KSH_SDPA_SLOTS: {
        const int64_t n_slots = d[4];
        int64_t nwg = d[5];
        if (n_slots <= 0 || n_slots > 65535) return set_error("sdpa_slots: n_slots=%lld", (long long)n_slots);
        if (nwg == 0 && k.desc.sched.k_split) nwg = k.desc.sched.k_split;   // K-split from the schedule
        if (nwg == 0 && lanes) {
            // two workgroups per CU, at least 64 rows each, and few enough partials for one workgroup to fold
            nwg = (512 + n_slots * n_kv - 1) / (n_slots * n_kv);
            const int64_t cap = (max_t + 63) / 64;
            if (nwg > cap) nwg = cap;
            if (nwg > 64) nwg = 64;
            if (nwg < 1) nwg = 1;
        }
        if (nwg == 0) {
            // enough partitions to put ~4 workgroups on each of the 256 CUs, rows permitting
            nwg = (1024 + n_slots * n_kv - 1) / (n_slots * n_kv);
            const int64_t cap = (max_t + 4 * kTile - 1) / (4 * kTile);
            if (nwg > cap) nwg = cap;
            if (nwg < 1) nwg = 1;
        }
        if (nwg < 0 || nwg > 4096) return set_error("sdpa_slots: nwg=%lld", (long long)nwg);
        // dims[6] = slots in the K / V pools when the launch's entries are a subset of them in any order (one decode
        // step for several sequences): a 5th input f32[n_slots] names each entry's slot
        const int64_t pool_slots = d[6];
        if (pool_slots < 0 || pool_slots > 65535) return set_error("sdpa_slots: pool slots=%lld", (long long)pool_slots);
        // dims[7] = bytes from one slot of the pools to the next (0: max_t rows; a pool sized for wider heads has more)
        const int64_t slot_stride = d[7];
        if (slot_stride < 0 || (slot_stride && (!pool_slots || (size_t)slot_stride < kvb || slot_stride % 2)))
            return set_error("sdpa_slots: slot stride %lld", (long long)slot_stride);
        if (pool_slots && !lanes) return set_error("sdpa_slots: entries that name their pool slot are built for the register form only (hd 128 / 256 / 512, up to 8 q heads per kv head)");
        k.info.n_inputs = pool_slots ? 5 : 4;
        k.info.n_outputs = 2;
        k.in_bytes[0] = (size_t)n_slots * n_q * hd * 4;
        k.in_bytes[1] = k.in_bytes[2] = pool_slots ? (size_t)(pool_slots - 1) * (slot_stride ? (size_t)slot_stride : kvb) + kvb : kvb * (size_t)n_slots;
        k.in_bytes[3] = (size_t)n_slots * 16;
        k.in_bytes[4] = pool_slots ? (size_t)n_slots * 4 : 0;
        k.in_align[4] = 4;
        k.out_bytes[0] = (size_t)n_slots * n_q * nwg * (hd + 2) * 4;
        k.out_bytes[1] = (size_t)n_slots * n_q * hd * 4;
        k.out_align[1] = 4;
        if (k.desc.params[1] != 0.f) {
            // params[1] != 0: out[1] is the prepared operand of a decode round's GEMM (KSH_MATVEC_ROUND) over the n_q * hd
            // columns, row = slot
            const int64_t cols = n_q * hd;
            if (!lanes || n_slots < 2 || n_slots > 16 || nwg < 2 || nwg > 64 || cols % 256)
                return set_error("sdpa_slots: the result as a prepared operand takes 2 to 16 slots, 2 to 64 partitions and n_q * hd a multiple of 256");
            k.out_bytes[1] = (size_t)(64 * cols + 2048 * (cols / 256));
            k.out_align[1] = 16;
        }
        set_launch(k, (uint32_t)nwg, (uint32_t)n_kv, (uint32_t)n_slots, kThreads, lds);
        set_name(k, "sdpa_slots_hd%d_nwg%d", (int)hd, (int)nwg);
        k.variant = (int)nwg;
        k.info.sched.k_split = (uint32_t)nwg;
        k.info.sched.lds_tile = kTile;
        k.launch = launch_slots;
        lanes_nwg = (int)nwg;
        lanes_slots = (int)n_slots;
        break;
    }
    case KSH_SDPA_BATCH: {
        // sdpa_hybrid_kv_batch (crates/ksearch_kernels/src/lib.rs:1592-1623): n_tok consecutive prompt tokens over one cache
        const int64_t n_tok = d[4];
        int64_t nwg = d[5];
        if (n_tok <= 0 || n_tok > 4096) return set_error("sdpa_batch: n_tok=%lld", (long long)n_tok);
        if (nwg == 0 && k.desc.sched.k_split) nwg = k.desc.sched.k_split;
        if (nwg == 0 && (hd == 256 || hd == 512) && n_q / n_kv <= 8 && n_tok > 16 && k.desc.sched.vec != 1 && k.desc.sched.vec != 3) {
            nwg = 1;   // the matrix-core form of a chunk (one workgroup per token) is fastest with one partition per token
        }
        if (nwg == 0) {
            // ~4 workgroups per compute unit over all tokens, at least 64 rows per partition, at most 16 partitions
            nwg = (1024 + n_tok * n_kv - 1) / (n_tok * n_kv);
            const int64_t cap = (max_t + 63) / 64;
            if (nwg > cap) nwg = cap;
            if (nwg > 16) nwg = 16;
            if (nwg < 1) nwg = 1;
        }
        if (nwg < 0 || nwg > 64) return set_error("sdpa_batch: nwg=%lld", (long long)nwg);
        k.info.n_inputs = 4;
        k.info.n_outputs = 2;
        k.in_bytes[0] = (size_t)n_tok * n_q * hd * 4;
        k.in_bytes[1] = k.in_bytes[2] = kvb;
        k.in_bytes[3] = 12;
        k.out_bytes[0] = (size_t)n_tok * n_q * nwg * (hd + 2) * 4;
        k.out_bytes[1] = (size_t)n_tok * n_q * hd * 4;
        k.out_align[1] = 4;
        set_launch(k, (uint32_t)nwg, (uint32_t)n_kv, (uint32_t)n_tok, kThreads, lds);
        set_name(k, "sdpa_batch_hd%d_t%d_nwg%d", (int)hd, (int)n_tok, (int)nwg);
        k.variant = (int)nwg;
        k.info.sched.k_split = (uint32_t)nwg;
        k.info.sched.lds_tile = kTile;
        k.scratch_bytes = (size_t)n_tok * 16;
        k.launch = launch_batch;
        lanes_nwg = (int)nwg;
        lanes_slots = (int)n_tok;
        break;
    }
    default: return set_error("bind_sdpa: kind %d", k.desc.kind);
    }
    k.in_align[0] = 4; k.in_align[1] = k.in_align[2] = 2; k.in_align[3] = 4; k.out_align[0] = 4;
    if (lanes) {
        k.in_align[0] = 16;
        if (bind_sdpa_lanes(k, lanes_nwg, lanes_slots)) return 1;
        char name[64];
        snprintf(name, sizeof(name), "%s", k.info.name);
        set_name(k, k.info.sched.vec == 2 ? "%s_mfma_w%d" : "%s_regs_w%d", name, (int)k.info.sched.nsg);
    }
    return 0;
}

}  // namespace ksh
