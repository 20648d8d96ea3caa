// Q6_K packed-weight GEMV for gfx950 (the LM head: 262144 x 2048).
//
// Takes the place of lower_matvec_q6k_coop
// (crates/ksearch_codegen/src/lower.rs:2086-2472) and
// ksearch_q6k_coop_frag_nr4_dev (crates/ksearch_codegen/src/render.rs:886-930),
// which give 2 lanes x 16 positions per superblock with byte loads on a
// 32-lane simdgroup.  Here:
//
//   - a superblock (210 B: ql[128] qh[64] sc[16] d) is owned by 8 lanes; lane
//     (ip, il) takes, in half ip of the block, positions l0 = 8*il .. +7 of all
//     four quadrants: 8 B of ql, 8 B of ql+32, 8 B of qh, the half's 8 scale
//     bytes and d.  Blocks are only 2-byte aligned, so these are unaligned
//     64-bit loads, which gfx950 global loads support;
//   - a wave sweeps 8 superblocks (2048 columns) per step; the activation
//     vector is staged once per workgroup in LDS as three int8 digit planes of
//     X = rint(x / s), s = max|x| / (2^20 - 1) per 128 elements (optionally
//     after an RMSNorm / add-then-RMSNorm computed by the workgroup itself,
//     gemv_prologue.hpp), and a lane keeps its 32 positions' digits in
//     registers across every row it owns;
//   - the 6-bit values are assembled four at a time with dword logic and meet
//     the digit planes in v_dot4_i32_i8 (exact integer sums per quadrant); the
//     -32 offset is applied through the pre-summed X of each run of 8:
//       y += d * s * sum_k sc_k * (sum(v*X) - 32*SX_k)
//     |x - s X| <= s/2 = 2^-21 of the run's largest magnitude, below the f32
//     summation noise of a 2048-term dot;
//   - a workgroup walks a long run of rows (x staged once), issuing the loads
//     of the next R rows before it consumes the current ones.
//
// The result differs from dequant-then-dot (gguf_impl.rs:761-791 +
// check_mul_mm.rs:60-71) by reassociation and by that rounding of x.
#include "gemv_prologue.hpp"
#include "ksh_internal.hpp"

KSH_STAMP_BUFFER
KSH_STAMP_READER(ksh_stamps_matvec_q6k)

namespace ksh {
namespace {

constexpr int kQ6kBytes = 210;

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ u32x2 ld64_unaligned(const uint8_t *p)
{
    // 2-byte-aligned address: the compiler emits one global_load_dwordx2
    u32x2 v;
    __builtin_memcpy(&v, p, 8);
    return v;
}

__device__ __forceinline__ int dot4_start(int a, int b)
{
    int r;
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

struct Q6kLane {
    u32x2 q1, q2, qh, sc;
    uint32_t d;      // half bits
};

__device__ __forceinline__ Q6kLane q6k_load(const uint8_t *blk, int ip, int il)
{
    Q6kLane r;
    r.q1 = ld64_unaligned(blk + 64 * ip + 8 * il);
    r.q2 = ld64_unaligned(blk + 64 * ip + 32 + 8 * il);
    r.qh = ld64_unaligned(blk + 128 + 32 * ip + 8 * il);
    r.sc = ld64_unaligned(blk + 192 + 8 * ip);
    uint16_t d;
    __builtin_memcpy(&d, blk + 208, 2);
    r.d = d;
    return r;
}

// a lane's share of the staged vector for one superblock: digit planes of its
// 8 positions in each quadrant k (two dwords each), minus the sum of X over
// them, and the scale of its 128-element half
struct XQ6 {
    uint32_t H[4][2], M[4][2], L[4][2];
    int nsx5[4];   // -32 * sum of X over the lane's 8 positions of quadrant k
    float s;
    __device__ __forceinline__ void load(const uint8_t *lds, int blk, int ip, int il, bool valid)
    {
        const uint8_t *half = lds + (blk * 2 + ip) * kQ6HalfBytes;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int o = 32 * k + 8 * il;
            const uint2 h = *reinterpret_cast<const uint2 *>(half + o);
            const uint2 m = *reinterpret_cast<const uint2 *>(half + 128 + o);
            const uint2 l = *reinterpret_cast<const uint2 *>(half + 256 + o);
            H[k][0] = h.x; H[k][1] = h.y; M[k][0] = m.x; M[k][1] = m.y; L[k][0] = l.x; L[k][1] = l.y;
            nsx5[k] = reinterpret_cast<const int *>(half + 384)[4 * k + il] * 32;
        }
        s = valid ? *reinterpret_cast<const float *>(half + 448) : 0.f;   // a lane past the row's end contributes nothing
    }
};

__device__ __forceinline__ float q6k_lane_dot(const Q6kLane &B, int il, const XQ6 &X)
{
    const uint32_t q1[2] = {B.q1.x, B.q1.y}, q2[2] = {B.q2.x, B.q2.y}, qh[2] = {B.qh.x, B.qh.y};
    int hs[4], ms[4], ls[4];
#pragma unroll
    for (int w = 0; w < 2; w++) {
        uint32_t a[4];
        a[0] = (q1[w] & 0x0F0F0F0Fu) | ((qh[w] << 4) & 0x30303030u);
        a[1] = (q2[w] & 0x0F0F0F0Fu) | ((qh[w] << 2) & 0x30303030u);
        a[2] = ((q1[w] >> 4) & 0x0F0F0F0Fu) | (qh[w] & 0x30303030u);
        a[3] = ((q2[w] >> 4) & 0x0F0F0F0Fu) | ((qh[w] >> 2) & 0x30303030u);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            if (w == 0) {
                // three-operand form with a literal zero: the accumulating form would need a zeroed register first
                hs[k] = dot4_start((int)a[k], (int)X.H[k][0]);
                ms[k] = dot4_start((int)a[k], (int)X.M[k][0]);
                ls[k] = __builtin_amdgcn_sdot4((int)a[k], (int)X.L[k][0], X.nsx5[k], false);   // starts at -32*sum(X)
            } else {
                hs[k] = __builtin_amdgcn_sdot4((int)a[k], (int)X.H[k][w], hs[k], false);
                ms[k] = __builtin_amdgcn_sdot4((int)a[k], (int)X.M[k][w], ms[k], false);
                ls[k] = __builtin_amdgcn_sdot4((int)a[k], (int)X.L[k][w], ls[k], false);
            }
        }
    }
    // the lane's 8 positions share is = l0/16 = il/2; scales sc[is + 2k]
    const uint32_t scw = (il & 2) ? ((B.sc.x >> 8) | (B.sc.y << 24)) : B.sc.x;
    const uint32_t sch = (il & 2) ? (B.sc.y >> 8) : B.sc.y;
    const float c[4] = {(float)(int8_t)(scw & 0xFF), (float)(int8_t)((scw >> 16) & 0xFF), (float)(int8_t)(sch & 0xFF),
                        (float)(int8_t)((sch >> 16) & 0xFF)};
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        // sum(v*X) - 32*sum(X), exact: |.| < 2^30
        const int xk = (((hs[k] << 7) + ms[k]) << 7) + ls[k];
        t = fmaf(c[k], (float)xk, t);
    }
    return (half_bits_to_f32(B.d) * X.s) * t;
}

struct Q6kParams {
    const uint8_t *W;
    float *y;
    Prologue pro;
    int rows, bpr, rows_per_wave;
};

// One step == 8 superblocks.  STEPS = ceil(bpr / 8); lanes whose superblock lies
// past the row's end re-read the last one against a zero scale.
template <int R, int NW, int STEPS>
__global__ __launch_bounds__(NW * 64) void q6k_gemv_kernel(Q6kParams p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bl = lane >> 3, ip = (lane >> 2) & 1, il = lane & 3;
    const int cols = p.bpr * 256;
    const size_t row_bytes = (size_t)p.bpr * kQ6kBytes;
    const int w0 = (blockIdx.x * NW + wave) * p.rows_per_wave;
    const int w1 = min(w0 + p.rows_per_wave, p.rows);

    Q6kLane cur[STEPS][R], nxt[STEPS][R];
    auto load_rows = [&](Q6kLane (&dst)[STEPS][R], int row0) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint8_t *rp = p.W + (size_t)min(row0 + r, p.rows - 1) * row_bytes;
#pragma unroll
            for (int s = 0; s < STEPS; s++)
                dst[s][r] = q6k_load(rp + (size_t)min(s * 8 + bl, p.bpr - 1) * kQ6kBytes, ip, il);
        }
    };
    constexpr int KMAX = (STEPS * 512 + NW * 64 - 1) / (NW * 64);   // float4 of the vector per thread: cols <= STEPS * 2048
    StageRegs sr;
    stage_fetch<NW * 64, false, KMAX>(p.pro, cols, sr);
    load_rows(cur, min(w0, p.rows - 1));   // unconditional (clamped): the staging wait can then leave these in flight
    stage_finish<kXQ6, NW * 64, false, KMAX>(p.pro, xs, cols, sr);
    __syncthreads();
    if (w0 >= w1) return;

    XQ6 X[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; s++) X[s].load(xs, min(s * 8 + bl, p.bpr - 1), ip, il, s * 8 + bl < p.bpr);

    for (int row0 = w0; row0 < w1; row0 += R) {
        load_rows(nxt, min(row0 + R, p.rows - 1));
#pragma unroll
        for (int r = 0; r < R; r++) {
            float acc = 0.f;
#pragma unroll
            for (int s = 0; s < STEPS; s++) acc += q6k_lane_dot(cur[s][r], il, X[s]);
            acc = wave_sum(acc);
            if (lane == 0 && row0 + r < w1) p.y[row0 + r] = acc;
        }
#pragma unroll
        for (int s = 0; s < STEPS; s++)
#pragma unroll
            for (int r = 0; r < R; r++) cur[s][r] = nxt[s][r];
    }
}

// ---- Q6K_ROWS: the same weights with every row regrouped by field ------------
// Row of bpr superblocks: ql [bpr][128] | qh [bpr][64] | sc [bpr][16] | d [bpr][2], each section 16-byte
// aligned, the row padded to a multiple of 16 bytes (q6r_row_bytes: 1264 for the 1260 bytes of a 1536-column
// row; nothing for 2048 or 4096 columns).  A step covers 8 superblocks with ONE 128-bit load per lane over 1 KB of ql, lane
// after lane: lane j = lane % 8 of superblock b = lane / 8 holds ql bytes 16j .. 16j+15, i.e. in half ip = j / 4
// the positions l0 = 16 * (j % 2) .. +15 of the quadrants k = part (low nibbles) and part + 2 (high nibbles),
// part = (j / 2) % 2.  It fetches the 16 qh bytes of those positions (lanes j and j ^ 2 the same ones), the
// half's 8 scale bytes and d.  A row is then fetched through the fewest cache lines it spans (14) instead of
// the ~80 that the per-field loads of the 210-byte superblocks touch.
__host__ __device__ constexpr size_t q6r_row_bytes(int bpr) { return ((size_t)bpr * 210 + 15) / 16 * 16; }

struct Q6rLane {
    u32x4_t ql, qh;
    u32x2 sc;
    uint32_t d;
};

__device__ __forceinline__ Q6rLane q6r_load(const uint8_t *row, int bpr, int blk, int lane)
{
    const int j = lane & 7, ip = j >> 2;
    Q6rLane r;
    // (streamed once per launch and never reused: loads marked non-temporal, 88.6 -> 85.8 us on 262144 x 2048; the same
    // mark on the Q4_K GEMVs' weights costs them 5 %)
    r.ql = __builtin_nontemporal_load((const KSH_GLOBAL u32x4_t *)(row + (size_t)blk * 128 + 16 * j));
    r.qh = __builtin_nontemporal_load((const KSH_GLOBAL u32x4_t *)(row + (size_t)bpr * 128 + (size_t)blk * 64 + 32 * ip + 16 * (j & 1)));
    r.sc = *(const KSH_GLOBAL u32x2 *)(row + (size_t)bpr * 192 + (size_t)blk * 16 + 8 * ip);
    r.d = *(const KSH_GLOBAL uint16_t *)(row + (size_t)bpr * 208 + (size_t)blk * 2);
    return r;
}

// the lane's share of the staged vector: digit planes of its 16 positions in its two quadrants, minus 32 times
// the sum of X over each 16, and the scale of its 128-element half
struct XQ6r {
    u32x4_t H[2], M[2], L[2];
    int nsx5[2];
    float s;
    __device__ __forceinline__ void load(const uint8_t *lds, int blk, int lane, bool valid)
    {
        const int j = lane & 7, ip = j >> 2, part = (j >> 1) & 1, l0 = 16 * (j & 1);
        const uint8_t *half = lds + (blk * 2 + ip) * kQ6HalfBytes;
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const int k = part + 2 * q, o = 32 * k + l0;
            H[q] = *reinterpret_cast<const u32x4_t *>(half + o);
            M[q] = *reinterpret_cast<const u32x4_t *>(half + 128 + o);
            L[q] = *reinterpret_cast<const u32x4_t *>(half + 256 + o);
            const int *nsx = reinterpret_cast<const int *>(half + 384) + 4 * k + 2 * (j & 1);   // runs of 8
            nsx5[q] = (nsx[0] + nsx[1]) * 32;
        }
        s = valid ? *reinterpret_cast<const float *>(half + 448) : 0.f;
    }
};

__device__ __forceinline__ float q6r_lane_dot(const Q6rLane &B, int lane, const XQ6r &X)
{
    const int j = lane & 7, part = (j >> 1) & 1;
    int hs[2], ms[2], ls[2];
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const uint32_t t = B.qh[w] >> (2 * part);
        const uint32_t a[2] = {(B.ql[w] & 0x0F0F0F0Fu) | ((t << 4) & 0x30303030u), ((B.ql[w] >> 4) & 0x0F0F0F0Fu) | (t & 0x30303030u)};
#pragma unroll
        for (int q = 0; q < 2; q++) {
            if (w == 0) {
                hs[q] = dot4_start((int)a[q], (int)X.H[q][0]);
                ms[q] = dot4_start((int)a[q], (int)X.M[q][0]);
                ls[q] = __builtin_amdgcn_sdot4((int)a[q], (int)X.L[q][0], X.nsx5[q], false);   // starts at -32*sum(X)
            } else {
                hs[q] = __builtin_amdgcn_sdot4((int)a[q], (int)X.H[q][w], hs[q], false);
                ms[q] = __builtin_amdgcn_sdot4((int)a[q], (int)X.M[q][w], ms[q], false);
                ls[q] = __builtin_amdgcn_sdot4((int)a[q], (int)X.L[q][w], ls[q], false);
            }
        }
    }
    // scales of the half: index 2k + l0/16 for k = part and part + 2: byte 2*part + (j&1) of each dword
    const int sh = 8 * (2 * part + (j & 1));
    const float c0 = (float)(int8_t)(B.sc.x >> sh), c1 = (float)(int8_t)(B.sc.y >> sh);
    const int x0 = (((hs[0] << 7) + ms[0]) << 7) + ls[0], x1 = (((hs[1] << 7) + ms[1]) << 7) + ls[1];
    return (half_bits_to_f32(B.d) * X.s) * fmaf(c1, (float)x1, c0 * (float)x0);
}

template <int R, int NW, int STEPS>
__global__ __launch_bounds__(NW * 64) void q6r_gemv_kernel(Q6kParams p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // timeline build (tag 0): slots 0 entry, 1 loads issued, 2 vector staged, 3 barrier passed, 4 first row done, 5 last row stored, 6 acknowledged
    // (every fourth workgroup leaves records: 2048 workgroups of 8 waves are more than the buffer holds)
    const int sw = (blockIdx.x & 3) ? kStampWaves : (int)(blockIdx.x >> 2) * NW + wave;
    (void)sw;
    KSH_STAMP_BEGIN
    const int bl = lane >> 3;
    const int cols = p.bpr * 256;
    const size_t row_bytes = q6r_row_bytes(p.bpr);
    const int w0 = (blockIdx.x * NW + wave) * p.rows_per_wave;
    const int w1 = min(w0 + p.rows_per_wave, p.rows);

    Q6rLane cur[STEPS][R], nxt[STEPS][R];
    auto load_rows = [&](Q6rLane (&dst)[STEPS][R], int row0) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint8_t *rp = p.W + (size_t)min(row0 + r, p.rows - 1) * row_bytes;
#pragma unroll
            for (int s = 0; s < STEPS; s++) dst[s][r] = q6r_load(rp, p.bpr, min(s * 8 + bl, p.bpr - 1), lane);   // past the row's end: the last superblock again, against a zero scale
        }
    };
    constexpr int KMAX = (STEPS * 512 + NW * 64 - 1) / (NW * 64);   // float4 of the vector per thread: cols == STEPS * 2048
    StageRegs sr;
    stage_fetch<NW * 64, false, KMAX>(p.pro, cols, sr);
    load_rows(cur, min(w0, p.rows - 1));
    KSH_STAMP(1);
    stage_finish<kXQ6, NW * 64, false, KMAX>(p.pro, xs, cols, sr);
    KSH_STAMP(2);
    __syncthreads();
    KSH_STAMP(3);
    if (w0 >= w1) return;

    XQ6r X[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; s++) X[s].load(xs, min(s * 8 + bl, p.bpr - 1), lane, s * 8 + bl < p.bpr);

    for (int row0 = w0; row0 < w1; row0 += R) {
        load_rows(nxt, min(row0 + R, p.rows - 1));
#pragma unroll
        for (int r = 0; r < R; r++) {
            float acc = 0.f;
#pragma unroll
            for (int s = 0; s < STEPS; s++) acc += q6r_lane_dot(cur[s][r], lane, X[s]);
            acc = wave_sum(acc);
            if (lane == 0 && row0 + r < w1) p.y[row0 + r] = acc;
        }
        if (row0 == w0) KSH_STAMP(4);
#pragma unroll
        for (int s = 0; s < STEPS; s++)
#pragma unroll
            for (int r = 0; r < R; r++) cur[s][r] = nxt[s][r];
    }
    KSH_STAMP(5);
    KSH_STAMP_FLUSH(0, sw, 6);
}

struct Q6kGeom {
    int R, NW, rpw;
};

Q6kGeom pick_geom6(const ksh_sched &s, int rows)
{
    Q6kGeom G;
    G.NW = s.nsg ? (int)s.nsg : 4;
    G.R = s.nr0 ? (int)s.nr0 : 2;
    // rows a wave walks: long enough to amortise the x staging, short enough
    // to leave >= 8 workgroups per CU
    int rpw = s.unroll ? (int)s.unroll * G.R : 16;
    if (!s.unroll) while (rpw > G.R && rows / (rpw * G.NW) < 2048) rpw >>= 1;   // (an explicit count is taken as given)
    if (rpw < G.R) rpw = G.R;
    G.rpw = rpw;
    return G;
}

template <int R, int NW>
int launch_steps(int steps, bool by_rows, const Q6kParams &p, unsigned grid, size_t lds, hipStream_t st)
{
    if (by_rows) {
        switch (steps) {
        case 1: hipLaunchKernelGGL((q6r_gemv_kernel<R, NW, 1>), dim3(grid), dim3(NW * 64), lds, st, p); break;
        case 2: hipLaunchKernelGGL((q6r_gemv_kernel<(R > 2 ? 2 : R), NW, 2>), dim3(grid), dim3(NW * 64), lds, st, p); break;
        default: return set_error("matvec_q6k: cols=%d is not built for row-grouped weights (2048 and 4096 are)", p.bpr * 256);
        }
        const hipError_t e = hipGetLastError();
        return e == hipSuccess ? 0 : hip_fail(e, "q6k_gemv launch");
    }
    switch (steps) {
    case 1: hipLaunchKernelGGL((q6k_gemv_kernel<R, NW, 1>), dim3(grid), dim3(NW * 64), lds, st, p); break;
    case 2: hipLaunchKernelGGL((q6k_gemv_kernel<(R > 2 ? 2 : R), NW, 2>), dim3(grid), dim3(NW * 64), lds, st, p); break;
    case 3: hipLaunchKernelGGL((q6k_gemv_kernel<1, NW, 3>), dim3(grid), dim3(NW * 64), lds, st, p); break;
    case 4: hipLaunchKernelGGL((q6k_gemv_kernel<1, NW, 4>), dim3(grid), dim3(NW * 64), lds, st, p); break;
    default: return set_error("matvec_q6k: cols=%d is not built (up to 8192 are)", p.bpr * 256);
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "q6k_gemv launch");
}

int launch_matvec_q6k(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    Q6kParams p{};
    p.W = (const uint8_t *)a.in[0];
    p.y = (float *)a.out[0];
    p.pro.x = (const float *)a.in[1];
    p.pro.eps = k.desc.params[0];
    p.pro.kind = k.desc.kind == KSH_MATVEC ? kPlain : (k.desc.dims[2] ? kAddThenRms : kRms);
    if (p.pro.kind != kPlain) p.pro.w_norm = (const float *)a.in[2];
    if (p.pro.kind == kAddThenRms) {
        p.pro.nwg = __builtin_bit_cast(int, k.desc.params[1] != 0.f ? k.desc.params[1] : 1.0f);   // the stream scale
        p.pro.w_post = (const float *)a.in[3];
        p.pro.res = (const float *)a.in[4];
        p.pro.x_out = (float *)a.out[1];
    }
    p.rows = (int)k.desc.dims[0];
    p.bpr = (int)(k.desc.dims[1] / 256);
    const int R = k.variant & 0xFF, NW = (k.variant >> 8) & 0xFF;
    p.rows_per_wave = k.variant >> 16;
    const unsigned grid = k.info.grid[0];
    const size_t lds = k.info.lds_bytes;
    const int steps = (p.bpr + 7) / 8;
#define KSH_CASE(r, w) \
    if (R == r && NW == w) return launch_steps<r, w>(steps, k.desc.dtypes[0] == KSH_Q6K_ROWS, p, grid, lds, st);
    KSH_CASE(1, 4) KSH_CASE(2, 4) KSH_CASE(4, 4)
    KSH_CASE(1, 2) KSH_CASE(2, 2) KSH_CASE(4, 2)
    KSH_CASE(1, 8) KSH_CASE(2, 8) KSH_CASE(4, 8)
#undef KSH_CASE
    return set_error("matvec_q6k: no instance for nr0=%d nsg=%d", R, NW);
}

}  // namespace

int bind_matvec_q6k(ksh_kernel &k)
{
    const int64_t rows = k.desc.dims[0], cols = k.desc.dims[1];
    const bool pro = k.desc.kind == KSH_RMSNORM_MATVEC, has_res = pro && k.desc.dims[2] != 0;
    if (k.desc.kind != KSH_MATVEC && !pro) return set_error("matvec_q6k: kind %d is not built for Q6_K weights", k.desc.kind);
    if (rows <= 0 || rows > (1 << 30)) return set_error("matvec: rows=%lld", (long long)rows);
    if (cols <= 0 || cols % 256 || cols > 8192)
        return set_error("matvec_q6k: cols=%lld is not a positive multiple of 256 up to 8192", (long long)cols);
    const bool by_rows = k.desc.dtypes[0] == KSH_Q6K_ROWS;
    if (by_rows && cols != 1536 && cols != 2048 && cols != 4096)
        return set_error("matvec_q6k: row-grouped weights are built for 1536, 2048 and 4096 columns (got %lld)", (long long)cols);
    Q6kGeom G = pick_geom6(k.desc.sched, (int)rows);
    if (k.desc.dtypes[0] == KSH_Q6K_ROWS && sched_is_zero(k.desc.sched)) {   // measured best on 262144 x 2048
        G.NW = 8;
        G.R = 1;
        G.rpw = 16;
        while (G.rpw > 1 && rows / (G.rpw * G.NW) < 2048) G.rpw >>= 1;
    }
    // keeps the double buffer and the digit planes in registers
    if (cols > 4096) { G.rpw = G.rpw / G.R; G.R = 1; }
    else if (cols > 2048 && G.R > 2) { G.rpw = G.rpw / G.R * 2; G.R = 2; }
    if (!((G.R == 1 || G.R == 2 || G.R == 4) && (G.NW == 2 || G.NW == 4 || G.NW == 8)) || G.rpw % G.R || G.rpw > 32767)
        return set_error("matvec_q6k: unsupported schedule nr0=%d nsg=%d unroll=%u", G.R, G.NW, k.desc.sched.unroll);
    const int bpr = (int)(cols / 256);
    if (pro && cols > (int64_t)4 * G.NW * 64 * kStageP)
        return set_error("rmsnorm_matvec requires LOCAL staging of the vector (cols=%lld too large)", (long long)cols);
    k.info.n_inputs = pro ? (has_res ? 5 : 3) : 2;
    k.info.n_outputs = has_res ? 2 : 1;
    k.in_bytes[0] = by_rows ? (size_t)rows * q6r_row_bytes(bpr) : (size_t)rows * bpr * kQ6kBytes;
    k.in_align[0] = by_rows ? 16 : 2;
    for (int i = 1; i < k.info.n_inputs; i++) { k.in_bytes[i] = (size_t)cols * 4; k.in_align[i] = 16; }
    k.out_bytes[0] = (size_t)rows * 4;
    k.out_align[0] = 4;
    if (has_res) { k.out_bytes[1] = (size_t)cols * 4; k.out_align[1] = 16; }
    const int rows_per_wg = G.rpw * G.NW;
    set_launch(k, (uint32_t)((rows + rows_per_wg - 1) / rows_per_wg), 1, 1, (uint32_t)G.NW * 64,
               (uint32_t)xs_bytes<kXQ6>((int)cols));
    k.info.sched = k.desc.sched;
    k.info.sched.tg = (uint64_t)G.NW * 64;
    k.info.sched.nsg = (uint32_t)G.NW;
    k.info.sched.nr0 = (uint32_t)G.R;
    k.info.sched.unroll = (uint32_t)(G.rpw / G.R);
    k.info.sched.vec = 3;
    k.info.sched.k_split = 1;
    set_name(k, "%smatvec_q6k%s_r%d_w%d_u%d", pro ? (has_res ? "addrms_" : "rms_") : "", by_rows ? "rows" : "", G.R, G.NW, G.rpw / G.R);
    k.variant = G.R | (G.NW << 8) | (G.rpw << 16);
    k.launch = launch_matvec_q6k;
    return 0;
}

int matvec_q6k_candidates(const ksh_kernel_desc &d, ksh_sched *out, int cap)
{
    (void)d;
    int n = 0;
    for (uint32_t nsg : {2u, 4u, 8u})
        for (uint32_t nr0 : {1u, 2u, 4u})
            for (uint32_t unroll : {2u, 8u}) {
                if (n >= cap) return n;
                ksh_sched s{};
                s.tg = 64ull * nsg; s.vec = 3; s.unroll = unroll; s.nsg = nsg; s.nr0 = nr0; s.k_split = 1;
                out[n++] = s;
            }
    return n;
}

}  // namespace ksh
