// Batched prefill GEMM over Q4_K weights on the gfx950 matrix cores:
//   Y[t, r] = sum_c deq(W[r, c]) * X[t, c]      X bf16 [batch, cols], Y f32 [batch, rows]
//
// Takes the place of KirStmt::Q4kMulMm / ksearch_q4k_mul_mm
// (crates/ksearch_codegen/src/lower.rs:404-424, 788-818,
// crates/ksearch_codegen/src/render.rs:1073-1191), which dequantizes a 64x32
// weight tile to half (rounding every weight) and runs 8x8 simdgroup MMAs.
//
// Here no weight is rounded.  With w = d*sc_j*n - dmin*m_j (n the 4-bit code,
// j the 32-wide sub-block):
//
//   sum_c w*x = sum_sb [ d * sum_k (sc_j*n_k) x_k  -  sum_j dmin*m_j * Sx_j ],   Sx_j = sum_{k in j} x_k
//
// sc_j*n_k is an integer <= 945, exact in f16, and is produced two at a time
// by one 24-bit multiply-add that also ORs it into the mantissa of half 1024.0:
// (q & 0x000F000F) * sc + 0x64006400 = (1024 + sc*n_a, 1024 + sc*n_b).  The
// matrix cores accumulate C' = sum_k (1024 + sc*n) x_k per superblock in f32;
// the per-row f16 scale d is applied once per superblock (F += d * C'), and
// the bias and the mins go through a second, short matrix product against the
// per-sub-block sums of x:  F -= sum_j (dmin*m_j + 1024*d) * Sx_j, with both
// factors split into f16 hi + lo parts so that this term keeps f32 accuracy.
// X is bf16, which converts to f16 without loss for |x| >= 2^-17 (smaller
// values lose at most 2^-25 absolutely).
//
// Tiling: a workgroup owns 128 tokens x 128 weight rows; each of its four
// multiplying waves owns 32 tokens x 128 rows as 1 x 4 v_mfma_f32_32x32x16_f16
// tiles (four more waves load and convert).  M = tokens, N = weight
// rows, so a lane's accumulator column is one weight row (one d per lane) and
// stores are contiguous along Y's row index.  K advances 64 columns (one
// 64-element group: 32 quant bytes per row) per step through a double-buffered
// LDS stage, with the next step's global loads in flight under the MFMAs.
#include <type_traits>

#include "ksh_device.hpp"
#include "ksh_internal.hpp"
#include "q4k_lane.hpp"
#include "round_operand.hpp"

namespace ksh {
namespace {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int BM = 128, BN = 128, KS = 64;
constexpr int PITCH = KS + 8;      // halves per LDS row of the main tiles (144 B: conflict-free 16 B reads)
constexpr int PITCH2 = 32 + 8;     // halves per LDS row of the min-term tiles

// X bf16 -> f16 (permuted) in the order the matrix instruction wants its A operand, plus the min-term
// operand per (token, superblock): 32 halves = Sx_hi[8] | Sx_hi[8] | Sx_lo[8] | 0[8].
// Xf[token / 32][k / 16][lane][8] with lane = token % 32 + 32 * ((k / 8) % 2): one 32 x 16 fragment is 1 KB,
// lane after lane, so that a multiplying wave fetches it with a single 128-bit load per lane and the
// activations never pass through LDS.
// A wave takes 32 tokens x one 32-column sub-block: lane (token % 32, h) converts the 8-element runs h and 2 + h
// of the sub-block and is lane token % 32 + 32 h of the sub-block's two fragments, so both leave as whole
// kilobytes, lane after lane (with a thread per run in row order, the eight 16-byte pieces of a 128-byte line of
// Xf came from eight workgroups: 5.7 us for 2 MB).  The four waves of a workgroup take neighbouring sub-blocks, so
// that together they read whole lines of X.  The sub-block's sum is (run 0 + run 1) + (run 2 + run 3), the two
// halves of the wave trading their runs' sums.
__global__ __launch_bounds__(256) void mm_prep_x_kernel(const uint16_t *__restrict__ X, _Float16 *__restrict__ Xf,
                                                        _Float16 *__restrict__ SxA, int batch, int cols)
{
    const int lane = threadIdx.x & 63, wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int nsub = cols / 32, tb = wave / nsub, s = wave - tb * nsub;
    const int t = tb * 32 + (lane & 31), h = lane >> 5;
    if (tb * 32 >= batch) return;
    const bool live = t < batch;
    const u32x4_t *row = reinterpret_cast<const u32x4_t *>(X + (size_t)min(t, batch - 1) * cols);   // (rows past the batch: read a real row, store nothing)
    float c[2];
    h8 o[2];
#pragma unroll
    for (int r = 0; r < 2; r++) {
        const u32x4_t in = row[4 * s + 2 * r + h];
        const uint32_t w[4] = {in.x, in.y, in.z, in.w};
        float f[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f[2 * i] = as_f32(w[i] << 16);
            f[2 * i + 1] = as_f32(w[i] & 0xFFFF0000u);
        }
        c[r] = ((f[0] + f[1]) + (f[2] + f[3])) + ((f[4] + f[5]) + (f[6] + f[7]));
#pragma unroll
        for (int i = 0; i < 8; i++) o[r][kperm(i)] = (_Float16)f[i];
    }
    // the other half's runs: (run 0 + run 1) and (run 2 + run 3), the same in both halves
    const auto x0 = __builtin_amdgcn_permlane32_swap(as_u32(c[0]), as_u32(c[0]), false, false);
    const auto x1 = __builtin_amdgcn_permlane32_swap(as_u32(c[1]), as_u32(c[1]), false, false);
    float sum = (as_f32(x0[0]) + as_f32(x0[1])) + (as_f32(x1[0]) + as_f32(x1[1]));
    if (!live) return;
    h8 *frag = reinterpret_cast<h8 *>(Xf) + ((size_t)tb * (cols / 16) + 2 * s) * 64 + lane;
    frag[0] = o[0];
    frag[64] = o[1];
    if (h == 0) {
        sum = pinned(sum);
        const _Float16 hi = (_Float16)sum;
        const _Float16 lo = (_Float16)(sum - (float)hi);
        _Float16 *a2 = SxA + ((size_t)t * (cols / 256) + s / 8) * 32;
        const int jj = s % 8;
        a2[jj] = hi;
        a2[8 + jj] = hi;
        a2[16 + jj] = lo;
        a2[24 + jj] = (_Float16)0.f;
    }
}

// The same for f32 activations (the decode loops' prompt chunks): x = hi + 2^-11 lo with hi = f16(x) and
// lo = f16(2^11 (x - hi)), 22 bits of x, each part with its own fragments and its own sums.  The product then runs
// twice, the second pass adding 2^-11 times its result to the first.
__global__ __launch_bounds__(256) void mm_prep_x_f32_kernel(const float *__restrict__ X, _Float16 *__restrict__ Xf_hi,
                                                            _Float16 *__restrict__ Xf_lo, _Float16 *__restrict__ SxA_hi,
                                                            _Float16 *__restrict__ SxA_lo, int batch, int cols)
{
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= batch * (cols / 8)) return;   // (whole quads: cols is a multiple of 32)
    const f32x4_t in0 = reinterpret_cast<const f32x4_t *>(X)[2 * (size_t)idx], in1 = reinterpret_cast<const f32x4_t *>(X)[2 * (size_t)idx + 1];
    const float f[8] = {in0.x, in0.y, in0.z, in0.w, in1.x, in1.y, in1.z, in1.w};
    h8 oh, ol;
    float fh[8], fl[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const _Float16 hi = (_Float16)f[i];
        const _Float16 lo = (_Float16)((f[i] - (float)hi) * 2048.0f);   // kept 2^11 up, in the normal range wherever hi is
        oh[kperm(i)] = hi;
        ol[kperm(i)] = lo;
        fh[i] = (float)hi;
        fl[i] = (float)lo;
    }
    float sh = ((fh[0] + fh[1]) + (fh[2] + fh[3])) + ((fh[4] + fh[5]) + (fh[6] + fh[7]));
    float sl = ((fl[0] + fl[1]) + (fl[2] + fl[3])) + ((fl[4] + fl[5]) + (fl[6] + fl[7]));
    sh += dpp_f32<0xB1>(sh);
    sh += dpp_f32<0x4E>(sh);
    sl += dpp_f32<0xB1>(sl);
    sl += dpp_f32<0x4E>(sl);
    const int k8 = cols / 8, t = idx / k8, j = idx - t * k8;
    const size_t frag = ((size_t)(t >> 5) * (cols / 16) + (j >> 1)) * 64 + (t & 31) + 32 * (j & 1);
    reinterpret_cast<h8 *>(Xf_hi)[frag] = oh;
    reinterpret_cast<h8 *>(Xf_lo)[frag] = ol;
    if ((threadIdx.x & 3) == 0) {
        const int s = j / 4, jj = s % 8;
        const size_t o = ((size_t)t * (cols / 256) + s / 8) * 32;
        const float sums[2] = {sh, sl};
        _Float16 *dst[2] = {SxA_hi + o, SxA_lo + o};
#pragma unroll
        for (int part = 0; part < 2; part++) {
            const float sum = pinned(sums[part]);
            const _Float16 hi = (_Float16)sum;
            const _Float16 lo = (_Float16)(sum - (float)hi);
            dst[part][jj] = hi;
            dst[part][8 + jj] = hi;
            dst[part][16 + jj] = lo;
            dst[part][24 + jj] = (_Float16)0.f;
        }
    }
}

// The same preparation with the producer of the rows folded in (f32 activations), one workgroup per row, cols / 8
// threads (1024 at most) with 8 consecutive elements each per trip:
//   MODE 0  x = X
//   MODE 1  x = rmsnorm(X, w)                                  (rmsnorm_rows, crates/ksearch_kernels/src/lib.rs:1478-1500)
//   MODE 2  x_new = res + rmsnorm(X, w_post), stored; x = rmsnorm(x_new, w_norm)   (rmsnorm_add_then_rmsnorm_rows)
//   MODE 3  x = gelu(X) * up                                   (gelu_mul on rows, gemma_prim.rs:1516-1538)
// in the operation order of the kernels that do these alone (every product and sum rounded by itself).
//
// inv_s = nullptr: the two parts as above (lo kept 2^11 up, each part with its own sums), for the small-batch form.
// inv_s != nullptr (the tile): the row is first scaled by the power of two s that puts its largest magnitude into
// [2^9, 2^10) -- exact, and any f32 row fits f16 then, sums of 32 elements included -- and x s = hi + lo with BOTH
// parts at that scale, so that one accumulator takes hi * w and lo * w of the same converted weight.  lo is a
// subnormal f16 for elements below 2^-13 of the row's largest; what that costs is below 2^-35 of the largest.  The
// sums of a sub-block are those of hi + lo, split in two halves as for bf16 rows; 1 / s goes to inv_s[row] for the
// tile's last step.
template <int MODE>
__global__ __launch_bounds__(1024) void mm_prep_rows_kernel(const float *__restrict__ X, const float *__restrict__ P0, const float *P1,
                                                             const float *__restrict__ P2, float *x_out, _Float16 *__restrict__ Xf_hi,
                                                             _Float16 *__restrict__ Xf_lo, _Float16 *__restrict__ SxA_hi,
                                                             _Float16 *__restrict__ SxA_lo, int cols, float eps, int x_slices,
                                                             float *__restrict__ inv_s)
{
    // x_slices != 0: X is the unfolded partial sums of the GEMM that produced it, [slice][row][stride] with stride =
    // cols (MODE 3: 2 * cols, gate | up side by side, and `up` is read from there); the slices are added here in the
    // fold's order
    __shared__ float red[3][16];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    auto ld8 = [](const float *p, float (&v)[8]) __attribute__((always_inline)) {
        const f32x4_t a = reinterpret_cast<const f32x4_t *>(p)[0], b = reinterpret_cast<const f32x4_t *>(p)[1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    };
    auto row_sum = [&](float v, int which) __attribute__((always_inline)) {
        v = wave_sum(v);
        if (lane == 0) red[which][wave] = v;
        __syncthreads();
        float s = 0.f;
        for (int i = 0; i < nw; i++) s += red[which][i];
        return s;
    };
    const size_t x_stride = MODE == 3 ? 2 * (size_t)cols : (size_t)cols, x_plane = (size_t)gridDim.x * x_stride;
    auto ldx = [&](int j, size_t col0, float (&v)[8]) __attribute__((always_inline)) {
        const float *src = X + (size_t)t * x_stride + col0 + 8 * (size_t)j;
        ld8(src, v);
        for (int k = 1; k < x_slices; k++) {
            float a[8];
            ld8(src + (size_t)k * x_plane, a);
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] += a[i];
        }
    };
    // the row's elements 8j .. 8j+7 (the norms run with cols / 8 threads, one trip; plain rows and gelu * up of longer
    // rows take several)
    auto produce = [&](int j, float (&f)[8]) __attribute__((always_inline)) {
        const size_t e0 = (size_t)t * cols + 8 * (size_t)j;
        if (x_slices) ldx(j, 0, f);
        else ld8(X + e0, f);
        if (MODE == 1 || MODE == 2) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) ss += f[i] * f[i];
            const float inv = 1.0f / sqrtf(row_sum(ss, 0) / (float)cols + eps);
            float w[8];
            ld8(P0 + 8 * j, w);
#pragma unroll
            for (int i = 0; i < 8; i++) f[i] = __fmul_rn(__fmul_rn(f[i], inv), w[i]);
            if (MODE == 2) {
                float r[8], wn[8];
                ld8(P1 + e0, r);
                float ss2 = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    f[i] = __fadd_rn(r[i], f[i]);
                    ss2 += f[i] * f[i];
                }
                reinterpret_cast<f32x4_t *>(x_out + e0)[0] = f32x4_t{f[0], f[1], f[2], f[3]};
                reinterpret_cast<f32x4_t *>(x_out + e0)[1] = f32x4_t{f[4], f[5], f[6], f[7]};
                const float inv2 = 1.0f / sqrtf(row_sum(ss2, 1) / (float)cols + eps);
                ld8(P2 + 8 * j, wn);
#pragma unroll
                for (int i = 0; i < 8; i++) f[i] = __fmul_rn(__fmul_rn(f[i], inv2), wn[i]);
            }
        }
        if (MODE == 3) {
            float u[8];
            if (x_slices) ldx(j, (size_t)cols, u);
            else ld8(P0 + e0, u);
#pragma unroll
            for (int i = 0; i < 8; i++) f[i] = gelu_mul_f32(f[i], u[i]);
        }
    };
    const int octets = cols / 8;
    const bool one_trip = octets <= (int)blockDim.x;
    float kept[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float s = 1.0f;
    if (inv_s) {
        // the row's largest magnitude (rows of one trip keep their elements; longer ones are produced again below)
        float m = 0.f;
        for (int j = threadIdx.x; j < octets; j += blockDim.x) {
            produce(j, kept);
#pragma unroll
            for (int i = 0; i < 8; i++) m = fmaxf(m, fabsf(kept[i]));
        }
        m = wave_max(m);
        if (lane == 0) red[2][wave] = m;
        __syncthreads();
        for (int i = 0; i < nw; i++) m = fmaxf(m, red[2][i]);
        // s = 2^(9 - floor(log2 m)); rows of zeros (and anything below 2^-112) take 2^121, infinities and NaNs 2^-118
        const uint32_t e = (uint32_t)max((int)((as_u32(m) >> 23) & 0xFFu), 15);
        s = as_f32((263u - e) << 23);
        if (threadIdx.x == 0) inv_s[t] = as_f32((e - 9u) << 23);
    }
    for (int j = threadIdx.x; j < octets; j += blockDim.x) {
        float f[8];
        if (inv_s && one_trip) {
#pragma unroll
            for (int i = 0; i < 8; i++) f[i] = kept[i];
        } else {
            produce(j, f);
        }
        h8 oh, ol;
        float fh[8], fl[8];
        const float lo_up = inv_s ? 1.0f : 2048.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float x = pinned(f[i]) * s;
            const _Float16 hi = (_Float16)x;
            const _Float16 lo = (_Float16)((x - (float)hi) * lo_up);
            oh[kperm(i)] = hi;
            ol[kperm(i)] = lo;
            fh[i] = (float)hi;
            fl[i] = (float)lo;
        }
        float sh = ((fh[0] + fh[1]) + (fh[2] + fh[3])) + ((fh[4] + fh[5]) + (fh[6] + fh[7]));
        float sl = ((fl[0] + fl[1]) + (fl[2] + fl[3])) + ((fl[4] + fl[5]) + (fl[6] + fl[7]));
        sh += dpp_f32<0xB1>(sh);
        sh += dpp_f32<0x4E>(sh);
        sl += dpp_f32<0xB1>(sl);
        sl += dpp_f32<0x4E>(sl);
        const size_t frag = ((size_t)(t >> 5) * (cols / 16) + (j >> 1)) * 64 + (t & 31) + 32 * (j & 1);
        reinterpret_cast<h8 *>(Xf_hi)[frag] = oh;
        reinterpret_cast<h8 *>(Xf_lo)[frag] = ol;
        if ((threadIdx.x & 3) == 0) {
            const int sbk = j / 4, jj = sbk % 8;
            const size_t o = ((size_t)t * (cols / 256) + sbk / 8) * 32;
            const float sums[2] = {inv_s ? sh + sl : sh, sl};
            _Float16 *dst[2] = {SxA_hi + o, SxA_lo + o};
#pragma unroll
            for (int part = 0; part < 2; part++) {
                if (part && inv_s) break;       // (one set of sums; the other operand's place holds inv_s)
                const float sum = pinned(sums[part]);
                const _Float16 hi = (_Float16)sum;
                const _Float16 lo = (_Float16)(sum - (float)hi);
                dst[part][jj] = hi;
                dst[part][8 + jj] = hi;
                dst[part][16 + jj] = lo;
                dst[part][24 + jj] = (_Float16)0.f;
            }
        }
    }
}

struct MmParams {
    const uint8_t *W;
    const _Float16 *Xf, *SxA;   // fragment-ordered f16 activations (mm_prep_x_kernel), sums of x
    float *Y;
    int rows, cols, batch;
    // Small grids (few tokens x few weight rows): blockIdx.z = K slice.  A workgroup then takes the superblocks of
    // its slice only and every z stores its own batch x rows partial sums behind Y_parts for the fold (ksplit = 0:
    // full K, results in Y).
    int ksplit;
    float *Y_parts;
    // Up to three matrices that share the activations (q | k | v of a prompt chunk) in one launch of the 128 x 128
    // tile: blockIdx.y counts the row tiles of W, then of W1, then of W2, each with its own result.
    const uint8_t *W1, *W2;
    float *Y1, *Y2;
    int rows1, rows2;
    // f32 activations (the kernel's LO form): the lo parts' fragments and 1 / s per token row (see mm_prep_rows_kernel)
    const _Float16 *Xf_lo;
    const float *inv_s;
};

__device__ __forceinline__ uint32_t pair_f16(uint32_t masked, uint32_t sc)
{
    return __umul24(masked, sc) + 0x64006400u;     // half 1024.0 twice
}

// what a loader thread (two per tile row) holds per superblock: of each of the four 64-column groups the 16 quant
// bytes it converts (all requested when the superblock opens, so that a weight row's cache lines are fetched once,
// not once per step), the header and half of the token's sums of x
// (native vector types: with HIP's uint4 class the copies become memcpys that keep these sets in scratch memory)
struct SbRegs {
    u32x4_t q[4];      // of each of the four 64-column groups, the 16 quant bytes this thread converts
    u32x4_t hdr, sx0, sx1;
};

constexpr int kThreadsMM = 512;
constexpr int kLdsMain = BN * PITCH;             // halves per main stage (the dequantized weight tile)
constexpr int kLdsMin = (BM + BN) * PITCH2;      // halves per min-term stage
constexpr size_t kLdsBytes = 2 * (size_t)(kLdsMain + kLdsMin) * 2 + 2 * BN * 4;
constexpr size_t kLdsBytes64 = 2 * (size_t)(kLdsMain + (64 + BN) * PITCH2) * 2 + 2 * BN * 4;   // the 64-token tile

// Eight waves in two roles, one of each per SIMD.  Waves 0..3 only multiply:
// each owns 32 tokens x 128 columns of the 128-token tile (1 x 4 MFMA tiles; of
// the 64-token tile 32 x 64) and works on LDS stage s&1.  Waves 4..7 only
// load and convert: during the same step they request the activations of step
// s+4 (and, when a superblock opens, the next superblock's weights) and write
// step s+1 into stage (s+1)&1.  One barrier per K step joins them, so the
// conversions and the LDS writes of one role run in the shadow of the other
// role's matrix instructions.  The min-term operands of a superblock are
// written together with its first step into their own double buffer and
// consumed after its fourth.
//
// Q6 = true: the same tile and roles over Q6_K weights (K3b of the reference's plan: Q6_K tensors in prefill).
// w = d * sc_j * q with q = code - 32 in [-32, 31] and sc_j an int8 per 16 columns; the loaders build the f16
// pair (1024 + code) by an OR into the mantissa, subtract 1056 and multiply by sc_j, both as packed f16.
// sc_j * q is exact in f16 up to 2048; beyond that (needs |sc_j| > 64) it rounds to the nearest even integer, a
// relative 2^-11 at most and on those weights only (the reference's tile rounds every weight to half, the same
// bound).  There is no min term, so the short second product is skipped; d is applied per superblock as for Q4_K.
// TM = tokens per workgroup.  128: each multiplying wave owns 32 x 128.  64: each owns 32 x 64 with half the
// accumulators, the kernel fits 128 registers and 70 KB of LDS, and two workgroups share a compute unit, so that one's
// barriers and first loads fall into the other's products (the weights are converted once per 64 tokens then).
// LO = true: f32 activations as two f16 parts at the row's own scale.  Every converted weight meets the hi and the lo
// fragment of a token tile in the same accumulator (twice the matrix instructions per conversion, and the
// conversions are what a step waits for), and the finished sums are multiplied by 1 / s of their token.
template <bool Q6, int TM, bool LO>
__global__ __launch_bounds__(kThreadsMM, TM == 64 ? 2 : 1) void q_mul_mm_kernel(MmParams p)
{
    constexpr int MT = TM / 64, kLdsMinT = (TM + BN) * PITCH2;
    extern __shared__ __attribute__((aligned(16))) _Float16 lds[];
    auto main_stage = [&](int i) { return lds + (i & 1) * kLdsMain; };
    auto min_stage = [&](int i) { return lds + 2 * kLdsMain + (i & 1) * kLdsMinT; };
    auto dsc_stage = [&](int i) { return reinterpret_cast<float *>(lds + 2 * kLdsMain + 2 * kLdsMinT) + (i & 1) * BN; };

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // which matrix this row tile belongs to (the copy of the arguments is this workgroup's own)
    int by = blockIdx.y, ycol = 0;
    const int rows_all = p.rows + p.rows1 + p.rows2;
    if (p.rows1) {
        const int ty0 = (p.rows + BN - 1) / BN, ty1 = (p.rows1 + BN - 1) / BN;
        if (by >= ty0 + ty1) { by -= ty0 + ty1; ycol = p.rows + p.rows1; p.W = p.W2; p.Y = p.Y2; p.rows = p.rows2; }
        else if (by >= ty0) { by -= ty0; ycol = p.rows; p.W = p.W1; p.Y = p.Y1; p.rows = p.rows1; }
    }
    const int t0 = blockIdx.x * TM, r0 = by * BN;
    const int nsb_row = p.cols / 256;                            // superblocks per weight row
    int nsb = nsb_row, sb0 = 0;                                  // this workgroup's share of them
    size_t ystride = (size_t)p.rows;
    if (p.ksplit) {
        const int slice = blockIdx.z;
        nsb = nsb_row / p.ksplit;
        sb0 = slice * nsb;
        p.Y = p.Y_parts + (size_t)blockIdx.z * p.batch * rows_all + ycol;   // partial sums: all matrices' columns side by side
        ystride = (size_t)rows_all;
    }
    const int nsteps = nsb * 4;

    if (Q6 && wave >= 4) {
        // ------------------------------------------------------------------ loaders, Q6_K
        // thread lh of a row's pair converts columns 32*lh .. 32*lh+31 of every 64-column step: step (h, part)
        // of a superblock = ql bytes 64h + 32lh .. +31 (nibble `part`), qh bytes 32h .. +31 (bit pair
        // 4*part + 2*lh), scales 8h + 4*part + 2*lh and the next one.  Blocks are 2-byte aligned.
        const int lt = tid - 256, lrow = lt >> 1, lh = lt & 1;
        const size_t row_bytes = (size_t)nsb_row * 210;
        const uint8_t *wrow = p.W + (size_t)min(r0 + lrow, p.rows - 1) * row_bytes + (size_t)sb0 * 210;
        struct Sb6Regs {
            u32x2_t ql[8];    // [4h + i]: ql bytes 64h + 32lh + 8i .. +7
            u32x2_t qh[8];    // all 64 qh bytes
            u32x2_t sc[2];    // the 16 int8 scales
            uint32_t d;
        };
        auto ld64 = [](const uint8_t *a) __attribute__((always_inline)) {
            u32x2_t v;
            __builtin_memcpy(&v, a, 8);
            return v;
        };
        auto fetch_sb = [&](int sb, Sb6Regs &r) __attribute__((always_inline)) {
            const uint8_t *blk = wrow + (size_t)sb * 210;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                r.ql[i] = ld64(blk + 32 * lh + 8 * i);
                r.ql[4 + i] = ld64(blk + 64 + 32 * lh + 8 * i);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) r.qh[i] = ld64(blk + 128 + 8 * i);
            r.sc[0] = ld64(blk + 192);
            r.sc[1] = ld64(blk + 200);
            uint16_t d;
            __builtin_memcpy(&d, blk + 208, 2);
            r.d = d;
        };
        auto stage = [&](int step, auto gtag, const Sb6Regs &w) __attribute__((always_inline)) {
            constexpr int G = decltype(gtag)::value, H = G >> 1, P = G & 1;
            _Float16 *Bs = main_stage(step);
            const uint32_t s16 = (w.sc[H][P] >> (16 * lh)) & 0xFFFFu;
            const _Float16 sa = (_Float16)(int)(int8_t)(s16 & 0xFFu), sb_ = (_Float16)(int)(int8_t)(s16 >> 8);
            const h2 sc2[2] = {h2{sa, sa}, h2{sb_, sb_}};
            const h2 bias = {(_Float16)1056.f, (_Float16)1056.f};
            const int hsh = 4 * P + 2 * lh;
            uint32_t o[16];
#pragma unroll
            for (int j = 0; j < 8; j++) {   // 4 columns per dword; dwords 0..3 take the first scale, 4..7 the second
                const uint32_t L = w.ql[4 * H + (j >> 1)][j & 1], Q = w.qh[4 * H + (j >> 1)][j & 1];
                const uint32_t nib = (P ? (L >> 4) : L) & 0x0F0F0F0Fu;
                const uint32_t c = nib | (((Q >> hsh) & 0x03030303u) << 4);   // four 6-bit codes
                const uint32_t pa = (c & 0x00FF00FFu) | 0x64006400u;          // columns (0, 2) as 1024 + code
                const uint32_t pb = ((c >> 8) & 0x00FF00FFu) | 0x64006400u;   // columns (1, 3)
                const h2 va = (__builtin_bit_cast(h2, pa) - bias) * sc2[j >> 2];
                const h2 vb = (__builtin_bit_cast(h2, pb) - bias) * sc2[j >> 2];
                o[2 * j] = __builtin_bit_cast(uint32_t, va);
                o[2 * j + 1] = __builtin_bit_cast(uint32_t, vb);
            }
            uint4 *dst = reinterpret_cast<uint4 *>(&Bs[lrow * PITCH + 32 * lh]);
#pragma unroll
            for (int i = 0; i < 4; i++) dst[i] = make_uint4(o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]);
            if (G == 0 && lh == 0) dsc_stage(step >> 2)[lrow] = half_bits_to_f32(w.d);
        };
        Sb6Regs wcur, wnext;
        fetch_sb(0, wcur);
        stage(0, std::integral_constant<int, 0>{}, wcur);
        __syncthreads();
        auto step_body = [&](int sb, auto gtag) __attribute__((always_inline)) {
            constexpr int g = decltype(gtag)::value;
            const int step = 4 * sb + g;
            if (g == 0) fetch_sb(min(sb + 1, nsb - 1), wnext);
            if (step + 1 < nsteps) {
                if (g == 3) wcur = wnext;
                stage(step + 1, std::integral_constant<int, (g + 1) & 3>{}, wcur);
            }
            __syncthreads();
        };
        for (int sb = 0; sb < nsb; sb++) {
            step_body(sb, std::integral_constant<int, 0>{});
            step_body(sb, std::integral_constant<int, 1>{});
            step_body(sb, std::integral_constant<int, 2>{});
            step_body(sb, std::integral_constant<int, 3>{});
        }
        return;
    }

    if (!Q6 && wave >= 4) {
        // ------------------------------------------------------------------ loaders
        const int lt = tid - 256, lrow = lt >> 1, lh = lt & 1;   // two threads per tile row
        const size_t row_bytes = (size_t)nsb_row * 144;
        const uint8_t *wrow = p.W + (size_t)min(r0 + lrow, p.rows - 1) * row_bytes + (size_t)sb0 * 144;
        const size_t sx_off = ((size_t)min(t0 + lrow, p.batch - 1) * nsb_row + sb0) * 32;
        const _Float16 *sxrow = p.SxA + sx_off;

        auto fetch_sb = [&](int sb, SbRegs &r) __attribute__((always_inline)) {
            const u32x4_t *w = reinterpret_cast<const u32x4_t *>(wrow + (size_t)sb * 144);
            r.hdr = w[0];
#pragma unroll
            for (int i = 0; i < 4; i++) r.q[i] = w[1 + 2 * i + lh];     // the 16 bytes of group i that this thread converts
            const u32x4_t *sx = reinterpret_cast<const u32x4_t *>(sxrow + sb * 32 + 16 * lh);
            r.sx0 = sx[0];
            r.sx1 = sx[1];
        };
        // G = the step's group: this thread converts bytes 16*lh .. 16*lh+15 of its 32 quant bytes
        auto stage = [&](int step, auto gtag, const SbRegs &w) __attribute__((always_inline)) {
            constexpr int G = decltype(gtag)::value;
            const int sb = step >> 2;
            _Float16 *Bs = main_stage(step);
            {
                const u32x4_t c = w.q[G];
                const uint32_t q[4] = {c[0], c[1], c[2], c[3]};
                const uint4 s = q4k_group_scales(w.hdr.y, w.hdr.z, w.hdr.w, G);   // sc_lo, mn_lo, sc_hi, mn_hi
                uint32_t lo[8], hi[8];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t t4 = q[i] >> 4;
                    lo[2 * i] = pair_f16(q[i] & 0x000F000Fu, s.x);
                    lo[2 * i + 1] = pair_f16((q[i] >> 8) & 0x000F000Fu, s.x);
                    hi[2 * i] = pair_f16(t4 & 0x000F000Fu, s.z);
                    hi[2 * i + 1] = pair_f16((t4 >> 8) & 0x000F000Fu, s.z);
                }
                uint4 *dlo = reinterpret_cast<uint4 *>(&Bs[lrow * PITCH + 16 * lh]);
                uint4 *dhi = reinterpret_cast<uint4 *>(&Bs[lrow * PITCH + 32 + 16 * lh]);
                dlo[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
                dlo[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
                dhi[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
                dhi[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
            }
            if (G == 0) {
                // bias + mins of this superblock, for the short second product after its fourth step
                _Float16 *A2s = min_stage(sb), *B2s = A2s + TM * PITCH2;
                const float d = half_bits_to_f32(w.hdr.x & 0xFFFFu), dmin = half_bits_to_f32(w.hdr.x >> 16);
                // this thread covers sub-blocks 4*lh .. 4*lh+3 of its row: groups 2*lh, 2*lh+1
                uint32_t hi2[2], lo2[2];
#pragma unroll
                for (int gg = 0; gg < 2; gg++) {
                    const uint4 s = q4k_group_scales(w.hdr.y, w.hdr.z, w.hdr.w, 2 * lh + gg);
                    const float c0 = pinned(-(dmin * (float)s.y + 1024.f * d)), c1 = pinned(-(dmin * (float)s.w + 1024.f * d));
                    const _Float16 h0 = (_Float16)c0, h1 = (_Float16)c1;
                    const _Float16 l0 = (_Float16)(c0 - (float)h0), l1 = (_Float16)(c1 - (float)h1);
                    hi2[gg] = (uint32_t)__builtin_bit_cast(uint16_t, h0) | ((uint32_t)__builtin_bit_cast(uint16_t, h1) << 16);
                    lo2[gg] = (uint32_t)__builtin_bit_cast(uint16_t, l0) | ((uint32_t)__builtin_bit_cast(uint16_t, l1) << 16);
                }
                // row layout (32 halves): hi[8] | lo[8] | hi[8] | 0[8]; this thread owns halves 4*lh .. +3 of each octet
                uint2 *b2 = reinterpret_cast<uint2 *>(&B2s[lrow * PITCH2 + 4 * lh]);
                b2[0] = make_uint2(hi2[0], hi2[1]);
                b2[2] = make_uint2(lo2[0], lo2[1]);
                b2[4] = make_uint2(hi2[0], hi2[1]);
                b2[6] = make_uint2(0u, 0u);
                if (lh == 0) dsc_stage(sb)[lrow] = d;
                if (lrow < TM) {
                    u32x4_t *dst = reinterpret_cast<u32x4_t *>(&A2s[lrow * PITCH2 + 16 * lh]);
                    dst[0] = w.sx0;
                    dst[1] = w.sx1;
                }
            }
        };

        // the next superblock's weights are requested when a superblock opens: four steps to arrive
        SbRegs wcur, wnext;
        fetch_sb(0, wcur);
        stage(0, std::integral_constant<int, 0>{}, wcur);
        __syncthreads();
        auto step_body = [&](int sb, auto gtag) __attribute__((always_inline)) {
            constexpr int g = decltype(gtag)::value;
            const int step = 4 * sb + g;
            if (g == 0) fetch_sb(min(sb + 1, nsb - 1), wnext);
            if (step + 1 < nsteps) {
                if (g == 3) wcur = wnext;
                stage(step + 1, std::integral_constant<int, (g + 1) & 3>{}, wcur);
            }
            __syncthreads();
        };
        for (int sb = 0; sb < nsb; sb++) {
            step_body(sb, std::integral_constant<int, 0>{});
            step_body(sb, std::integral_constant<int, 1>{});
            step_body(sb, std::integral_constant<int, 2>{});
            step_body(sb, std::integral_constant<int, 3>{});
        }
        return;
    }

    // ---------------------------------------------------------------------- multipliers
    // WIDE (the 128-token tiles): a multiplying wave owns 32 tokens x all 128 columns instead of 64 x 64 -- one A fragment
    // per k slice serves four products, so the activations cross the vector-memory path once per workgroup instead of
    // twice (that path was busy for two thirds of the kernel), and all four waves read every B operand from LDS (twice
    // the LDS reads, which the operands requested a slice ahead hide): cfg2 31.5 -> 30.5 us per pair.
    constexpr bool WIDE = TM == 128;
    constexpr int MW = WIDE ? 1 : MT, NW_ = WIDE ? 4 : 2, NSPAN = WIDE ? 0 : 64;
    const int wm = WIDE ? wave : wave >> 1, wn = WIDE ? 0 : wave & 1;
    f16v F[MW][NW_], Cp[MW][NW_];
#pragma unroll
    for (int a = 0; a < MW; a++)
#pragma unroll
        for (int b = 0; b < NW_; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) { F[a][b][i] = 0.f; Cp[a][b][i] = 0.f; }
    const int lm = lane & 31, lk = (lane >> 5) * 8;
    const f16v kZero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // A operands straight from memory: fragment (token tile, k / 16) is 64 lanes x 16 bytes, 1 KB apart along k.
    // Two register sets, each refilled for two steps ahead as soon as its own step's instructions are issued (LO: one
    // set of hi and lo fragments, refilled for the next step -- a step is long against the way to the cache).
    const int ntt = (p.batch + 31) / 32;
    const h8 *xa[MW];
#pragma unroll
    for (int mt = 0; mt < MW; mt++)
        xa[mt] = reinterpret_cast<const h8 *>(p.Xf) + ((size_t)min((t0 + (wm * MW + mt) * 32) / 32, ntt - 1) * (p.cols / 16) + (size_t)sb0 * 16) * 64 + lane;
    const ptrdiff_t lo_delta = LO ? reinterpret_cast<const h8 *>(p.Xf_lo) - reinterpret_cast<const h8 *>(p.Xf) : 0;
    auto afrag = [&](int mt, int step, int ks) __attribute__((always_inline)) {
        return xa[mt][(ptrdiff_t)(step * (KS / 16) + ks) * 64];
    };
    auto afrag_lo = [&](int mt, int step, int ks) __attribute__((always_inline)) {
        return xa[mt][(ptrdiff_t)(step * (KS / 16) + ks) * 64 + lo_delta];
    };
    constexpr int AHEAD = LO ? 1 : 2;
    struct ARegs { h8 a[MW][KS / 16], al[LO ? MW : 1][KS / 16]; };
    auto fetch_a = [&](int step, ARegs &r) __attribute__((always_inline)) {
#pragma unroll
        for (int mt = 0; mt < MW; mt++)
#pragma unroll
            for (int ks = 0; ks < KS / 16; ks++) {
                r.a[mt][ks] = afrag(mt, step, ks);
                if (LO) r.al[mt][ks] = afrag_lo(mt, step, ks);
            }
    };
    ARegs a0, a1;
    fetch_a(0, a0);
    if (!LO) fetch_a(min(1, nsteps - 1), a1);
    __syncthreads();   // stage 0 is written
    auto mul_step = [&](int sb, auto gtag, ARegs &A) __attribute__((always_inline)) {
        constexpr int g = decltype(gtag)::value;
        const int step = 4 * sb + g;
        const _Float16 *Bs = main_stage(step);
        // B operands a k slice ahead (bf16 / f16 activations on the 128-token tile): left to itself the compiler reads a
        // slice's two operands into the registers the previous slice's products have just released, so every slice
        // begins with an LDS round trip in front of its four matrix instructions (cfg2: 32.5 -> 31.1 us per pair; with
        // f32 activations a slice has eight products to hide it behind: prompts of 1024 / 4000 tokens 14.1 / 67.6 ->
        // 14.0 / 67.1 ms).  The 64-token tile loses by it (a 256-token prompt 5.1 -> 5.3 ms) and keeps the plain order.
        constexpr bool BPIPE = TM == 128;
        h8 bb[2][NW_];
        if (BPIPE) {
#pragma unroll
            for (int nt = 0; nt < NW_; nt++)
                bb[0][nt] = *reinterpret_cast<const h8 *>(&Bs[(wn * NSPAN + nt * 32 + lm) * PITCH + lk]);
        }
#pragma unroll
        for (int ks = 0; ks < KS / 16; ks++) {
            h8 b[NW_];
            if (BPIPE) {
                if (ks + 1 < KS / 16) {
#pragma unroll
                    for (int nt = 0; nt < NW_; nt++)
                        bb[(ks + 1) & 1][nt] = *reinterpret_cast<const h8 *>(&Bs[(wn * NSPAN + nt * 32 + lm) * PITCH + 16 * (ks + 1) + lk]);
                }
                __builtin_amdgcn_sched_barrier(0);   // (the requests stay in front of this slice's products)
#pragma unroll
                for (int nt = 0; nt < NW_; nt++) b[nt] = bb[ks & 1][nt];
            } else {
#pragma unroll
                for (int nt = 0; nt < NW_; nt++)
                    b[nt] = *reinterpret_cast<const h8 *>(&Bs[(wn * NSPAN + nt * 32 + lm) * PITCH + 16 * ks + lk]);
            }
#pragma unroll
            for (int mt = 0; mt < MW; mt++)
#pragma unroll
                for (int nt = 0; nt < NW_; nt++)
                    // a superblock's first product starts from the constant zero: no pass over the accumulators to clear them
                    Cp[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A.a[mt][ks], b[nt], (g == 0 && ks == 0) ? kZero16 : Cp[mt][nt], 0, 0, 0);
            if (LO) {
#pragma unroll
                for (int mt = 0; mt < MW; mt++)
#pragma unroll
                    for (int nt = 0; nt < NW_; nt++)
                        Cp[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A.al[mt][ks], b[nt], Cp[mt][nt], 0, 0, 0);
            }
            // this k slice's fragments are spent: ask for the ones of AHEAD steps on right away
#pragma unroll
            for (int mt = 0; mt < MW; mt++) {
                A.a[mt][ks] = afrag(mt, min(step + AHEAD, nsteps - 1), ks);
                if (LO) A.al[mt][ks] = afrag_lo(mt, min(step + AHEAD, nsteps - 1), ks);
            }
            if (BPIPE) __builtin_amdgcn_sched_barrier(0);
        }
        if (g == 3) {
            // ---- end of the superblock: bias + mins through the short second product, then the row scale
            const _Float16 *A2s = min_stage(sb), *B2s = A2s + TM * PITCH2;
            const float *dsc = dsc_stage(sb);
#pragma unroll
            for (int ks = 0; ks < (Q6 ? 0 : 2); ks++) {
                h8 a[MW], b[NW_];
#pragma unroll
                for (int mt = 0; mt < MW; mt++)
                    a[mt] = *reinterpret_cast<const h8 *>(&A2s[((wm * MW + mt) * 32 + lm) * PITCH2 + 16 * ks + lk]);
#pragma unroll
                for (int nt = 0; nt < NW_; nt++)
                    b[nt] = *reinterpret_cast<const h8 *>(&B2s[(wn * NSPAN + nt * 32 + lm) * PITCH2 + 16 * ks + lk]);
#pragma unroll
                for (int mt = 0; mt < MW; mt++)
#pragma unroll
                    for (int nt = 0; nt < NW_; nt++)
                        F[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt], b[nt], F[mt][nt], 0, 0, 0);
            }
#pragma unroll
            for (int nt = 0; nt < NW_; nt++) {
                const float dn = dsc[wn * NSPAN + nt * 32 + lm];
#pragma unroll
                for (int mt = 0; mt < MW; mt++)
#pragma unroll
                    for (int i = 0; i < 16; i++)
                        F[mt][nt][i] = fmaf(dn, Cp[mt][nt][i], F[mt][nt][i]);
            }
        }
        __syncthreads();
    };
    for (int sb = 0; sb < nsb; sb++) {
        mul_step(sb, std::integral_constant<int, 0>{}, a0);
        mul_step(sb, std::integral_constant<int, 1>{}, LO ? a0 : a1);
        mul_step(sb, std::integral_constant<int, 2>{}, a0);
        mul_step(sb, std::integral_constant<int, 3>{}, LO ? a0 : a1);
    }

    // accumulator layout of the 32x32 tile: column = lane % 32, row = 8*(i/4) + 4*(lane/32) + i%4
#pragma unroll
    for (int mt = 0; mt < MW; mt++)
#pragma unroll
        for (int nt = 0; nt < NW_; nt++) {
            const int r = r0 + wn * NSPAN + nt * 32 + lm;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int t = t0 + (wm * MW + mt) * 32 + 8 * (i / 4) + 4 * (lane >> 5) + (i & 3);
                if (t < p.batch && r < p.rows) p.Y[(size_t)t * ystride + r] = LO ? F[mt][nt][i] * p.inv_s[t] : F[mt][nt][i];
            }
        }
}

// ---- small batches (up to 64 tokens): a GEMV-shaped launch on the matrix cores ---------------------------------
// A prompt remainder or a round of decoding slots is a few dozen tokens: the 128 x 128 tile then leaves most of the
// chip idle (rows / 128 workgroups) and half of every tile empty.  Here a workgroup owns 32 weight rows and all
// tokens; its 8 waves split the row's superblocks between them (K-split inside the workgroup, folded through LDS at
// the end, so the sum order is fixed) and every wave reads its weights straight from memory in the order the matrix
// instruction wants its B operand: lane (n, h) = (lane % 32, lane / 32) owns row n and, in every 16-column slice,
// columns 8h .. 8h+7 -- per 64-column group the low and the high nibbles of bytes 8h .. 8h+7 and 16+8h .. 16+8h+7,
// two 8-byte loads.  Conversion (sc*n as exact f16, biased by 1024), the per-superblock scale and the bias / min
// product are those of the big tile; the activations come as the same fragments, hi and lo part in the same pass
// (each converted weight is used for both), so f32 activations cost one launch.
template <int MT, bool HAS_LO>
__global__ __launch_bounds__(512) void q4k_mm_skinny_kernel(MmParams p, const _Float16 *__restrict__ Xf_lo, const _Float16 *__restrict__ SxA_lo,
                                                             float lo_scale)
{
    extern __shared__ __attribute__((aligned(16))) float red[];   // [8][MT][16][64]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;
    const int r0 = blockIdx.x * 32, nsb = p.cols / 256;
    const size_t row_bytes = (size_t)nsb * 144;
    const uint8_t *wrow = p.W + (size_t)min(r0 + n, p.rows - 1) * row_bytes;
    const int ntt = (p.batch + 31) / 32;
    const h8 *xa[MT], *xl[MT];
    const _Float16 *sxa[MT], *sxl[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        const size_t frag0 = (size_t)min(mt, ntt - 1) * (p.cols / 16) * 64 + lane;
        xa[mt] = reinterpret_cast<const h8 *>(p.Xf) + frag0;
        xl[mt] = reinterpret_cast<const h8 *>(HAS_LO ? Xf_lo : p.Xf) + frag0;
        const size_t so = (size_t)min(mt * 32 + n, p.batch - 1) * nsb * 32 + 8 * h;   // + sb * 32 + 16 * ks
        sxa[mt] = p.SxA + so;
        sxl[mt] = (HAS_LO ? SxA_lo : p.SxA) + so;
    }
    f16v F[MT], Fl[MT];
    const f16v kZero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mt = 0; mt < MT; mt++) { F[mt] = kZero16; Fl[mt] = kZero16; }

    for (int sb = wave; sb < nsb; sb += 8) {
        const uint8_t *blk = wrow + (size_t)sb * 144;
        const u32x4_t hdr = *reinterpret_cast<const u32x4_t *>(blk);
        u32x2_t q[4][2];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            q[g][0] = *reinterpret_cast<const u32x2_t *>(blk + 16 + 32 * g + 8 * h);
            q[g][1] = *reinterpret_cast<const u32x2_t *>(blk + 16 + 32 * g + 16 + 8 * h);
        }
        f16v C[MT], Cl[MT];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            // this group's activation fragments: slices 4g .. 4g+3 of the superblock
            h8 a[MT][4], al[MT][4];
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const size_t o = (size_t)(sb * 16 + 4 * g + j) * 64;
                    a[mt][j] = xa[mt][o];
                    if (HAS_LO) al[mt][j] = xl[mt][o];
                }
            const uint4 s = q4k_group_scales(hdr.y, hdr.z, hdr.w, g);   // sc_lo, mn_lo, sc_hi, mn_hi
#pragma unroll
            for (int j = 0; j < 4; j++) {
                // slice j: bytes (j & 1 ? 16 + 8h : 8h) .. +7, low nibbles for j < 2, high nibbles after
                const u32x2_t qq = q[g][j & 1];
                const uint32_t sc = j < 2 ? s.x : s.z;
                uint32_t o[4];
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    const uint32_t d = j < 2 ? qq[i] : qq[i] >> 4;
                    o[2 * i] = pair_f16(d & 0x000F000Fu, sc);
                    o[2 * i + 1] = pair_f16((d >> 8) & 0x000F000Fu, sc);
                }
                const u32x4_t ov = {o[0], o[1], o[2], o[3]};
                const h8 b = __builtin_bit_cast(h8, ov);
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    C[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt][j], b, (g == 0 && j == 0) ? kZero16 : C[mt], 0, 0, 0);
                    if (HAS_LO) Cl[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[mt][j], b, (g == 0 && j == 0) ? kZero16 : Cl[mt], 0, 0, 0);
                }
            }
        }
        // bias + mins of the superblock: the row's eight coefficients -(dmin*m_j + 1024*d) as f16 hi | lo, against the
        // tokens' sums of x (hi[8] hi[8] lo[8] 0[8] per token and superblock): hi*hi + hi*lo + lo*hi
        const float d = half_bits_to_f32(hdr.x & 0xFFFFu), dmin = half_bits_to_f32(hdr.x >> 16);
        _Float16 chi[8], clo[8];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint4 s = q4k_group_scales(hdr.y, hdr.z, hdr.w, g);
            const float c0 = pinned(-(dmin * (float)s.y + 1024.f * d)), c1 = pinned(-(dmin * (float)s.w + 1024.f * d));
            chi[2 * g] = (_Float16)c0; chi[2 * g + 1] = (_Float16)c1;
            clo[2 * g] = (_Float16)(c0 - (float)chi[2 * g]); clo[2 * g + 1] = (_Float16)(c1 - (float)chi[2 * g + 1]);
        }
        h8 b2[2];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            b2[0][i] = h ? clo[i] : chi[i];                 // columns 0..7: hi, 8..15: lo
            b2[1][i] = h ? (_Float16)0.f : chi[i];          // columns 16..23: hi, 24..31: zero
        }
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                const h8 a2 = *reinterpret_cast<const h8 *>(sxa[mt] + (size_t)sb * 32 + 16 * ks);
                F[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2, b2[ks], F[mt], 0, 0, 0);
                if (HAS_LO) {
                    const h8 a2l = *reinterpret_cast<const h8 *>(sxl[mt] + (size_t)sb * 32 + 16 * ks);
                    Fl[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2l, b2[ks], Fl[mt], 0, 0, 0);
                }
            }
#pragma unroll
            for (int i = 0; i < 16; i++) {
                F[mt][i] = fmaf(d, C[mt][i], F[mt][i]);
                if (HAS_LO) Fl[mt][i] = fmaf(d, Cl[mt][i], Fl[mt][i]);
            }
        }
    }
    // fold the eight waves' shares (fixed order), then store: accumulator i of lane (n, h) is token
    // 8*(i/4) + 4*h + i%4 of the tile, weight row n
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int i = 0; i < 16; i++)
            red[((wave * MT + mt) * 16 + i) * 64 + lane] = HAS_LO ? fmaf(lo_scale, Fl[mt][i], F[mt][i]) : F[mt][i];
    __syncthreads();
    for (int o = tid; o < MT * 16 * 64; o += 512) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < 8; w++) sum += red[w * MT * 16 * 64 + o];
        const int mt = o / (16 * 64), i = (o / 64) & 15, l = o & 63;
        const int t = mt * 32 + 8 * (i / 4) + 4 * (l >> 5) + (i & 3), r = r0 + (l & 31);
        if (t < p.batch && r < p.rows) p.Y[(size_t)t * p.rows + r] = sum;
    }
}

// ---- decode rounds (up to 16 tokens) --------------------------------------------------------------------------
// A round of decoding slots is at most 16 rows, and several GEMMs read the same rows (q | k | v, gate | up).  Two
// kinds serve it (neither has a counterpart in the reference, whose round is one decode step per request):
//   KSH_ROUND_PREP    x f32[batch, cols] -> a prepared operand: the fragments of the 32 x 32 x 16 matrix instruction
//                     with x = hi + 2^-11 lo in ONE tile -- rows 0..15 the tokens' hi parts, rows 16..31 their lo
//                     parts -- so that one instruction per weight slice serves both parts, and the sums of x per
//                     sub-block for the bias / min product, hi and lo.  Written once per distinct input.
//   KSH_MATVEC_ROUND  up to three Q4_K matrices of the same width against one prepared operand in one launch, or a
//                     gate | up pair whose workgroups hold the same 32 rows of both and store gelu(gate) * up.
// A workgroup owns 32 weight rows of one matrix and 8 superblocks of columns, one per wave: every load of the
// workgroup (80 bytes of weights and 288 of activations per lane) goes out before anything is used, so the launch is
// one memory round trip where the small-batch form above walks a wave's superblocks one round trip at a time.  Rows
// longer than 2048 columns split over blockIdx.y; the slices' sums go to a scratch buffer and a second launch adds
// them in a fixed order.  Conversion, scales and the bias / min product are those of the forms above.

// what one thread does with 8 consecutive elements (8 j .. 8 j + 7) of token row t; whole quads call it together
// (the four threads of a sub-block add their sums up over the quad)
__device__ __forceinline__ void round_prep_write(const float (&f)[8], int t, int j, int cols, _Float16 *__restrict__ Xp)
{
    h8 oh, ol;
    float sh, sl;
    round_split8(f, oh, ol, sh, sl);
    sh += dpp_f32<0xB1>(sh);
    sh += dpp_f32<0x4E>(sh);
    sl += dpp_f32<0xB1>(sl);
    sl += dpp_f32<0x4E>(sl);
    // fragment of 16 columns: lane = row + 32 * ((k / 8) % 2); row t is the token's hi part, row 16 + t its lo part
    const size_t frag = (size_t)(j >> 1) * 64 + t + 32 * (j & 1);
    reinterpret_cast<h8 *>(Xp)[frag] = oh;
    reinterpret_cast<h8 *>(Xp)[frag + 16] = ol;
    if ((threadIdx.x & 3) == 0) round_store_sums(Xp, cols, t, j / 4, sh, sl);
}

// one thread per 8 elements of the 16 token rows (rows past the batch are written as zeros)
__global__ __launch_bounds__(256) void mm_round_prep_kernel(const float *__restrict__ X, _Float16 *__restrict__ Xp, int batch, int cols)
{
    const int idx = blockIdx.x * 256 + threadIdx.x;
    const int k8 = cols / 8;
    if (idx >= kRoundTokens * k8) return;   // (whole quads: cols is a multiple of 32)
    const int t = idx / k8, j = idx - t * k8;
    f32x4_t in0 = {0.f, 0.f, 0.f, 0.f}, in1 = in0;
    if (t < batch) {
        in0 = reinterpret_cast<const f32x4_t *>(X)[2 * ((size_t)t * k8 + j)];
        in1 = reinterpret_cast<const f32x4_t *>(X)[2 * ((size_t)t * k8 + j) + 1];
    }
    const float f[8] = {in0.x, in0.y, in0.z, in0.w, in1.x, in1.y, in1.z, in1.w};
    round_prep_write(f, t, j, cols, Xp);
}

// The rows forms of the norms (rmsnorm_rows, rmsnorm_add_then_rmsnorm rows: crates/ksearch_kernels/src/lib.rs:1478-1560)
// with the prepared operand as their output: one workgroup per token row, the same sums in the same order as the
// kernels that write f32 rows (explicitly rounded products and sums: nothing is contracted).
//   MODE 1:  v = (x * inv) * w                                                     -> xp
//   MODE 2:  x_new = [scale *] (res + (y * inv) * w_post);  v = (x_new * inv2) * w_norm   -> xp, x_new (may be res)
//   MODE 3:  x_new = res + (y * inv) * w_post;  v = x_new                          -> xp, x_new (may be res)
__device__ __forceinline__ float round_block_sum(float v, float *red)
{
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();                       // (red may still be read from the previous sum)
    if (lane == 0) red[wave] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

template <int MODE>
__global__ __launch_bounds__(256) void mm_round_prep_norm_kernel(const float *__restrict__ x, const float *__restrict__ w_first, const float *res,
                                                                 const float *__restrict__ w_norm, float *x_new, _Float16 *__restrict__ Xp,
                                                                 int batch, int cols, float eps, float scale)
{
    __shared__ float red[4];
    extern __shared__ float mid[];      // MODE 2: the row between the two norms
    const int t = blockIdx.x, k8 = cols / 8;
    if (t >= batch) {
        const float zero[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int j = threadIdx.x; j < k8; j += 256) round_prep_write(zero, t, j, cols, Xp);
        return;
    }
    x += (size_t)t * cols;
    float ss = 0.f;
    for (int i = threadIdx.x; i < cols; i += 256) ss = __fadd_rn(ss, __fmul_rn(x[i], x[i]));
    ss = round_block_sum(ss, red);
    float inv = 1.0f / sqrtf(__fadd_rn(ss / (float)cols, eps));
    if (MODE >= 2) {
        res += (size_t)t * cols;
        x_new += (size_t)t * cols;
        float ss2 = 0.f;
        for (int i = threadIdx.x; i < cols; i += 256) {
            float v = __fadd_rn(__fmul_rn(__fmul_rn(x[i], inv), w_first[i]), res[i]);
            if (scale != 0.f) v = __fmul_rn(scale, v);
            mid[i] = v;
            x_new[i] = v;
            ss2 = __fadd_rn(ss2, __fmul_rn(v, v));
        }
        if (MODE == 2) {
            ss2 = round_block_sum(ss2, red);
            inv = 1.0f / sqrtf(__fadd_rn(ss2 / (float)cols, eps));
        } else {
            __syncthreads();   // the row is read across threads below
        }
    }
    const float *src = MODE >= 2 ? mid : x, *w = MODE == 2 ? w_norm : w_first;
    for (int j = threadIdx.x; j < k8; j += 256) {
        float f[8];
#pragma unroll
        for (int i = 0; i < 8; i++) f[i] = MODE == 3 ? src[8 * j + i] : pinned(__fmul_rn(__fmul_rn(src[8 * j + i], inv), w[8 * j + i]));
        round_prep_write(f, t, j, cols, Xp);
    }
}

// The same for rows of up to 2048 columns (the widths of the models this serves): thread j owns elements 8 j .. 8 j + 7
// from the first load to the fragment it writes, every input is requested up front, and the row never passes through
// LDS -- the launch is one round trip and two block sums where the form above is three dependent passes.  (The sums
// of squares are taken in a different order than the kernels that write f32 rows: equal to the last bit or two.)
template <int MODE>
__global__ __launch_bounds__(256) void mm_round_prep_norm8_kernel(const float *__restrict__ x, const float *__restrict__ w_first, const float *res,
                                                                  const float *__restrict__ w_norm, float *x_new, _Float16 *__restrict__ Xp,
                                                                  int batch, int cols, float eps, float scale, int slices)
{
    __shared__ float red[4];
    const int t = blockIdx.x, k8 = cols / 8, j = threadIdx.x;
    const bool has = j < k8;                  // (whole quads: cols is a multiple of 32)
    if (t >= batch) {
        const float zero[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (has) round_prep_write(zero, t, j, cols, Xp);
        return;
    }
    const f32x4_t z4 = {0.f, 0.f, 0.f, 0.f};
    const size_t e = (size_t)t * cols + 8 * (size_t)min(j, k8 - 1), ew = 8 * (size_t)min(j, k8 - 1);
    auto ld8 = [&](const float *p, size_t off, float (&o)[8]) {
        const f32x4_t a = has ? *reinterpret_cast<const f32x4_t *>(p + off) : z4, b = has ? *reinterpret_cast<const f32x4_t *>(p + off + 4) : z4;
        o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
    };
    float y[8], w1[8], r[8], w2[8];
    ld8(x, e, y);
    // x as the column slices' partial sums of a split GEMM ([slices][batch][cols]): added here, slice after slice, in
    // the order the GEMM's own second launch adds them
    for (int sl = 1; sl < slices; sl++) {
        float ys[8];
        ld8(x, (size_t)sl * batch * cols + e, ys);
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = __fadd_rn(y[i], ys[i]);
    }
    ld8(w_first, ew, w1);
    if (MODE >= 2) ld8(res, e, r);
    if (MODE == 2) ld8(w_norm, ew, w2);
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) ss = __fadd_rn(ss, __fmul_rn(y[i], y[i]));
    ss = round_block_sum(ss, red);
    float inv = 1.0f / sqrtf(__fadd_rn(ss / (float)cols, eps));
    float f[8];
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] = __fmul_rn(__fmul_rn(y[i], inv), w1[i]);
    if (MODE >= 2) {
        float ss2 = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            f[i] = __fadd_rn(f[i], r[i]);
            if (scale != 0.f) f[i] = __fmul_rn(scale, f[i]);
            ss2 = __fadd_rn(ss2, __fmul_rn(f[i], f[i]));
        }
        if (has) {
            *reinterpret_cast<f32x4_t *>(x_new + e) = f32x4_t{f[0], f[1], f[2], f[3]};
            *reinterpret_cast<f32x4_t *>(x_new + e + 4) = f32x4_t{f[4], f[5], f[6], f[7]};
        }
        if (MODE == 2) {
            ss2 = round_block_sum(ss2, red);
            inv = 1.0f / sqrtf(__fadd_rn(ss2 / (float)cols, eps));
#pragma unroll
            for (int i = 0; i < 8; i++) f[i] = __fmul_rn(__fmul_rn(f[i], inv), w2[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] = pinned(f[i]);
    if (has) round_prep_write(f, t, j, cols, Xp);
}

struct RoundParams {
    const uint8_t *W0, *W1, *W2;
    float *Y0, *Y1, *Y2;
    int rows0, rows1, rows2, tiles0, tiles1;
    int cols, batch;
    const _Float16 *Xp;
    float *part;                 // [slices][batch][rows0] when the columns are split
    const float *mul;            // NM = 1: y = gelu(W0 x) * mul[t * mul_stride + r] (the per-layer-embedding gate)
    int mul_stride;
    _Float16 *emit;              // not null: the result goes out as the prepared operand of the next GEMM (rows0 columns)
};

// NM = 2: the gate | up pair (W0, W1 of rows0 rows each; gelu(W0 x) * (W1 x) to Y0)
template <int NM>
__global__ __launch_bounds__(512) void q4k_mm_round_kernel(RoundParams p)
{
    extern __shared__ __attribute__((aligned(16))) float red[];   // [8][NM][8][64]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;
    // the workgroup's matrix: a choice between arguments already fetched, not an indexed read of them
    int tile = blockIdx.x;
    const bool in1 = NM == 1 && tile >= p.tiles0, in2 = in1 && tile - p.tiles0 >= p.tiles1;
    if (in1) tile -= p.tiles0;
    if (in2) tile -= p.tiles1;
    const uint8_t *W = in2 ? p.W2 : in1 ? p.W1 : p.W0;
    float *Y = in2 ? p.Y2 : in1 ? p.Y1 : p.Y0;
    const int rows = in2 ? p.rows2 : in1 ? p.rows1 : p.rows0;
    const int r0 = tile * 32, nsb = p.cols / 256;
    const int sb = blockIdx.y * 8 + wave;
    const bool active = sb < nsb;                        // (wave-uniform: a row of 1536 columns leaves two waves idle)
    const int sbc = min(sb, nsb - 1);
    const size_t woff = (size_t)min(r0 + n, rows - 1) * nsb * 144 + (size_t)sbc * 144;

    // ---- every load of the wave, up front
    u32x4_t hdr[NM];
    u32x2_t q[NM][4][2];
#pragma unroll
    for (int m = 0; m < NM; m++) {
        const uint8_t *blk = (m ? p.W1 : W) + woff;
        hdr[m] = *reinterpret_cast<const u32x4_t *>(blk);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            q[m][g][0] = *reinterpret_cast<const u32x2_t *>(blk + 16 + 32 * g + 8 * h);
            q[m][g][1] = *reinterpret_cast<const u32x2_t *>(blk + 16 + 32 * g + 16 + 8 * h);
        }
    }
    const h8 *xa = reinterpret_cast<const h8 *>(p.Xp) + (size_t)sbc * 16 * 64 + lane;
    h8 a[16];
#pragma unroll
    for (int j = 0; j < 16; j++) a[j] = xa[(size_t)j * 64];
    // sums of x: rows 0..15 the tokens' hi parts, rows 16..31 their lo parts
    const _Float16 *sx = p.Xp + round_xf_halves(p.cols) + (n >= 16 ? round_sx_halves(p.cols) : 0) + ((size_t)(n & 15) * nsb + sbc) * 32 + 8 * h;
    const h8 a2[2] = {*reinterpret_cast<const h8 *>(sx), *reinterpret_cast<const h8 *>(sx + 16)};

    const f16v kZero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int m = 0; m < NM; m++) {
        f16v C = kZero16;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint4 s = q4k_group_scales(hdr[m].y, hdr[m].z, hdr[m].w, g);   // sc_lo, mn_lo, sc_hi, mn_hi
#pragma unroll
            for (int j = 0; j < 4; j++) {
                // slice j: bytes (j & 1 ? 16 + 8h : 8h) .. +7, low nibbles for j < 2, high nibbles after
                const u32x2_t qq = q[m][g][j & 1];
                const uint32_t sc = j < 2 ? s.x : s.z;
                uint32_t o[4];
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    const uint32_t d = j < 2 ? qq[i] : qq[i] >> 4;
                    o[2 * i] = pair_f16(d & 0x000F000Fu, sc);
                    o[2 * i + 1] = pair_f16((d >> 8) & 0x000F000Fu, sc);
                }
                const u32x4_t ov = {o[0], o[1], o[2], o[3]};
                C = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[4 * g + j], __builtin_bit_cast(h8, ov), C, 0, 0, 0);
            }
        }
        // bias + mins of the superblock: the row's eight coefficients -(dmin*m_j + 1024*d) as f16 hi | lo, against the
        // sums of x (hi[8] hi[8] lo[8] 0[8] per row and superblock): hi*hi + hi*lo + lo*hi
        const float d = half_bits_to_f32(hdr[m].x & 0xFFFFu), dmin = half_bits_to_f32(hdr[m].x >> 16);
        _Float16 chi[8], clo[8];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint4 s = q4k_group_scales(hdr[m].y, hdr[m].z, hdr[m].w, g);
            const float c0 = pinned(-(dmin * (float)s.y + 1024.f * d)), c1 = pinned(-(dmin * (float)s.w + 1024.f * d));
            chi[2 * g] = (_Float16)c0; chi[2 * g + 1] = (_Float16)c1;
            clo[2 * g] = (_Float16)(c0 - (float)chi[2 * g]); clo[2 * g + 1] = (_Float16)(c1 - (float)chi[2 * g + 1]);
        }
        h8 b2[2];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            b2[0][i] = h ? clo[i] : chi[i];                 // columns 0..7: hi, 8..15: lo
            b2[1][i] = h ? (_Float16)0.f : chi[i];          // columns 16..23: hi, 24..31: zero
        }
        f16v F = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2[0], b2[0], kZero16, 0, 0, 0);
        F = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2[1], b2[1], F, 0, 0, 0);
        // accumulator i of lane (n, h) is row 8*(i/4) + 4*h + i%4 of the tile: i < 8 a token's hi part, i + 8 its lo part
#pragma unroll
        for (int i = 0; i < 8; i++)
            red[((wave * NM + m) * 8 + i) * 64 + lane] = active ? fmaf(1.0f / 2048.0f, fmaf(d, C[i + 8], F[i + 8]), fmaf(d, C[i], F[i])) : 0.f;
    }
    __syncthreads();
    // one output per thread: the eight waves' shares in a fixed order
    const int i = tid >> 6, t = 8 * (i >> 2) + 4 * h + (i & 3), r = r0 + n;
    float v[NM];
#pragma unroll
    for (int m = 0; m < NM; m++) {
        v[m] = 0.f;
#pragma unroll
        for (int w = 0; w < 8; w++) v[m] += red[((w * NM + m) * 8 + i) * 64 + lane];
    }
    const bool mine = t < p.batch && r < rows;
    float y = NM == 2 ? gelu_mul_f32(v[0], v[NM - 1]) : v[0];
    if (NM == 1 && p.mul) y = gelu_mul_f32(y, p.mul[(size_t)min(t, p.batch - 1) * p.mul_stride + min(r, rows - 1)]);
    if (!p.emit) {
        if (mine) {
            if (gridDim.y == 1) Y[(size_t)t * rows + r] = y;
            else p.part[((size_t)blockIdx.y * p.batch + t) * rows + r] = y;
        }
        return;
    }
    // The tile's 16 x 32 results are 32 columns of the next GEMM's input: two fragments' worth of every token row and
    // exactly one sub-block of sums, so the workgroup writes its share of the prepared operand itself (rows0 is a
    // multiple of 256 and the columns are not split: host-checked).  Rows past the batch are written as zeros.
    float *T = red + 8 * NM * 8 * 64;             // [16][33]
    T[t * 33 + n] = mine ? y : 0.f;
    __syncthreads();
    if (tid < 64) {
        const int tt = tid & 15, ks = (tid >> 4) & 1, kh = tid >> 5;
        float f[8];
#pragma unroll
        for (int e = 0; e < 8; e++) f[e] = T[tt * 33 + 16 * ks + 8 * kh + e];
        h8 oh, ol;
        float sh, sl;
        round_split8(f, oh, ol, sh, sl);
        const size_t frag = (size_t)(r0 / 16 + ks) * 64 + tt + 32 * kh;
        reinterpret_cast<h8 *>(p.emit)[frag] = oh;
        reinterpret_cast<h8 *>(p.emit)[frag + 16] = ol;
    } else if (tid < 80) {
        const int tt = tid - 64;
        float sh4[4], sl4[4];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            float f[8];
#pragma unroll
            for (int e = 0; e < 8; e++) f[e] = T[tt * 33 + 8 * g + e];
            h8 oh, ol;
            round_split8(f, oh, ol, sh4[g], sl4[g]);
        }
        round_store_sums(p.emit, rows, tt, r0 / 32, (sh4[0] + sh4[1]) + (sh4[2] + sh4[3]), (sl4[0] + sl4[1]) + (sl4[2] + sl4[3]));
    }
}

// y[i] = the slices' partial sums of element i, slice after slice
__global__ __launch_bounds__(256) void mm_round_fold_kernel(const float *__restrict__ part, float *__restrict__ y, int n, int slices)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float s = part[i];
    for (int k = 1; k < slices; k++) s += part[(size_t)k * n + i];
    y[i] = s;
}

// y[i] = the K slices' partial sums of element i, slice after slice; the slices of the low parts of f32 activations
// (parts = 2) come in scaled.  The partial sums hold the columns of up to three matrices side by side (rows0 | rows1 |
// rows2 per token), each with a result buffer of its own.
__global__ __launch_bounds__(256) void mm_parts_fold_kernel(const float *__restrict__ part, float *__restrict__ y0, float *__restrict__ y1, float *__restrict__ y2,
                                                             int batch, int rows0, int rows1, int rows2, int slices)
{
    const int rows_all = rows0 + rows1 + rows2, n = batch * rows_all;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float s = part[i];
    for (int k = 1; k < slices; k++) s += part[(size_t)k * n + i];
    if (!rows1) { y0[i] = s; return; }
    const int t = i / rows_all, c = i - t * rows_all;
    if (c < rows0) y0[(size_t)t * rows0 + c] = s;
    else if (c < rows0 + rows1) y1[(size_t)t * rows1 + c - rows0] = s;
    else y2[(size_t)t * rows2 + c - rows0 - rows1] = s;
}

// The same round against a Q6_K matrix with row-grouped fields (KSH_Q6K_ROWS: the LM head as the decode loops keep it;
// rows of up to 2048 columns).  The B operand is the 6-bit code minus 32 as an exact f16 integer (the code OR-ed into
// the mantissa of 1024.0, minus 1056 with one packed subtraction per two weights); Q6_K has one int8 scale per 16
// columns, which is the K depth of the matrix instruction, so the scale is applied in f32 to the instruction's
// result: nothing is rounded (folded into the f16 operand as the 128 x 128 tile does it, sc * q above 2048 loses
// its last bit).  A workgroup keeps the activations of the whole row in registers -- wave w the 16 fragments of
// superblock w -- and walks tiles of 32 weight rows, the next tile's bytes in flight under the current one; the waves'
// shares of a tile meet in LDS (two buffers, one barrier per tile).
constexpr int kQ6rRowAlign = 16;
__host__ __device__ inline size_t round_q6r_row_bytes(int bpr) { return ((size_t)bpr * 210 + kQ6rRowAlign - 1) / kQ6rRowAlign * kQ6rRowAlign; }

struct Round6Params {
    const uint8_t *W;
    float *Y;
    int rows, cols, batch, tiles, tiles_per_wg;
    const _Float16 *Xp;
};

struct Q6Tile {
    u32x2_t ql[2][2][2];   // [half][quadrant parity][low / high 16 positions]: bytes 8h .. 8h+7 of them
    u32x2_t qh[2][2];      // [half][low / high 16 positions]
    u32x4_t sc;            // the superblock's 16 int8 scales
    uint32_t d;
};

__global__ __launch_bounds__(512) void q6r_mm_round_kernel(Round6Params p)
{
    extern __shared__ __attribute__((aligned(16))) float red[];   // [2][8 waves][8][64]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;
    const int bpr = p.cols / 256;
    const bool active = wave < bpr;                       // (wave-uniform: a row of 1536 columns leaves two waves idle)
    const int sbc = min(wave, bpr - 1);
    const size_t row_bytes = round_q6r_row_bytes(bpr);
    const h8 *xa = reinterpret_cast<const h8 *>(p.Xp) + (size_t)sbc * 16 * 64 + lane;
    h8 a[16];
#pragma unroll
    for (int j = 0; j < 16; j++) a[j] = xa[(size_t)j * 64];
    auto load_tile = [&](Q6Tile &dst, int tile) {
        const uint8_t *rp = p.W + (size_t)min(tile * 32 + n, p.rows - 1) * row_bytes;
#pragma unroll
        for (int ip = 0; ip < 2; ip++)
#pragma unroll
            for (int lh = 0; lh < 2; lh++) {
#pragma unroll
                for (int par = 0; par < 2; par++)
                    dst.ql[ip][par][lh] = *reinterpret_cast<const u32x2_t *>(rp + (size_t)sbc * 128 + 64 * ip + 32 * par + 16 * lh + 8 * h);
                dst.qh[ip][lh] = *reinterpret_cast<const u32x2_t *>(rp + (size_t)bpr * 128 + (size_t)sbc * 64 + 32 * ip + 16 * lh + 8 * h);
            }
        dst.sc = *reinterpret_cast<const u32x4_t *>(rp + (size_t)bpr * 192 + (size_t)sbc * 16);
        dst.d = *reinterpret_cast<const uint16_t *>(rp + (size_t)bpr * 208 + (size_t)sbc * 2);
    };
    const int tile0 = blockIdx.x * p.tiles_per_wg, tile1 = min(tile0 + p.tiles_per_wg, p.tiles);
    if (tile0 >= tile1) return;
    uint32_t byte_mask = 0x00FF00FFu, bias = 0x64006400u;   // in registers: the and-or is then one instruction
    asm volatile("" : "+v"(byte_mask), "+v"(bias));
    const h8 k1056 = {(_Float16)1056.f, (_Float16)1056.f, (_Float16)1056.f, (_Float16)1056.f,
                      (_Float16)1056.f, (_Float16)1056.f, (_Float16)1056.f, (_Float16)1056.f};
    const f16v kZero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    Q6Tile cur, nxt;
    load_tile(cur, tile0);
    int buf = 0;
    for (int tile = tile0; tile < tile1; tile++) {
        load_tile(nxt, min(tile + 1, tile1 - 1));
        f16v G = kZero16;
#pragma unroll
        for (int j = 0; j < 16; j++) {
            // group j: half ip, quadrant q, positions 16 lh .. +15; element 16 j of the superblock onwards
            const int ip = j >> 3, q = (j >> 1) & 3, lh = j & 1;
            const u32x2_t ql2 = cur.ql[ip][q & 1][lh], qh2 = cur.qh[ip][lh];
            uint32_t o[4];
#pragma unroll
            for (int dw = 0; dw < 2; dw++) {
                const uint32_t lo4 = (ql2[dw] >> (4 * (q >> 1))) & 0x0F0F0F0Fu, hi2 = (qh2[dw] >> (2 * q)) & 0x03030303u;
                const uint32_t code = lo4 | (hi2 << 4);
                o[2 * dw] = (code & byte_mask) | bias;              // codes of bytes 0 and 2 as 1024 + c
                o[2 * dw + 1] = ((code >> 8) & byte_mask) | bias;   // bytes 1 and 3: the order the fragments keep
            }
            const u32x4_t ov = {o[0], o[1], o[2], o[3]};
            const h8 b = __builtin_bit_cast(h8, ov) - k1056;
            const f16v C = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j], b, kZero16, 0, 0, 0);
            const float sc = (float)(int)(int8_t)(cur.sc[j >> 2] >> (8 * (j & 3)));
#pragma unroll
            for (int i = 0; i < 16; i++) G[i] = fmaf(sc, C[i], G[i]);
        }
        // accumulator i of lane (n, h) is row 8*(i/4) + 4*h + i%4 of the tile: i < 8 a token's hi part, i + 8 its lo part
        const float d = active ? half_bits_to_f32(cur.d) : 0.f;
        float *mine = red + (size_t)(buf * 8 + wave) * 8 * 64 + lane;
#pragma unroll
        for (int i = 0; i < 8; i++) mine[i * 64] = d * fmaf(1.0f / 2048.0f, G[i + 8], G[i]);
        __syncthreads();
        {
            const int i = wave, t = 8 * (i >> 2) + 4 * h + (i & 3), r = tile * 32 + n;
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < 8; w++) sum += red[(size_t)((buf * 8 + w) * 8 + i) * 64 + lane];
            if (t < p.batch && r < p.rows) p.Y[(size_t)t * p.rows + r] = sum;
        }
        buf ^= 1;
        cur = nxt;
    }
}

int launch_round_prep(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int cols = (int)k.desc.dims[0], batch = (int)k.desc.dims[1], mode = (int)k.desc.dims[2];
    const int n = kRoundTokens * (cols / 8);
    const float *in1 = mode ? (const float *)a.in[1] : nullptr, *in2 = mode >= 2 ? (const float *)a.in[2] : nullptr,
                *in3 = mode == 2 ? (const float *)a.in[3] : nullptr;
    float *x_new = mode >= 2 ? (float *)a.out[1] : nullptr;
    const float scale = mode == 2 ? k.desc.params[1] : 0.f;
    const int slices = (int)std::max<int64_t>(1, k.desc.dims[3]);
#define KSH_PN(KERNEL, M, LDS) \
    hipLaunchKernelGGL(KERNEL<M>, dim3(kRoundTokens), dim3(256), LDS, st, (const float *)a.in[0], in1, in2, in3, x_new, (_Float16 *)a.out[0], batch, cols, \
                       k.desc.params[0], scale)
#define KSH_PN8(M) \
    hipLaunchKernelGGL(mm_round_prep_norm8_kernel<M>, dim3(kRoundTokens), dim3(256), 0, st, (const float *)a.in[0], in1, in2, in3, x_new, \
                       (_Float16 *)a.out[0], batch, cols, k.desc.params[0], scale, slices)
    if (mode && cols <= 2048) {
        if (mode == 1) KSH_PN8(1);
        else if (mode == 2) KSH_PN8(2);
        else KSH_PN8(3);
    } else if (mode == 1) {
        KSH_PN(mm_round_prep_norm_kernel, 1, 0);
    } else if (mode == 2) {
        KSH_PN(mm_round_prep_norm_kernel, 2, (size_t)cols * 4);
    } else if (mode == 3) {
        KSH_PN(mm_round_prep_norm_kernel, 3, (size_t)cols * 4);
    }
#undef KSH_PN
#undef KSH_PN8
    else
        hipLaunchKernelGGL(mm_round_prep_kernel, dim3((n + 255) / 256), dim3(256), 0, st, (const float *)a.in[0], (_Float16 *)a.out[0], batch, cols);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "round_prep launch");
}

int launch_matvec_round(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int64_t *d = k.desc.dims;
    if (k.desc.dtypes[0] == KSH_Q6K_ROWS) {
        Round6Params p6{};
        p6.W = (const uint8_t *)a.in[0];
        p6.Xp = (const _Float16 *)a.in[1];
        p6.Y = (float *)a.out[0];
        p6.rows = (int)d[0]; p6.cols = (int)d[1]; p6.batch = (int)d[2];
        p6.tiles = (p6.rows + 31) / 32;
        p6.tiles_per_wg = (p6.tiles + (int)k.info.grid[0] - 1) / (int)k.info.grid[0];
        hipLaunchKernelGGL(q6r_mm_round_kernel, dim3(k.info.grid[0]), dim3(512), k.info.lds_bytes, st, p6);
        const hipError_t e6 = hipGetLastError();
        return e6 == hipSuccess ? 0 : hip_fail(e6, "matvec_round (Q6_K rows) launch");
    }
    const bool pair = d[5] != 0;
    const int n_mat = pair ? 2 : d[4] ? 3 : d[3] ? 2 : 1;
    RoundParams p{};
    p.W0 = (const uint8_t *)a.in[0];
    p.Xp = (const _Float16 *)a.in[1];
    p.W1 = n_mat > 1 ? (const uint8_t *)a.in[2] : p.W0;
    p.W2 = n_mat > 2 ? (const uint8_t *)a.in[3] : p.W0;
    p.Y0 = (float *)a.out[0];
    p.Y1 = (!pair && n_mat > 1) ? (float *)a.out[1] : p.Y0;
    p.Y2 = n_mat > 2 ? (float *)a.out[2] : p.Y0;
    p.rows0 = (int)d[0]; p.rows1 = pair ? (int)d[0] : (int)d[3]; p.rows2 = (int)d[4];
    p.tiles0 = (p.rows0 + 31) / 32; p.tiles1 = pair ? 0 : (p.rows1 + 31) / 32;
    p.cols = (int)d[1]; p.batch = (int)d[2];
    p.part = (float *)k.scratch;
    if (d[7]) { p.mul = (const float *)a.in[2]; p.mul_stride = (int)d[7]; }
    if (d[6] == 1) { p.emit = (_Float16 *)a.out[0]; p.Y0 = p.Y1 = p.Y2 = nullptr; }
    if (d[6] == 2) p.part = (float *)a.out[0];     // the slices' partial sums are the result
    const dim3 grid(k.info.grid[0], k.info.grid[1]);
    if (pair) hipLaunchKernelGGL(q4k_mm_round_kernel<2>, grid, dim3(512), k.info.lds_bytes, st, p);
    else hipLaunchKernelGGL(q4k_mm_round_kernel<1>, grid, dim3(512), k.info.lds_bytes, st, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, "matvec_round launch");
    if (grid.y > 1 && d[6] != 2) {
        const int n = p.batch * p.rows0;
        hipLaunchKernelGGL(mm_round_fold_kernel, dim3((n + 255) / 256), dim3(256), 0, st, (const float *)k.scratch, p.Y0, n, (int)grid.y);
        e = hipGetLastError();
        if (e != hipSuccess) return hip_fail(e, "matvec_round fold launch");
    }
    return 0;
}

constexpr int kSkinnyMaxBatch = 64;

// Tokens per workgroup of the tile.  64 (Q4_K): up to 64 tokens (the other half of a 128-token tile would be empty
// rows), and wherever the 128-token tiles and their K slices are fewer than the compute units (bf16 activations) or
// than twice the compute units (f32 activations, whose tile runs two products per converted weight) -- two
// workgroups share a compute unit then, and twice as many of them fill the chip.  Beyond that the 128-token tile
// (bf16, cfg2: 33.7 us against 40.3 with 64-token tiles; f32, prompts of 256 / 1024 / 4000 tokens through cfg4's
// model: 5.05 / 14.1 / 67.7 ms with this rule, 5.07 / 14.25 / 68.0 with 64-token tiles throughout, 5.3 / 14.9 / 72.7
// with 128-token tiles from 65 tokens on).
int mm_tile_tokens(const ksh_kernel_desc &d, int64_t ks)
{
    if (d.dtypes[0] == KSH_Q6K) return 128;
    const int64_t row_tiles = (d.dims[0] + BN - 1) / BN + (d.dims[3] + BN - 1) / BN + (d.dims[4] + BN - 1) / BN;
    const int64_t fill = d.dtypes[1] == KSH_F32 ? 512 : 256;
    return d.dims[2] <= 64 || ((d.dims[2] + BM - 1) / BM) * row_tiles * ks < fill ? 64 : 128;
}

int launch_mul_mm(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int rows = (int)k.desc.dims[0], cols = (int)k.desc.dims[1], batch = (int)k.desc.dims[2];
    const bool f32x = k.desc.dtypes[1] == KSH_F32;
    const size_t xf_halves = (size_t)((batch + 31) / 32 * 32) * cols, sx_halves = (size_t)batch * (cols / 256) * 32;
    _Float16 *Xf = (_Float16 *)k.scratch;
    _Float16 *SxA = Xf + xf_halves;
    _Float16 *Xf_lo = SxA + sx_halves, *SxA_lo = Xf_lo + xf_halves;     // f32 activations only
    const int n = batch * (cols / 8);
    const int n_mat0 = 1 + (k.desc.dims[3] > 0) + (k.desc.dims[4] > 0), prologue = (int)k.desc.dims[5];
    // f32 activations of the tile: both parts at the row's own scale, 1 / s per row where the small-batch form keeps
    // the sums of the lo parts (which the tile does not use)
    const bool tile = k.variant != 1;
    float *inv_s = f32x && tile ? reinterpret_cast<float *>(SxA_lo) : nullptr;
    const dim3 pg((unsigned)batch), pb((unsigned)std::min((cols / 8 + 63) / 64 * 64, 1024));     // whole waves: the row-wide reductions read every lane
    if (prologue) {
        // the rows' producer runs inside the preparation: in = W, X, [W1, W2,] then the prologue's operands
        const int xs = (int)k.desc.dims[7];
        const int n_out0 = k.desc.dims[6] ? 1 : n_mat0;                    // (unfolded partial sums are one buffer)
        const float *X = (const float *)a.in[1], *q0 = (const float *)a.in[1 + n_mat0];
        const float eps = k.desc.params[0];
        if (prologue == 1)
            hipLaunchKernelGGL(mm_prep_rows_kernel<1>, pg, pb, 0, st, X, q0, nullptr, nullptr, nullptr, Xf, Xf_lo, SxA, SxA_lo, cols, eps, xs, inv_s);
        else if (prologue == 2)
            hipLaunchKernelGGL(mm_prep_rows_kernel<2>, pg, pb, 0, st, X, q0, (const float *)a.in[2 + n_mat0], (const float *)a.in[3 + n_mat0], (float *)a.out[n_out0],
                               Xf, Xf_lo, SxA, SxA_lo, cols, eps, xs, inv_s);
        else
            hipLaunchKernelGGL(mm_prep_rows_kernel<3>, pg, pb, 0, st, X, xs ? X : q0, nullptr, nullptr, nullptr, Xf, Xf_lo, SxA, SxA_lo, cols, eps, xs, inv_s);
    } else if (f32x && tile)
        hipLaunchKernelGGL(mm_prep_rows_kernel<0>, pg, pb, 0, st, (const float *)a.in[1], nullptr, nullptr, nullptr, nullptr, Xf, Xf_lo, SxA, SxA_lo, cols, 0.f, 0, inv_s);
    else if (f32x) hipLaunchKernelGGL(mm_prep_x_f32_kernel, dim3((n + 255) / 256), dim3(256), 0, st, (const float *)a.in[1], Xf, Xf_lo, SxA, SxA_lo, batch, cols);
    else hipLaunchKernelGGL(mm_prep_x_kernel, dim3(((batch + 31) / 32 * (cols / 32) + 3) / 4), dim3(256), 0, st, (const uint16_t *)a.in[1], Xf, SxA, batch, cols);
    MmParams p;
    p.W = (const uint8_t *)a.in[0];
    p.Y = (float *)a.out[0];
    p.rows = rows; p.cols = cols; p.batch = batch;
    const int rows1 = (int)k.desc.dims[3], rows2 = (int)k.desc.dims[4];
    p.rows1 = rows1; p.rows2 = rows2;
    p.W1 = rows1 ? (const uint8_t *)a.in[2] : p.W; p.W2 = rows2 ? (const uint8_t *)a.in[3] : p.W;
    const bool unfolded_out = k.desc.dims[6] != 0;
    p.Y1 = rows1 && !unfolded_out ? (float *)a.out[1] : p.Y; p.Y2 = rows2 && !unfolded_out ? (float *)a.out[2] : p.Y;
    if (k.variant == 1) {
        // the small-batch form: one launch, the low parts riding along
        p.Xf = Xf; p.SxA = SxA;
        const dim3 sg((rows + 31) / 32);
        const int mt = batch <= 32 ? 1 : 2;
        const size_t lds = (size_t)8 * mt * 16 * 64 * 4;
        if (f32x && mt == 1) hipLaunchKernelGGL((q4k_mm_skinny_kernel<1, true>), sg, dim3(512), lds, st, p, Xf_lo, SxA_lo, 1.0f / 2048.0f);
        else if (f32x) hipLaunchKernelGGL((q4k_mm_skinny_kernel<2, true>), sg, dim3(512), lds, st, p, Xf_lo, SxA_lo, 1.0f / 2048.0f);
        else if (mt == 1) hipLaunchKernelGGL((q4k_mm_skinny_kernel<1, false>), sg, dim3(512), lds, st, p, Xf, SxA, 0.f);
        else hipLaunchKernelGGL((q4k_mm_skinny_kernel<2, false>), sg, dim3(512), lds, st, p, Xf, SxA, 0.f);
        const hipError_t e2 = hipGetLastError();
        return e2 == hipSuccess ? 0 : hip_fail(e2, "mul_mm (small batch) launch");
    }
    const int tm = mm_tile_tokens(k.desc, k.variant >= 2 ? k.variant >> 1 : 1);
    const dim3 grid((batch + tm - 1) / tm, (rows + BN - 1) / BN + (rows1 + BN - 1) / BN + (rows2 + BN - 1) / BN);
    p.Xf = Xf; p.SxA = SxA; p.Xf_lo = Xf_lo; p.inv_s = inv_s;
    p.ksplit = 0; p.Y_parts = nullptr;
    const bool q6 = k.desc.dtypes[0] == KSH_Q6K;
    auto launch_tile = [&](dim3 g) {
#define KSH_TILE(Q6, TM, LDS) \
    do { \
        if (f32x) hipLaunchKernelGGL((q_mul_mm_kernel<Q6, TM, true>), g, dim3(kThreadsMM), LDS, st, p); \
        else hipLaunchKernelGGL((q_mul_mm_kernel<Q6, TM, false>), g, dim3(kThreadsMM), LDS, st, p); \
    } while (0)
        if (q6) KSH_TILE(true, 128, kLdsBytes);
        else if (tm == 64) KSH_TILE(false, 64, kLdsBytes64);
        else KSH_TILE(false, 128, kLdsBytes);
#undef KSH_TILE
    };
    if (k.variant >= 2) {
        // few tiles: K slices as blockIdx.z of one launch, then the fold
        const int ks = k.variant >> 1;
        p.ksplit = ks;
        const bool unfolded = k.desc.dims[6] != 0;                    // the partial sums are the result: the reader adds them
        p.Y_parts = unfolded ? (float *)a.out[0] : (float *)((f32x ? SxA_lo : SxA) + sx_halves);     // (else behind the prepared activations)
        launch_tile(dim3(grid.x, grid.y, ks));
        hipError_t e3 = hipGetLastError();
        if (e3 != hipSuccess) return hip_fail(e3, "mul_mm (K slices) launch");
        if (unfolded) return 0;
        const int n2 = batch * (rows + rows1 + rows2);
        hipLaunchKernelGGL(mm_parts_fold_kernel, dim3((n2 + 255) / 256), dim3(256), 0, st, (const float *)p.Y_parts, p.Y, p.Y1, p.Y2, batch, rows, rows1, rows2,
                           ks);
        e3 = hipGetLastError();
        return e3 == hipSuccess ? 0 : hip_fail(e3, "mul_mm fold launch");
    }
    launch_tile(grid);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "mul_mm launch");
}

}  // namespace

int bind_matvec_batch(ksh_kernel &k)
{
    const int64_t rows = k.desc.dims[0], cols = k.desc.dims[1], batch = k.desc.dims[2];
    const bool q6 = k.desc.dtypes[0] == KSH_Q6K;
    if (k.desc.dtypes[0] != KSH_Q4K && !q6) return set_error("matvec_batch: weight dtype %d is not built (Q4_K and Q6_K are)", k.desc.dtypes[0]);
    const bool f32x = k.desc.dtypes[1] == KSH_F32;
    if (k.desc.dtypes[1] != KSH_BF16 && !f32x) return set_error("matvec_batch: activation dtype %d is not built (BF16 and F32 are)", k.desc.dtypes[1]);
    if (rows <= 0 || batch <= 0 || rows > (1 << 24) || batch > (1 << 20)) return set_error("matvec_batch: rows=%lld batch=%lld", (long long)rows, (long long)batch);
    if (cols <= 0 || cols % 256 || cols > (1 << 20)) return set_error("matvec_batch: cols=%lld is not a positive multiple of 256", (long long)cols);
    // dims[3], dims[4]: the rows of a second and a third matrix over the same activations (q | k | v of a prompt
    // chunk), taken by the 128 x 128 tile in the same launch
    const int64_t rows1 = k.desc.dims[3], rows2 = k.desc.dims[4], rows_all = rows + rows1 + rows2;
    if (rows1 < 0 || rows2 < 0 || (rows2 && !rows1) || rows_all > (1 << 24)) return set_error("matvec_batch: rows of the further matrices %lld, %lld", (long long)rows1, (long long)rows2);
    const int n_mat = 1 + (rows1 > 0) + (rows2 > 0);
    k.info.n_inputs = 1 + n_mat;
    k.info.n_outputs = n_mat;
    const size_t row_bytes = (size_t)(cols / 256) * (q6 ? 210 : 144);
    k.in_bytes[0] = (size_t)rows * row_bytes; k.in_align[0] = q6 ? 2 : 16;
    k.in_bytes[1] = (size_t)batch * cols * (f32x ? 4 : 2); k.in_align[1] = 16;
    k.out_bytes[0] = (size_t)batch * rows * 4; k.out_align[0] = 4;
    if (rows1) { k.in_bytes[2] = (size_t)rows1 * row_bytes; k.in_align[2] = k.in_align[0]; k.out_bytes[1] = (size_t)batch * rows1 * 4; k.out_align[1] = 4; }
    if (rows2) { k.in_bytes[3] = (size_t)rows2 * row_bytes; k.in_align[3] = k.in_align[0]; k.out_bytes[2] = (size_t)batch * rows2 * 4; k.out_align[2] = 4; }
    // dims[5]: the producer of the rows, run inside the preparation of f32 activations (params[0] = eps):
    //   1 rmsnorm(X, w)                 in: ..., w[cols]
    //   2 add then norm                 in: ..., w_post[cols], res[batch, cols], w_norm[cols]   out: ..., x_new[batch, cols] (may be res)
    //   3 gelu(X) * up                  in: ..., up[batch, cols]
    const int64_t prologue = k.desc.dims[5];
    if (prologue < 0 || prologue > 3) return set_error("matvec_batch: prologue %lld (0 none, 1 rmsnorm, 2 add then norm, 3 gelu * up)", (long long)prologue);
    // dims[6] = 1: the K slices' partial sums are the result, unfolded: out[0] = f32[slices][batch][all rows] (the
    // matrices' columns side by side; slices = grid[2] of the bound kernel), for a reader that adds them itself --
    // dims[7] = the slices (grid[2]) of the GEMM whose unfolded result this one's X is (prologues 1 to 3; prologue 3
    // then reads gate | up from that one buffer and takes no `up` operand)
    const int64_t unfolded = k.desc.dims[6], x_slices = k.desc.dims[7];
    if (unfolded < 0 || unfolded > 1) return set_error("matvec_batch: dims[6]=%lld (0, or 1 for unfolded partial sums)", (long long)unfolded);
    if (x_slices && (!prologue || x_slices < 1 || x_slices > 64))
        return set_error("matvec_batch: X as unfolded partial sums (dims[7]=%lld) takes a prologue and 1 to 64 slices", (long long)k.desc.dims[7]);
    if (prologue) {
        if (!f32x) return set_error("matvec_batch: a prologue takes F32 activations");
        if (prologue != 3 && (cols > 8192 || cols % 512)) return set_error("matvec_batch: a norm prologue takes rows of a multiple of 512 up to 8192 columns, got %lld", (long long)cols);
        int ni = 1 + n_mat;
        const size_t vec = (size_t)cols * 4, mat = (size_t)batch * cols * 4;
        auto add_in = [&](size_t bytes) { k.in_bytes[ni] = bytes; k.in_align[ni] = 16; ni++; };
        if (prologue == 1) add_in(vec);
        if (prologue == 2) { add_in(vec); add_in(mat); add_in(vec); k.out_bytes[n_mat] = mat; k.out_align[n_mat] = 16; k.info.n_outputs = n_mat + 1; }
        if (prologue == 3 && !x_slices) add_in(mat);
        k.info.n_inputs = ni;
        if (x_slices) k.in_bytes[1] = (size_t)x_slices * mat * (prologue == 3 ? 2 : 1);
    }
    // f16 copy of X plus the min-term operand (32 halves per token and superblock)
    k.scratch_bytes = ((size_t)((batch + 31) / 32 * 32) * cols * 2 + (size_t)batch * (cols / 256) * 64) * (f32x ? 2 : 1);
    // schedule: nr0 = weight rows per workgroup.  32 = the small-batch form (Q4_K, up to 64 tokens: the default
    // there), 128 = the 128 x 128 tile.
    const uint32_t want = k.desc.sched.nr0;
    if (want && want != 32 && want != BN) return set_error("matvec_batch: unsupported schedule nr0=%u (32 or %d)", want, BN);
    const bool can_skinny = !q6 && batch <= kSkinnyMaxBatch && n_mat == 1 && !unfolded;
    if (want == 32 && !can_skinny) return set_error("matvec_batch: the small-batch form takes Q4_K weights and up to %d tokens", kSkinnyMaxBatch);
    // (long rows of a short matrix leave the small-batch form 64 workgroups with four superblocks per wave: from 33
    // tokens on the tile over K slices is faster there -- 2048 x 8192 at 63 tokens: 27.5 us against 41.0)
    const bool long_rows = batch > 32 && rows <= 2048 && cols >= 8192;
    k.variant = (want == 32 || (want == 0 && can_skinny && !long_rows)) ? 1 : 0;
    k.info.sched = k.desc.sched;
    if (k.variant == 1) {
        set_launch(k, (uint32_t)((rows + 31) / 32), 1, 1, 512, (uint32_t)(8 * (batch <= 32 ? 1 : 2) * 16 * 64 * 4));
        k.info.sched.tg = 512; k.info.sched.nsg = 8; k.info.sched.nr0 = 32; k.info.sched.k_split = 8; k.info.sched.lds_tile = 16;
        set_name(k, "mul_mm_q4k_skinny_32xT%d%s", batch <= 32 ? 32 : 64, f32x ? "_f32x" : "");
        k.launch = launch_mul_mm;
        return 0;
    }
    // Few tiles (a prompt of a few hundred tokens, or a narrow matrix): the superblocks of a row are split into K
    // slices and, for f32 activations, the hi and the lo part become workgroups of the same launch, until the grid is
    // about one workgroup per compute unit; every slice stores its partial sums and a second launch adds them in a
    // fixed order.  sched.k_split names the slice count (a divisor of cols / 256; 1 = none).
    const int64_t row_tiles = (rows + BN - 1) / BN + (rows1 + BN - 1) / BN + (rows2 + BN - 1) / BN;
    const int64_t nsb = cols / 256;
    int64_t ks = 1;
    if (k.desc.sched.k_split) {
        ks = k.desc.sched.k_split;
        if (nsb % ks) return set_error("matvec_batch: k_split=%lld does not divide the %lld superblocks of a row", (long long)ks, (long long)nsb);
    } else {
        // (a slice of one superblock is all prologue; the workgroups are counted with the token tile they will have)
        auto workgroups = [&](int64_t s) { const int64_t tm_s = mm_tile_tokens(k.desc, s); return ((batch + tm_s - 1) / tm_s) * row_tiles * s; };
        while (nsb % (ks * 2) == 0 && nsb / (ks * 2) >= 2 && workgroups(ks * 2) <= 256) ks *= 2;
    }
    const bool z_form = unfolded || ks > 1;
    k.variant = z_form ? (int)(ks << 1) : 0;
    if (z_form && !unfolded) k.scratch_bytes += (size_t)ks * batch * rows_all * 4;
    if (unfolded) {
        const int keep = prologue == 2 ? 1 : 0;                       // (the add-then-norm prologue's x_new stays an output)
        if (keep) { k.out_bytes[1] = k.out_bytes[n_mat]; k.out_align[1] = 16; }
        k.out_bytes[0] = (size_t)ks * batch * rows_all * 4; k.out_align[0] = 16;
        k.info.n_outputs = 1 + keep;
    }
    const int tm = mm_tile_tokens(k.desc, ks);
    set_launch(k, (uint32_t)((batch + tm - 1) / tm), (uint32_t)row_tiles, z_form ? (uint32_t)ks : 1, kThreadsMM,
               (uint32_t)(tm == 64 ? kLdsBytes64 : kLdsBytes));
    k.info.sched.tg = kThreadsMM; k.info.sched.nsg = kThreadsMM / 64; k.info.sched.nr0 = BN; k.info.sched.k_split = (uint32_t)ks; k.info.sched.lds_tile = KS;
    set_name(k, "mul_mm_%s_%dx%dx%d%s%s%s%s", q6 ? "q6k" : "q4k", BM, BN, KS, f32x ? "_f32x" : "", z_form ? "_kz" : "", n_mat == 3 ? "_x3" : n_mat == 2 ? "_x2" : "",
             prologue == 1 ? "_rms" : prologue == 2 ? "_addrms" : prologue == 3 ? "_gelu" : "");
    if (unfolded) { char nm[64]; snprintf(nm, sizeof(nm), "%s", k.info.name); set_name(k, "%s_unfolded", nm); }
    k.launch = launch_mul_mm;
    return 0;
}

int bind_round_prep(ksh_kernel &k)
{
    const int64_t cols = k.desc.dims[0], batch = k.desc.dims[1], mode = k.desc.dims[2];
    if (cols <= 0 || cols % 256 || cols > (1 << 16)) return set_error("round_prep: cols=%lld is not a positive multiple of 256 up to 65536", (long long)cols);
    if (batch < 1 || batch > kRoundTokens) return set_error("round_prep: %lld rows (1 to %d)", (long long)batch, kRoundTokens);
    if (mode < 0 || mode > 3) return set_error("round_prep: mode %lld (0 plain, 1 rmsnorm, 2 add then rmsnorm, 3 rmsnorm add)", (long long)mode);
    if (mode >= 2 && cols > 8192) return set_error("round_prep: the add-then-norm form keeps a row in LDS (cols=%lld, up to 8192)", (long long)cols);
    const int64_t slices = std::max<int64_t>(1, k.desc.dims[3]);
    if (k.desc.dims[3] < 0 || slices > 64 || (slices > 1 && (!mode || cols > 2048)))
        return set_error("round_prep: an input in %lld column slices takes a norm (mode 1 to 3) and rows of up to 2048 columns", (long long)k.desc.dims[3]);
    k.info.n_inputs = mode == 2 ? 4 : mode == 3 ? 3 : mode == 1 ? 2 : 1;
    k.info.n_outputs = mode >= 2 ? 2 : 1;
    k.in_bytes[0] = (size_t)slices * batch * cols * 4; k.in_align[0] = 16;
    // (128-bit loads and stores of every operand)
    if (mode) { k.in_bytes[1] = (size_t)cols * 4; k.in_align[1] = 16; }
    if (mode >= 2) {
        k.in_bytes[2] = (size_t)batch * cols * 4; k.in_align[2] = 16;
        if (mode == 2) { k.in_bytes[3] = (size_t)cols * 4; k.in_align[3] = 16; }
        k.out_bytes[1] = (size_t)batch * cols * 4; k.out_align[1] = 16;
    }
    k.out_bytes[0] = (round_xf_halves((int)cols) + 2 * round_sx_halves((int)cols)) * 2; k.out_align[0] = 16;
    if (mode) set_launch(k, kRoundTokens, 1, 1, 256, mode >= 2 ? (uint32_t)cols * 4 : 0);
    else set_launch(k, (uint32_t)((kRoundTokens * (cols / 8) + 255) / 256), 1, 1, 256, 0);
    set_name(k, mode == 3 ? "round_prep_rmsnorm_add" : mode == 2 ? "round_prep_add_then_rmsnorm" : mode == 1 ? "round_prep_rmsnorm" : "round_prep_f32x");
    k.launch = launch_round_prep;
    return 0;
}

int bind_matvec_round(ksh_kernel &k)
{
    const int64_t *d = k.desc.dims;
    const int64_t rows0 = d[0], cols = d[1], batch = d[2], rows1 = d[3], rows2 = d[4];
    const bool pair = d[5] != 0;
    const bool q6r = k.desc.dtypes[0] == KSH_Q6K_ROWS;
    if (k.desc.dtypes[0] != KSH_Q4K && !q6r) return set_error("matvec_round: weight dtype %d is not built (Q4_K and row-grouped Q6_K are)", k.desc.dtypes[0]);
    if (cols <= 0 || cols % 256 || cols > (1 << 16)) return set_error("matvec_round: cols=%lld is not a positive multiple of 256 up to 65536", (long long)cols);
    if (batch < 1 || batch > kRoundTokens) return set_error("matvec_round: %lld rows (1 to %d)", (long long)batch, kRoundTokens);
    if (q6r) {
        if (rows1 || rows2 || pair) return set_error("matvec_round: row-grouped Q6_K takes one matrix per launch");
        if (cols > 2048) return set_error("matvec_round: row-grouped Q6_K rows of up to 2048 columns (cols=%lld)", (long long)cols);
        if (rows0 <= 0 || rows0 > (1 << 24)) return set_error("matvec_round: rows %lld", (long long)rows0);
        k.info.n_inputs = 2;
        k.info.n_outputs = 1;
        k.in_bytes[0] = (size_t)rows0 * round_q6r_row_bytes((int)(cols / 256)); k.in_align[0] = 16;
        k.in_bytes[1] = (round_xf_halves((int)cols) + 2 * round_sx_halves((int)cols)) * 2; k.in_align[1] = 16;
        k.out_bytes[0] = (size_t)batch * rows0 * 4; k.out_align[0] = 4;
        // one workgroup per compute unit (its registers hold the activations of a whole row), tiles shared out evenly
        const int64_t tiles = (rows0 + 31) / 32, per = (tiles + 255) / 256;
        set_launch(k, (uint32_t)((tiles + per - 1) / per), 1, 1, 512, (uint32_t)(2 * 8 * 8 * 64 * 4));
        k.info.sched = k.desc.sched;
        k.info.sched.tg = 512; k.info.sched.nsg = 8; k.info.sched.nr0 = 32; k.info.sched.k_split = 1; k.info.sched.lds_tile = 16;
        set_name(k, "matvec_round_q6krows");
        k.launch = launch_matvec_round;
        return 0;
    }
    if (rows0 <= 0 || rows1 < 0 || rows2 < 0 || (rows2 && !rows1) || rows0 + rows1 + rows2 > (1 << 24))
        return set_error("matvec_round: rows %lld / %lld / %lld", (long long)rows0, (long long)rows1, (long long)rows2);
    if (pair && (rows1 || rows2)) return set_error("matvec_round: a gate | up pair names one row count (both matrices have it)");
    const int slices = (int)((cols / 256 + 7) / 8);
    if (slices > 1 && (pair || rows1)) return set_error("matvec_round: rows longer than 2048 columns take one matrix per launch");
    const bool emit = d[6] == 1, unfolded = d[6] == 2;
    if (d[6] < 0 || d[6] > 2) return set_error("matvec_round: result form %lld (0 rows, 1 prepared operand, 2 the column slices' partial sums)", (long long)d[6]);
    const int64_t mul_stride = d[7];
    if (mul_stride && (pair || rows1 || mul_stride < rows0)) return set_error("matvec_round: the gate multiplier takes one matrix and a row stride of at least its rows");
    if (emit && (rows1 || slices > 1 || rows0 % 256))
        return set_error("matvec_round: the result as a prepared operand takes one matrix (or a pair) of up to 2048 columns whose rows are a multiple of 256");
    const int n_mat = pair ? 2 : rows2 ? 3 : rows1 ? 2 : 1;
    const int64_t rows[3] = {rows0, pair ? rows0 : rows1, rows2};
    k.info.n_inputs = 1 + n_mat;
    k.info.n_outputs = pair ? 1 : n_mat;
    k.in_bytes[0] = (size_t)rows0 * (cols / 256) * 144; k.in_align[0] = 16;
    k.in_bytes[1] = (round_xf_halves((int)cols) + 2 * round_sx_halves((int)cols)) * 2; k.in_align[1] = 16;
    for (int i = 1; i < n_mat; i++) { k.in_bytes[1 + i] = (size_t)rows[i] * (cols / 256) * 144; k.in_align[1 + i] = 16; }
    if (mul_stride) { k.info.n_inputs = 3; k.in_bytes[2] = ((size_t)(batch - 1) * mul_stride + rows0) * 4; k.in_align[2] = 4; }
    for (int i = 0; i < k.info.n_outputs; i++) { k.out_bytes[i] = (size_t)batch * rows[i] * 4; k.out_align[i] = 4; }
    if (emit) { k.out_bytes[0] = (round_xf_halves((int)rows0) + 2 * round_sx_halves((int)rows0)) * 2; k.out_align[0] = 16; }
    if (unfolded && (rows1 || pair)) return set_error("matvec_round: partial sums as the result take one matrix");
    k.scratch_bytes = slices > 1 && !unfolded ? (size_t)slices * batch * rows0 * 4 : 0;
    if (unfolded) k.out_bytes[0] = (size_t)slices * batch * rows0 * 4;
    const int64_t tiles = pair ? (rows0 + 31) / 32 : (rows0 + 31) / 32 + (rows1 + 31) / 32 + (rows2 + 31) / 32;
    set_launch(k, (uint32_t)tiles, (uint32_t)slices, 1, 512, (uint32_t)(8 * (pair ? 2 : 1) * 8 * 64 * 4 + (emit ? 16 * 33 * 4 : 0)));
    k.info.sched = k.desc.sched;
    k.info.sched.tg = 512; k.info.sched.nsg = 8; k.info.sched.nr0 = 32; k.info.sched.k_split = (uint32_t)slices; k.info.sched.lds_tile = 16;
    set_name(k, "matvec_round_q4k_%s%s%s", pair ? "gate_up_gelu" : mul_stride ? "gelu_mul" : n_mat == 3 ? "x3" : n_mat == 2 ? "x2" : "x1",
             slices > 1 ? "_ksplit" : "", emit ? "_prepared" : "");
    k.launch = launch_matvec_round;
    return 0;
}

// schedules of the prefill GEMM: the 128 x 128 tile with K depth 64 (LDS-staged, one K range per workgroup) and, for
// Q4_K weights and up to 64 tokens, 32 weight rows per workgroup with the K range split over its 8 waves
int mul_mm_candidates(const ksh_kernel_desc &d, ksh_sched *out, int cap)
{
    int n = 0;
    if (n < cap) {
        ksh_sched s{};
        s.tg = kThreadsMM; s.nsg = kThreadsMM / 64; s.nr0 = BN; s.lds_tile = KS; s.unroll = 1; s.vec = 0; s.k_split = 1;
        out[n++] = s;
    }
    if (n < cap && d.dtypes[0] == KSH_Q4K && d.dims[2] <= kSkinnyMaxBatch && !d.dims[3]) {
        ksh_sched s{};
        s.tg = 512; s.nsg = 8; s.nr0 = 32; s.lds_tile = 16; s.unroll = 1; s.vec = 0; s.k_split = 8;
        out[n++] = s;
    }
    // the 128 x 128 tile over K slices, where whole rows leave the grid short of one workgroup per compute unit
    const int64_t tiles = ((d.dims[2] + BM - 1) / BM) * ((d.dims[0] + BN - 1) / BN + (d.dims[3] + BN - 1) / BN + (d.dims[4] + BN - 1) / BN) * (d.dtypes[1] == KSH_F32 ? 2 : 1),
                  nsb = d.dims[1] / 256;
    for (uint32_t ks : {2u, 4u, 8u, 16u}) {
        if (n >= cap || nsb % ks || tiles * (ks / 2) >= 256) continue;
        ksh_sched s{};
        s.tg = kThreadsMM; s.nsg = kThreadsMM / 64; s.nr0 = BN; s.lds_tile = KS; s.unroll = 1; s.vec = 0; s.k_split = ks;
        out[n++] = s;
    }
    return n;
}

}  // namespace ksh
