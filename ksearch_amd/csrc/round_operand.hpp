// The prepared GEMM operand of a decode round (up to 16 rows; KSH_ROUND_PREP writes it, KSH_MATVEC_ROUND reads it), for
// the kernels that write it as their own result: the fragments of the 32 x 32 x 16 matrix instruction with
// x = hi + 2^-11 lo in one tile (rows 0..15 the tokens' hi parts, rows 16..31 their lo parts), and the sums of x per
// sub-block of 32 columns, hi and lo.
//   fragments  [cols / 16][64 lanes][8 halves], lane = row + 32 * ((k / 8) % 2), position kperm(i) holds k = 8 * (..) + i
//   sums       [2 parts][16 rows][cols / 256][32 halves] = hi[8] hi[8] lo[8] 0[8] of the superblock's eight sub-blocks
#pragma once
#include "ksh_device.hpp"

namespace ksh {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));

// within every 4 consecutive k the stored order is (0, 2, 1, 3): that is the
// order the paired nibble extraction produces, applied to X as well
__device__ __forceinline__ int kperm(int i) { return (i & ~3) | ((i & 1) << 1) | ((i >> 1) & 1); }

constexpr int kRoundTokens = 16;

__host__ __device__ inline size_t round_xf_halves(int cols) { return (size_t)32 * cols; }
__host__ __device__ inline size_t round_sx_halves(int cols) { return (size_t)kRoundTokens * (cols / 256) * 32; }

// 8 consecutive values as the hi and lo halves of a fragment lane, and the sums of the two parts
__device__ __forceinline__ void round_split8(const float (&f)[8], h8 &oh, h8 &ol, float &sh, float &sl)
{
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
    sh = ((fh[0] + fh[1]) + (fh[2] + fh[3])) + ((fh[4] + fh[5]) + (fh[6] + fh[7]));
    sl = ((fl[0] + fl[1]) + (fl[2] + fl[3])) + ((fl[4] + fl[5]) + (fl[6] + fl[7]));
}

// the sums of a sub-block's hi and lo parts as the bias / min product reads them: hi[8] hi[8] lo[8] 0[8] per row and
// superblock, entry jj of each
__device__ __forceinline__ void round_store_sums(_Float16 *__restrict__ Xp, int cols, int t, int sub_block, float sh, float sl)
{
    const int jj = sub_block % 8;
    _Float16 *sx = Xp + round_xf_halves(cols) + ((size_t)t * (cols / 256) + sub_block / 8) * 32;
    const float sums[2] = {sh, sl};
#pragma unroll
    for (int part = 0; part < 2; part++) {
        _Float16 *dst = sx + part * round_sx_halves(cols);
        const float sum = pinned(sums[part]);
        const _Float16 hi = (_Float16)sum;
        const _Float16 lo = (_Float16)(sum - (float)hi);
        dst[jj] = hi;
        dst[8 + jj] = hi;
        dst[16 + jj] = lo;
        dst[24 + jj] = (_Float16)0.f;
    }
}

}  // namespace
}  // namespace ksh
