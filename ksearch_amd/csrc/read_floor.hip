// Memory-only floors of the Q4_K GEMV (KSH_READ_FLOOR): launches of the same grid, workgroup size and LDS
// reservation as the 4096 x 4096 default schedule (2 rows per wave, 8 waves per workgroup) that do nothing, or only
// read the matrix.  They give a single launch of that size its lower bound on this part: what is left when all
// arithmetic, the activation vector and the reduction are taken away.  Measurement aid; no counterpart in the
// reference.
#include "ksh_device.hpp"
#include "ksh_internal.hpp"

namespace ksh {
namespace {

constexpr int kR = 2, kNW = 8, kBlk = 144;

// mode 0: nothing.  mode 1: every lane issues the GEMV's loads (a superblock is owned by 4 lanes: 16-byte header +
// the lane's 32 quant bytes, 2 rows per wave, all loads up front).  mode 2: the same bytes as flat 128-bit loads,
// lane after lane.
template <int MODE>
__global__ __launch_bounds__(kNW * 64) void read_floor_kernel(const uint8_t *__restrict__ W, int rows, int bpr, float *sink)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];
    if (MODE == 0) {
        if (threadIdx.x == 0xFFFF) sink[0] = (float)xs[0];
        return;
    }
    uint32_t acc = 0;
    if (MODE == 1) {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane & 3, bl = lane >> 2;
        const size_t row_bytes = (size_t)bpr * kBlk;
        const int row0 = (blockIdx.x * kNW + wave) * kR;
        uint4 v[kR][3];
#pragma unroll
        for (int r = 0; r < kR; r++) {
            const uint8_t *blk = W + (size_t)min(row0 + r, rows - 1) * row_bytes + (size_t)min(bl, bpr - 1) * kBlk;
            v[r][0] = ldg_u4(blk, 0);
            v[r][1] = ldg_u4(blk, 1 + 2 * g);
            v[r][2] = ldg_u4(blk, 2 + 2 * g);
        }
#pragma unroll
        for (int r = 0; r < kR; r++)
#pragma unroll
            for (int i = 0; i < 3; i++) acc ^= v[r][i].x ^ v[r][i].y ^ v[r][i].z ^ v[r][i].w;
    } else {
        // rows * bpr * 9 vectors of 16 bytes over gridDim * 512 threads: 4096 x 4096 gives 4.5 per thread
        const size_t n16 = (size_t)rows * bpr * 9, nthr = (size_t)gridDim.x * blockDim.x;
        const size_t i0 = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
        uint4 v[5];
#pragma unroll
        for (int u = 0; u < 5; u++) v[u] = ldg_u4(W, min(i0 + u * nthr, n16 - 1));
#pragma unroll
        for (int u = 0; u < 5; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x12345678u) sink[0] = 1.0f;      // keeps the loads alive; random weights never take this branch
}

// the empty launch again with an argument block of the GEMV's size (19 pointers and integers: 136 bytes)
struct PaddedArgs {
    const uint8_t *p[9];
    float *sink;
    int v[14];
};
__global__ __launch_bounds__(kNW * 64) void read_floor_empty_args_kernel(PaddedArgs a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];
    if (threadIdx.x == 0xFFFF) a.sink[0] = (float)xs[0] + (float)a.v[13];
}

int launch_read_floor(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const int rows = (int)k.desc.dims[0], bpr = (int)(k.desc.dims[1] / 256), mode = (int)k.desc.dims[2];
    const dim3 grid(k.info.grid[0]), block(k.info.block[0]);
    const size_t lds = k.info.lds_bytes;
    const uint8_t *W = (const uint8_t *)a.in[0];
    float *sink = (float *)a.out[0];
    if (mode == 0 && k.desc.dims[6]) {
        PaddedArgs pa{};
        pa.p[0] = W; pa.sink = sink; pa.v[0] = rows; pa.v[1] = bpr;
        hipLaunchKernelGGL(read_floor_empty_args_kernel, grid, block, lds, st, pa);
    } else if (mode == 0) hipLaunchKernelGGL(read_floor_kernel<0>, grid, block, lds, st, W, rows, bpr, sink);
    else if (mode == 1) hipLaunchKernelGGL(read_floor_kernel<1>, grid, block, lds, st, W, rows, bpr, sink);
    else hipLaunchKernelGGL(read_floor_kernel<2>, grid, block, lds, st, W, rows, bpr, sink);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "read_floor launch");
}

}  // namespace

int bind_read_floor(ksh_kernel &k)
{
    const int64_t rows = k.desc.dims[0], cols = k.desc.dims[1], mode = k.desc.dims[2];
    if (k.desc.dtypes[0] != KSH_Q4K) return set_error("read_floor: only Q4_K matrices (dtype %d)", k.desc.dtypes[0]);
    if (rows <= 0 || rows > (1 << 20) || cols <= 0 || cols % 256 || cols > 4096)
        return set_error("read_floor: rows=%lld cols=%lld (cols: a multiple of 256 up to 4096)", (long long)rows, (long long)cols);
    if (mode < 0 || mode > 2) return set_error("read_floor: mode %lld (0 empty, 1 GEMV lane pattern, 2 flat loads)", (long long)mode);
    // the flat form reads five vectors per thread: enough for rows of 4096 columns, clamped beyond the end
    k.info.n_inputs = 1;
    k.info.n_outputs = 1;
    k.in_bytes[0] = (size_t)rows * (cols / 256) * kBlk; k.in_align[0] = 16;
    k.out_bytes[0] = 4; k.out_align[0] = 4;
    uint32_t grid = (uint32_t)((rows + kR * kNW - 1) / (kR * kNW)), threads = kNW * 64;
    // LDS as the GEMV's int8 digit-plane image of the vector: 208 bytes per 64 columns + 16 per group + 128
    uint32_t lds = (uint32_t)((cols / 64) * 224 + 128);
    // the empty launch in other shapes: dims[3] workgroups, dims[4] threads per workgroup (a multiple of 64 up to 512),
    // dims[5] = 1 without the LDS reservation, dims[6] = 1 with an argument block of the GEMV's size
    if (mode == 0) {
        const int64_t g = k.desc.dims[3], t = k.desc.dims[4];
        if (g < 0 || g > (1 << 20) || t < 0 || t > kNW * 64 || t % 64) return set_error("read_floor: %lld workgroups of %lld threads", (long long)g, (long long)t);
        if (g) grid = (uint32_t)g;
        if (t) threads = (uint32_t)t;
        if (k.desc.dims[5]) lds = 0;
    } else if (k.desc.dims[3] || k.desc.dims[4] || k.desc.dims[5] || k.desc.dims[6]) {
        return set_error("read_floor: the launch shape is a parameter of the empty launch (mode 0) only");
    }
    set_launch(k, grid, 1, 1, threads, lds);
    set_name(k, "read_floor_q4k_%s", mode == 0 ? "empty" : mode == 1 ? "lanes" : "flat");
    k.launch = launch_read_floor;
    return 0;
}

}  // namespace ksh
