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
//   - a wave sweeps 8 superblocks (2048 columns) per step and keeps the 32
//     matching activations per lane in registers across every row it owns, so
//     x comes out of LDS once per wave, not once per row;
//   - the 6-bit values are assembled four at a time with dword logic, turned
//     into floats with the byte converts, and the -32 offset is applied
//     through per-16 sums of x:  y += d * sum_k sc_k * (sum(v*x) - 32*Sx_k);
//   - a workgroup walks a long run of rows (x staged in LDS once), issuing the
//     loads of the next R rows before it consumes the current ones.
//
// The result differs from dequant-then-dot (gguf_impl.rs:761-791 +
// check_mul_mm.rs:60-71) by reassociation only.
#include "ksh_device.hpp"
#include "ksh_internal.hpp"

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
    r.d = (uint32_t)blk[208] | ((uint32_t)blk[209] << 8);
    return r;
}

__device__ __forceinline__ float dot4_bytes(uint32_t a, const float *x, float acc)
{
    acc = fmaf(ubyte_f32<0>(a), x[0], acc);
    acc = fmaf(ubyte_f32<1>(a), x[1], acc);
    acc = fmaf(ubyte_f32<2>(a), x[2], acc);
    acc = fmaf(ubyte_f32<3>(a), x[3], acc);
    return acc;
}

// xr: x[l0..l0+7], x[32+l0..], x[64+l0..], x[96+l0..] of the lane's half (32 floats)
// sx[k]: sum of xr[8k..8k+7]
__device__ __forceinline__ float q6k_lane_dot(const Q6kLane &L, int il, const float *xr, const float *sx)
{
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    const uint32_t q1[2] = {L.q1.x, L.q1.y}, q2[2] = {L.q2.x, L.q2.y}, qh[2] = {L.qh.x, L.qh.y};
#pragma unroll
    for (int w = 0; w < 2; w++) {
        const uint32_t a1 = (q1[w] & 0x0F0F0F0Fu) | ((qh[w] << 4) & 0x30303030u);
        const uint32_t a2 = (q2[w] & 0x0F0F0F0Fu) | ((qh[w] << 2) & 0x30303030u);
        const uint32_t a3 = ((q1[w] >> 4) & 0x0F0F0F0Fu) | (qh[w] & 0x30303030u);
        const uint32_t a4 = ((q2[w] >> 4) & 0x0F0F0F0Fu) | ((qh[w] >> 2) & 0x30303030u);
        s0 = dot4_bytes(a1, xr + 4 * w, s0);
        s1 = dot4_bytes(a2, xr + 8 + 4 * w, s1);
        s2 = dot4_bytes(a3, xr + 16 + 4 * w, s2);
        s3 = dot4_bytes(a4, xr + 24 + 4 * w, s3);
    }
    // the lane's 8 positions share is = l0/16 = il/2; scales sc[is + 2k]
    const uint32_t scw = (il & 2) ? ((L.sc.x >> 8) | (L.sc.y << 24)) : L.sc.x;   // bytes is, is+1, is+2, is+3 .. need is+{0,2,4,6}
    const uint32_t sch = (il & 2) ? (L.sc.y >> 8) : L.sc.y;
    const float c0 = (float)(int8_t)(scw & 0xFF);
    const float c1 = (float)(int8_t)((scw >> 16) & 0xFF);
    const float c2 = (float)(int8_t)(sch & 0xFF);
    const float c3 = (float)(int8_t)((sch >> 16) & 0xFF);
    s0 = fmaf(-32.f, sx[0], s0);
    s1 = fmaf(-32.f, sx[1], s1);
    s2 = fmaf(-32.f, sx[2], s2);
    s3 = fmaf(-32.f, sx[3], s3);
    const float t = fmaf(c0, s0, c1 * s1) + fmaf(c2, s2, c3 * s3);
    return half_bits_to_f32(L.d) * t;
}

__device__ __forceinline__ int xs6_index(int e) { return e + ((e >> 7) << 2); }
__host__ __device__ constexpr int xs6_floats(int cols) { return cols + (cols >> 7) * 4; }

struct Q6kParams {
    const uint8_t *W;
    const float *x;
    float *y;
    int rows, bpr, rows_per_wave;
};

// One step == 8 superblocks.  STEPS = ceil(bpr / 8); lanes whose superblock lies
// past the row's end re-read the last one against zeroed activations.
template <int R, int NW, int STEPS>
__global__ __launch_bounds__(NW * 64) void q6k_gemv_kernel(Q6kParams p)
{
    extern __shared__ float xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bl = lane >> 3, ip = (lane >> 2) & 1, il = lane & 3;
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
    if (w0 < w1) load_rows(cur, w0);

    {
        const float4 *x4 = reinterpret_cast<const float4 *>(p.x);
        for (int i = tid; i < p.bpr * 64; i += NW * 64) {
            const float4 v = x4[i];
            *reinterpret_cast<float4 *>(&xs[xs6_index(i * 4)]) = v;
        }
    }
    __syncthreads();
    if (w0 >= w1) return;

    float xr[STEPS][32], sx[STEPS][4];
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
        const bool valid = s * 8 + bl < p.bpr;
        const int e0 = min(s * 8 + bl, p.bpr - 1) * 256 + 128 * ip + 8 * il;
        const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const float *src = &xs[xs6_index(e0 + 32 * k)];
            const float4 a = valid ? *reinterpret_cast<const float4 *>(src) : zero;
            const float4 b = valid ? *reinterpret_cast<const float4 *>(src + 4) : zero;
            float *d = &xr[s][8 * k];
            d[0] = a.x; d[1] = a.y; d[2] = a.z; d[3] = a.w;
            d[4] = b.x; d[5] = b.y; d[6] = b.z; d[7] = b.w;
            sx[s][k] = ((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w));
        }
    }

    for (int row0 = w0; row0 < w1; row0 += R) {
        const bool more = row0 + R < w1;
        if (more) load_rows(nxt, row0 + R);
#pragma unroll
        for (int r = 0; r < R; r++) {
            float acc = 0.f;
#pragma unroll
            for (int s = 0; s < STEPS; s++) acc += q6k_lane_dot(cur[s][r], il, xr[s], sx[s]);
            acc = wave_sum(acc);
            if (lane == 0 && row0 + r < w1) p.y[row0 + r] = acc;
        }
        if (more) {
#pragma unroll
            for (int s = 0; s < STEPS; s++)
#pragma unroll
                for (int r = 0; r < R; r++) cur[s][r] = nxt[s][r];
        }
    }
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
    int rpw = s.unroll ? (int)s.unroll * G.R : 32;
    while (rpw > G.R && rows / (rpw * G.NW) < 2048) rpw >>= 1;
    if (rpw < G.R) rpw = G.R;
    G.rpw = rpw;
    return G;
}

template <int R, int NW>
int launch_steps(int steps, const Q6kParams &p, unsigned grid, size_t lds, hipStream_t st)
{
    switch (steps) {
    case 1: hipLaunchKernelGGL((q6k_gemv_kernel<R, NW, 1>), dim3(grid), dim3(NW * 64), lds, st, p); break;
    case 2: hipLaunchKernelGGL((q6k_gemv_kernel<R, NW, 2>), dim3(grid), dim3(NW * 64), lds, st, p); break;
    case 3: hipLaunchKernelGGL((q6k_gemv_kernel<R, NW, 3>), dim3(grid), dim3(NW * 64), lds, st, p); break;
    case 4: hipLaunchKernelGGL((q6k_gemv_kernel<R, NW, 4>), dim3(grid), dim3(NW * 64), lds, st, p); break;
    default: return set_error("matvec_q6k: cols=%d is not built (up to 8192 are)", p.bpr * 256);
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "q6k_gemv launch");
}

int launch_matvec_q6k(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    Q6kParams p;
    p.W = (const uint8_t *)a.in[0];
    p.x = (const float *)a.in[1];
    p.y = (float *)a.out[0];
    p.rows = (int)k.desc.dims[0];
    p.bpr = (int)(k.desc.dims[1] / 256);
    const int R = k.variant & 0xFF, NW = (k.variant >> 8) & 0xFF;
    p.rows_per_wave = k.variant >> 16;
    const unsigned grid = k.info.grid[0];
    const size_t lds = k.info.lds_bytes;
    const int steps = (p.bpr + 7) / 8;
#define KSH_CASE(r, w) \
    if (R == r && NW == w) return launch_steps<r, w>(steps, p, grid, lds, st);
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
    if (k.desc.kind != KSH_MATVEC) return set_error("rmsnorm_matvec: Q6_K weights are not built for this kind");
    if (rows <= 0 || rows > (1 << 30)) return set_error("matvec: rows=%lld", (long long)rows);
    if (cols <= 0 || cols % 256 || cols > 8192)
        return set_error("matvec_q6k: cols=%lld is not a positive multiple of 256 up to 8192", (long long)cols);
    Q6kGeom G = pick_geom6(k.desc.sched, (int)rows);
    if (cols > 4096 && G.R > 2) { G.rpw = G.rpw / G.R * 2; G.R = 2; }   // keeps the double buffer in registers
    if (!((G.R == 1 || G.R == 2 || G.R == 4) && (G.NW == 2 || G.NW == 4 || G.NW == 8)) || G.rpw % G.R || G.rpw > 32767)
        return set_error("matvec_q6k: unsupported schedule nr0=%d nsg=%d unroll=%u", G.R, G.NW, k.desc.sched.unroll);
    const int bpr = (int)(cols / 256);
    k.info.n_inputs = 2;
    k.info.n_outputs = 1;
    k.in_bytes[0] = (size_t)rows * bpr * kQ6kBytes;
    k.in_bytes[1] = (size_t)cols * 4;
    k.out_bytes[0] = (size_t)rows * 4;
    k.in_align[0] = 2; k.in_align[1] = 16; k.out_align[0] = 4;
    const int rows_per_wg = G.rpw * G.NW;
    set_launch(k, (uint32_t)((rows + rows_per_wg - 1) / rows_per_wg), 1, 1, (uint32_t)G.NW * 64,
               (uint32_t)(xs6_floats((int)cols) * sizeof(float)));
    k.info.sched = k.desc.sched;
    k.info.sched.tg = (uint64_t)G.NW * 64;
    k.info.sched.nsg = (uint32_t)G.NW;
    k.info.sched.nr0 = (uint32_t)G.R;
    k.info.sched.unroll = (uint32_t)(G.rpw / G.R);
    k.info.sched.vec = 0;
    k.info.sched.k_split = 1;
    set_name(k, "matvec_q6k_r%d_w%d_u%d", G.R, G.NW, G.rpw / G.R);
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
                s.tg = 64ull * nsg; s.vec = 0; s.unroll = unroll; s.nsg = nsg; s.nr0 = nr0; s.k_split = 1;
                out[n++] = s;
            }
    return n;
}

}  // namespace ksh
