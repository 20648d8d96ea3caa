// Q4_K packed-weight GEMV family for gfx950: y = W x, the fused QKV triple and
// the fused gate||up + GELU.
//
// Takes the place of lower_matvec_q4k_coop / lower_matvec_qkv_q4k_coop /
// lower_matvec_gate_up_q4k_coop (crates/ksearch_codegen/src/lower.rs:1763-2082,
// 3343-3462, 2673-2968) and the ksearch_q4k_coop_frag_nr4* bodies
// (crates/ksearch_codegen/src/render.rs:459-607).  Those are 32-lane maps with
// 8 lanes per superblock and 2-byte loads; this one is laid out for wave64 and
// 128-bit loads:
//
//   - a superblock (144 B = 9 x 16 B) is owned by 4 lanes; lane g of the four
//     takes the 64-element group g: its 32 quant bytes (two dwordx4) plus the
//     16-byte header (broadcast across the four lanes by the memory system);
//   - a wave therefore sweeps 16 superblocks (4096 columns) per step, and keeps
//     the matching 64 activations per lane in registers across R rows, so x is
//     read once per R rows;
//   - x is staged once per workgroup in LDS (stride-padded so that the
//     256-byte lane stride is bank-conflict free);
//   - every row's loads are issued before the first use, so one workgroup
//     keeps R * 192 B per lane in flight;
//   - the 6-bit scales/mins are unpacked in registers, the mins are applied
//     through per-sub-block sums of x, and rows are reduced with DPP.
//
// Arithmetic per (row, superblock, group), all f32:
//   acc += d*sc_lo * sum(n_lo*x) + d*sc_hi * sum(n_hi*x) - dmin*(m_lo*Sx_lo + m_hi*Sx_hi)
// which is the reference's coop form (render.rs:506-511) and differs from the
// CPU dequant-then-dot (gguf_impl.rs:690-721 + check_mul_mm.rs:60-71) by
// reassociation only.
#include "ksh_device.hpp"
#include "ksh_internal.hpp"

namespace ksh {
namespace {

constexpr int kQ4kBytes = 144;

// LDS layout of x: 4 floats of padding after every 64, so lanes that are 64
// floats apart land 68 dwords apart and eight consecutive lanes cover all 32
// banks with their 16-byte reads.
__device__ __forceinline__ int xs_index(int e) { return e + ((e >> 6) << 2); }
__host__ __device__ constexpr int xs_floats(int cols) { return cols + (cols >> 6) * 4; }

struct Q4kLane {
    uint4 hdr;   // d | dmin<<16, then the 12 scale bytes
    uint4 qa;    // quant bytes 0..15 of the lane's group
    uint4 qb;    // quant bytes 16..31
};

__device__ __forceinline__ Q4kLane q4k_load(const uint8_t *blk, int g)
{
    Q4kLane r;
    const uint4 *p = reinterpret_cast<const uint4 *>(blk);
    r.hdr = p[0];
    r.qa = p[1 + 2 * g];
    r.qb = p[2 + 2 * g];
    return r;
}

// VAR 0: byte->float converts (v_cvt_f32_ubyteN) feeding plain FMAs.  `lo` gets
// sum(n_lo*x[l]), `hi` gets 16*sum(n_hi*x[32+l]) (the high nibbles are left in
// place; the 1/16 is folded into the scale, exactly).
__device__ __forceinline__ void dot_dword_cvt(uint32_t w, const float *xl, const float *xh,
                                              float &lo, float &hi)
{
    const uint32_t t = w & 0x0F0F0F0Fu, u = w & 0xF0F0F0F0u;
    lo = fmaf(ubyte_f32<0>(t), xl[0], lo);
    hi = fmaf(ubyte_f32<0>(u), xh[0], hi);
    lo = fmaf(ubyte_f32<1>(t), xl[1], lo);
    hi = fmaf(ubyte_f32<1>(u), xh[1], hi);
    lo = fmaf(ubyte_f32<2>(t), xl[2], lo);
    hi = fmaf(ubyte_f32<2>(u), xh[2], hi);
    lo = fmaf(ubyte_f32<3>(t), xl[3], lo);
    hi = fmaf(ubyte_f32<3>(u), xh[3], hi);
}

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// VAR 2: nibbles are OR-ed into the mantissa of half 1024.0 (0x6400), two per
// instruction, and consumed by mixed-precision FMAs (f16 * f32 + f32, exact
// products).  `lo` gets sum((1024+n_lo)*x), `hi` gets sum((1024+16 n_hi)*x);
// the 1024*Sx terms are removed in the epilogue.
// (a & mask) | magic in one VOP3 instruction; the masks live in VGPRs and the
// magic in an SGPR because gfx950's VOP3 encoding takes no 32-bit literals
// (left to itself the compiler emits a v_and + v_or pair per use).
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic)
{
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(mask), "s"(magic));
    return r;
}

__device__ __forceinline__ void dot_dword_mix(uint32_t w, const float *xl, const float *xh,
                                              float &lo, float &hi)
{
    const uint32_t w8 = w >> 8;
    const uint32_t mlo = 0x000F000Fu, mhi = 0x00F000F0u, magic = 0x64006400u;
    const half2_t p0 = __builtin_bit_cast(half2_t, and_or(w, mlo, magic));    // bytes 0,2 low
    const half2_t p1 = __builtin_bit_cast(half2_t, and_or(w, mhi, magic));    // bytes 0,2 high
    const half2_t p2 = __builtin_bit_cast(half2_t, and_or(w8, mlo, magic));   // bytes 1,3 low
    const half2_t p3 = __builtin_bit_cast(half2_t, and_or(w8, mhi, magic));   // bytes 1,3 high
    lo = fmaf((float)p0.x, xl[0], lo);
    hi = fmaf((float)p1.x, xh[0], hi);
    lo = fmaf((float)p2.x, xl[1], lo);
    hi = fmaf((float)p3.x, xh[1], hi);
    lo = fmaf((float)p0.y, xl[2], lo);
    hi = fmaf((float)p1.y, xh[2], hi);
    lo = fmaf((float)p2.y, xl[3], lo);
    hi = fmaf((float)p3.y, xh[3], hi);
}

// one (row, superblock, group): returns the f32 contribution to y[row]
template <int VAR>
__device__ __forceinline__ float q4k_group_dot(const Q4kLane &L, int g, const float *xr, float sx_lo,
                                               float sx_hi)
{
    float lo0 = 0.f, lo1 = 0.f, hi0 = 0.f, hi1 = 0.f;
    const uint32_t q[8] = {L.qa.x, L.qa.y, L.qa.z, L.qa.w, L.qb.x, L.qb.y, L.qb.z, L.qb.w};
#pragma unroll
    for (int k = 0; k < 8; k += 2) {
        if (VAR == 2) {
            dot_dword_mix(q[k], xr + 4 * k, xr + 32 + 4 * k, lo0, hi0);
            dot_dword_mix(q[k + 1], xr + 4 * k + 4, xr + 32 + 4 * k + 4, lo1, hi1);
        } else {
            dot_dword_cvt(q[k], xr + 4 * k, xr + 32 + 4 * k, lo0, hi0);
            dot_dword_cvt(q[k + 1], xr + 4 * k + 4, xr + 32 + 4 * k + 4, lo1, hi1);
        }
    }
    float lo = lo0 + lo1, hi = hi0 + hi1;
    const float d = half_bits_to_f32(L.hdr.x & 0xFFFFu), dmin = half_bits_to_f32(L.hdr.x >> 16);
    const uint4 s = q4k_group_scales(L.hdr.y, L.hdr.z, L.hdr.w, g);
    const float sc_lo = (float)s.x, mn_lo = (float)s.y, sc_hi = (float)s.z, mn_hi = (float)s.w;
    if (VAR == 2) {
        lo = fmaf(-1024.f, sx_lo, lo);
        hi = fmaf(-1024.f, sx_hi, hi);
    }
    const float pos = fmaf(sc_lo, lo, sc_hi * 0.0625f * hi);
    const float neg = fmaf(mn_lo, sx_lo, mn_hi * sx_hi);
    return fmaf(d, pos, -(dmin * neg));
}

__device__ __forceinline__ float gelu_mul_f32(float g, float u)
{
    // lower.rs:2926-2955: clamp, tanh-GELU on the f32 accumulator, times up
    const float ax = fminf(20.0f, fmaxf(-20.0f, g));
    const float t = 0.79788456f * (ax + 0.044715f * ((ax * ax) * ax));
    return (0.5f * ax) * (1.0f + tanhf(t)) * u;
}

// One launch covers up to three weight matrices that share x.
//   mode 0: the matrices are independent row ranges (plain GEMV: one; QKV:
//           three).  Every wave owns RPW consecutive rows of ONE matrix.
//   mode 1: gate || up: every wave owns the same RPW rows of W[0] and W[1] and
//           stores gelu(W0.x) * (W1.x).
struct MatvecParams {
    const uint8_t *W[3];
    float *y[3];
    int rows[3];
    int waves[3];      // waves assigned to each matrix (mode 0)
    const float *x;
    int bpr;           // superblocks per row (cols / 256)
    int mode;
};

struct WaveTask {
    const uint8_t *W0, *W1;
    float *y;
    int row0, rows;    // first row of this wave (or half-wave), rows in its matrix
    bool active;
};

// maps a global wave index onto (matrix, first row).  rpw = rows per wave.
__device__ __forceinline__ WaveTask wave_task(const MatvecParams &p, int wv, int rpw)
{
    WaveTask t;
    int m = 0;
    if (p.mode == 0) {
        if (wv >= p.waves[0]) { wv -= p.waves[0]; m = 1; }
        if (m == 1 && wv >= p.waves[1]) { wv -= p.waves[1]; m = 2; }
    }
    t.W0 = p.W[m];
    t.W1 = p.W[1];
    t.y = p.y[m];
    t.rows = p.rows[m];
    t.row0 = wv * rpw;
    t.active = t.row0 < t.rows && (p.mode == 1 || wv < p.waves[m]);
    return t;
}

template <int NW>
__device__ __forceinline__ void stage_x(const float *x, float *xs, int n_float4, int tid)
{
    const float4 *x4 = reinterpret_cast<const float4 *>(x);
    for (int i = tid; i < n_float4; i += NW * 64) {
        const float4 v = x4[i];
        *reinterpret_cast<float4 *>(&xs[xs_index(i * 4)]) = v;
    }
}

__device__ __forceinline__ void load_x_group(const float *xs, int b, int g, float *xr, float &sx_lo,
                                             float &sx_hi)
{
    const float *xg = &xs[xs_index(b * 256 + g * 64)];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float4 v = *reinterpret_cast<const float4 *>(xg + 4 * i);
        xr[4 * i] = v.x; xr[4 * i + 1] = v.y; xr[4 * i + 2] = v.z; xr[4 * i + 3] = v.w;
    }
    float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
#pragma unroll
    for (int i = 0; i < 32; i += 2) { a0 += xr[i]; a1 += xr[i + 1]; b0 += xr[32 + i]; b1 += xr[33 + i]; }
    sx_lo = a0 + a1;
    sx_hi = b0 + b1;
}

// Full-wave form: a wave owns R rows and sweeps 16 superblocks per step.
// NM = 1 (mode 0) or 2 (mode 1).  The weight loads of step s+1 are issued
// before step s is consumed, and step 0's before x is staged, so the first
// HBM round trip overlaps the LDS fill.
template <int R, int NW, int NM, int VAR, bool MULTI>
__global__ __launch_bounds__(NW * 64) void q4k_gemv_kernel(MatvecParams p)
{
    extern __shared__ float xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane & 3, bl = lane >> 2;
    const int bpr = p.bpr;
    const size_t row_bytes = (size_t)bpr * kQ4kBytes;
    const WaveTask t = wave_task(p, blockIdx.x * NW + wave, R);

    const uint8_t *rowp[NM][R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        // rows past the end re-read the last row; their sums are never stored
        const size_t off = (size_t)min(t.row0 + r, t.rows - 1) * row_bytes;
        rowp[0][r] = t.W0 + off;
        if (NM == 2) rowp[NM - 1][r] = t.W1 + off;
    }

    // MULTI: rows longer than 16 superblocks take several steps and double-buffer
    Q4kLane cur[NM][R], nxt[MULTI ? NM : 1][MULTI ? R : 1];
    if (t.active && bl < bpr) {
#pragma unroll
        for (int m = 0; m < NM; m++)
#pragma unroll
            for (int r = 0; r < R; r++) cur[m][r] = q4k_load(rowp[m][r] + (size_t)bl * kQ4kBytes, g);
    }
    stage_x<NW>(p.x, xs, bpr * 64, tid);
    __syncthreads();
    if (!t.active) return;

    float acc[NM][R];
#pragma unroll
    for (int m = 0; m < NM; m++)
#pragma unroll
        for (int r = 0; r < R; r++) acc[m][r] = 0.f;

    for (int b = bl; b < bpr; b += 16) {
        const bool more = MULTI && b + 16 < bpr;
        if (MULTI && more) {
#pragma unroll
            for (int m = 0; m < NM; m++)
#pragma unroll
                for (int r = 0; r < R; r++) nxt[m][r] = q4k_load(rowp[m][r] + (size_t)(b + 16) * kQ4kBytes, g);
        }
        float xr[64], sx_lo, sx_hi;
        load_x_group(xs, b, g, xr, sx_lo, sx_hi);
#pragma unroll
        for (int m = 0; m < NM; m++)
#pragma unroll
            for (int r = 0; r < R; r++) acc[m][r] += q4k_group_dot<VAR>(cur[m][r], g, xr, sx_lo, sx_hi);
        if (MULTI && more) {
#pragma unroll
            for (int m = 0; m < NM; m++)
#pragma unroll
                for (int r = 0; r < R; r++) cur[m][r] = nxt[m][r];
        }
    }

#pragma unroll
    for (int r = 0; r < R; r++) {
        float s[NM];
#pragma unroll
        for (int m = 0; m < NM; m++) s[m] = wave_sum(acc[m][r]);
        const int row = t.row0 + r;
        if (lane == 0 && row < t.rows) t.y[row] = (NM == 2) ? gelu_mul_f32(s[0], s[NM - 1]) : s[0];
    }
}

// Half-wave form for rows of exactly 8 superblocks (2048 columns): lanes
// 0..31 and 32..63 work on different rows, so a wave covers 2R rows in a single
// step and no lane idles.
template <int R, int NW, int NM, int VAR>
__global__ __launch_bounds__(NW * 64) void q4k_gemv_half_kernel(MatvecParams p)
{
    extern __shared__ float xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane & 3, bl = (lane >> 2) & 7, hw = lane >> 5;
    constexpr int bpr = 8;
    constexpr size_t row_bytes = (size_t)bpr * kQ4kBytes;
    WaveTask t = wave_task(p, blockIdx.x * NW + wave, 2 * R);
    const int row0 = t.row0 + hw * R;

    Q4kLane L[NM][R];
    if (t.active) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const size_t off = (size_t)min(row0 + r, t.rows - 1) * row_bytes + (size_t)bl * kQ4kBytes;
            L[0][r] = q4k_load(t.W0 + off, g);
            if (NM == 2) L[NM - 1][r] = q4k_load(t.W1 + off, g);
        }
    }
    stage_x<NW>(p.x, xs, bpr * 64, tid);
    __syncthreads();
    if (!t.active) return;

    float xr[64], sx_lo, sx_hi;
    load_x_group(xs, bl, g, xr, sx_lo, sx_hi);

#pragma unroll
    for (int r = 0; r < R; r++) {
        float s[NM];
#pragma unroll
        for (int m = 0; m < NM; m++) {
            const float2 hs = wave_half_sums(q4k_group_dot<VAR>(L[m][r], g, xr, sx_lo, sx_hi));
            s[m] = hw ? hs.y : hs.x;
        }
        const int row = row0 + r;
        if ((lane & 31) == 0 && row < t.rows) t.y[row] = (NM == 2) ? gelu_mul_f32(s[0], s[NM - 1]) : s[0];
    }
}

struct Q4kGeom {
    int R, NW, var;
    bool half;
    int rpw() const { return R * (half ? 2 : 1); }   // rows per wave
};

int waves_for(int rows, int rpw) { return (rows + rpw - 1) / rpw; }

template <int R, int NW, int NM, int VAR>
int launch_inst(bool half, const MatvecParams &p, int total_waves, hipStream_t st)
{
    const unsigned grid = (unsigned)((total_waves + NW - 1) / NW);
    const size_t lds = (size_t)xs_floats(p.bpr * 256) * sizeof(float);
    if (half)
        hipLaunchKernelGGL((q4k_gemv_half_kernel<R, NW, NM, VAR>), dim3(grid), dim3(NW * 64), lds, st, p);
    else if (p.bpr > 16)
        hipLaunchKernelGGL((q4k_gemv_kernel<R, NW, NM, VAR, true>), dim3(grid), dim3(NW * 64), lds, st, p);
    else
        hipLaunchKernelGGL((q4k_gemv_kernel<R, NW, NM, VAR, false>), dim3(grid), dim3(NW * 64), lds, st, p);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "q4k_gemv launch");
}

template <int NM, int VAR>
int launch_rn(const Q4kGeom &G, const MatvecParams &p, int total_waves, hipStream_t st)
{
#define KSH_CASE(r, w) \
    if (G.R == r && G.NW == w) return launch_inst<r, w, NM, VAR>(G.half, p, total_waves, st);
    KSH_CASE(1, 4) KSH_CASE(2, 4) KSH_CASE(4, 4)
    KSH_CASE(1, 2) KSH_CASE(2, 2) KSH_CASE(4, 2)
    KSH_CASE(1, 8) KSH_CASE(2, 8) KSH_CASE(4, 8)
    KSH_CASE(1, 1) KSH_CASE(2, 1) KSH_CASE(4, 1)
#undef KSH_CASE
    return set_error("q4k gemv: no instance for nr0=%d nsg=%d", G.R, G.NW);
}

template <int NM>
int launch_q4k(const Q4kGeom &G, const MatvecParams &p, int total_waves, hipStream_t st)
{
    return G.var == 2 ? launch_rn<NM, 2>(G, p, total_waves, st) : launch_rn<NM, 0>(G, p, total_waves, st);
}

// default schedule: rows per wave as high as still leaves >= 2 workgroups per
// CU (x reuse vs. filling 256 CUs), 4 waves per workgroup.
Q4kGeom pick_geom(const ksh_sched &s, int total_rows, int bpr)
{
    Q4kGeom G;
    G.half = (bpr == 8);
    G.var = s.vec == 2 ? 2 : 0;
    G.NW = s.nsg ? (int)s.nsg : 4;
    if (s.nr0) {
        G.R = (int)s.nr0;
    } else {
        G.R = 4;
        while (G.R > 1 && total_rows / (G.NW * G.rpw()) < 512) G.R >>= 1;
    }
    return G;
}

bool geom_ok(const Q4kGeom &G)
{
    return (G.R == 1 || G.R == 2 || G.R == 4) && (G.NW == 1 || G.NW == 2 || G.NW == 4 || G.NW == 8);
}

void fill_info(ksh_kernel &k, const Q4kGeom &G, int total_waves, int bpr, const char *base)
{
    set_launch(k, (uint32_t)((total_waves + G.NW - 1) / G.NW), 1, 1, (uint32_t)G.NW * 64,
               (uint32_t)(xs_floats(bpr * 256) * sizeof(float)));
    k.info.sched = k.desc.sched;
    k.info.sched.tg = (uint64_t)G.NW * 64;
    k.info.sched.nsg = (uint32_t)G.NW;
    k.info.sched.nr0 = (uint32_t)G.R;
    k.info.sched.vec = (uint32_t)G.var;
    k.info.sched.unroll = 1;
    k.info.sched.k_split = 1;
    set_name(k, "%s_q4k_r%d_w%d_v%d%s", base, G.R, G.NW, G.var, G.half ? "_h" : "");
    k.variant = G.R | (G.NW << 8) | (G.var << 16) | ((int)G.half << 24);
}

Q4kGeom geom_of(const ksh_kernel &k)
{
    Q4kGeom G;
    G.R = k.variant & 0xFF;
    G.NW = (k.variant >> 8) & 0xFF;
    G.var = (k.variant >> 16) & 0xFF;
    G.half = (k.variant >> 24) & 1;
    return G;
}

int launch_matvec_q4k(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const Q4kGeom G = geom_of(k);
    MatvecParams p{};
    p.W[0] = (const uint8_t *)a.in[0];
    p.x = (const float *)a.in[1];
    p.y[0] = (float *)a.out[0];
    p.rows[0] = (int)k.desc.dims[0];
    p.waves[0] = waves_for(p.rows[0], G.rpw());
    p.bpr = (int)(k.desc.dims[1] / 256);
    return launch_q4k<1>(G, p, p.waves[0], st);
}

int launch_qkv_q4k(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const Q4kGeom G = geom_of(k);
    MatvecParams p{};
    int total = 0;
    for (int m = 0; m < 3; m++) {
        p.W[m] = (const uint8_t *)a.in[m];
        p.y[m] = (float *)a.out[m];
        p.rows[m] = (int)k.desc.dims[m == 0 ? 0 : 1];
        p.waves[m] = waves_for(p.rows[m], G.rpw());
        total += p.waves[m];
    }
    p.x = (const float *)a.in[3];
    p.bpr = (int)(k.desc.dims[2] / 256);
    return launch_q4k<1>(G, p, total, st);
}

int launch_gate_up_q4k(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const Q4kGeom G = geom_of(k);
    MatvecParams p{};
    p.W[0] = (const uint8_t *)a.in[0];
    p.W[1] = (const uint8_t *)a.in[1];
    p.x = (const float *)a.in[2];
    p.y[0] = (float *)a.out[0];
    p.rows[0] = p.rows[1] = (int)k.desc.dims[0];
    p.waves[0] = waves_for(p.rows[0], G.rpw());
    p.bpr = (int)(k.desc.dims[1] / 256);
    p.mode = 1;
    return launch_q4k<2>(G, p, p.waves[0], st);
}

int check_cols(int64_t cols)
{
    if (cols <= 0 || cols % 256)
        return set_error("Q4_K matvec: cols=%lld is not a positive multiple of 256", (long long)cols);
    if (cols > 32768)
        return set_error("Q4_K matvec: cols=%lld does not fit the LDS staging buffer", (long long)cols);
    return 0;
}

}  // namespace

int bind_matvec_q4k(ksh_kernel &k)
{
    const int64_t rows = k.desc.dims[0], cols = k.desc.dims[1];
    if (rows <= 0 || rows > (1 << 30)) return set_error("matvec: rows=%lld", (long long)rows);
    if (check_cols(cols)) return 1;
    const int bpr = (int)(cols / 256);
    const Q4kGeom G = pick_geom(k.desc.sched, (int)rows, bpr);
    if (!geom_ok(G)) return set_error("matvec_q4k: unsupported schedule nr0=%d nsg=%d", G.R, G.NW);
    k.info.n_inputs = 2;
    k.info.n_outputs = 1;
    k.in_bytes[0] = (size_t)rows * bpr * kQ4kBytes;
    k.in_bytes[1] = (size_t)cols * 4;
    k.out_bytes[0] = (size_t)rows * 4;
    k.in_align[0] = 16; k.in_align[1] = 16; k.out_align[0] = 4;
    fill_info(k, G, waves_for((int)rows, G.rpw()), bpr, "matvec");
    k.launch = launch_matvec_q4k;
    return 0;
}

int bind_matvec_qkv(ksh_kernel &k)
{
    const int64_t qr = k.desc.dims[0], kvr = k.desc.dims[1], cols = k.desc.dims[2];
    if (k.desc.dtypes[0] != KSH_Q4K) return set_error("matvec_qkv: only Q4_K weights are built");
    if (qr <= 0 || kvr <= 0 || qr > (1 << 30) || kvr > (1 << 30))
        return set_error("matvec_qkv: q_rows=%lld kv_rows=%lld", (long long)qr, (long long)kvr);
    if (check_cols(cols)) return 1;
    const int bpr = (int)(cols / 256);
    const Q4kGeom G = pick_geom(k.desc.sched, (int)(qr + 2 * kvr), bpr);
    if (!geom_ok(G)) return set_error("matvec_qkv: unsupported schedule nr0=%d nsg=%d", G.R, G.NW);
    k.info.n_inputs = 4;
    k.info.n_outputs = 3;
    const size_t rb = (size_t)bpr * kQ4kBytes;
    k.in_bytes[0] = (size_t)qr * rb; k.in_bytes[1] = k.in_bytes[2] = (size_t)kvr * rb;
    k.in_bytes[3] = (size_t)cols * 4;
    k.out_bytes[0] = (size_t)qr * 4; k.out_bytes[1] = k.out_bytes[2] = (size_t)kvr * 4;
    for (int i = 0; i < 4; i++) k.in_align[i] = 16;
    for (int i = 0; i < 3; i++) k.out_align[i] = 4;
    fill_info(k, G, waves_for((int)qr, G.rpw()) + 2 * waves_for((int)kvr, G.rpw()), bpr, "matvec_qkv");
    k.launch = launch_qkv_q4k;
    return 0;
}

int bind_matvec_gate_up_gelu(ksh_kernel &k)
{
    const int64_t rows = k.desc.dims[0], cols = k.desc.dims[1];
    if (k.desc.dtypes[0] != KSH_Q4K) return set_error("matvec_gate_up_gelu: only Q4_K weights are built");
    if (rows <= 0 || rows > (1 << 30)) return set_error("matvec_gate_up_gelu: rows=%lld", (long long)rows);
    if (check_cols(cols)) return 1;
    const int bpr = (int)(cols / 256);
    Q4kGeom G = pick_geom(k.desc.sched, (int)rows * 2, bpr);
    if (!geom_ok(G)) return set_error("matvec_gate_up_gelu: unsupported schedule nr0=%d nsg=%d", G.R, G.NW);
    k.info.n_inputs = 3;
    k.info.n_outputs = 1;
    const size_t rb = (size_t)bpr * kQ4kBytes;
    k.in_bytes[0] = k.in_bytes[1] = (size_t)rows * rb;
    k.in_bytes[2] = (size_t)cols * 4;
    k.out_bytes[0] = (size_t)rows * 4;
    for (int i = 0; i < 3; i++) k.in_align[i] = 16;
    k.out_align[0] = 4;
    fill_info(k, G, waves_for((int)rows, G.rpw()), bpr, "matvec_gate_up_gelu");
    k.launch = launch_gate_up_q4k;
    return 0;
}

int matvec_q4k_candidates(const ksh_kernel_desc &d, ksh_sched *out, int cap)
{
    (void)d;
    int n = 0;
    for (uint32_t var : {0u, 2u})
        for (uint32_t nsg : {1u, 2u, 4u, 8u})
            for (uint32_t nr0 : {1u, 2u, 4u}) {
                if (n >= cap) return n;
                ksh_sched s{};
                s.tg = 64ull * nsg; s.vec = var; s.unroll = 1; s.nsg = nsg; s.nr0 = nr0; s.k_split = 1;
                out[n++] = s;
            }
    return n;
}

}  // namespace ksh
