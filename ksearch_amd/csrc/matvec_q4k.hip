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
//   - the activation vector is staged once per workgroup in LDS, either as
//     padded f32 or as three int8 digit planes (gemv_prologue.hpp), optionally
//     after an RMSNorm / add-then-RMSNorm computed by the workgroup itself;
//   - every row's loads are issued before the first use, so one workgroup
//     keeps R * 192 B per lane in flight;
//   - the 6-bit scales/mins are unpacked in registers, the mins are applied
//     through per-sub-block sums of x, and rows are reduced with DPP;
//   - inner product variant 0: nibble -> f32 byte converts + FMAs; variant 3:
//     nibbles unpacked to bytes and v_dot4_i32_i8 against the digit planes
//     (exact integer sums per 32-wide sub-block, one f32 scale per sub-block).
//
// Arithmetic per (row, superblock, group), all f32:
//   acc += d*sc_lo * sum(n_lo*x) + d*sc_hi * sum(n_hi*x) - dmin*(m_lo*Sx_lo + m_hi*Sx_hi)
// which is the reference's coop form (render.rs:506-511) and differs from the
// CPU dequant-then-dot (gguf_impl.rs:690-721 + check_mul_mm.rs:60-71) by
// reassociation only.
#include "gemv_prologue.hpp"
#include "ksh_internal.hpp"
#include "q4k_lane.hpp"

KSH_STAMP_BUFFER
KSH_STAMP_READER(ksh_stamps_matvec_q4k)

namespace ksh {
namespace {

// timeline build: one record set per decode-step shape -- tag = prologue kind * 2 + (two matrices per wave)
// slots: 0 entry, 1 every load issued, 2 vector staged, 3 barrier passed, 4 inner products done, 5 stores issued, 6 stores acknowledged,
//        7 (half-wave form) the vector's loads issued, in front of the barrier that holds the weight loads back
#define KSH_GEMV_TAG(p, NM) ((p).pro.kind * 2 + ((NM) - 1))

// One launch covers up to three weight matrices that share the input vector.
//   mode 0: the matrices are independent row ranges (plain GEMV: one; QKV:
//           three).  Every wave owns RPW consecutive rows of ONE matrix.
//   mode 1: gate || up: every wave owns the same RPW rows of W[0] and W[1] and
//           stores gelu(W0.x) * (W1.x).
// (Named fields, not arrays: a run-time index into a by-value kernel argument
// makes the compiler copy the whole struct to scratch memory.)
struct MatvecParams {
    const uint8_t *W0, *W1, *W2;
    float *y0, *y1, *y2;
    int rows0, rows1, rows2;
    int waves0, waves1, waves2;   // waves assigned to each matrix (mode 0)
    Prologue pro;
    int bpr;                      // superblocks per row (cols / 256)
    int mode;
};

// Kernel arguments are fetched with scalar loads where they are first used;
// left alone the compiler sinks each into the branch that needs it, and a wave
// then pays one scalar-cache round trip after another before its first weight
// load.  Copying the fields through two opaque statements at the top turns
// that into a few wide loads and two waits.
__device__ __forceinline__ MatvecParams fetch_params(const MatvecParams &p)
{
    const uint8_t *W0 = p.W0, *W1 = p.W1, *W2 = p.W2;
    float *y0 = p.y0, *y1 = p.y1, *y2 = p.y2;
    int rows0 = p.rows0, rows1 = p.rows1, rows2 = p.rows2, waves0 = p.waves0, waves1 = p.waves1, waves2 = p.waves2;
    const float *x = p.pro.x, *w_norm = p.pro.w_norm, *w_post = p.pro.w_post, *res = p.pro.res;
    float *x_out = p.pro.x_out;
    int eps = __float_as_int(p.pro.eps), kind = p.pro.kind, bpr = p.bpr, mode = p.mode, nwg = p.pro.nwg, hd_log2 = p.pro.hd_log2;
    asm volatile("" : "+s"(W0), "+s"(W1), "+s"(W2), "+s"(y0), "+s"(y1), "+s"(y2), "+s"(rows0), "+s"(rows1), "+s"(rows2),
                 "+s"(waves0), "+s"(waves1), "+s"(waves2));
    asm volatile("" : "+s"(x), "+s"(w_norm), "+s"(w_post), "+s"(res), "+s"(x_out), "+s"(eps), "+s"(kind), "+s"(bpr), "+s"(mode),
                 "+s"(nwg), "+s"(hd_log2));
    MatvecParams q;
    q.W0 = W0; q.W1 = W1; q.W2 = W2;
    q.y0 = y0; q.y1 = y1; q.y2 = y2;
    q.rows0 = rows0; q.rows1 = rows1; q.rows2 = rows2;
    q.waves0 = waves0; q.waves1 = waves1; q.waves2 = waves2;
    q.pro.x = x; q.pro.w_norm = w_norm; q.pro.w_post = w_post; q.pro.res = res; q.pro.x_out = x_out;
    q.pro.eps = __int_as_float(eps); q.pro.kind = kind; q.pro.nwg = nwg; q.pro.hd_log2 = hd_log2;
    q.bpr = bpr; q.mode = mode;
    return q;
}

struct WaveTask {
    const uint8_t *W0, *W1;
    float *y;
    int row0, rows;    // first row of this wave (or half-wave), rows in its matrix
    bool active;
};

// (by-value arguments: all three are read before the choice, so nothing turns
// this into a choice of address followed by a dependent load)
template <class T>
__device__ __forceinline__ T sel3(bool in1, bool in2, T a0, T a1, T a2)
{
    return in2 ? a2 : in1 ? a1 : a0;
}

// maps a global wave index onto (matrix, first row).  rpw = rows per wave.  The
// index must live in scalar registers (readfirstlane): the matrix is then
// picked with scalar loads of the kernel arguments instead of a per-lane
// gather from them, which would put a memory round trip in front of every load.
template <int NM>
__device__ __forceinline__ WaveTask wave_task(const MatvecParams &p, int wv, int rpw)
{
    WaveTask t;
    // one matrix, or a gate | up pair whose waves all own rows of both: nothing to choose between (a scalar branch
    // instead of thirty selects in front of the first weight load)
    if (NM == 2 || (p.waves1 == 0 && p.waves2 == 0)) {
        t.W0 = p.W0;
        t.W1 = p.W1;
        t.y = p.y0;
        t.rows = p.rows0;
        t.row0 = wv * rpw;
        t.active = t.row0 < t.rows;
        if (!t.active) t.row0 = 0;
        return t;
    }
    // selects between already-fetched arguments rather than indexing them
    const bool in1 = p.mode == 0 && wv >= p.waves0;
    const bool in2 = in1 && wv - p.waves0 >= p.waves1;
    if (in1) wv -= p.waves0;
    if (in2) wv -= p.waves1;
    t.W0 = sel3(in1, in2, p.W0, p.W1, p.W2);
    t.W1 = p.W1;
    t.y = sel3(in1, in2, p.y0, p.y1, p.y2);
    t.rows = sel3(in1, in2, p.rows0, p.rows1, p.rows2);
    const int nw = sel3(in1, in2, p.waves0, p.waves1, p.waves2);
    t.row0 = wv * rpw;
    t.active = t.row0 < t.rows && (p.mode == 1 || wv < nw);
    if (!t.active) {   // keeps its loads (so that every wave issues the same number) but points them at row 0
        t.W0 = p.W0;
        t.rows = p.rows0;
        t.row0 = 0;
    }
    return t;
}

// Full-wave form: a wave owns R rows and sweeps 16 superblocks per step.
// NM = 1 (mode 0) or 2 (mode 1).  The weight loads of step s+1 are issued
// before step s is consumed, and step 0's before the input is staged, so the
// first HBM round trip overlaps the prologue.
// MERGE: built with the partition-merging prologue (kept out of every other instance: a longer program in front
// of the first weight load costs 0.1 us at 4096 x 4096)
// CB: superblocks per row when the instance is built for one row length (0: p.bpr); KIND: its prologue kind (-1:
// p.pro.kind).  The instances with both (the plain GEMV over 4096 and 8192 columns) reach their weight loads in a
// fraction of the instructions the general form needs.
template <int R, int NW, int NM, int XF, bool MULTI, bool MERGE, int CB = 0, int KIND = -1>
__global__ __launch_bounds__(NW * 64) void q4k_gemv_kernel(MatvecParams p_in)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];
    const MatvecParams p = fetch_params(p_in);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    KSH_STAMP_BEGIN
    const int g = lane & 3, bl = lane >> 2;
    const int bpr = CB ? CB : p.bpr, cols = bpr * 256;
    const size_t row_bytes = (size_t)bpr * kQ4kBytes;
    constexpr int KMAX = CB ? (CB * 64 + NW * 64 - 1) / (NW * 64) : kStageX;   // float4 of the vector per thread
    const WaveTask t = wave_task<NM>(p, blockIdx.x * NW + wave, R);

    const uint8_t *rowp[NM][R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        // rows past the end re-read the last row; their sums are never stored
        const size_t off = (size_t)min(t.row0 + r, t.rows - 1) * row_bytes;
        rowp[0][r] = t.W0 + off;
        if (NM == 2) rowp[NM - 1][r] = t.W1 + off;
    }

    // Every wave and lane issues the same loads, unconditionally (lanes past the
    // row's end re-read its last superblock and drop the product): the wait for
    // the staged vector can then be an exact count that leaves the weight loads
    // in flight, where a conditional load would force a wait for everything.
    // MULTI: rows longer than 16 superblocks take several steps and double-buffer.
    Q4kLane cur[NM][R], nxt[MULTI ? NM : 1][MULTI ? R : 1];
    StageRegs sr;
    constexpr int RPRE = R;   // (splitting the issue as the half-wave form does costs 0.5 us at 4096 x 4096)
    stage_fetch<NW * 64, MERGE, KMAX, KIND>(p.pro, cols, sr);
    // The short front reaches its weight loads a few dozen instructions behind the vector's, and loads of different
    // waves share one in-order path per compute unit: without this barrier a wave's vector loads queue behind another
    // wave's HBM-cold weights (vector staged in the slowest wave at 2.3 us instead of 1.7).  The general form's long
    // front keeps the two apart by itself.
    if (CB) __syncthreads();
#pragma unroll
    for (int m = 0; m < NM; m++)
#pragma unroll
        for (int r = 0; r < RPRE; r++) cur[m][r] = q4k_load(rowp[m][r] + (size_t)min(bl, bpr - 1) * kQ4kBytes, g);
    KSH_STAMP(1);
    stage_finish<XF, NW * 64, MERGE, KMAX, KIND>(p.pro, xs, cols, sr);
    KSH_STAMP(2);
    __syncthreads();
    KSH_STAMP(3);
    if (!t.active) return;
#pragma unroll
    for (int m = 0; m < NM; m++)
#pragma unroll
        for (int r = RPRE; r < R; r++) cur[m][r] = q4k_load(rowp[m][r] + (size_t)min(bl, bpr - 1) * kQ4kBytes, g);

    float acc[NM][R];
#pragma unroll
    for (int m = 0; m < NM; m++)
#pragma unroll
        for (int r = 0; r < R; r++) acc[m][r] = 0.f;

    for (int b0 = 0; b0 < bpr; b0 += 16) {
        const int b = min(b0 + bl, bpr - 1);
        const bool mine = b0 + bl < bpr;
        if (MULTI) {
            const int bn = min(b0 + 16 + bl, bpr - 1);
#pragma unroll
            for (int m = 0; m < NM; m++)
#pragma unroll
                for (int r = 0; r < R; r++) nxt[m][r] = q4k_load(rowp[m][r] + (size_t)bn * kQ4kBytes, g);
        }
        XGroup<XF> X;
        X.load(xs, cols, b, g);
#pragma unroll
        for (int m = 0; m < NM; m++)
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float v = q4k_group_dot<XF>(cur[m][r], g, X);
                acc[m][r] += mine ? v : 0.f;
            }
        if (MULTI) {
#pragma unroll
            for (int m = 0; m < NM; m++)
#pragma unroll
                for (int r = 0; r < R; r++) cur[m][r] = nxt[m][r];
        }
    }

    KSH_STAMP_USE(acc[NM - 1][R - 1]);
    KSH_STAMP(4);
    // every row is reduced before the first is stored: a store in front of a later row's wait makes that wait one for
    // the store's acknowledgement as well (loads and stores retire in order)
    float res[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        float s[NM];
#pragma unroll
        for (int m = 0; m < NM; m++) s[m] = wave_sum(acc[m][r]);
        res[r] = (NM == 2) ? gelu_mul_f32(s[0], s[NM - 1]) : s[0];
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int row = t.row0 + r;
        if (lane == 0 && row < t.rows) stg_f32(t.y, row, res[r]);
    }
    KSH_STAMP(5);
    KSH_STAMP_FLUSH(KSH_GEMV_TAG(p, NM), blockIdx.x * NW + wave, 6);
}

// Half-wave form for rows of at most 8 superblocks (BPR = 8: 2048 columns, no lane idles; BPR = 6: 1536 columns,
// a quarter of the lanes re-read the row's last superblock and drop the product): lanes 0..31 and 32..63 work
// on different rows, so a wave covers 2R rows in a single step.
template <int R, int NW, int NM, int XF, bool MERGE, int BPR>
__global__ __launch_bounds__(NW * 64) void q4k_gemv_half_kernel(MatvecParams p_in)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];
    const MatvecParams p = fetch_params(p_in);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    KSH_STAMP_BEGIN
    const int g = lane & 3, slot = (lane >> 2) & 7, hw = lane >> 5;
    constexpr int bpr = BPR;
    const int bl = BPR == 8 ? slot : min(slot, BPR - 1);
    const bool mine = BPR == 8 || slot < BPR;
    constexpr size_t row_bytes = (size_t)bpr * kQ4kBytes;
    WaveTask t = wave_task<NM>(p, blockIdx.x * NW + wave, 2 * R);
    const int row0 = t.row0 + hw * R;

    Q4kLane L[NM][R];
    StageRegs sr;
    // (the instances that merge attention partitions are launched for that prologue alone: the other kinds' loads
    // and arithmetic are not compiled into them)
    constexpr int KIND = MERGE ? kMergeParts : -1;
    stage_fetch<NW * 64, MERGE, kStageX, KIND>(p.pro, bpr * 256, sr);
    // With a normalising prologue every wave's vector loads are queued before any wave's weight loads: behind
    // another wave's HBM-cold weights in the compute unit's memory pipeline they came back up to 1.3 us late, and
    // the prologue's reduction waits for the slowest wave.
    KSH_STAMP(7);
    if (MERGE || p.pro.kind != kPlain) __syncthreads();
    auto load_r = [&](int r) {
        const size_t off = (size_t)min(row0 + r, t.rows - 1) * row_bytes + (size_t)bl * kQ4kBytes;
        L[0][r] = q4k_load(t.W0 + off, g);
        if (NM == 2) L[NM - 1][r] = q4k_load(t.W1 + off, g);
    };
    // Only the first row's loads go out before the input is staged: a compute
    // unit's memory queue is finite, a wave that cannot issue cannot reach the
    // staging barrier either, and one row per half-wave already covers the HBM
    // round trips that the staging takes.  The other rows follow the barrier
    // and stream in while the first is being multiplied (gate || up, 2048 ->
    // 8192 with the add-then-norm prologue: 8.1 -> 7.1 us).
    load_r(0);
    KSH_STAMP(1);
    stage_finish<XF, NW * 64, MERGE, kStageX, KIND>(p.pro, xs, bpr * 256, sr);
    KSH_STAMP(2);
    __syncthreads();
    KSH_STAMP(3);
    if (!t.active) return;
#pragma unroll
    for (int r = 1; r < R; r++) load_r(r);

    XGroup<XF> X;
    X.load(xs, bpr * 256, bl, g);

    // (every row is multiplied and reduced before the first is stored, as in the full-wave form)
    float res[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        float s[NM];
#pragma unroll
        for (int m = 0; m < NM; m++) {
            const float v = q4k_group_dot<XF>(L[m][r], g, X);
            const float2 hs = wave_half_sums(mine ? v : 0.f);
            s[m] = hw ? hs.y : hs.x;
        }
        res[r] = (NM == 2) ? gelu_mul_f32(s[0], s[NM - 1]) : s[0];
    }
    KSH_STAMP_USE(res[R - 1]);
    KSH_STAMP(4);
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int row = row0 + r;
        if ((lane & 31) == 0 && row < t.rows) stg_f32(t.y, row, res[r]);
    }
    KSH_STAMP(5);
    KSH_STAMP_FLUSH(KSH_GEMV_TAG(p, NM), blockIdx.x * NW + wave, 6);
}

struct Q4kGeom {
    int R, NW, var;
    bool half;
    int rpw() const { return R * (half ? 2 : 1); }   // rows per wave
};

int waves_for(int rows, int rpw) { return (rows + rpw - 1) / rpw; }

size_t lds_for(int var, int cols) { return var == kXI8 ? xs_bytes<kXI8>(cols) : var == kXI2 ? xs_bytes<kXI2>(cols) : xs_bytes<kXF32>(cols); }

template <int R, int NW, int NM, int XF, bool MERGE>
void launch_pro(bool half, const MatvecParams &p, unsigned grid, size_t lds, hipStream_t st)
{
    if (half && p.bpr == 8)
        hipLaunchKernelGGL((q4k_gemv_half_kernel<R, NW, NM, XF, MERGE, 8>), dim3(grid), dim3(NW * 64), lds, st, p);
    else if (half)
        hipLaunchKernelGGL((q4k_gemv_half_kernel<R, NW, NM, XF, MERGE, 6>), dim3(grid), dim3(NW * 64), lds, st, p);
    // the plain GEMV over 4096 columns, built for that row length (4.25 against 4.35 us at 4096 x 4096; the same for 8192
    // columns -- the down projection -- was slower inside the decode loop, 1111 against 1123 tok/s, and is not built)
    else if (NM == 1 && !MERGE && NW == 8 && R <= 2 && p.pro.kind == kPlain && p.bpr == 16)
        hipLaunchKernelGGL((q4k_gemv_kernel<(R <= 2 ? R : 1), 8, 1, XF, false, false, 16, kPlain>), dim3(grid), dim3(NW * 64), lds, st, p);
    else if (p.bpr > 16)
        hipLaunchKernelGGL((q4k_gemv_kernel<R, NW, NM, XF, true, MERGE>), dim3(grid), dim3(NW * 64), lds, st, p);
    else
        hipLaunchKernelGGL((q4k_gemv_kernel<R, NW, NM, XF, false, MERGE>), dim3(grid), dim3(NW * 64), lds, st, p);
}

template <int R, int NW, int NM, int XF>
int launch_inst(bool half, const MatvecParams &p, int total_waves, hipStream_t st)
{
    const unsigned grid = (unsigned)((total_waves + NW - 1) / NW);
    const size_t lds = xs_bytes<XF>(p.bpr * 256);
    if (NM == 1 && p.pro.kind == kMergeParts) launch_pro<R, NW, 1, XF, true>(half, p, grid, lds, st);
    else launch_pro<R, NW, NM, XF, false>(half, p, grid, lds, st);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "q4k_gemv launch");
}

template <int NM, int XF>
int launch_rn(const Q4kGeom &G, const MatvecParams &p, int total_waves, hipStream_t st)
{
#define KSH_CASE(r, w) \
    if (G.R == r && G.NW == w) return launch_inst<r, w, NM, XF>(G.half, p, total_waves, st);
    KSH_CASE(1, 4) KSH_CASE(2, 4) KSH_CASE(4, 4)
    KSH_CASE(1, 8) KSH_CASE(2, 8) KSH_CASE(4, 8)
#undef KSH_CASE
    return set_error("q4k gemv: no instance for nr0=%d nsg=%d", G.R, G.NW);
}

template <int NM>
int launch_q4k(const Q4kGeom &G, const MatvecParams &p, int total_waves, hipStream_t st)
{
    return G.var == kXI8 ? launch_rn<NM, kXI8>(G, p, total_waves, st)
         : G.var == kXI2 ? launch_rn<NM, kXI2>(G, p, total_waves, st) : launch_rn<NM, kXF32>(G, p, total_waves, st);
}

// default schedule, from cold-cache timings of the candidate set on the decode
// shapes and the 4096 x 4096 case: 8 waves per workgroup and 2 rows per wave
// where that still leaves ~150 workgroups, else fewer rows, else smaller
// workgroups; int8 dot, except for rows longer than one 16-superblock step,
// where the f32 form is the faster one.
Q4kGeom pick_geom(const ksh_sched &s, int total_rows, int bpr)
{
    Q4kGeom G;
    G.half = (bpr == 8 || bpr == 6);
    G.var = sched_is_zero(s) ? (bpr > 16 ? kXF32 : kXI8) : (s.vec == 3 ? kXI8 : s.vec == 2 ? kXI2 : kXF32);
    if (s.nsg && s.nr0) {
        G.NW = (int)s.nsg;
        G.R = (int)s.nr0;
        return G;
    }
    // 1536-column matrices of 12288 rows and more (the wide feed-forward of the cache-reading layers): 4-wave
    // workgroups, twice as many of them (in the decode loop 1.398 against 1.410 ms per token)
    if (bpr == 6 && total_rows >= 12288 && !s.nsg && !s.nr0) {
        G.NW = 4;
        G.R = 2;
        return G;
    }
    for (int nw : {8, 4})
        for (int r : {2, 1}) {
            if (s.nsg && (int)s.nsg != nw) continue;
            if (s.nr0 && (int)s.nr0 != r) continue;
            G.NW = nw;
            G.R = r;
            if (total_rows / (nw * G.rpw()) >= 144) return G;
        }
    G.NW = s.nsg ? (int)s.nsg : 4;
    G.R = s.nr0 ? (int)s.nr0 : 1;
    return G;
}

bool geom_ok(const Q4kGeom &G) { return (G.R == 1 || G.R == 2 || G.R == 4) && (G.NW == 4 || G.NW == 8); }

void fill_info(ksh_kernel &k, const Q4kGeom &G, int total_waves, int bpr, const char *base)
{
    set_launch(k, (uint32_t)((total_waves + G.NW - 1) / G.NW), 1, 1, (uint32_t)G.NW * 64,
               (uint32_t)lds_for(G.var, bpr * 256));
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

// The three shapes (plain / QKV / gate-up), each with an optional normalising
// prologue.  Binding order of inputs: weight matrices, the vector, then for a
// prologue w_norm, and with a residual w_post, res; outputs: the GEMV results,
// then with a residual the new residual stream.
struct Shape {
    int n_mat;        // weight matrices bound
    int nm;           // matrices per wave (2 for gate||up)
    int64_t rows[3];
    int64_t cols;
    int prologue;     // kPlain / kRms / kAddThenRms / kMergeParts
    float eps;
    int nwg, hd;      // kMergeParts
};

Shape shape_of(const ksh_kernel_desc &d)
{
    Shape s{};
    const int64_t *D = d.dims;
    switch (d.kind) {
    case KSH_MATVEC: s.n_mat = 1; s.nm = 1; s.rows[0] = D[0]; s.cols = D[1]; break;
    case KSH_RMSNORM_MATVEC: s.n_mat = 1; s.nm = 1; s.rows[0] = D[0]; s.cols = D[1]; s.prologue = D[2] ? kAddThenRms : kRms; break;
    case KSH_MATVEC_QKV: s.n_mat = 3; s.nm = 1; s.rows[0] = D[0]; s.rows[1] = s.rows[2] = D[1]; s.cols = D[2]; break;
    case KSH_RMSNORM_MATVEC_QKV:
        s.n_mat = 3; s.nm = 1; s.rows[0] = D[0]; s.rows[1] = s.rows[2] = D[1]; s.cols = D[2];
        s.prologue = D[3] ? kAddThenRms : kRms;
        break;
    case KSH_MATVEC_GATE_UP_GELU: s.n_mat = 2; s.nm = 2; s.rows[0] = s.rows[1] = D[0]; s.cols = D[1]; break;
    case KSH_RMSNORM_MATVEC_GATE_UP_GELU:
        s.n_mat = 2; s.nm = 2; s.rows[0] = s.rows[1] = D[0]; s.cols = D[1];
        s.prologue = D[2] ? kAddThenRms : kRms;
        break;
    case KSH_ATTN_MERGE_MATVEC:
        s.n_mat = 1; s.nm = 1; s.rows[0] = D[0]; s.cols = D[1] * D[2]; s.prologue = kMergeParts;
        s.hd = (int)D[2]; s.nwg = (int)D[3];
        break;
    }
    s.eps = d.params[0];
    return s;
}

int launch_any(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const Q4kGeom G = geom_of(k);
    const Shape s = shape_of(k.desc);
    MatvecParams p{};
    int total = 0;
    const int n_y = s.nm == 2 ? 1 : s.n_mat;
    const uint8_t **W[3] = {&p.W0, &p.W1, &p.W2};
    float **y[3] = {&p.y0, &p.y1, &p.y2};
    int *rows[3] = {&p.rows0, &p.rows1, &p.rows2}, *waves[3] = {&p.waves0, &p.waves1, &p.waves2};
    for (int m = 0; m < s.n_mat; m++) {
        *W[m] = (const uint8_t *)a.in[m];
        *rows[m] = (int)s.rows[m];
        *waves[m] = waves_for(*rows[m], G.rpw());
        if (s.nm == 1) total += *waves[m];
    }
    for (int m = 0; m < n_y; m++) *y[m] = (float *)a.out[m];
    if (s.nm == 2) total = p.waves0;
    p.mode = s.nm == 2 ? 1 : 0;
    p.bpr = (int)(s.cols / 256);
    p.pro.kind = s.prologue;
    p.pro.eps = s.eps;
    p.pro.x = (const float *)a.in[s.n_mat];
    if (s.prologue == kMergeParts) {
        p.pro.w_norm = p.pro.x + (size_t)s.cols * s.nwg;   // the (m, l) pairs follow the values
        p.pro.nwg = s.nwg;
        p.pro.hd_log2 = __builtin_ctz((unsigned)s.hd);
        return launch_q4k<1>(G, p, total, st);
    }
    if (s.prologue != kPlain) p.pro.w_norm = (const float *)a.in[s.n_mat + 1];
    if (s.prologue == kAddThenRms) {
        p.pro.nwg = __builtin_bit_cast(int, k.desc.params[1] != 0.f ? k.desc.params[1] : 1.0f);   // the stream scale
        p.pro.w_post = (const float *)a.in[s.n_mat + 2];
        p.pro.res = (const float *)a.in[s.n_mat + 3];
        p.pro.x_out = (float *)a.out[n_y];
    }
    return s.nm == 2 ? launch_q4k<2>(G, p, total, st) : launch_q4k<1>(G, p, total, st);
}

}  // namespace

int bind_matvec_q4k_family(ksh_kernel &k)
{
    const Shape s = shape_of(k.desc);
    if (!s.n_mat) return set_error("q4k gemv: kind %d", k.desc.kind);
    if (k.desc.dtypes[0] != KSH_Q4K) return set_error("%d: only Q4_K weights are built for this kind", k.desc.kind);
    if (k.desc.dtypes[1] != KSH_F32 && k.desc.dtypes[1] != 0)
        return set_error("matvec: activation dtype %d is not built (f32 only)", k.desc.dtypes[1]);
    int64_t total_rows = 0;
    for (int m = 0; m < s.n_mat; m++) {
        if (s.rows[m] <= 0 || s.rows[m] > (1 << 30)) return set_error("matvec: rows=%lld", (long long)s.rows[m]);
        total_rows += s.rows[m];
    }
    if (s.cols <= 0 || s.cols % 256) return set_error("Q4_K matvec: cols=%lld is not a positive multiple of 256", (long long)s.cols);
    if (s.cols > 32768) return set_error("Q4_K matvec: cols=%lld does not fit the LDS staging buffer", (long long)s.cols);
    const int bpr = (int)(s.cols / 256);
    Q4kGeom G = pick_geom(k.desc.sched, (int)(s.nm == 2 ? s.rows[0] : total_rows), bpr);
    // QKV at one row per half-wave: one dot per lane does not pay for turning the vector into digit planes (3.86 vs 4.08 us)
    if (sched_is_zero(k.desc.sched) && s.n_mat == 3 && G.half && G.R == 1) G.var = kXF32;
    if (s.prologue == kMergeParts) {
        if (s.hd < 4 || (s.hd & (s.hd - 1)) || s.nwg < 1 || s.nwg > kMergeMaxParts)
            return set_error("attn_merge_matvec: hd=%d must be a power of two, nwg=%d at most %d", s.hd, s.nwg, kMergeMaxParts);
        if (!k.desc.sched.nsg) { G.NW = 8; if (!k.desc.sched.nr0) G.R = 1; }   // one float4 of the merged vector per thread
        if (s.cols > (int64_t)4 * G.NW * 64)
            return set_error("attn_merge_matvec: n_q*hd=%lld exceeds one float4 per thread (%d)", (long long)s.cols, 4 * G.NW * 64);
    }
    if (lds_for(G.var, (int)s.cols) > 65536)
        return set_error("Q4_K matvec: cols=%lld does not fit the LDS staging buffer", (long long)s.cols);
    if (!geom_ok(G)) return set_error("matvec_q4k: unsupported schedule nr0=%d nsg=%d (nr0 in 1,2,4; nsg in 4,8)", G.R, G.NW);
    if (s.prologue != kPlain && s.prologue != kMergeParts && s.cols > (int64_t)4 * G.NW * 64 * kStageP)
        return set_error("rmsnorm_matvec requires LOCAL staging of the vector (cols=%lld too large)", (long long)s.cols);
    const size_t rb = (size_t)bpr * kQ4kBytes, vb = (size_t)s.cols * 4;
    const int n_y = s.nm == 2 ? 1 : s.n_mat;
    int ni = 0, no = 0;
    for (int m = 0; m < s.n_mat; m++) { k.in_bytes[ni] = (size_t)s.rows[m] * rb; k.in_align[ni++] = 16; }
    k.in_bytes[ni] = s.prologue == kMergeParts ? (size_t)s.nwg * (s.cols + 2 * (s.cols / s.hd)) * 4 : vb; k.in_align[ni++] = 16;
    if (s.prologue == kRms || s.prologue == kAddThenRms) { k.in_bytes[ni] = vb; k.in_align[ni++] = 16; }
    if (s.prologue == kAddThenRms) {
        k.in_bytes[ni] = vb; k.in_align[ni++] = 16;
        k.in_bytes[ni] = vb; k.in_align[ni++] = 16;
    }
    for (int m = 0; m < n_y; m++) { k.out_bytes[no] = (size_t)s.rows[m] * 4; k.out_align[no++] = 4; }
    if (s.prologue == kAddThenRms) { k.out_bytes[no] = vb; k.out_align[no++] = 16; }
    k.info.n_inputs = ni;
    k.info.n_outputs = no;
    int waves = 0;
    if (s.nm == 2) waves = waves_for((int)s.rows[0], G.rpw());
    else for (int m = 0; m < s.n_mat; m++) waves += waves_for((int)s.rows[m], G.rpw());
    static const char *pre[] = {"", "rms_", "addrms_", "attn_merge_"};
    char base[48];
    snprintf(base, sizeof(base), "%smatvec%s", pre[s.prologue], s.n_mat == 3 ? "_qkv" : s.nm == 2 ? "_gate_up_gelu" : "");
    fill_info(k, G, waves, bpr, base);
    k.launch = launch_any;
    return 0;
}

int bind_matvec_q4k(ksh_kernel &k) { return bind_matvec_q4k_family(k); }
int bind_matvec_qkv(ksh_kernel &k) { return bind_matvec_q4k_family(k); }
int bind_matvec_gate_up_gelu(ksh_kernel &k) { return bind_matvec_q4k_family(k); }

int matvec_q4k_candidates(const ksh_kernel_desc &d, ksh_sched *out, int cap)
{
    (void)d;
    int n = 0;
    // (vec = 2, the two-plane form, is built and can be asked for by schedule, but the search does not offer it: its
    // error is 2^-16 of a 32-element sub-block's largest magnitude, which is 1e-3 of an element next to an outlier
    // sixty times its size -- the three-plane form has 2^-21)
    for (uint32_t var : {3u, 1u})
        for (uint32_t nsg : {4u, 8u})
            for (uint32_t nr0 : {1u, 2u, 4u}) {
                if (n >= cap) return n;
                ksh_sched s{};
                s.tg = 64ull * nsg; s.vec = var; s.unroll = 1; s.nsg = nsg; s.nr0 = nr0; s.k_split = 1;
                out[n++] = s;
            }
    return n;
}

}  // namespace ksh
