// Decode attention over a Q4_0 KV cache, register form, for head sizes 128, 256
// and 512 with up to 8 q heads per kv head; optionally with the per-head RMSNorm +
// RoPE + Q4_0 KV append in front of it and always with the split-KV merge
// behind it, so that a decode step's attention is one launch.
//
// Same semantics as the tile form next door (which stays for the other
// shapes): lower_sdpa_online / lower_sdpa_mwg_part / lower_sdpa_mwg_reduce
// (crates/ksearch_codegen/src/lower.rs:4897-5359, 5367-5894, 5897-6087) and,
// for the fused prologue, RmsNormPerHeadQkvQ40 (lower.rs:4080-4440,
// gemma_prim.rs:984-1008).
//
// Layout of the work:
//   - a KV row of hd elements is hd/8 dwords of nibbles; hd/8 consecutive
//     lanes take one row, lane j owning dword j: Q4_0 block b = j/4, bytes
//     4w..4w+3 (w = j%4), i.e. elements 32b+4w+{0..3} (low nibbles) and
//     32b+16+4w+{0..3} (high nibbles).  A wave therefore works on 64/(hd/8)
//     rows at once, and the four lanes of a DPP quad share a block and its
//     scale;
//   - every lane keeps the matching 8 elements of q for all heads in registers
//     (pre-multiplied by the softmax scale) and its 8 elements of the output
//     accumulator for all heads;
//   - scores: 8 FMAs per head on the lane's nibbles, times the block scale,
//     then a transposing butterfly (two quad steps that halve the number of
//     heads a lane carries, then row rotations and one row swap) leaves every
//     lane with the finished scores of GP/4 heads of its row;
//   - softmax bookkeeping is lane-local: rows are taken four at a time, their
//     maximum and the rescale factor are per lane, and the probabilities are
//     handed to the other three lanes of the quad with quad broadcasts;
//   - P.V: p*scale per head, then 8 FMAs per head; the -8 offset of the codes
//     is applied once at the end through the running sum of p*scale;
//   - every row group ends with its own (m, l, O); the workgroup folds them
//     through LDS, writes one partial per partition, and the last partition
//     to arrive (a device-scope counter) folds the partials into the output.
#include "ksh_device.hpp"
#include "round_operand.hpp"
#include "q40_pack.hpp"
#include "ksh_internal.hpp"

KSH_STAMP_BUFFER
KSH_STAMP_READER(ksh_stamps_sdpa_lanes)

namespace ksh {
namespace {

// timeline build, register-form kernel: tag 0 plain attention, 1 the fused decode step; tag 2 the matrix-core row phase in
// its V-block form (slots: 1 the deal is known, 2 q operands shared, 3 tile and scale tables in LDS, 4 probabilities
// written, 5 products done, 6 stores acknowledged)
// slots: 0 entry, 1 every load of the front issued, 2 length and position in, 3 q (and the new row) ready,
//        4 rows done, 5 row groups folded, 6 records stored (acknowledged)
#define KSH_LANES_WAVE ((((int)blockIdx.z * (int)gridDim.y + (int)blockIdx.y) * (int)gridDim.x + (int)blockIdx.x) * NW + wave)

enum { kModeDirect = 0, kModePart = 1, kModeMerge = 2, kModeSplitPart = 3 };   // SplitPart: values and (m, l) pairs in separate arrays, no merge
constexpr int kRT = 4;   // row steps per softmax update

struct LaneParams {
    const float *q;          // [n_slots][n_q*hd]; fused: the raw q of the QKV GEMV
    const uint8_t *k, *v;    // [n_slots][max_t*n_kv*row_bytes]
    const float *meta;       // [n_slots][meta_stride]: tlen, start, window(, pos)
    const float *slot_ids;   // nullptr, or [n_slots]: which slot of the K / V pools entry i attends (entries of a decode round)
    size_t slot_stride;      // bytes from one slot of the pools to the next; 0: max_t * n_kv * row bytes
    float *tmp;              // [n_slots][n_q][nwg][hd+2]
    float *out;              // [n_slots][n_q*hd]
    uint32_t *counters;      // [n_slots*n_kv], zero between launches
    const float *qw, *kw, *rope, *k_raw, *v_raw;   // fused prologue
    uint8_t *k_w, *v_w;                            // the caches again, writable
    float eps, scale;
    int n_q, n_kv, max_t, nwg, meta_stride, mode, fused;
    int groups;   // q heads this workgroup handles: (n_q / n_kv) / hsplit
    int hsplit;   // workgroups that share a kv head's rows, each with its own q heads
    int balance;  // the launch's nwg * n_slots partitions are dealt to the slots by length (kModeMerge, several slots)
    int rope_row; // fused: `rope` is the current position's row of the table, not the table
    int kv_shared; // every slot attends the same cache (a chunk of prompt tokens, one meta record and one q per token)
    int no_append; // fused: the step's K / V row is in the cache already (a layer that reuses another layer's cache): q is normed and
                   // roped as usual, nothing is appended, every attended row comes from the cache
};

// Kernel arguments are fetched with scalar loads where they are first used; left alone the compiler spreads them
// over the kernel's front (four groups here), and a wave pays one scalar-cache round trip after another before its
// first vector load.  An empty statement at the top that reads every field makes them a few wide loads issued
// together and one wait.  (The fields are only read, not passed through the statement: a pointer that comes out of
// an opaque statement is no longer known to point to global memory and would be accessed with flat instructions.)
__device__ __forceinline__ void touch_lane_params(const LaneParams &p)
{
    asm volatile("" ::"s"(p.q), "s"(p.k), "s"(p.v), "s"(p.meta), "s"(p.slot_ids), "s"(p.slot_stride), "s"(p.tmp), "s"(p.out), "s"(p.counters));
    asm volatile("" ::"s"(p.qw), "s"(p.kw), "s"(p.rope), "s"(p.k_raw), "s"(p.v_raw), "s"(p.k_w), "s"(p.v_w));
    asm volatile("" ::"s"(p.eps), "s"(p.scale), "s"(p.n_q), "s"(p.n_kv), "s"(p.max_t), "s"(p.nwg), "s"(p.meta_stride), "s"(p.mode), "s"(p.fused),
                 "s"(p.groups), "s"(p.hsplit), "s"(p.balance), "s"(p.rope_row), "s"(p.kv_shared), "s"(p.no_append));
}

__device__ __forceinline__ uint32_t ld32_a2(const uint8_t *p)
{
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}
__device__ __forceinline__ uint32_t ld16_a2(const uint8_t *p)
{
    uint16_t v;
    __builtin_memcpy(&v, p, 2);
    return v;
}

__device__ __forceinline__ float xor16_sum(float x)
{
    // rows 1 and 3 of the first copy trade places with rows 0 and 2 of the second
    const auto r = __builtin_amdgcn_permlane16_swap(as_u32(x), as_u32(x), false, false);
    return as_f32(r[0]) + as_f32(r[1]);
}

__device__ __forceinline__ float xor32_sum(float x)
{
    // the two halves of the wave trade places
    const auto r = __builtin_amdgcn_permlane32_swap(as_u32(x), as_u32(x), false, false);
    return as_f32(r[0]) + as_f32(r[1]);
}

struct RowRegs {
    uint32_t kd, ks, vd, vs;
};

// (GP = 1: a workgroup with a single q head -- the decode step's unmerged form with the heads spread over the
// workgroups -- where the instances for four heads would carry three heads of zeros through every row)
template <int GP>
struct State {
    float m[(GP + 3) / 4], l[(GP + 3) / 4];
    float O[GP][8], S[GP];
};

// the head whose finished score ends up in slot i of the lane at quad position c
template <int GP>
__device__ __forceinline__ int head_of(int c, int i)
{
    return (c & 1) * (GP / 2) + ((c >> 1) & 1) * (GP / 4) + i;
}

// per-lane partial dots of GP heads -> finished dots of GP/4 heads, in every lane of the row group
template <int HD, int GP>
__device__ __forceinline__ void reduce_heads(const float (&v)[GP], int c, float (&out)[(GP + 3) / 4])
{
    if constexpr (GP == 1) {
        float x = v[0] + dpp_f32<0xB1>(v[0]);   // the quad's four dwords of the block ...
        x += dpp_f32<0x4E>(x);
        x += dpp_f32<0x124>(x);                 // ... and the row group's blocks
        x += dpp_f32<0x128>(x);
        if (HD >= 256) x = xor16_sum(x);
        if (HD == 512) x = xor32_sum(x);
        out[0] = x;
    } else if constexpr (GP == 2) {
        // lanes with c & 1 = 0 end up with head 0, the others with head 1
        const bool b0 = c & 1;
        const float keep = b0 ? v[1] : v[0], send = b0 ? v[0] : v[1];
        float x = keep + dpp_f32<0xB1>(send);   // quad_perm [1,0,3,2]
        x += dpp_f32<0x4E>(x);                  // quad_perm [2,3,0,1]
        x += dpp_f32<0x124>(x);
        x += dpp_f32<0x128>(x);
        if (HD >= 256) x = xor16_sum(x);
        if (HD == 512) x = xor32_sum(x);
        out[0] = x;
    } else {
        const bool b0 = c & 1, b1 = c & 2;
        float a[GP / 2];
#pragma unroll
        for (int i = 0; i < GP / 2; i++) {
            const float keep = b0 ? v[i + GP / 2] : v[i], send = b0 ? v[i] : v[i + GP / 2];
            a[i] = keep + dpp_f32<0xB1>(send);   // quad_perm [1,0,3,2]
        }
#pragma unroll
        for (int i = 0; i < GP / 4; i++) {
            const float keep = b1 ? a[i + GP / 4] : a[i], send = b1 ? a[i] : a[i + GP / 4];
            float x = keep + dpp_f32<0x4E>(send);   // quad_perm [2,3,0,1]
            x += dpp_f32<0x124>(x);                 // row_ror:4
            x += dpp_f32<0x128>(x);                 // row_ror:8
            if (HD >= 256) x = xor16_sum(x);
            if (HD == 512) x = xor32_sum(x);
            out[i] = x;
        }
    }
}

// one lane's GP/4 values -> all GP, through the quad
template <int GP>
__device__ __forceinline__ void quad_gather(const float (&x)[(GP + 3) / 4], float (&all)[GP])
{
    if constexpr (GP == 1) {
        all[0] = x[0];
    } else if constexpr (GP == 2) {
        all[0] = dpp_f32<0x00>(x[0]);
        all[1] = dpp_f32<0x55>(x[0]);
    } else {
#pragma unroll
        for (int i = 0; i < GP / 4; i++) {
            all[i] = dpp_f32<0x00>(x[i]);
            all[GP / 2 + i] = dpp_f32<0x55>(x[i]);
            all[GP / 4 + i] = dpp_f32<0xAA>(x[i]);
            all[GP / 2 + GP / 4 + i] = dpp_f32<0xFF>(x[i]);
        }
    }
}

__device__ __forceinline__ void unpack8(uint32_t d, float (&n)[8])
{
    const uint32_t lo = d & 0x0F0F0F0Fu, hi = (d >> 4) & 0x0F0F0F0Fu;
    n[0] = ubyte_f32<0>(lo); n[1] = ubyte_f32<1>(lo); n[2] = ubyte_f32<2>(lo); n[3] = ubyte_f32<3>(lo);
    n[4] = ubyte_f32<0>(hi); n[5] = ubyte_f32<1>(hi); n[6] = ubyte_f32<2>(hi); n[7] = ubyte_f32<3>(hi);
}

// NR row steps: scores, one online-softmax update, P.V
template <int HD, int GP, int NR>
__device__ __forceinline__ void process_rows(const RowRegs (&r)[NR], const bool (&valid)[NR], const bool (&live)[NR],
                                             const float (&qv)[GP][8], const float (&Sq)[GP], State<GP> &st, int c)
{
    // valid: this lane's row exists; live: some row of this wave's step exists (wave-uniform: dead steps are skipped)
    constexpr int HPL = (GP + 3) / 4;
    float s[NR][HPL];
#pragma unroll
    for (int t = 0; t < NR; t++) {
#pragma unroll
        for (int i = 0; i < HPL; i++) s[t][i] = -INFINITY;
        if (!live[t]) continue;
        float n[8], part[GP];
        unpack8(r[t].kd, n);
        const float ks = half_bits_to_f32(r[t].ks);
#pragma unroll
        for (int h = 0; h < GP; h++) {
            float acc = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) acc = fmaf(n[e], qv[h][e], acc);
            part[h] = ks * fmaf(-8.f, Sq[h], acc);
        }
        float fin[HPL];
        reduce_heads<HD, GP>(part, c, fin);
#pragma unroll
        for (int i = 0; i < HPL; i++) s[t][i] = valid[t] ? fin[i] : -INFINITY;
    }
    float alpha[HPL], pr[NR][HPL];
#pragma unroll
    for (int i = 0; i < HPL; i++) {
        float mt = s[0][i];
#pragma unroll
        for (int t = 1; t < NR; t++) mt = fmaxf(mt, s[t][i]);
        const float m2 = fmaxf(st.m[i], mt);
        alpha[i] = __expf(st.m[i] - m2);
        float ls = 0.f;
#pragma unroll
        for (int t = 0; t < NR; t++) {
            pr[t][i] = __expf(s[t][i] - m2);
            ls += pr[t][i];
        }
        st.l[i] = fmaf(st.l[i], alpha[i], ls);
        st.m[i] = m2;
    }
    float aall[GP];
    quad_gather<GP>(alpha, aall);
#pragma unroll
    for (int h = 0; h < GP; h++) {
        st.S[h] *= aall[h];
#pragma unroll
        for (int e = 0; e < 8; e++) st.O[h][e] *= aall[h];
    }
#pragma unroll
    for (int t = 0; t < NR; t++) {
        if (!live[t]) continue;
        float n[8], pall[GP];
        unpack8(r[t].vd, n);
        const float vs = half_bits_to_f32(r[t].vs);
        quad_gather<GP>(pr[t], pall);
#pragma unroll
        for (int h = 0; h < GP; h++) {
            const float pd = pall[h] * vs;
            st.S[h] += pd;
#pragma unroll
            for (int e = 0; e < 8; e++) st.O[h][e] = fmaf(pd, n[e], st.O[h][e]);
        }
    }
}

// Device-scope traffic between workgroups that may sit on different XCDs (each
// with its own L2): the partials are written and read with agent-scope atomic
// accesses, which go through to the memory side instead of staying in the
// writer's L2, so that the hand-over needs no L2 write-back / invalidate
// (a full __threadfence() costs about a microsecond per workgroup here, and
// they serialise).
__device__ __forceinline__ void st_agent(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float ld_agent(const float *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// One wave computes, for one head, the log-sum-exp weights of n partial states
// whose (m, l) pairs sit `stride` floats apart: w[i] = exp(m_i - M), and
// (M, L = sum w_i l_i) into ML.  Lane-parallel, so no chain of LDS round trips.
// w is written up to npad >= n with zeros, so that the consumer needs no bound checks.
__device__ __forceinline__ void merge_weights(const float *ml, int stride, int n, int npad, float *w, float *ML, int lane)
{
    float m = -1.0e30f;
    for (int i = lane; i < n; i += 64) m = fmaxf(m, ml[i * stride]);
    const float M = wave_max(m);
    float ls = 0.f;
    for (int i = lane; i < npad; i += 64) {
        const int ic = min(i, n - 1);
        const float wt = i < n ? __expf(ml[ic * stride] - M) : 0.f;
        w[i] = wt;
        ls = fmaf(wt, ml[ic * stride + 1], ls);
    }
    const float L = wave_sum(ls);
    if (lane == 0) { ML[0] = M; ML[1] = L; }
}

// RMSNorm (optionally weighted), optional RoPE, of one head already in
// registers as element lane + 64*j
template <int HD>
__device__ __forceinline__ void norm_rope_regs(const float (&xv)[HD / 64], const float *wv, const float *cs, const float *sn,
                                               float eps, float (&ro)[HD / 64])
{
    constexpr int PER = HD / 64;
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) ss += xv[j] * xv[j];
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)HD + eps);
    float nv[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) nv[j] = wv ? xv[j] * inv * wv[j] : xv[j] * inv;
    if (!cs) {
#pragma unroll
        for (int j = 0; j < PER; j++) ro[j] = nv[j];
        return;
    }
#pragma unroll
    for (int j = 0; j < PER / 2; j++) {
        const float u = nv[j], vv = nv[j + PER / 2];
        ro[j] = u * cs[j] - vv * sn[j];
        ro[j + PER / 2] = u * sn[j] + vv * cs[j];
    }
}

// Slots of unequal length share a launch's P = nwg * n_slots workgroups by length: ceil(tlen / c) to a slot (at
// least one), with c = ceil(T / (P - n_slots)) rows, so that they sum to at most P; what is left over exits.
// Every workgroup derives the same table from the slots' lengths.  Slot s's partitions are the consecutive
// flat indices from the sum of its predecessors' counts, and its records sit in that order.
// round > 1: the rows per partition are rounded up to a multiple of it (the matrix-core form works in tiles of rows).
//
// A whole wave works the deal out at once, as one short chain of vector instructions (a launch of this kind is a chain
// of dependent steps: the first form of this routine -- two loops over the slots with a lane read each, three integer
// divisions, uniform values moving between the vector and the scalar unit -- was 0.8 us of the merge launch and as much
// of the row launch): lane s of every 16-lane row holds slot s's length (one load per lane, all in flight together), the
// total is a row sum that every lane ends up with, the two divisions go through a reciprocal with an exact fix-up and no
// branch, the running count of partitions is a prefix sum over the row (row shifts), the owner of a flat index is the
// number of slots whose running count does not exceed it, and only the answer is read out of the lanes.
// `f` is the flat partition index of the caller (wave-uniform); slot < 0 says that the deal has fewer partitions than
// that.  With `of_slot` >= 0 the answer is that slot's range of partitions instead (first, nparts).  Up to 64 slots
// (more than 16: one slot per lane of the wave, and the rows' totals cross through lane reads); `round` is a power of
// two; lengths and their total below 2^22.
struct Deal {
    int slot, part, nparts, first, tlen, start, c;
};
// ceil(a / b) with rb ~ 1 / b (one ulp): the truncated product is off by one at most, either way, and the remainder
// against it says which
__device__ __forceinline__ uint32_t ceil_div_rcp(uint32_t a, uint32_t b, float rb)
{
    const uint32_t q = (uint32_t)((float)a * rb);
    const int32_t t = (int32_t)(a - q * b);      // in (-b, 2b)
    return q + (t > 0 ? 1u : 0u) + (t > (int32_t)b ? 1u : 0u);
}
template <int SHR>
__device__ __forceinline__ int row_shr_i32(int v)   // lane i of a 16-lane row reads lane i - SHR of it, 0 below the row's start
{
    return __builtin_amdgcn_update_dpp(0, v, 0x110 + SHR, 0xF, 0xF, true);
}
__device__ __forceinline__ Deal deal_wave(const float *meta, int stride, int n_slots, int nwg, int round, int f, int of_slot = -1)
{
    const int lane = threadIdx.x & 63;
    const bool wide = n_slots > 16;
    const int sl = wide ? lane : (lane & 15), ls = min(sl, n_slots - 1);
    const bool live = sl < n_slots;
    const float lenf = meta[(size_t)ls * stride];
    const int st = (int)meta[(size_t)ls * stride + 1];
    const uint32_t spare = (uint32_t)max(1, nwg * n_slots - n_slots);
    const float rspare = __builtin_amdgcn_rcpf((float)spare);
    const uint32_t len = live ? (uint32_t)lenf : 0u;
    float Tf = row16_sum(live ? lenf : 0.f);      // (integers below 2^24: exact in f32)
    if (wide) {
        const float a = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(Tf), 0)), b = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(Tf), 16));
        const float c = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(Tf), 32)), d = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(Tf), 48));
        Tf = (a + b) + (c + d);
    }
    uint32_t c = max(1u, ceil_div_rcp((uint32_t)Tf, spare, rspare));
    c = (c + (uint32_t)round - 1u) & ~((uint32_t)round - 1u);
    const int n = live ? (int)max(1u, ceil_div_rcp(len, c, __builtin_amdgcn_rcpf((float)c))) : 0;
    // partitions up to and with each lane's slot
    int incl = n;
    incl += row_shr_i32<1>(incl);
    incl += row_shr_i32<2>(incl);
    incl += row_shr_i32<4>(incl);
    incl += row_shr_i32<8>(incl);
    if (wide) {
        const int t0 = __builtin_amdgcn_readlane(incl, 15), t1 = __builtin_amdgcn_readlane(incl, 31), t2 = __builtin_amdgcn_readlane(incl, 47);
        incl += lane >= 48 ? t0 + t1 + t2 : lane >= 32 ? t0 + t1 : lane >= 16 ? t0 : 0;
    }
    const int excl = incl - n;
    const int slot = of_slot >= 0 ? of_slot : (int)__builtin_popcountll(__builtin_amdgcn_ballot_w64(live && (wide || lane < 16) && incl <= f));
    Deal d{-1, 0, 0, 0, 0, 0, __builtin_amdgcn_readfirstlane((int)c)};
    if (slot < n_slots) {
        d.slot = slot;
        d.first = __builtin_amdgcn_readlane(excl, slot);
        d.nparts = __builtin_amdgcn_readlane(n, slot);
        d.part = f - d.first;
        d.tlen = __builtin_amdgcn_readlane((int)len, slot);
        d.start = __builtin_amdgcn_readlane(st, slot);
    }
    return d;
}

// The merge of a balanced launch's partials, as a second launch: with a hundred partitions to a long slot a
// single (last-arriving) workgroup would pull them all through one compute unit.  A workgroup takes 64
// dimensions of one (slot, head): thread (g, j) = (tid / 16, tid % 16) holds a float4 of them for the partitions
// g, g + 16, ..., so that a slot's whole set of records is requested in one go, while the weights
// exp(m_i - M) are still being worked out.  grid = (n_q * HD / 64, n_slots), 256 threads.
// Records of a balanced launch: values [flat][n_q][HD], then (m, l) [flat][n_q][2].
// xp != nullptr: the result leaves as the prepared operand of a decode round's GEMM (row = slot, n_q * HD columns) instead
// of f32 rows: a workgroup's 64 dimensions are eight fragment lanes and two sub-blocks of sums of its row.
template <int HD>
__global__ __launch_bounds__(256) void sdpa_dealt_merge_kernel(const float *tmp, const float *meta, int meta_stride, int nwg,
                                                                int n_q, float *out, int round, _Float16 *xp)
{
    constexpr int kMaxParts = 16 * 64;   // host-checked: nwg * n_slots
    constexpr int QB = 8;                // partitions per thread in flight
    __shared__ float w[kMaxParts];
    __shared__ float red[8];
    __shared__ __attribute__((aligned(16))) float part4[16][64];
    const int head = blockIdx.x / (HD / 64), dq = blockIdx.x % (HD / 64), slot = blockIdx.y, S = gridDim.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = tid >> 4, j = tid & 15;
    const Deal deal = deal_wave(meta, meta_stride, S, nwg, round, 0, slot);
    const int first = deal.first, n = deal.nparts;
    const size_t P = (size_t)nwg * S;
    const float *ov = tmp + ((size_t)first * n_q + head) * HD + dq * 64 + 4 * j;   // + i * n_q * HD
    const float *ml = tmp + P * n_q * HD + ((size_t)first * n_q + head) * 2;      // + i * n_q * 2
    const size_t ops = (size_t)n_q * HD, mps = (size_t)n_q * 2;
    // a thread's (m, l) pairs first (loads come back in the order they went out, and the weights are made of these),
    // read once and kept in registers across the barrier; then the first batch of values, requested before the
    // weights exist
    float2 p2[kMaxParts / 256];
#pragma unroll
    for (int u = 0; u < kMaxParts / 256; u++) p2[u] = ldg_f2(ml + (size_t)min(tid + 256 * u, n - 1) * mps, 0);
    float4 v[QB];
#pragma unroll
    for (int u = 0; u < QB; u++) v[u] = ldg_f4(ov + (size_t)min(g + 16 * u, n - 1) * ops, 0);
    float m = -1.0e30f;
#pragma unroll
    for (int u = 0; u < kMaxParts / 256; u++)
        if (tid + 256 * u < n) m = fmaxf(m, p2[u].x);
    m = wave_max(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
    const float M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float ls = 0.f;
#pragma unroll
    for (int u = 0; u < kMaxParts / 256; u++) {
        const int i = tid + 256 * u;
        if (i < n) {
            const float wt = __expf(p2[u].x - M);
            w[i] = wt;
            ls = fmaf(wt, p2[u].y, ls);
        }
    }
    ls = wave_sum(ls);
    if (lane == 0) red[4 + wave] = ls;
    __syncthreads();
    const float L = (red[4] + red[5]) + (red[6] + red[7]);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int i0 = 0; i0 < n; i0 += 16 * QB) {
        if (i0) {
#pragma unroll
            for (int u = 0; u < QB; u++) v[u] = ldg_f4(ov + (size_t)min(i0 + g + 16 * u, n - 1) * ops, 0);
        }
#pragma unroll
        for (int u = 0; u < QB; u++) {
            const int i = i0 + g + 16 * u;
            const float wt = i < n ? w[i] : 0.f;
            acc.x = fmaf(wt, v[u].x, acc.x);
            acc.y = fmaf(wt, v[u].y, acc.y);
            acc.z = fmaf(wt, v[u].z, acc.z);
            acc.w = fmaf(wt, v[u].w, acc.w);
        }
    }
    *reinterpret_cast<float4 *>(&part4[g][4 * j]) = acc;
    __syncthreads();
    if (tid < 64) {
        float sum = 0.f;
#pragma unroll
        for (int q = 0; q < 16; q++) sum += part4[q][tid];
        const float y = sum / L;
        if (!xp) {
            out[((size_t)slot * n_q + head) * HD + dq * 64 + tid] = y;
        } else {
            // (one wave: its LDS operations complete in order; the fences keep the compiler from moving them)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            part4[0][tid] = y;
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            const int cols = n_q * HD, c0 = head * HD + dq * 64 + 8 * (tid & 7);
            float f[8];
#pragma unroll
            for (int e = 0; e < 8; e++) f[e] = part4[0][8 * (tid & 7) + e];
            h8 oh, ol;
            float sh, sl;
            round_split8(f, oh, ol, sh, sl);
            sh += dpp_f32<0xB1>(sh);      // the four lanes of a sub-block
            sh += dpp_f32<0x4E>(sh);
            sl += dpp_f32<0xB1>(sl);
            sl += dpp_f32<0x4E>(sl);
            if (tid < 8) {
                const int j = c0 / 8;
                const size_t frag = (size_t)(j >> 1) * 64 + slot + 32 * (j & 1);
                reinterpret_cast<h8 *>(xp)[frag] = oh;
                reinterpret_cast<h8 *>(xp)[frag + 16] = ol;
                if ((tid & 3) == 0) round_store_sums(xp, cols, slot, c0 / 32, sh, sl);
            }
        }
    }
}

// Per-token records of a chunk of consecutive prompt tokens (crates/ksearch_codegen/src/lower.rs:4961-4983): token i
// attends tlen_i = min(tlen0 + i, window) rows from start_i = tlen0 + i - tlen_i; in: {tlen0, -, window}.
__global__ void sdpa_batch_meta_kernel(const float *meta, float *tok_meta, int n_tok)
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

// grid = (nwg, n_kv, n_slots)
// FUSED: the decode step's form (p.fused), a kernel of its own: with the choice made at compile time the front of
// either form is one run of loads without the other form's branches in it, and the wait for the record in front of
// the rows counts exactly the loads behind it.
template <int HD, int GP, int NW, bool FUSED>
__global__ __launch_bounds__(NW * 64) void sdpa_lanes_kernel(LaneParams p_in)
{
    touch_lane_params(p_in);
    LaneParams p = p_in;
    p.fused = FUSED;
    if (FUSED) {   // one sequence, its own cache, partitions of equal size: what the other kinds' fields would select is not compiled in
        p.balance = 0;
        p.slot_ids = nullptr;
        p.kv_shared = 0;
    }
    constexpr int LPR = HD / 8, RPS = 64 / LPR, HPL = (GP + 3) / 4, NSLOT = NW * RPS, NT = NW * 64;
    constexpr int MLF = (2 * GP + 3) / 4 * 4;  // the (m, l) pairs in front of a row group's values, padded so that those stay 16-byte aligned
    constexpr int SLOTF = GP * HD + MLF;      // floats of one row group's state
    constexpr int ROWB = HD / 32 * 18;
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *qs = smem;                            // [GP][HD]            fused prologue only
    float *slots = qs + GP * HD;                 // [NSLOT][SLOTF]      later [groups][nwg] merge weights
    float *wts = slots + NSLOT * SLOTF;          // [GP][NSLOT]
    float *mlh = wts + GP * NSLOT;               // [GP][2]
    uint8_t *newrow = reinterpret_cast<uint8_t *>(mlh + 2 * GP);   // K row, V row of the appended position
    __shared__ int last_flag;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    KSH_STAMP_BEGIN
    const int j = lane % LPR, sub = lane / LPR, b = j >> 2, w = j & 3, c = w;
    int part = blockIdx.x, slot = FUSED ? 0 : blockIdx.z, nparts = p.nwg;
    const int kvh = p.n_kv == 1 ? 0 : blockIdx.y / p.hsplit, hg = blockIdx.y - kvh * p.hsplit;   // (one kv head: no division in the front)
    const int groups = p.groups;
    const int head0 = (kvh * p.hsplit + hg) * groups;   // first q head of this workgroup
    // partial records: rec(head, part) = tmp + rec_base + head * rec_hs + part * rec_ps
    size_t rec_base = (size_t)slot * p.n_q * p.nwg * (HD + 2), rec_hs = (size_t)p.nwg * (HD + 2), rec_ps = HD + 2;
    if (p.balance) {
        const Deal d = deal_wave(p.meta, p.meta_stride, (int)gridDim.z, p.nwg, 1, blockIdx.z * p.nwg + blockIdx.x);
        if (d.slot < 0) return;   // left over
        slot = d.slot; part = d.part; nparts = d.nparts;
        rec_base = (size_t)d.first + part;   // flat partition index: values [flat][n_q][HD], then (m, l) [flat][n_q][2]
    }

    const size_t slot_bytes = p.kv_shared ? 0 : p.slot_stride ? p.slot_stride : (size_t)p.max_t * p.n_kv * ROWB;
    const size_t kv_slot = p.slot_ids ? (size_t)max((int)p.slot_ids[slot], 0) : (size_t)slot;
    const uint8_t *kbase = p.k + kv_slot * slot_bytes + (size_t)kvh * ROWB + 18 * b;
    const uint8_t *vbase = p.v + kv_slot * slot_bytes + (size_t)kvh * ROWB + 18 * b;
    const size_t row_stride = (size_t)p.n_kv * ROWB;
    const float *qg = p.q + ((size_t)slot * p.n_q + head0) * HD;

    auto load_row_at = [&](int first, int t) {
        RowRegs r;
        const size_t off = (size_t)(first + t) * row_stride;
        r.kd = ld32_a2(kbase + off + 2 + 4 * w);
        r.ks = ld16_a2(kbase + off);
        r.vd = ld32_a2(vbase + off + 2 + 4 * w);
        r.vs = ld16_a2(vbase + off);
        return r;
    };

    // The fused decode step deals rows to the partitions in groups of GRP (one step of the workgroup), round
    // robin: which rows a workgroup starts with then does not depend on the attended length, and its first
    // loads go out before the length has come back from memory (rows past the end are read -- the cache is
    // max_t rows long -- and dropped).  The other kinds give every partition one contiguous range.
    constexpr int GRP = NW * RPS, TILE = GRP * kRT;
    const bool dealt = p.fused != 0;
    // The last partition of a fused step takes no cached rows: it norms, ropes and packs the new K / V row,
    // stores it and attends it.  That work (0.7 us) would otherwise sit in front of one row partition's rows.
    const bool appender = p.nwg > 1 && !p.no_append;          // (nothing to append: every partition takes rows)
    const int rparts = appender ? p.nwg - 1 : p.nwg;          // partitions that share the cached rows
    const bool has_rows = !appender || part < p.nwg - 1;
    auto dealt_row = [&](int it, int t) { return ((it * kRT + t) * rparts + part) * GRP + wave * RPS + sub; };   // relative to start
    RowRegs cur[kRT], nxt[kRT];

    // Vector loads return in the order they were issued: the length and position first, then what the fused
    // prologue needs (raw q / k / v of this workgroup's head tasks, the norm weights, the position's rope row
    // when it is given directly), then the rows.
    // The record is read with vector loads (opaque_zero_v) and without a branch around the position (the other kinds'
    // record may end after three floats, so they read its first again): as scalar loads, or behind a branch, the
    // values -- which end up in scalar registers -- were waited for right here, two memory round trips one after the
    // other in front of every other load of the launch.
    const float *meta = p.meta + (size_t)slot * p.meta_stride + opaque_zero_v();
    const float meta_tlen = meta[0], meta_start = meta[1], meta_pos = meta[dealt ? 3 : 0];
    // head tasks: q heads 0..groups-1, then K and V (used by the owner only); a wave takes tasks wave, wave+NW, ...
    constexpr int PER = HD / 64, MAXT = GP / NW + 1;
    float xv[MAXT][PER], wq[PER], wk[PER], cs[PER / 2], sn[PER / 2];
    if (dealt) {
#pragma unroll
        for (int t = 0; t < MAXT; t++) {
            const int task = min(wave + t * NW, groups + 1);
            const float *src = task < groups ? qg + (size_t)task * HD
                                             : (task == groups ? p.k_raw : p.v_raw) + (size_t)kvh * HD;
#pragma unroll
            for (int jj = 0; jj < PER; jj++) xv[t][jj] = src[lane + 64 * jj];
        }
#pragma unroll
        for (int jj = 0; jj < PER; jj++) {
            wq[jj] = p.qw[lane + 64 * jj];
            wk[jj] = p.kw[lane + 64 * jj];
        }
        if (p.rope_row) {
#pragma unroll
            for (int jj = 0; jj < PER / 2; jj++) {
                cs[jj] = p.rope[lane + 64 * jj];
                sn[jj] = p.rope[HD / 2 + lane + 64 * jj];
            }
        }
#pragma unroll
        for (int t = 0; t < kRT; t++) cur[t] = load_row_at(0, min(dealt_row(0, t), p.max_t - 1));   // as if start == 0
    }
    KSH_STAMP(1);
    __builtin_amdgcn_sched_barrier(0);   // the record's first use stays behind the front's last load
    const int tlen = (int)meta_tlen, start = (int)meta_start;
    KSH_STAMP_USE(tlen);
    KSH_STAMP(2);
    const int chunk = (tlen + nparts - 1) / nparts;
    const int p0 = part * chunk;
    int p1 = min(p0 + chunk, tlen);
    auto load_row = [&](int t) { return load_row_at(start, t); };

    // the row this step appends is attended from LDS by the last partition (other kinds: by the one whose range holds it)
    const bool owner = p.fused && !p.no_append && (p.nwg == 1 || part == p.nwg - 1);   // (p.fused kinds are always dealt)
    const int tend = p.no_append ? tlen : tlen - 1;   // dealt: rows [0, tend) come from the cache
    if (dealt) {
        if (start != 0) {                // a window that has begun to slide: ask again
#pragma unroll
            for (int t = 0; t < kRT; t++) cur[t] = load_row(min(dealt_row(0, t), p.max_t - 1 - start));
        }
    } else {
        if (owner) p1 = min(p1, tlen - 1);
        const int last = max(p1 - 1, p0 < tlen ? p0 : 0);   // an empty partition still loads (a valid row) and drops it
#pragma unroll
        for (int t = 0; t < kRT; t++) cur[t] = load_row(min(p0 + (t * NW + wave) * RPS + sub, last));
    }

    // ---- q into registers (and, fused, the new K/V row into the cache) -------
    float qv[GP][8], Sq[GP];
    if (p.fused) {
        const int pos = dealt ? min(max((int)meta_pos, 0), p.max_t - 1) : 0;
        const int ntask = groups + (owner ? 2 : 0);
        if (!p.rope_row) {
            const float *rope = p.rope + (size_t)pos * HD;
#pragma unroll
            for (int jj = 0; jj < PER / 2; jj++) {
                cs[jj] = rope[lane + 64 * jj];
                sn[jj] = rope[HD / 2 + lane + 64 * jj];
            }
        }
#pragma unroll
        for (int t = 0; t < MAXT; t++) {
            const int task = wave + t * NW;
            if (task >= ntask) continue;
            float ro[PER];
            if (task < groups) {
                norm_rope_regs<HD>(xv[t], wq, cs, sn, p.eps, ro);
#pragma unroll
                for (int jj = 0; jj < PER; jj++) qs[task * HD + lane + 64 * jj] = ro[jj] * p.scale;
            } else {
                const bool is_k = task == groups;
                if (is_k) norm_rope_regs<HD>(xv[t], wk, cs, sn, p.eps, ro);
                else norm_rope_regs<HD>(xv[t], nullptr, nullptr, nullptr, p.eps, ro);
                uint8_t *dst = newrow + (is_k ? 0 : ROWB);
#pragma unroll
                for (int jj = 0; jj < PER; jj++) pack_q40_group(ro[jj], lane & 31, dst + (2 * jj + (lane >> 5)) * 18, true);
            }
        }
        __syncthreads();
        if (owner && hg == 0) {
            // the appended row goes to the cache; the owners attend it from LDS
            const size_t off = kv_slot * slot_bytes + ((size_t)pos * p.n_kv + kvh) * ROWB;
            for (int i = tid; i < ROWB; i += NT) {   // (one pass, except 512-wide heads on four waves)
                if (i < ROWB / 2)
                    reinterpret_cast<uint16_t *>(p.k_w + off)[i] = reinterpret_cast<const uint16_t *>(newrow)[i];
                else
                    reinterpret_cast<uint16_t *>(p.v_w + off)[i - ROWB / 2] = reinterpret_cast<const uint16_t *>(newrow + ROWB)[i - ROWB / 2];
            }
        }
#pragma unroll
        for (int h = 0; h < GP; h++) {
            const float4 a = h < groups ? *reinterpret_cast<const float4 *>(qs + h * HD + 32 * b + 4 * w) : make_float4(0.f, 0.f, 0.f, 0.f);
            const float4 d = h < groups ? *reinterpret_cast<const float4 *>(qs + h * HD + 32 * b + 16 + 4 * w) : make_float4(0.f, 0.f, 0.f, 0.f);
            qv[h][0] = a.x; qv[h][1] = a.y; qv[h][2] = a.z; qv[h][3] = a.w;
            qv[h][4] = d.x; qv[h][5] = d.y; qv[h][6] = d.z; qv[h][7] = d.w;
        }
    } else {
#pragma unroll
        for (int h = 0; h < GP; h++) {
            const float *qh = qg + (size_t)min(h, groups - 1) * HD + 32 * b + 4 * w;
            const float4 a = *reinterpret_cast<const float4 *>(qh), d = *reinterpret_cast<const float4 *>(qh + 16);
            const float sc = h < groups ? p.scale : 0.f;
            qv[h][0] = a.x * sc; qv[h][1] = a.y * sc; qv[h][2] = a.z * sc; qv[h][3] = a.w * sc;
            qv[h][4] = d.x * sc; qv[h][5] = d.y * sc; qv[h][6] = d.z * sc; qv[h][7] = d.w * sc;
        }
    }
#pragma unroll
    for (int h = 0; h < GP; h++)
        Sq[h] = ((qv[h][0] + qv[h][1]) + (qv[h][2] + qv[h][3])) + ((qv[h][4] + qv[h][5]) + (qv[h][6] + qv[h][7]));
    KSH_STAMP_USE(Sq[0]);
    KSH_STAMP(3);

    State<GP> st;
#pragma unroll
    for (int i = 0; i < HPL; i++) { st.m[i] = -1.0e30f; st.l[i] = 0.f; }
#pragma unroll
    for (int h = 0; h < GP; h++) {
        st.S[h] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) st.O[h][e] = 0.f;
    }

    // ---- the partition's rows: kRT steps of RPS rows per wave at a time -----
    if (dealt) {
        for (int it = 0; has_rows && (it * kRT * rparts + part) * GRP < tend; it++) {
            bool valid[kRT], live[kRT];
#pragma unroll
            for (int t = 0; t < kRT; t++) {
                valid[t] = dealt_row(it, t) < tend;
                live[t] = ((it * kRT + t) * rparts + part) * GRP + wave * RPS < tend;
                nxt[t] = load_row(min(dealt_row(it + 1, t), p.max_t - 1 - start));   // unconditional: keeps the wait counts exact
            }
            process_rows<HD, GP, kRT>(cur, valid, live, qv, Sq, st, c);
#pragma unroll
            for (int t = 0; t < kRT; t++) cur[t] = nxt[t];
        }
    } else if (p0 < p1) {
        for (int base = p0; base < p1; base += TILE) {
            bool valid[kRT], live[kRT];
#pragma unroll
            for (int t = 0; t < kRT; t++) {
                const int row = base + (t * NW + wave) * RPS + sub;
                valid[t] = row < p1;
                live[t] = base + (t * NW + wave) * RPS < p1;
                nxt[t] = load_row(min(row + TILE, p1 - 1));   // unconditional: keeps the wait counts exact
            }
            process_rows<HD, GP, kRT>(cur, valid, live, qv, Sq, st, c);
#pragma unroll
            for (int t = 0; t < kRT; t++) cur[t] = nxt[t];
        }
    }
    if (p.fused && owner) {
        RowRegs r[1];
        const uint16_t *kr = reinterpret_cast<const uint16_t *>(newrow + 18 * b);
        const uint16_t *vr = reinterpret_cast<const uint16_t *>(newrow + ROWB + 18 * b);
        r[0].ks = kr[0];
        r[0].kd = (uint32_t)kr[1 + 2 * w] | ((uint32_t)kr[2 + 2 * w] << 16);
        r[0].vs = vr[0];
        r[0].vd = (uint32_t)vr[1 + 2 * w] | ((uint32_t)vr[2 + 2 * w] << 16);
        const bool valid[1] = {wave == 0 && sub == 0}, live[1] = {wave == 0};
        process_rows<HD, GP, 1>(r, valid, live, qv, Sq, st, c);
    }

    KSH_STAMP_USE(st.O[0][0]);
    KSH_STAMP(4);
    // ---- fold the row groups of this workgroup ------------------------------
    {
        float *my = slots + (wave * RPS + sub) * SLOTF;
        if (j < 4) {
#pragma unroll
            for (int i = 0; i < HPL; i++) {
                const int h = head_of<GP>(c, i);
                my[2 * h] = st.m[i];
                my[2 * h + 1] = st.l[i];
            }
        }
#pragma unroll
        for (int h = 0; h < GP; h++) {
            if (h >= groups) break;   // heads past the workgroup's share carry nothing
            const float o8 = 8.f * st.S[h];
            float *o = my + MLF + h * HD + 32 * b + 4 * w;
            *reinterpret_cast<float4 *>(o) = make_float4(st.O[h][0] - o8, st.O[h][1] - o8, st.O[h][2] - o8, st.O[h][3] - o8);
            *reinterpret_cast<float4 *>(o + 16) = make_float4(st.O[h][4] - o8, st.O[h][5] - o8, st.O[h][6] - o8, st.O[h][7] - o8);
        }
    }
    __syncthreads();
    {
        // One barrier: every thread works out its head's weights exp(m_s - M) itself (NSLOT broadcast reads and
        // exponentials) instead of waiting for a wave per head to publish them behind a second barrier.
        // Fully unrolled: one wave per SIMD has nothing to hide an LDS round trip behind, so all reads go out first.
        // (With four outputs per thread -- eight heads -- that is four times the exponentials: there a wave per head
        // publishes the weights and a second barrier follows, 1 us less at 4 slots x 64 partitions.)
        constexpr int OBW = GP * HD >= NT ? GP * HD / NT : 1;
        constexpr bool kOwnWeights = OBW <= 2;
        float accw[OBW], Mh[OBW], Lh[OBW];
        if (!kOwnWeights) {
            for (int h = wave; h < groups; h += NW) merge_weights(slots + 2 * h, SLOTF, NSLOT, NSLOT, wts + h * NSLOT, mlh + 2 * h, lane);
            __syncthreads();
        }
#pragma unroll
        for (int ob = 0; ob < OBW; ob++) {
            accw[ob] = 0.f; Mh[ob] = 0.f; Lh[ob] = 1.f;
            if (ob * NT >= groups * HD) continue;   // (the same for the whole workgroup)
            const int o = min(tid + ob * NT, groups * HD - 1), h = o / HD, d = o % HD;
            float M = -1.0e30f, L = 0.f, a = 0.f;
            if (kOwnWeights) {
                float mv[NSLOT];
#pragma unroll
                for (int s = 0; s < NSLOT; s++) { mv[s] = slots[s * SLOTF + 2 * h]; M = fmaxf(M, mv[s]); }
#pragma unroll
                for (int s = 0; s < NSLOT; s++) {
                    const float wt = __expf(mv[s] - M);
                    L = fmaf(wt, slots[s * SLOTF + 2 * h + 1], L);
                    a = fmaf(wt, slots[s * SLOTF + MLF + h * HD + d], a);
                }
            } else {
#pragma unroll
                for (int s = 0; s < NSLOT; s++) a = fmaf(wts[h * NSLOT + s], slots[s * SLOTF + MLF + h * HD + d], a);
                M = mlh[2 * h];
                L = mlh[2 * h + 1];
            }
            accw[ob] = a; Mh[ob] = M; Lh[ob] = L;
        }
        KSH_STAMP(5);
#pragma unroll
        for (int ob = 0; ob < OBW; ob++) {
            const int o = tid + ob * NT;
            if (o >= groups * HD) continue;
            const int h = o / HD, d = o % HD, head = head0 + h;
            if (p.mode == kModeDirect) {
                p.out[((size_t)slot * p.n_q + head) * HD + d] = accw[ob] / Lh[ob];
            } else if (p.balance) {
                const size_t r = rec_base * p.n_q + head;
                float *ml = p.tmp + (size_t)gridDim.z * p.nwg * p.n_q * HD;
                p.tmp[r * HD + d] = accw[ob];
                if (d == 0) { ml[2 * r] = Mh[ob]; ml[2 * r + 1] = Lh[ob]; }
            } else if (p.mode == kModeSplitPart) {
                const size_t r = ((size_t)slot * p.n_q + head) * p.nwg + part;
                float *ml = p.tmp + (size_t)gridDim.z * p.n_q * p.nwg * HD;
                p.tmp[r * HD + d] = accw[ob];
                if (d == 0) { ml[2 * r] = Mh[ob]; ml[2 * r + 1] = Lh[ob]; }
            } else {
                float *rec = p.tmp + rec_base + head * rec_hs + part * rec_ps;
                st_agent(rec + 2 + d, accw[ob]);
                if (d == 0) { st_agent(rec, Mh[ob]); st_agent(rec + 1, Lh[ob]); }
            }
        }
    }
    KSH_STAMP_FLUSH(p.fused ? 1 : 0, KSH_LANES_WAVE, 6);
    if (p.mode != kModeMerge) return;

    // ---- the last partition to arrive folds the partials (lower.rs:5897-6087) -
    // every thread's record stores have completed (they are write-through) before the barrier lets thread 0 count
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0) {
        const uint32_t arrived = __hip_atomic_fetch_add(&p.counters[slot * gridDim.y + blockIdx.y], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_flag = arrived == (uint32_t)nparts - 1u;
    }
    __syncthreads();
    if (!last_flag) return;
    // The records come from the memory side (about a microsecond away), so all of
    // a thread's loads -- its output elements' values from up to QB partitions,
    // then its share of the (m, l) pairs -- are issued before anything is used.
    constexpr int QB = 16, OB = GP * HD >= NT ? GP * HD / NT : 1;   // partitions in flight x output elements per thread
    const int nwgp = (nparts + QB - 1) / QB * QB;
    float *w2 = slots;                          // [groups][nwgp] weights, zero past nparts
    float *mq = slots + groups * nwgp;          // [groups][nparts][2]
    const float *recs = p.tmp + rec_base + head0 * rec_hs;
    float acc[OB], val[OB][QB];
#pragma unroll
    for (int ob = 0; ob < OB; ob++) {
        acc[ob] = 0.f;
        const int o = min(tid + ob * NT, groups * HD - 1), h = o / HD, d = o % HD;
        const float *rh = recs + h * rec_hs + 2 + d;
#pragma unroll
        for (int u = 0; u < QB; u++) val[ob][u] = ld_agent(rh + (size_t)min(u, nparts - 1) * rec_ps);
    }
    for (int i = tid; i < groups * nparts; i += NT) {
        const int h = i / nparts, q = i - h * nparts;
        const float *rec = recs + h * rec_hs + q * rec_ps;
        mq[2 * i] = ld_agent(rec);
        mq[2 * i + 1] = ld_agent(rec + 1);
    }
    __syncthreads();
    for (int h = wave; h < groups; h += NW) merge_weights(mq + 2 * h * nparts, 2, nparts, nwgp, w2 + h * nwgp, mlh + 2 * h, lane);
    __syncthreads();
    for (int q0 = 0; q0 < nparts; q0 += QB) {
#pragma unroll
        for (int ob = 0; ob < OB; ob++) {
            const int o = min(tid + ob * NT, groups * HD - 1), h = o / HD, d = o % HD;
            if (q0) {
                const float *rh = recs + h * rec_hs + 2 + d;
#pragma unroll
                for (int u = 0; u < QB; u++) val[ob][u] = ld_agent(rh + (size_t)min(q0 + u, nparts - 1) * rec_ps);
            }
#pragma unroll
            for (int u = 0; u < QB; u++) acc[ob] = fmaf(w2[h * nwgp + q0 + u], val[ob][u], acc[ob]);
        }
    }
#pragma unroll
    for (int ob = 0; ob < OB; ob++) {
        const int o = tid + ob * NT;
        if (o < groups * HD) {
            const int h = o / HD, d = o % HD;
            p.out[((size_t)slot * p.n_q + head0 + h) * HD + d] = acc[ob] / mlh[2 * h + 1];
        }
    }
    if (tid == 0) __hip_atomic_store(&p.counters[slot * gridDim.y + blockIdx.y], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
}

// ---------------------------------------------------------------------------------------------------------------
// Matrix-core form of the row phase (split-KV partials), for head size 256 and up to 8 q heads per kv head.
//
// The vector-ALU form above spends ~200 instructions per KV row and wave (8 FMAs per head and dword for the scores,
// as many for P.V, the butterflies between them).  Here both products run on v_mfma_f32_16x16x32_f16 with exact
// operands and the vector ALU only converts and scales:
//   - a wave takes tiles of 32 rows.  The tile's K and V bytes are copied to the wave's LDS strip with whole 128-bit
//     loads (a row is 9 of them), and its 2 x 256 block scales are converted once into two f32 tables.
//   - scores: per 16 rows and Q4_0 block b, A = the block's codes as f16 (16 + n: the nibble ORed into the mantissa
//     of 16.0, two ops per pair), B = the 8 heads' q of that block as f16 hi parts in columns 0..7 and lo parts in
//     columns 8..15 (22 bits of q; fixed for the whole launch).  The 16 x 16 result is exact up to f32 summation;
//     S += d[row, b] * (C - 24 * sum_b(q)) applies the block scale and takes the 16 + 8 offset out again.
//   - softmax bookkeeping on the accumulator layout (a lane holds 8 rows of one column); hi and lo columns are
//     added across lanes, the running maximum is shared across the wave.
//   - P.V: A = P' = p * dv[row, b] per block b, again split hi | lo over the 16 output rows, which needs no data
//     movement because the accumulator layout of the scores is the A-operand layout of this product when k runs
//     over a lane's own rows; B = the V codes of 8 rows and one element per lane, gathered bytewise from the LDS
//     strip (the one transposition of the kernel).  A third product against ones keeps sum(P') per block for the
//     code offset.
// A workgroup folds its waves' states through LDS and writes one partial record per head, in the layout of the
// vector-ALU form, so the same merge kernels follow.
typedef _Float16 h8v __attribute__((ext_vector_type(8)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef _Float16 h4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
// A workgroup takes rounds of 128 rows: four waves with tiles of 32 rows (the P.V product is a full 16x16x32), or eight
// waves with tiles of 16 (16x16x16: half the work per wave and two waves per SIMD, for launches whose partitions are a
// round or two and whose time is therefore one wave's chain of dependent steps).
constexpr int kMfmaRound = 128;

__device__ __forceinline__ float xor16_max(float x)
{
    const auto r = __builtin_amdgcn_permlane16_swap(as_u32(x), as_u32(x), false, false);
    return fmaxf(as_f32(r[0]), as_f32(r[1]));
}
__device__ __forceinline__ float xor32_max(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(as_u32(x), as_u32(x), false, false);
    return fmaxf(as_f32(r[0]), as_f32(r[1]));
}

// 8 nibbles of a dword as f16 (16 + n), in the order (n0, n4), (n1, n5), (n2, n6), (n3, n7)
// (M = 0x03C003C0 and G = 0x4C004C00 come in registers: the and-or is then one instruction, which takes no literals)
__device__ __forceinline__ h8v nibbles_f16(uint32_t d, uint32_t M, uint32_t G)
{
    const u32x4_t o = {((d << 6) & M) | G, ((d << 2) & M) | G, ((d >> 2) & M) | G, ((d >> 6) & M) | G};
    return __builtin_bit_cast(h8v, o);
}

// the element of a 32-wide Q4_0 block that slot s of lane group kq holds in the score products (see nibbles_f16:
// byte i of the lane's dword carries elements 4kq + i (low nibble) and 16 + 4kq + i (high nibble))
__device__ __forceinline__ int mfma_k_elem(int s, int kq)
{
    const int byte = ((s >> 2) & 1) + 2 * (s & 1);   // s: 0 1 2 3 4 5 6 7 -> byte 0 2 0 2 1 3 1 3
    return 4 * kq + byte + ((s >> 1) & 1) * 16;      //    nibble: lo lo hi hi lo lo hi hi
}

// HDV < HD (heads of 512 as two halves of 256): the workgroups of blockIdx.y = 2 * kvh + half both work out the scores
// and the softmax over all HD dimensions (the same numbers twice) and each takes P.V for its HDV dimensions of V,
// whose accumulators are what limits the head size a wave can hold.
// BAL: the launch whose partitions are dealt to the slots by length (p.balance), known when the kernel is built: either
// form's front then holds its own way to its rows only.
// PVX (eight waves with tiles of 16 rows, heads of 256): the waves share P.V by V block instead of by rows.  Every wave
// still takes the scores of its own 16 rows, the round's maximum and the probabilities meet in LDS (two barriers), and
// wave w then multiplies all 128 rows of the round into the 32 dimensions of block w -- its accumulators are final for
// the workgroup, so the eight-way fold of whole states through LDS and the pass that merges them fall away (they took
// a quarter of the launch) and every wave stores its own slice of the record.
template <int HD, int TR, int HDV = HD, bool BAL = false, bool PVX = false>
__global__ __launch_bounds__(kMfmaRound / TR * 64, TR == 32 ? 2 : 1) void sdpa_mfma_kernel(LaneParams p_in)
{
    LaneParams p = p_in;
    p.balance = BAL;
    static_assert(TR == 16 || TR == 32, "tile rows");
    static_assert(!PVX || (TR == 16 && HDV == HD && HD / 32 == kMfmaRound / TR), "a V block per wave");
    static_assert(HD % HDV == 0 && (HDV == HD || TR == 32), "V halves come with tiles of 32 rows");
    touch_lane_params(p_in);   // every kernel argument in one round trip
    KSH_STAMP_BEGIN
    constexpr int NW = kMfmaRound / TR, NT = NW * 64, NB = HD / 32, ROWB = NB * 18, TILEB = TR * ROWB;
    constexpr int NBV = HDV / 32, ROWBV = NBV * 18, TILEBV = TR * ROWBV;   // this workgroup's share of a V row
    constexpr int STRIP = TILEB + TILEBV + TR * NB * 4 + TR * NBV * 4;     // K bytes, V bytes, K scales, V scales
    constexpr int PIECES = TR * ROWB / 16, PIECESV = TR * ROWBV / 16;      // 128-bit pieces of a tile
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15, q4 = lane >> 4, head = col & 7, is_lo = col >> 3;
    const uint32_t odd_mask = 0u - (uint32_t)(q4 & 1);     // all ones in the lane groups whose accumulator rows are heads 4..7
    uint32_t nib_mask = 0x03C003C0u, nib_one = 0x4C004C00u;  // a nibble's place in an f16 mantissa; 16.0 twice
    asm volatile("" : "+v"(nib_mask), "+v"(nib_one));
    // the two parts of x = p * dv: hi lanes keep x cut to 11 bits, lo lanes what the cut left over
    const uint32_t keep = is_lo ? 0xFFFFFFFFu : 0xFFFFE000u, drop = is_lo ? 0xFFFFE000u : 0u;
    uint8_t *strip = lds_raw + (size_t)wave * STRIP;
    uint8_t *kraw = strip, *vraw = strip + TILEB;
    float *ksc = reinterpret_cast<float *>(strip + TILEB + TILEBV), *vsc = ksc + TR * NB;

    int part = blockIdx.x, slot = blockIdx.z, nparts = p.nwg;
    const int kvh = blockIdx.y / (HD / HDV), vhalf = blockIdx.y % (HD / HDV), groups = p.groups, head0 = kvh * groups;
    size_t rec_base = 0;
    int p0, p1, start;
    if (p.balance) {
        const Deal d = deal_wave(p.meta, p.meta_stride, (int)gridDim.z, p.nwg, kMfmaRound, blockIdx.z * p.nwg + blockIdx.x);
        if (d.slot < 0) return;   // left over
        slot = d.slot; part = d.part; nparts = d.nparts;
        rec_base = (size_t)d.first + part;
        p0 = part * d.c;
        p1 = min(p0 + d.c, d.tlen);
        start = d.start;
        if (PVX) { KSH_STAMP_USE(start); KSH_STAMP(1); }
    } else {
        int tlen;
        if (p.kv_shared) {
            // token `slot` of a prompt chunk (crates/ksearch_codegen/src/lower.rs:4961-4983): meta = {rows attended by token 0, -, window}
            const int abs_t = (int)p.meta[0] + slot;
            tlen = min(abs_t, (int)p.meta[2]);
            start = abs_t - tlen;
        } else {
            tlen = (int)p.meta[(size_t)slot * p.meta_stride];
            start = (int)p.meta[(size_t)slot * p.meta_stride + 1];
        }
        const int chunk = ((tlen + nparts - 1) / nparts + TR - 1) / TR * TR;
        p0 = min(part * chunk, tlen);
        p1 = min(p0 + chunk, tlen);
    }
    const size_t slot_bytes = p.kv_shared ? 0 : p.slot_stride ? p.slot_stride : (size_t)p.max_t * p.n_kv * ROWB;
    const size_t row_stride = (size_t)p.n_kv * ROWB;
    const size_t kv_slot = p.slot_ids ? (size_t)max((int)p.slot_ids[slot], 0) : (size_t)slot;
    const uint8_t *kbase = p.k + kv_slot * slot_bytes + (size_t)kvh * ROWB;
    const uint8_t *vbase = p.v + kv_slot * slot_bytes + (size_t)kvh * ROWB + (size_t)vhalf * ROWBV;

    // ---- a tile's bytes as whole 128-bit pieces, into registers (the first tile's are requested right behind q)
    constexpr int NPC = (PIECES + 63) / 64, NPCV = (PIECESV + 63) / 64;
    u32x4_t kpre[NPC], vpre[NPCV];
    auto fetch_tile = [&](int it) __attribute__((always_inline)) {
        const int row0 = p0 + (it * NW + wave) * TR;
        const int nvalid = max(0, min(TR, p1 - row0));
#pragma unroll
        for (int u = 0; u < NPC; u++) {
            const int idx = lane + 64 * u, row = idx / (ROWB / 16), pc = idx % (ROWB / 16);
            kpre[u] = u32x4_t{0u, 0u, 0u, 0u};
            if (HDV == HD) vpre[u] = u32x4_t{0u, 0u, 0u, 0u};
            if (idx < PIECES && row < nvalid) {
                const size_t off = (size_t)(start + row0 + row) * row_stride + (size_t)pc * 16;
                kpre[u] = *reinterpret_cast<const u32x4_t *>(kbase + off);
                if (HDV == HD) vpre[u] = *reinterpret_cast<const u32x4_t *>(vbase + off);
            }
        }
        if (HDV != HD) {
#pragma unroll
            for (int u = 0; u < NPCV; u++) {
                const int idx = lane + 64 * u, row = idx / (ROWBV / 16), pc = idx % (ROWBV / 16);
                vpre[u] = u32x4_t{0u, 0u, 0u, 0u};
                if (idx < PIECESV && row < nvalid)
                    vpre[u] = *reinterpret_cast<const u32x4_t *>(vbase + (size_t)(start + row0 + row) * row_stride + (size_t)pc * 16);
            }
        }
    };

    // ---- q: the B operands of the score products and 24 * sum_b(q), fixed for the launch.  Wave w prepares blocks
    // w, w + NW, ... and the workgroup shares them through LDS (behind the strips).  q is asked for before the tile:
    // loads come back in the order they went out, q is the short way (it was just written) and its preparation
    // then runs while the tile is on its way.
    static_assert(NB % NW == 0, "the q blocks divide among the waves");
    constexpr int QPW = NB / NW;
    h8v qop[NB];
    float qs24[NB];
    {
        // (heads of 512: the shared operands lie over the strips, which nothing has written yet, so that two workgroups fit a compute unit)
        h8v *qshare = reinterpret_cast<h8v *>(lds_raw + (HDV == HD ? (size_t)NW * STRIP : 0));       // [NB][64] operands
        float *qsum_share = HDV == HD ? reinterpret_cast<float *>(qshare + NB * 64) : reinterpret_cast<float *>(lds_raw + (size_t)NW * STRIP);   // [NB][64]
        const float *qh = p.q + ((size_t)slot * p.n_q + head0 + min(head, groups - 1)) * HD;
        const bool have = head < groups;
        float4 qlo[QPW], qhi[QPW];
#pragma unroll
        for (int u = 0; u < QPW; u++) {
            const int b = wave + NW * u;
            qlo[u] = *reinterpret_cast<const float4 *>(qh + 32 * b + 4 * q4);        // elements 4kq .. 4kq+3
            qhi[u] = *reinterpret_cast<const float4 *>(qh + 32 * b + 16 + 4 * q4);   // 16+4kq .. 16+4kq+3
        }
        if (HDV == HD) fetch_tile(0);      // (heads of 512 have no registers to hold a tile across the q preparation)
#pragma unroll
        for (int u = 0; u < QPW; u++) {
            const int b = wave + NW * u;
            const float4 lo4 = qlo[u], hi4 = qhi[u];
            const float x[8] = {lo4.x, lo4.z, hi4.x, hi4.z, lo4.y, lo4.w, hi4.y, hi4.w};       // slot order (mfma_k_elem)
            h8v op;
            float sum = 0.f;
#pragma unroll
            for (int s2 = 0; s2 < 8; s2++) {
                const float xs = pinned(have ? x[s2] * p.scale : 0.f);   // (a product on its way into a hi | lo split)
                const _Float16 hi = (_Float16)xs;
                const _Float16 lo = (_Float16)(xs - (float)hi);
                const _Float16 v = is_lo ? lo : hi;
                op[s2] = v;
                sum += (float)v;
            }
            sum = xor32_sum(xor16_sum(sum));      // the column's four lane groups hold the block's 32 elements
            qshare[b * 64 + lane] = op;
            qsum_share[b * 64 + lane] = 24.f * sum;
        }
        __syncthreads();
#pragma unroll
        for (int b = 0; b < NB; b++) {
            qop[b] = qshare[b * 64 + lane];
            if (HDV == HD) qs24[b] = qsum_share[b * 64 + lane];     // (heads of 512 read theirs from LDS block by block: sixteen registers less)
        }
        if (HDV != HD) __syncthreads();      // every wave has its copy before a strip is written
        if (PVX) { KSH_STAMP_USE(qs24[NB - 1]); KSH_STAMP(2); }
    }

    constexpr int NACC = PVX ? 1 : NBV;                     // V blocks a wave accumulates
    f4v O[2 * NACC];
    float Tl[NACC];
#pragma unroll
    for (int c = 0; c < 2 * NACC; c++) O[c] = f4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int b = 0; b < NACC; b++) Tl[b] = 0.f;
    float m_run = -1.0e30f, l_run = 0.f;
    // PVX: what the waves exchange per round, behind the shared q operands
    float *Psh = reinterpret_cast<float *>(lds_raw + (size_t)NW * STRIP + (size_t)NB * 64 * (16 + 4));   // [8 heads][128 rows]
    float *mxs = Psh + 8 * kMfmaRound, *lws = mxs + NW * 8;                                               // [wave][head] each

    const int ntiles = (p1 - p0 + TR - 1) / TR;
    const int nsteps = (ntiles + NW - 1) / NW;               // the same for every wave: the barriers below are uniform
    for (int it = 0; it < nsteps; it++) {
        const int row0 = p0 + (it * NW + wave) * TR;
        const int nvalid = max(0, min(TR, p1 - row0));         // wave-uniform
        // The strip belongs to this wave alone, and a wave's LDS operations complete in the order they were issued:
        // no workgroup barrier in this loop, only fences that keep the compiler from moving accesses across them.
        // (Later tiles are requested here, not a tile ahead: forty registers less make room for a second wave per
        // SIMD, which covers the wait better than the look-ahead did.)
        if (it > 0 || HDV != HD) fetch_tile(it);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
#pragma unroll
        for (int u = 0; u < NPC; u++) {
            const int idx = lane + 64 * u;
            if (idx < PIECES) {
                *reinterpret_cast<u32x4_t *>(kraw + idx * 16) = kpre[u];
                if (HDV == HD) *reinterpret_cast<u32x4_t *>(vraw + idx * 16) = vpre[u];
            }
        }
        if (HDV != HD) {
#pragma unroll
            for (int u = 0; u < NPCV; u++) {
                const int idx = lane + 64 * u;
                if (idx < PIECESV) *reinterpret_cast<u32x4_t *>(vraw + idx * 16) = vpre[u];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        // ---- block scales as f32 tables [row][block]; rows past the end get 0 (their codes are zeros too)
#pragma unroll
        for (int u = 0; u < TR * NB / 64; u++) {
            const int idx = lane + 64 * u, b = idx / TR, row = idx % TR;      // tables are [block][row]
            const uint32_t kb = *reinterpret_cast<const uint16_t *>(kraw + row * ROWB + 18 * b);
            ksc[idx] = row < nvalid ? half_bits_to_f32(kb) : 0.f;
            if (HDV == HD) {
                const uint32_t vb = *reinterpret_cast<const uint16_t *>(vraw + row * ROWBV + 18 * b);
                vsc[idx] = row < nvalid ? half_bits_to_f32(vb) : 0.f;
            }
        }
        if (HDV != HD) {
#pragma unroll
            for (int u = 0; u < TR * NBV / 64; u++) {
                const int idx = lane + 64 * u, b = idx / TR, row = idx % TR;
                const uint32_t vb = *reinterpret_cast<const uint16_t *>(vraw + row * ROWBV + 18 * b);
                vsc[idx] = row < nvalid ? half_bits_to_f32(vb) : 0.f;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        if constexpr (PVX) {
            if (it == 0) KSH_STAMP(3);
            // ---- scores of the wave's 16 rows (as below): lane (col, q4) ends up with rows 4*q4 + r
            float sv[4] = {-1.0e30f, -1.0e30f, -1.0e30f, -1.0e30f};
            if (nvalid > 0) {
                float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    const float4 dk4 = *reinterpret_cast<const float4 *>(ksc + b * TR + 4 * q4);
                    const float dk[4] = {dk4.x, dk4.y, dk4.z, dk4.w};
                    const uint8_t *src = kraw + col * ROWB + 18 * b + 2 + 4 * q4;
                    const uint32_t d = (uint32_t)*reinterpret_cast<const uint16_t *>(src) |
                                       ((uint32_t)*reinterpret_cast<const uint16_t *>(src + 2) << 16);
                    const f4v c = __builtin_amdgcn_mfma_f32_16x16x32_f16(nibbles_f16(d, nib_mask, nib_one), qop[b], f4v{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[r] = fmaf(dk[r], c[r] - qs24[b], acc[r]);
                }
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float tot = acc[r] + dpp_f32<0x128>(acc[r]);        // hi + lo column (row_ror:8)
                    sv[r] = (4 * q4 + r) < nvalid ? tot : -1.0e30f;
                }
            }
            // ---- probabilities against the wave's own maximum; maxima, sums and probabilities meet in LDS behind one
            // barrier (which also makes every wave's V bytes and scale tables visible to the others), and a tile's factor
            // exp(m_tile - m) rides on its V scales in the product below
            float mt = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
            mt = xor32_max(xor16_max(mt));
            float pr[4], ls = 0.f;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                pr[r] = (4 * q4 + r) < nvalid ? __expf(sv[r] - mt) : 0.f;
                ls += pr[r];
            }
            ls = xor32_sum(xor16_sum(ls));                     // the wave's 16 rows of this column's head
            if (!is_lo) *reinterpret_cast<float4 *>(Psh + head * kMfmaRound + TR * wave + 4 * q4) = make_float4(pr[0], pr[1], pr[2], pr[3]);
            if (lane < 8) { mxs[wave * 8 + lane] = mt; lws[wave * 8 + lane] = ls; }
            if (it == 0) KSH_STAMP(4);
            __syncthreads();
            float mw[NW], mr = -1.0e30f;
#pragma unroll
            for (int w = 0; w < NW; w++) { mw[w] = mxs[w * 8 + head]; mr = fmaxf(mr, mw[w]); }
            const float m_new = fmaxf(m_run, mr);
            const float alpha = __expf(m_run - m_new);
            float fw[NW], lr = 0.f;
#pragma unroll
            for (int w = 0; w < NW; w++) {
                fw[w] = __expf(mw[w] - m_new);
                lr = fmaf(fw[w], lws[w * 8 + head], lr);
            }
            l_run = fmaf(l_run, alpha, lr);
            m_run = m_new;
            if (it > 0) {
                // (the first round's factor multiplies zeros)
                float ah[8], ar[4];
#pragma unroll
                for (int h = 0; h < 8; h++) ah[h] = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(alpha), h));
#pragma unroll
                for (int r = 0; r < 4; r++) ar[r] = as_f32((as_u32(ah[r]) & ~odd_mask) | (as_u32(ah[4 + r]) & odd_mask));
#pragma unroll
                for (int c = 0; c < 2; c++)
#pragma unroll
                    for (int r = 0; r < 4; r++) O[c][r] *= ar[r];
                Tl[0] *= alpha;
            }
            // ---- P.V of block `wave` over the round's eight tiles: tile j lies in wave j's strip
            float tsum = 0.f;
#pragma unroll
            for (int j = 0; j < NW; j++) {
                const uint8_t *vj = lds_raw + (size_t)j * STRIP + TILEB;
                const float *vscj = reinterpret_cast<const float *>(lds_raw + (size_t)j * STRIP + TILEB + TILEBV) + TR * NB;
                const float4 p4 = *reinterpret_cast<const float4 *>(Psh + head * kMfmaRound + TR * j + 4 * q4);
                const float4 d4 = *reinterpret_cast<const float4 *>(vscj + wave * TR + 4 * q4);
                const float x[4] = {p4.x * (d4.x * fw[j]), p4.y * (d4.y * fw[j]), p4.z * (d4.z * fw[j]), p4.w * (d4.w * fw[j])};
                uint32_t pa[2], vlo[2], vhi[2];
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    const float y0 = as_f32(as_u32(x[2 * i]) & keep) - as_f32(as_u32(x[2 * i]) & drop);
                    const float y1 = as_f32(as_u32(x[2 * i + 1]) & keep) - as_f32(as_u32(x[2 * i + 1]) & drop);
                    pa[i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(y0, y1));
                    tsum += x[2 * i] + x[2 * i + 1];
                    const int ra = 4 * q4 + 2 * i;
                    const uint32_t t2 = (uint32_t)vj[ra * ROWBV + 18 * wave + 2 + col] | ((uint32_t)vj[(ra + 1) * ROWBV + 18 * wave + 2 + col] << 16);
                    vlo[i] = ((t2 << 6) & nib_mask) | nib_one;
                    vhi[i] = ((t2 << 2) & nib_mask) | nib_one;
                }
                const h4v pa4 = __builtin_bit_cast(h4v, u32x2_t{pa[0], pa[1]});
                const u32x2_t lo2 = {vlo[0], vlo[1]}, hi2 = {vhi[0], vhi[1]};
                O[0] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa4, __builtin_bit_cast(h4v, lo2), O[0], 0, 0, 0);
                O[1] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa4, __builtin_bit_cast(h4v, hi2), O[1], 0, 0, 0);
            }
            Tl[0] += tsum;
            if (it + 1 == nsteps) { KSH_STAMP_USE(O[1][3]); KSH_STAMP(5); }
            if (it + 1 < nsteps) __syncthreads();      // the strips and the exchange are written again
        } else
        if (nvalid > 0) {
            // ---- scores of the tile's two 16-row halves: lane (col, q4) ends up with rows 4*q4 + r of each
            constexpr int NS = TR / 4;                       // scores (rows) per lane
            float sv[NS];
#pragma unroll
            for (int t = 0; t < TR / 16; t++) {
                float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    const float4 dk4 = *reinterpret_cast<const float4 *>(ksc + b * TR + 16 * t + 4 * q4);   // rows 4*q4 .. +3
                    const float dk[4] = {dk4.x, dk4.y, dk4.z, dk4.w};
                    // A operand: row (16t + lane % 16), bytes 4*q4 .. 4*q4+3 of block b (2-byte aligned)
                    const uint8_t *src = kraw + (16 * t + col) * ROWB + 18 * b + 2 + 4 * q4;
                    const uint32_t d = (uint32_t)*reinterpret_cast<const uint16_t *>(src) |
                                       ((uint32_t)*reinterpret_cast<const uint16_t *>(src + 2) << 16);
                    const f4v c = __builtin_amdgcn_mfma_f32_16x16x32_f16(nibbles_f16(d, nib_mask, nib_one), qop[b], f4v{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    const float q24 = HDV == HD ? qs24[b] : reinterpret_cast<const float *>(lds_raw + (size_t)NW * STRIP)[b * 64 + lane];
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[r] = fmaf(dk[r], c[r] - q24, acc[r]);
                }
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float tot = acc[r] + dpp_f32<0x128>(acc[r]);        // hi + lo column (row_ror:8)
                    sv[4 * t + r] = (16 * t + 4 * q4 + r) < nvalid ? tot : -1.0e30f;
                }
            }
            // ---- online softmax over the tile (per column; the maximum across the wave's four lane groups)
            float mt = sv[0];
#pragma unroll
            for (int i = 1; i < NS; i++) mt = fmaxf(mt, sv[i]);
            mt = xor32_max(xor16_max(mt));
            const float m_new = fmaxf(m_run, mt);
            const float alpha = __expf(m_run - m_new);
            float pr[NS], ls = 0.f;
#pragma unroll
            for (int i = 0; i < NS; i++) {
                const int row = 16 * (i >> 2) + 4 * q4 + (i & 3);
                pr[i] = row < nvalid ? __expf(sv[i] - m_new) : 0.f;
                ls += pr[i];
            }
            l_run = fmaf(l_run, alpha, ls);
            m_run = m_new;
            // the accumulators of P.V hold output rows 4*q4 + r = columns of the scores: heads 4*(q4 & 1) + r
            float ah[8];
#pragma unroll
            for (int h = 0; h < 8; h++) ah[h] = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(alpha), h));
            bool rescale = false;
#pragma unroll
            for (int h = 0; h < 8; h++) rescale = rescale || ah[h] != 1.0f;
            if (rescale) {
                // (a bitwise select between the two scalars: an indexed pick would put the eight factors in memory)
                float ar[4];
#pragma unroll
                for (int r = 0; r < 4; r++) ar[r] = as_f32((as_u32(ah[r]) & ~odd_mask) | (as_u32(ah[4 + r]) & odd_mask));
#pragma unroll
                for (int c = 0; c < 2 * NBV; c++)
#pragma unroll
                    for (int r = 0; r < 4; r++) O[c][r] *= ar[r];
            }
#pragma unroll
            for (int b = 0; b < NBV; b++) Tl[b] *= alpha;       // (a lane's own column: its own factor)
            // ---- P.V per block: P' = p * dv (hi | lo), V codes gathered bytewise: slot s of the lane <-> row
            // 16*(s/4) + 4*q4 + s%4, the rows its own scores belong to
#pragma unroll
            for (int b = 0; b < NBV; b++) {
                uint32_t pa[NS / 2], vlo[NS / 2], vhi[NS / 2];
                float dv[NS];
#pragma unroll
                for (int t = 0; t < TR / 16; t++) {
                    const float4 d4 = *reinterpret_cast<const float4 *>(vsc + b * TR + 16 * t + 4 * q4);   // rows 16t + 4*q4 .. +3
                    dv[4 * t] = d4.x; dv[4 * t + 1] = d4.y; dv[4 * t + 2] = d4.z; dv[4 * t + 3] = d4.w;
                }
                float tsum = 0.f;
#pragma unroll
                for (int i = 0; i < NS; i += 2) {
                    // (the conversion is exact for the hi part and cuts the lo part to 11 of its 13 bits)
                    const float x0 = pr[i] * dv[i], x1 = pr[i + 1] * dv[i + 1];
                    const float y0 = as_f32(as_u32(x0) & keep) - as_f32(as_u32(x0) & drop);
                    const float y1 = as_f32(as_u32(x1) & keep) - as_f32(as_u32(x1) & drop);
                    pa[i / 2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(y0, y1));
                    tsum += x0 + x1;
                }
                Tl[b] += tsum;                                  // sum(P') of the lane's own rows and column, for the code offset
#pragma unroll
                for (int i = 0; i < NS / 2; i++) {
                    const int ra = 16 * ((2 * i) >> 2) + 4 * q4 + ((2 * i) & 3), rb = ra + 1;
                    const uint32_t t2 = (uint32_t)vraw[ra * ROWBV + 18 * b + 2 + col] | ((uint32_t)vraw[rb * ROWBV + 18 * b + 2 + col] << 16);
                    vlo[i] = ((t2 << 6) & nib_mask) | nib_one;
                    vhi[i] = ((t2 << 2) & nib_mask) | nib_one;
                }
                if constexpr (TR == 32) {
                    const h8v pa8 = __builtin_bit_cast(h8v, u32x4_t{pa[0], pa[1], pa[2], pa[3]});
                    const u32x4_t lo4 = {vlo[0], vlo[1], vlo[2], vlo[3]}, hi4 = {vhi[0], vhi[1], vhi[2], vhi[3]};
                    O[2 * b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa8, __builtin_bit_cast(h8v, lo4), O[2 * b], 0, 0, 0);
                    O[2 * b + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa8, __builtin_bit_cast(h8v, hi4), O[2 * b + 1], 0, 0, 0);
                } else {
                    // 16 rows: k = 4 * q4 + i is the row itself in both operands
                    const h4v pa4 = __builtin_bit_cast(h4v, u32x2_t{pa[0], pa[1]});
                    const u32x2_t lo2 = {vlo[0], vlo[1]}, hi2 = {vhi[0], vhi[1]};
                    O[2 * b] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa4, __builtin_bit_cast(h4v, lo2), O[2 * b], 0, 0, 0);
                    O[2 * b + 1] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa4, __builtin_bit_cast(h4v, hi2), O[2 * b + 1], 0, 0, 0);
                }
            }
        }
    }

    if constexpr (PVX) {
        // ---- every wave stores the 32 dimensions of its block for all heads; wave 0 adds (m, l)
        const uint32_t tcol = as_u32(24.f * xor32_sum(xor16_sum(Tl[0])));
        const int odd = q4 >> 1, d = 32 * wave + col + 16 * odd;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const uint32_t t_lo = (uint32_t)__builtin_amdgcn_readlane((int)tcol, r), t_hi = (uint32_t)__builtin_amdgcn_readlane((int)tcol, 4 + r);
            const float t24 = as_f32((t_lo & ~odd_mask) | (t_hi & odd_mask));
            const uint32_t l_lo = (uint32_t)__builtin_amdgcn_readlane((int)as_u32(l_run), r), l_hi = (uint32_t)__builtin_amdgcn_readlane((int)as_u32(l_run), 4 + r);
            const float L = as_f32((l_lo & ~odd_mask) | (l_hi & odd_mask));
            const auto sw = __builtin_amdgcn_permlane32_swap(as_u32(O[0][r]), as_u32(O[1][r]), false, false);
            const float a = (as_f32(sw[0]) - t24) + as_f32(sw[1]);
            const int h = 4 * (q4 & 1) + r, hq = head0 + h;
            if (h >= groups) continue;
            if (p.balance) {
                p.tmp[(rec_base * p.n_q + hq) * HD + d] = a;
            } else if (p.nwg == 1 && p.out) {
                p.out[((size_t)slot * p.n_q + hq) * HD + d] = a / L;
            } else {
                p.tmp[(size_t)slot * p.n_q * p.nwg * (HD + 2) + (size_t)hq * p.nwg * (HD + 2) + (size_t)part * (HD + 2) + 2 + d] = a;
            }
        }
        if (wave == 0 && lane < 8 && lane < groups) {
            const int hq = head0 + lane;
            if (p.balance) {
                float *ml = p.tmp + (size_t)gridDim.z * p.nwg * p.n_q * HD;
                ml[2 * (rec_base * p.n_q + hq)] = m_run;
                ml[2 * (rec_base * p.n_q + hq) + 1] = l_run;
            } else if (!(p.nwg == 1 && p.out)) {
                float *rec = p.tmp + (size_t)slot * p.n_q * p.nwg * (HD + 2) + (size_t)hq * p.nwg * (HD + 2) + (size_t)part * (HD + 2);
                rec[0] = m_run;
                rec[1] = l_run;
            }
        }
        KSH_STAMP_FLUSH(2, ((int)blockIdx.z * (int)gridDim.x + (int)blockIdx.x) * NW + wave, 6);
        return;
    }
    // ---- fold: every wave's state to LDS (hi rows first, lo rows added), then one record per head
    __syncthreads();
    float *ow = reinterpret_cast<float *>(lds_raw);            // [NW][8][HDV]
    float *mlw = ow + NW * 8 * HDV;                            // [NW][8][2]
    const float l_tot = xor32_sum(xor16_sum(l_run));
    // sum(P') of head h and block b: the four lane groups of column h hold its parts.  The accumulator layout wants
    // it by row (head 4 * (q4 & 1) + r): read from lane h as a scalar, picked bitwise like the rescale factors.
    float t24[4][NBV];
#pragma unroll
    for (int b = 0; b < NBV; b++) {
        const uint32_t tcol = as_u32(24.f * xor32_sum(xor16_sum(Tl[b])));
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const uint32_t t_lo = (uint32_t)__builtin_amdgcn_readlane((int)tcol, r), t_hi = (uint32_t)__builtin_amdgcn_readlane((int)tcol, 4 + r);
            t24[r][b] = as_f32((t_lo & ~odd_mask) | (t_hi & odd_mask));
        }
    }
    {
        // A head's hi rows sit in the lower 32 lanes and its lo rows in the upper 32 (lane ^ 32).  One half-wave swap
        // per block brings both parts of the block's even 16 columns to the lower lanes and both parts of its odd 16
        // columns to the upper lanes: swap(a, b) returns {a.lower | b.lower, a.upper | b.upper} by (lower, upper)
        // lanes.  (The offset 24 * sum(P') of the whole value -- hi and lo part -- is taken off the hi part.)
        const int odd = q4 >> 1;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float *dst = ow + ((size_t)wave * 8 + 4 * (q4 & 1) + r) * HDV + col + 16 * odd;
#pragma unroll
            for (int b = 0; b < NBV; b++) {
                const auto sw = __builtin_amdgcn_permlane32_swap(as_u32(O[2 * b][r]), as_u32(O[2 * b + 1][r]), false, false);
                dst[32 * b] = (as_f32(sw[0]) - t24[r][b]) + as_f32(sw[1]);
            }
        }
    }
    if (lane < 8) { mlw[(wave * 8 + lane) * 2] = m_run; mlw[(wave * 8 + lane) * 2 + 1] = l_tot; }
    __syncthreads();
    static_assert(NT % HDV == 0 || HDV % NT == 0, "whole heads per pass, or whole passes per head");
#pragma unroll
    for (int o = tid; o < 8 * HDV; o += NT) {
        const int h = o / HDV, d = o % HDV, hq = head0 + h;      // (h is the same for a whole wave)
        if (h >= groups) break;
        float M = -1.0e30f;
#pragma unroll
        for (int w = 0; w < NW; w++) M = fmaxf(M, mlw[(w * 8 + h) * 2]);
        float L = 0.f, a = 0.f;
#pragma unroll
        for (int w = 0; w < NW; w++) {
            const float wt = __expf(mlw[(w * 8 + h) * 2] - M);
            L = fmaf(wt, mlw[(w * 8 + h) * 2 + 1], L);
            a = fmaf(wt, ow[((size_t)w * 8 + h) * HDV + d], a);
        }
        if (p.balance) {
            const size_t r = rec_base * p.n_q + hq;
            float *ml = p.tmp + (size_t)gridDim.z * p.nwg * p.n_q * HD;
            p.tmp[r * HD + vhalf * HDV + d] = a;
            if (d == 0 && vhalf == 0) { ml[2 * r] = M; ml[2 * r + 1] = L; }
        } else if (p.nwg == 1 && p.out) {
            p.out[((size_t)slot * p.n_q + hq) * HD + vhalf * HDV + d] = a / L;      // one partition: nothing left to merge
        } else {
            float *rec = p.tmp + (size_t)slot * p.n_q * p.nwg * (HD + 2) + (size_t)hq * p.nwg * (HD + 2) + (size_t)part * (HD + 2);
            rec[2 + vhalf * HDV + d] = a;
            if (d == 0 && vhalf == 0) { rec[0] = M; rec[1] = L; }
        }
    }
}

// Merge of split-KV partials kept as records (m, l, o[HD]) per (token, head, partition) -- the layout and the rule
// of SdpaMwgReduce (crates/ksearch_codegen/src/lower.rs:5897-6087) -- for the launch that gives every token of a long
// prompt chunk its own workgroups.  grid = (n_q, n_tok), HD threads.
template <int HD>
__global__ __launch_bounds__(HD) void sdpa_records_merge_kernel(const float *__restrict__ tmp, float *__restrict__ out, int n_q, int nwg)
{
    const int h = blockIdx.x, tok = blockIdx.y, d = threadIdx.x;
    const float *rec = tmp + ((size_t)tok * n_q + h) * nwg * (HD + 2);
    float M = -1.0e30f;
    for (int q = 0; q < nwg; q++) M = fmaxf(M, rec[(size_t)q * (HD + 2)]);
    float L = 0.f, a = 0.f;
    for (int q = 0; q < nwg; q++) {
        const float w = __expf(rec[(size_t)q * (HD + 2)] - M);
        L = fmaf(w, rec[(size_t)q * (HD + 2) + 1], L);
        a = fmaf(w, rec[(size_t)q * (HD + 2) + 2 + d], a);
    }
    out[((size_t)tok * n_q + h) * HD + d] = a / L;
}

template <int HD, int TR, int HDV = HD, bool PVX = false>
constexpr size_t mfma_lds_bytes()
{
    constexpr size_t waves = kMfmaRound / TR;
    constexpr size_t strip = (size_t)TR * (HD / 32 * 18) + (size_t)TR * (HDV / 32 * 18) + (size_t)TR * (HD / 32) * 4 + (size_t)TR * (HDV / 32) * 4;
    constexpr size_t qshare = (size_t)(HD / 32) * 64 * (16 + 4);                 // the shared q operands and sums
    constexpr size_t fold = waves * 8 * HDV * 4 + waves * 8 * 2 * 4;
    constexpr size_t qsum = (size_t)(HD / 32) * 64 * 4;
    constexpr size_t front = HDV == HD ? strip * waves + qshare : strip * waves + qsum;   // (HDV < HD: the operands lie over the strips, the sums behind them)
    if (PVX) return front + (8 * kMfmaRound + 2 * waves * 8) * 4;                         // + the probabilities, maxima and sums the waves exchange; no fold
    return front > fold ? front : fold;
}

template <int HD, int GP, int NW>
constexpr size_t lanes_lds_bytes()
{
    constexpr int NSLOT = NW * (64 / (HD / 8));
    return ((size_t)GP * HD + (size_t)NSLOT * (GP * HD + (2 * GP + 3) / 4 * 4) + (size_t)GP * NSLOT + 2 * GP) * 4 + 2 * (HD / 32 * 18) + 16;
}

template <int HD, int GP, int NW>
int launch_inst(const LaneParams &p, int n_slots, hipStream_t st)
{
    const size_t lds = lanes_lds_bytes<HD, GP, NW>();
    if (p.fused) hipLaunchKernelGGL((sdpa_lanes_kernel<HD, GP, NW, true>), dim3(p.nwg, p.n_kv * p.hsplit, n_slots), dim3(NW * 64), lds, st, p);
    else hipLaunchKernelGGL((sdpa_lanes_kernel<HD, GP, NW, false>), dim3(p.nwg, p.n_kv * p.hsplit, n_slots), dim3(NW * 64), lds, st, p);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "sdpa (register form) launch");
}

// which launches take the instances for one or two q heads per workgroup: the fused decode step at heads of 256 and 512
bool lanes_few_heads(int fused, int mode, int groups, int hd)
{
    (void)mode;
    return fused && (hd == 256 || hd == 512) && groups <= 2;
}

int launch_lanes(const LaneParams &p, int hd, int nw, int n_slots, hipStream_t st)
{
    // the decode step with one or two q heads per workgroup (heads of 256): instances of their own
    if (lanes_few_heads(p.fused, p.mode, p.groups, hd) && (nw == 4 || nw == 8)) {
        const dim3 grid(p.nwg, p.n_kv * p.hsplit, n_slots);
        if (hd == 512 && p.groups == 1 && nw == 8) hipLaunchKernelGGL((sdpa_lanes_kernel<512, 1, 8, true>), grid, dim3(512), (lanes_lds_bytes<512, 1, 8>()), st, p);
        else if (hd == 512 && p.groups == 1) hipLaunchKernelGGL((sdpa_lanes_kernel<512, 1, 4, true>), grid, dim3(256), (lanes_lds_bytes<512, 1, 4>()), st, p);
        else if (hd == 512 && nw == 8) hipLaunchKernelGGL((sdpa_lanes_kernel<512, 2, 8, true>), grid, dim3(512), (lanes_lds_bytes<512, 2, 8>()), st, p);
        else if (hd == 512) hipLaunchKernelGGL((sdpa_lanes_kernel<512, 2, 4, true>), grid, dim3(256), (lanes_lds_bytes<512, 2, 4>()), st, p);
        else if (p.groups == 1 && nw == 8) hipLaunchKernelGGL((sdpa_lanes_kernel<256, 1, 8, true>), grid, dim3(512), (lanes_lds_bytes<256, 1, 8>()), st, p);
        else if (p.groups == 1) hipLaunchKernelGGL((sdpa_lanes_kernel<256, 1, 4, true>), grid, dim3(256), (lanes_lds_bytes<256, 1, 4>()), st, p);
        else if (nw == 8) hipLaunchKernelGGL((sdpa_lanes_kernel<256, 2, 8, true>), grid, dim3(512), (lanes_lds_bytes<256, 2, 8>()), st, p);
        else hipLaunchKernelGGL((sdpa_lanes_kernel<256, 2, 4, true>), grid, dim3(256), (lanes_lds_bytes<256, 2, 4>()), st, p);
        const hipError_t e = hipGetLastError();
        return e == hipSuccess ? 0 : hip_fail(e, "sdpa (register form, one or two heads) launch");
    }
    const int gp = p.groups <= 4 ? 4 : 8;
#define KSH_CASE(H, G, W) \
    if (hd == H && gp == G && nw == W) return launch_inst<H, G, W>(p, n_slots, st);
    KSH_CASE(128, 4, 4) KSH_CASE(128, 8, 4) KSH_CASE(256, 4, 4) KSH_CASE(256, 8, 4)
    KSH_CASE(128, 4, 8) KSH_CASE(128, 8, 8) KSH_CASE(256, 4, 8) KSH_CASE(256, 8, 8)
    KSH_CASE(512, 4, 4) KSH_CASE(512, 4, 8)     // (eight heads of 512 do not fit the fold's LDS: such shapes split the heads)
#undef KSH_CASE
    return set_error("sdpa (register form): no instance for hd=%d groups=%d nsg=%d", hd, p.groups, nw);
}

size_t lanes_lds(int hd, int groups, int nw, bool few_heads = false)
{
    const int gp = few_heads ? groups : groups <= 4 ? 4 : 8;
    const int nslot = nw * (64 / (hd / 8));
    return ((size_t)gp * hd + (size_t)nslot * (gp * hd + (2 * gp + 3) / 4 * 4) + (size_t)gp * nslot + 2 * gp) * 4 + 2 * (hd / 32 * 18) + 16;
}

LaneParams base_params(const ksh_kernel &k)
{
    LaneParams p{};
    p.n_q = (int)k.desc.dims[0];
    p.n_kv = (int)k.desc.dims[1];
    p.max_t = (int)k.desc.dims[3];
    p.hsplit = (k.variant >> 24) & 0xFF;
    p.groups = p.n_q / p.n_kv / p.hsplit;
    p.counters = (uint32_t *)k.scratch;
    return p;
}

// Several slots share one launch's partitions by length when there are few enough of them for every workgroup
// to derive the table itself.
bool balanced_slots(int n_slots, int nwg) { return n_slots > 1 && n_slots <= 16 && nwg >= 2 && nwg <= 64; }

// variant: nwg | NW << 16 | hsplit << 24
int launch_bound(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    LaneParams p = base_params(k);
    const int hd = (int)k.desc.dims[2], nw = (k.variant >> 16) & 0xFF;
    p.nwg = k.variant & 0xFFFF;
    // the matrix-core form of the row phase (bind_sdpa_lanes): 0xFF tiles of 32 rows, 0xFE of 16; 0xFD: tiles of 32
    // rows with every slot's partitions its own workgroups (a long prompt chunk: more tokens than the deal takes)
    const bool mfma = nw >= 0xFD, own_parts = nw == 0xFD;
    if (mfma) { p.hsplit = 1; p.groups = p.n_q / p.n_kv; }
    int n_slots = 1;
    // the row phase whose partitions are dealt to the slots by length (register or matrix-core form), then the merge launch
    auto launch_dealt = [&](_Float16 *xp) -> int {
        p.balance = 1;
        p.mode = kModePart;
        if (mfma) {
            if (nw == 0xFF)
                hipLaunchKernelGGL((sdpa_mfma_kernel<256, 32, 256, true>), dim3(p.nwg, p.n_kv, n_slots), dim3(kMfmaRound / 32 * 64), (mfma_lds_bytes<256, 32>()), st, p);
            else if ((size_t)p.max_t <= (size_t)3 * kMfmaRound * (p.nwg - 1))
                // partitions of at most three rounds even when every slot is full: the waves share P.V by V block (two
                // barriers a round, no fold: a round costs ~0.7 us more than in the barrier-free loop, the fold ~2.2 us once)
                hipLaunchKernelGGL((sdpa_mfma_kernel<256, 16, 256, true, true>), dim3(p.nwg, p.n_kv, n_slots), dim3(kMfmaRound / 16 * 64), (mfma_lds_bytes<256, 16, 256, true>()), st, p);
            else
                hipLaunchKernelGGL((sdpa_mfma_kernel<256, 16, 256, true>), dim3(p.nwg, p.n_kv, n_slots), dim3(kMfmaRound / 16 * 64), (mfma_lds_bytes<256, 16>()), st, p);
            const hipError_t e0 = hipGetLastError();
            if (e0 != hipSuccess) return hip_fail(e0, "sdpa (matrix-core form) launch");
        } else if (launch_lanes(p, hd, nw, n_slots, st)) {
            return 1;
        }
        if (hd == 512)
            hipLaunchKernelGGL(sdpa_dealt_merge_kernel<512>, dim3(p.n_q * 8, n_slots), dim3(256), 0, st, p.tmp, p.meta, p.meta_stride, p.nwg, p.n_q, p.out, mfma ? kMfmaRound : 1, xp);
        else if (hd == 256)
            hipLaunchKernelGGL(sdpa_dealt_merge_kernel<256>, dim3(p.n_q * 4, n_slots), dim3(256), 0, st, p.tmp, p.meta, p.meta_stride, p.nwg, p.n_q, p.out, mfma ? kMfmaRound : 1, xp);
        else
            hipLaunchKernelGGL(sdpa_dealt_merge_kernel<128>, dim3(p.n_q * 2, n_slots), dim3(256), 0, st, p.tmp, p.meta, p.meta_stride, p.nwg, p.n_q, p.out, mfma ? kMfmaRound : 1, xp);
        const hipError_t e = hipGetLastError();
        return e == hipSuccess ? 0 : hip_fail(e, "sdpa merge launch");
    };
    switch (k.desc.kind) {
    case KSH_SDPA_NAIVE:
        p.q = (const float *)a.in[0]; p.k = (const uint8_t *)a.in[1]; p.v = (const uint8_t *)a.in[2];
        p.meta = (const float *)a.in[3];
        p.out = (float *)a.out[0];
        p.scale = k.desc.params[0];
        p.mode = kModeDirect;
        break;
    case KSH_SDPA_MWG_PART:
        p.q = (const float *)a.in[0]; p.k = (const uint8_t *)a.in[1]; p.v = (const uint8_t *)a.in[2];
        p.meta = (const float *)a.in[3];
        p.tmp = (float *)a.out[0];
        p.scale = k.desc.params[0];
        p.mode = kModePart;
        break;
    case KSH_SDPA_SLOTS:
        n_slots = (int)k.desc.dims[4];
        p.q = (const float *)a.in[0]; p.k = (const uint8_t *)a.in[1]; p.v = (const uint8_t *)a.in[2];
        p.meta = (const float *)a.in[3];
        p.meta_stride = 4;
        if (k.desc.dims[6]) {   // entries of a decode round: each names its slot of the pools
            p.slot_ids = (const float *)a.in[4];
            p.slot_stride = (size_t)k.desc.dims[7];
        }
        p.tmp = (float *)a.out[0];
        p.out = (float *)a.out[1];
        p.scale = k.desc.params[0];
        p.mode = kModeMerge;
        if (k.desc.params[1] != 0.f && !(balanced_slots(n_slots, p.nwg) || mfma))
            return set_error("sdpa_slots: the result as a prepared operand needs the launch whose partitions are dealt by length (2 to 16 slots, 2 to 64 partitions)");
        if (balanced_slots(n_slots, p.nwg) || mfma) return launch_dealt(k.desc.params[1] != 0.f ? (_Float16 *)a.out[1] : nullptr);
        break;
    case KSH_SDPA_BATCH: {
        // in: q, K, V, meta{tlen of token 0, -, window}   out: tmp, o.  The per-token records are written by a small
        // kernel into the handle's scratch (behind the counters); K and V are shared by all tokens.
        n_slots = (int)k.desc.dims[4];
        float *tok_meta = (float *)((uint8_t *)k.scratch + (((size_t)n_slots * p.n_kv * p.hsplit * 4 + 15) & ~(size_t)15));
        // (the form with a workgroup per token works its token's record out itself)
        if (!own_parts) hipLaunchKernelGGL(sdpa_batch_meta_kernel, dim3((n_slots + 255) / 256), dim3(256), 0, st, (const float *)a.in[3], tok_meta, n_slots);
        p.q = (const float *)a.in[0]; p.k = (const uint8_t *)a.in[1]; p.v = (const uint8_t *)a.in[2];
        p.meta = tok_meta;
        p.meta_stride = 4;
        p.tmp = (float *)a.out[0];
        p.out = (float *)a.out[1];
        p.scale = k.desc.params[0];
        p.mode = kModeMerge;
        p.kv_shared = 1;
        if (own_parts) {
            p.meta = (const float *)a.in[3];
            p.balance = 0;
            p.mode = kModePart;
            if (hd == 512)   // two workgroups per kv head, each with half of the V dimensions
                hipLaunchKernelGGL((sdpa_mfma_kernel<512, 32, 256>), dim3(p.nwg, p.n_kv * 2, n_slots), dim3(kMfmaRound / 32 * 64), (mfma_lds_bytes<512, 32, 256>()), st, p);
            else
                hipLaunchKernelGGL((sdpa_mfma_kernel<256, 32>), dim3(p.nwg, p.n_kv, n_slots), dim3(kMfmaRound / 32 * 64), (mfma_lds_bytes<256, 32>()), st, p);
            const hipError_t e0 = hipGetLastError();
            if (e0 != hipSuccess) return hip_fail(e0, "sdpa_batch (matrix-core form) launch");
            if (p.nwg == 1) return 0;      // (the row launch has stored the finished heads)
            if (hd == 512) hipLaunchKernelGGL(sdpa_records_merge_kernel<512>, dim3(p.n_q, n_slots), dim3(512), 0, st, p.tmp, p.out, p.n_q, p.nwg);
            else hipLaunchKernelGGL(sdpa_records_merge_kernel<256>, dim3(p.n_q, n_slots), dim3(256), 0, st, p.tmp, p.out, p.n_q, p.nwg);
            const hipError_t e1 = hipGetLastError();
            return e1 == hipSuccess ? 0 : hip_fail(e1, "sdpa_batch merge launch");
        }
        if (mfma) return launch_dealt(nullptr);    // every token a slot of its own over the shared cache
        break;
    }
    case KSH_ATTEND_DECODE: {
        const bool reader = k.desc.dims[7] != 0;
        p.q = (const float *)a.in[0]; p.qw = (const float *)a.in[1]; p.rope = (const float *)a.in[2];
        int no = 0;
        if (reader) {
            // in: q, q_norm, rope, K cache, V cache, meta.  The loads of the raw k / v and of the key norm are issued
            // unconditionally: they read q and the query norm again and nothing uses them.
            p.k_raw = p.v_raw = p.q; p.kw = p.qw;
            p.k = (const uint8_t *)a.in[3]; p.v = (const uint8_t *)a.in[4];
            p.meta = (const float *)a.in[5];
            p.no_append = 1;
        } else {
            p.k_raw = (const float *)a.in[3]; p.kw = (const float *)a.in[4]; p.v_raw = (const float *)a.in[5];
            p.meta = (const float *)a.in[6];
            p.k_w = (uint8_t *)a.out[0]; p.v_w = (uint8_t *)a.out[1];
            p.k = p.k_w; p.v = p.v_w;
            no = 2;
        }
        p.meta_stride = 4;
        p.tmp = (float *)a.out[no];
        p.eps = k.desc.params[0];
        p.scale = k.desc.params[1];
        p.rope_row = k.desc.dims[6] != 0;
        if (k.desc.dims[5]) {
            p.mode = kModeSplitPart;
        } else {
            p.out = (float *)a.out[no + 1];
            p.mode = kModeMerge;
        }
        p.fused = 1;
        break;
    }
    default: return set_error("sdpa (register form): kind %d", k.desc.kind);
    }
    return launch_lanes(p, hd, nw, n_slots, st);
}

}  // namespace

bool sdpa_lanes_supports(int64_t n_q, int64_t n_kv, int64_t hd)
{
    return n_kv > 0 && n_q % n_kv == 0 && n_q / n_kv <= 8 && (hd == 128 || hd == 256 || hd == 512);
}

// Fills in the launch for a shape sdpa_lanes_supports(); the caller has
// validated the shape and set the buffer sizes of the SDPA kinds.
int bind_sdpa_lanes(ksh_kernel &k, int nwg, int n_slots)
{
    const int64_t *d = k.desc.dims;
    const int n_q = (int)d[0], n_kv = (int)d[1], hd = (int)d[2];
    // sched.vec = 2: the matrix-core form of the row phase -- several slots' (or one slot's) split-KV partials for
    // heads of 256 and up to 8 q heads per kv head, merged by a second launch
    // It is the default wherever it fits (from one slot of a few thousand rows to sixteen long ones it takes 0.5 to
    // 1.0 of the vector form's time); vec = 3 asks for the vector form by name.
    // (a chunk of up to 64 prompt tokens over one cache is 64 slots that share it: a schedule of KSH_SDPA_BATCH, not its
    // default -- timed alone it takes 0.65 to 0.8 of the register form's time, inside a prompt chunk's pass its second
    // launch costs more than that saves at 63 tokens)
    const bool batch_fits = k.desc.kind == KSH_SDPA_BATCH && hd == 256 && n_q / n_kv <= 8 && n_slots <= 64 && nwg >= 2 && nwg * n_slots <= 1024;
    const bool mfma_fits = (k.desc.kind == KSH_SDPA_SLOTS && hd == 256 && n_q / n_kv <= 8 && n_slots <= 16 && nwg >= 2 && nwg <= 64) || batch_fits;
    // A chunk of more than 16 tokens: every token's partitions are workgroups of their own (grid = partitions x kv
    // heads x tokens), records in the reference's layout, merged by a second launch.  Its tokens attend dozens to
    // thousands of rows each, where the register form's ~200 vector instructions per row and wave are the whole
    // cost (1024 tokens from an empty cache: 78 us against 422; heads of 512: 226 against 778): the default there;
    // vec = 3 asks for the register form, vec = 2 with up to 64 tokens for the form that deals the partitions by length.
    const bool long_batch = k.desc.kind == KSH_SDPA_BATCH && (hd == 256 || hd == 512) && n_q / n_kv <= 8 && n_slots > 16;
    if (long_batch && ((k.desc.sched.vec == 2 && !batch_fits) || k.desc.sched.vec == 0)) {
        if (k.desc.sched.lds_tile && k.desc.sched.lds_tile != 32) return set_error("sdpa_batch: the matrix-core form of a long chunk takes tiles of 32 rows (lds_tile=%u)", k.desc.sched.lds_tile);
        k.scratch_bytes = (((size_t)n_slots * n_kv * 4 + 15) & ~(size_t)15) + (size_t)n_slots * 16;
        // (heads of 512: two workgroups per kv head, each with all of the scores and half of the V dimensions)
        set_launch(k, (uint32_t)nwg, (uint32_t)(hd == 512 ? 2 * n_kv : n_kv), (uint32_t)n_slots, kMfmaRound / 32 * 64,
                   (uint32_t)(hd == 512 ? mfma_lds_bytes<512, 32, 256>() : mfma_lds_bytes<256, 32>()));
        k.info.sched = k.desc.sched;
        k.info.sched.vec = 2;
        k.info.sched.tg = kMfmaRound / 32 * 64;
        k.info.sched.nsg = kMfmaRound / 32;
        k.info.sched.k_split = (uint32_t)nwg;
        k.info.sched.lds_tile = 32;
        k.info.sched.unroll = 1;
        k.variant = nwg | (0xFD << 16) | (1 << 24);
        k.launch = launch_bound;
        return 0;
    }
    if (k.desc.sched.vec == 2 || (k.desc.sched.vec == 0 && mfma_fits && !batch_fits)) {
        if (!mfma_fits)
            return set_error("sdpa: the matrix-core form (vec=2) takes hd 256 and up to 8 q heads per kv head: KSH_SDPA_SLOTS with up to 16 slots "
                             "and 2..64 partitions, KSH_SDPA_BATCH with up to 64 tokens and 2 .. 1024 / tokens partitions");
        // sched.lds_tile: rows per wave tile, 32 (four waves) or 16 (eight waves).  0 takes 16 where the grid is at
        // most one workgroup per compute unit (eight-wave workgroups do not share one, so a larger grid would run in
        // two turns; within one turn the shorter chain per wave is worth about a microsecond)
        const int tile = k.desc.sched.lds_tile ? (int)k.desc.sched.lds_tile : (int64_t)nwg * n_kv * n_slots <= 256 ? 16 : 32;
        if (tile != 16 && tile != 32) return set_error("sdpa: the matrix-core form takes tiles of 16 or 32 rows (lds_tile=%d)", tile);
        const int waves = kMfmaRound / tile;
        // (the batch kind keeps its per-token records in the scratch, behind room for the register form's counters)
        k.scratch_bytes = batch_fits ? (((size_t)n_slots * n_kv * 4 + 15) & ~(size_t)15) + (size_t)n_slots * 16 : 16;
        set_launch(k, (uint32_t)nwg, (uint32_t)n_kv, (uint32_t)n_slots, waves * 64,
                   (uint32_t)(tile == 32 ? mfma_lds_bytes<256, 32>() : mfma_lds_bytes<256, 16>()));
        k.info.sched = k.desc.sched;
        k.info.sched.vec = 2;
        k.info.sched.tg = waves * 64;
        k.info.sched.nsg = waves;
        k.info.sched.k_split = (uint32_t)nwg;
        k.info.sched.lds_tile = tile;
        k.info.sched.unroll = 1;
        k.variant = nwg | ((tile == 32 ? 0xFF : 0xFE) << 16) | (1 << 24);
        k.launch = launch_bound;
        return 0;
    }
    int nw = k.desc.sched.nsg ? (int)k.desc.sched.nsg : 0;
    if (!nw) nw = (d[3] / nwg >= 256) ? 8 : 4;   // long partitions: more waves per workgroup
    if (nw != 4 && nw != 8) return set_error("sdpa: unsupported schedule nsg=%d (4 or 8)", nw);
    if (nwg < 1 || nwg > 4096) return set_error("sdpa: nwg=%d", nwg);
    // sched.unroll: workgroups per kv head, each with a share of its q heads (rows are then unpacked once per
    // share, but a decode step's latency is in the per-row work and the merge, both of which shrink with it)
    const int total_groups = n_q / n_kv;
    // (defaults from timing the decode shape: two heads per workgroup where the launch merges, one where it does not;
    // heads of 512, merging, 16 partitions, eight waves: one head per workgroup 8.3 / 9.6 / 15.2 us at 320 / 1000 / 3000
    // rows against 8.9 / 10.9 / 17.3 with two)
    int hsplit = k.desc.sched.unroll ? (int)k.desc.sched.unroll
                 : k.desc.kind != KSH_ATTEND_DECODE || total_groups < 4 ? 1
                 : k.desc.dims[5] || hd == 512 ? total_groups : (total_groups % 2 == 0 ? total_groups / 2 : 1);
    // heads of 512: at most four per workgroup (the fold's LDS)
    if (hd == 512 && !k.desc.sched.unroll && total_groups / hsplit > 4 && total_groups % 4 == 0) hsplit = total_groups / 4;
    if (hsplit < 1 || hsplit > 255 || total_groups % hsplit) return set_error("sdpa: unsupported schedule unroll=%d (must divide %d)", hsplit, total_groups);
    if (hd == 512 && total_groups / hsplit > 4) return set_error("sdpa: heads of 512 take at most four q heads per workgroup (unroll=%d leaves %d)", hsplit, total_groups / hsplit);
    const int wg_groups = total_groups / hsplit;
    // the unmerged decode step with one head per workgroup: four waves (eight row groups to fold instead of sixteen; in
    // cfg4's loop 1207-1210 against 1194-1197 tok/s with eight, per launch 4.1 against 4.7 us at 64 rows, equal at 300 - 600)
    if (!k.desc.sched.nsg && k.desc.kind == KSH_ATTEND_DECODE && k.desc.dims[5] != 0 && wg_groups == 1 && hd == 256) nw = 4;
    // heads of 512, one per workgroup, merging: eight waves at every partition length (16 row groups of 32 lanes)
    if (!k.desc.sched.nsg && k.desc.kind == KSH_ATTEND_DECODE && k.desc.dims[5] == 0 && wg_groups == 1 && hd == 512) nw = 8;
    const size_t lds = lanes_lds(hd, wg_groups, nw, k.desc.kind == KSH_ATTEND_DECODE && lanes_few_heads(1, k.desc.dims[5] ? kModeSplitPart : kModeMerge, wg_groups, hd));
    const bool merges = k.desc.kind == KSH_SDPA_SLOTS || k.desc.kind == KSH_SDPA_BATCH || (k.desc.kind == KSH_ATTEND_DECODE && !k.desc.dims[5]);
    if (merges && !(k.desc.kind == KSH_SDPA_SLOTS && balanced_slots(n_slots, nwg)) &&   // (those merge in a launch of their own)
        (size_t)wg_groups * (nwg + 16) * 3 * 4 > (size_t)nw * (64 / (hd / 8)) * ((wg_groups <= 4 ? 4 : 8) * hd) * 4)
        return set_error("sdpa: nwg=%d is too many partitions for the merge", nwg);
    k.scratch_bytes = (size_t)n_slots * n_kv * hsplit * 4;
    if (k.desc.kind == KSH_SDPA_BATCH) k.scratch_bytes = ((k.scratch_bytes + 15) & ~(size_t)15) + (size_t)n_slots * 16;   // + per-token records
    set_launch(k, (uint32_t)nwg, (uint32_t)(n_kv * hsplit), (uint32_t)n_slots, (uint32_t)nw * 64, (uint32_t)lds);
    k.info.sched = k.desc.sched;
    k.info.sched.tg = (uint64_t)nw * 64;
    k.info.sched.nsg = (uint32_t)nw;
    k.info.sched.k_split = (uint32_t)nwg;
    k.info.sched.lds_tile = 0;
    k.info.sched.unroll = (uint32_t)hsplit;
    k.variant = nwg | (nw << 16) | (hsplit << 24);
    k.launch = launch_bound;
    return 0;
}

// AttendDecode: RmsNormPerHeadQkvQ40 + split-KV attention + merge, one launch.
int bind_attend_decode(ksh_kernel &k)
{
    const int64_t *d = k.desc.dims;
    const int64_t n_q = d[0], n_kv = d[1], hd = d[2], max_t = d[3];
    int64_t nwg = d[4];
    if (n_q <= 0 || n_kv <= 0 || n_q % n_kv) return set_error("attend_decode: n_q=%lld n_kv=%lld", (long long)n_q, (long long)n_kv);
    if (!sdpa_lanes_supports(n_q, n_kv, hd))
        return set_error("attend_decode: built for hd 128, 256 or 512 and up to 8 q heads per kv head (got hd=%lld, %lld)",
                         (long long)hd, (long long)(n_q / n_kv));
    if (max_t <= 0 || max_t > (1 << 24)) return set_error("attend_decode: max_seq=%lld", (long long)max_t);
    if (nwg == 0 && k.desc.sched.k_split) nwg = k.desc.sched.k_split;   // K-split from the schedule
    if (nwg == 0) nwg = max_t >= 2048 ? 16 : (max_t + 127) / 128;
    const size_t kvb = (size_t)max_t * n_kv * (hd / 32) * 18, qb = (size_t)n_q * hd * 4, kb = (size_t)n_kv * hd * 4;
    const bool parts_only = d[5] != 0, reader = d[7] != 0;
    const size_t partb = (size_t)n_q * nwg * (hd + 2) * 4;
    for (int i = 0; i < 7; i++) k.in_align[i] = 4;
    k.in_align[0] = 16;
    k.in_bytes[0] = qb; k.in_bytes[1] = (size_t)hd * 4; k.in_bytes[2] = (d[6] ? 1 : (size_t)max_t) * hd * 4;
    if (reader) {
        // nothing to append: in: q, q_norm, rope, K cache, V cache, meta   out: parts | tmp, o
        k.info.n_inputs = 6;
        k.info.n_outputs = parts_only ? 1 : 2;
        k.in_bytes[3] = k.in_bytes[4] = kvb; k.in_bytes[5] = 16;
        k.in_align[3] = k.in_align[4] = 2;
        k.out_bytes[0] = partb; k.out_bytes[1] = qb;
        k.out_align[0] = parts_only ? 16 : 4; k.out_align[1] = 4;
    } else {
        k.info.n_inputs = 7;
        k.info.n_outputs = parts_only ? 3 : 4;
        k.in_bytes[3] = kb; k.in_bytes[4] = (size_t)hd * 4; k.in_bytes[5] = kb; k.in_bytes[6] = 16;
        k.out_bytes[0] = k.out_bytes[1] = kvb;
        k.out_bytes[2] = partb;
        k.out_bytes[3] = qb;
        k.out_align[0] = k.out_align[1] = 2; k.out_align[2] = parts_only ? 16 : 4; k.out_align[3] = 4;
    }
    if (bind_sdpa_lanes(k, (int)nwg, 1)) return 1;
    set_name(k, "attend_decode%s%s_hd%d_nwg%d_w%d_h%d", reader ? "_reader" : "", parts_only ? "_parts" : "", (int)hd, (int)nwg, (int)k.info.sched.nsg,
             (int)k.info.sched.unroll);
    return 0;
}

}  // namespace ksh
