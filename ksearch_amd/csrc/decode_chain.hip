// The four GEMVs between two attention launches of a decode step as ONE launch:
//
//   o-projection (of the attention output, or of its unmerged partitions)        -> o
//   x1 = x + rms(o) * post_attn_norm;  gelu(Wgate rms(x1) * ffn_norm) * (Wup ..) -> ff
//   down(ff)                                                                      -> y
//   x2 = x1 + rms(y) * post_ffw_norm;  Wq | Wk | Wv on rms(x2) * attn_norm'       -> q, k, v of the next layer
//
// (gemma_prim.rs:1062-1197 and, for the last phase, :946-961 of the next layer; the same arithmetic as the four
// launches KSH_ATTN_MERGE_MATVEC / KSH_MATVEC, KSH_RMSNORM_MATVEC_GATE_UP_GELU, KSH_MATVEC, KSH_RMSNORM_MATVEC_QKV
// that it replaces.)  Each phase needs the whole vector the phase before it produced, which between launches is
// what the kernel boundary provides.  Here the 256 workgroups stay resident, every workgroup owns a row slice of
// every matrix, and a phase's result vector is handed over THROUGH MEMORY WITH THE DATA AS ITS OWN FLAG: the vector
// was filled with a sentinel bit pattern beforehand, producers write their rows with write-through (agent-scope)
// stores, consumers poll the vector with agent-scope loads until no sentinel is left.  No counter, no fence, no
// cache maintenance; the next phases' weights are requested before the wait and stream under it.
//
// Sentinels: three vectors (o, ff, y) in two sets.  A launch uses one set and, first thing, resets its own slices of
// the OTHER set, which the previous launch used and the next one will: the kernel boundary between launches orders
// the reset before the next launch's polls and after the previous launch's.  (Launches alternate sets; a caller
// with an odd number of them per token refills both sets between tokens.)
//
// Every wait is bounded.  A wait that runs out raises *err; every wave polls that flag while it waits and stops
// waiting once it is up, so the grid always drains.  The results of such a launch are garbage and the host must
// check the flag (ksh::decode_chain_error) before it trusts them.
//
// Built for the benchmark shape's widths: hidden 2048, feed-forward 8192, q 2048 + k 256 + v 256 rows, Q4_K.
//
// Order of the requests: a wave that stalls issuing a long batch of cold loads cannot reach a barrier either, and
// loads come back in the order they were issued (per compute unit, across waves), so a poll queued behind megabytes
// of weights sees its vector late.  Each phase's weights are therefore requested behind the staging barrier of the
// phase before it, where they stream under that phase's arithmetic and the next wait.
//
// Off by default (KSEARCH_DECODE_CHAIN=1 switches it on): measured at the benchmark shape it is correct and slower
// than the four launches it replaces (20 - 22 us of phases per layer against 20.4 us), because every phase still pays
// its staging (1.3 - 1.8 us) and the three hand-overs cost 1.3 - 3.4 us each where a kernel boundary costs ~1.9.
#include "gemv_prologue.hpp"
#include "ksh_internal.hpp"
#include "q4k_lane.hpp"
#include "decode_chain.hpp"

namespace ksh {
namespace {

constexpr int NT = 512, NWG = kChainWorkgroups;
constexpr int HID = kChainHidden, FFN = kChainFfn;
constexpr int QROWS = 2048, KVROWS = 256;
constexpr uint32_t SENT = kChainSentinel;
constexpr size_t kRowBytesH = (size_t)(HID / 256) * 144, kRowBytesF = (size_t)(FFN / 256) * 144;

__device__ __forceinline__ uint32_t ld_agent(const uint32_t *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_agent(uint32_t *p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

struct Wait {
    int *err;
    int limit;
    bool dead;
};

// K float4 (elements 4 (i + k NT) ..) of a handed-over vector, once none of their words is the sentinel.  The loads
// are 128-bit and agent-coherent (sc1: past this XCD's L2, which other XCDs' write-through stores do not update).
template <int K>
__device__ __forceinline__ void poll_vec(const uint32_t *buf, int i, float4 (&out)[K], Wait &w)
{
    u32x4_t v[K];
    int spins = 0;
    for (;;) {
#pragma unroll
        for (int k = 0; k < K; k++) {
            const uint32_t *a = buf + 4 * (size_t)(i + k * NT);
            asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v[k]) : "v"(a) : "memory");
        }
#pragma unroll
        for (int k = 0; k < K; k++) asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[k]) : : "memory");
        bool ok = true;
#pragma unroll
        for (int k = 0; k < K; k++) ok &= v[k].x != SENT && v[k].y != SENT && v[k].z != SENT && v[k].w != SENT;
        if (ok || w.dead) break;
        if (++spins > w.limit) {
            __hip_atomic_store(w.err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            w.dead = true;
            break;
        }
        if ((spins & 31) == 31 && __hip_atomic_load(w.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
            w.dead = true;
            break;
        }
    }
#pragma unroll
    for (int k = 0; k < K; k++) out[k] = make_float4(as_f32(v[k].x), as_f32(v[k].y), as_f32(v[k].z), as_f32(v[k].w));
}

__global__ __launch_bounds__(NT) void decode_chain_kernel(ChainParams p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];   // the staged vector (digit planes) + reduction scratch
    __shared__ float red2[NT / 64][2];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), w = blockIdx.x;
    const int sb = (tid & 31) >> 2, g = tid & 3;       // this lane's (superblock, group) in a 2048-column row
    const int hw = tid >> 5;                            // half-wave 0..15: one 2048-column row per half-wave
    Wait wt{p.err, p.spin_limit, false};

    // ---- everything that does not depend on a hand-over is requested now, in the order it is needed
    // the other set's slices, for the launch after this one
    if (tid < 8) st_agent(p.o_other + 8 * w + tid, SENT);
    else if (tid < 16) st_agent(p.y_other + 8 * w + (tid - 8), SENT);
    else if (tid < 48) st_agent(p.ff_other + 32 * w + (tid - 16), SENT);
    Prologue prA{};
    prA.x = p.attn;
    prA.kind = p.attn_parts ? kMergeParts : kPlain;
    prA.w_norm = p.attn + (size_t)HID * p.attn_parts;   // the (m, l) pairs follow the values
    prA.nwg = p.attn_parts;
    prA.hd_log2 = p.hd_log2;
    StageRegs sA;
    stage_fetch<NT, true>(prA, HID, sA);
    const float4 res_in = ldg_f4(p.x, tid), w_post_b = ldg_f4(p.post_attn_norm, tid), w_norm_b = ldg_f4(p.ffn_norm, tid);
    float4 w_post_d = make_float4(0.f, 0.f, 0.f, 0.f), w_norm_d = w_post_d;
    if (!p.last) {
        w_post_d = ldg_f4(p.post_ffw_norm, tid);
        w_norm_d = ldg_f4(p.attn_norm_next, tid);
    }
    // o-projection: 8 rows per workgroup, one (row, superblock, group) per lane of the first four waves
    Q4kLane la{};
    if (wave < 4) la = q4k_load(p.wo + (size_t)(8 * w + hw) * kRowBytesH + (size_t)sb * 144, g);
    Q4kLane lb[4];

    // ---- phase A: o = Wo . attention output
    stage_finish<kXI8, NT, true>(prA, lds, HID, sA);
    __syncthreads();
    // gate || up: 32 + 32 rows per workgroup, four per half-wave: gate rows hw and hw + 16, up rows hw and hw + 16.
    // Behind the staging barrier: a wave that stalls issuing these cannot reach the barrier either.
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const uint8_t *base = k < 2 ? p.wgate : p.wup;
        lb[k] = q4k_load(base + (size_t)(32 * w + hw + 16 * (k & 1)) * kRowBytesH + (size_t)sb * 144, g);
    }
    XGroup<kXI8> X;
    X.load(lds, HID, sb, g);
    {
        const float v = wave < 4 ? q4k_group_dot<kXI8>(la, g, X) : 0.f;
        const float2 s2 = wave_half_sums(v);
        if (wave < 4 && lane == 0) {
            st_agent(p.o + 8 * w + 2 * wave, as_u32(s2.x));
            st_agent(p.o + 8 * w + 2 * wave + 1, as_u32(s2.y));
        }
    }
    __syncthreads();   // everybody has read the staged vector

    // ---- phase B: x1 = x + rms(o) w_post;  ff = gelu(Wgate n) * (Wup n),  n = rms(x1) w_ffn
    const int sbc = (tid & 127) >> 2;
    Q4kLane lc[2];
    float4 resid;
    {
        StageRegs sB;
        { float4 t4[1]; poll_vec<1>(p.o, tid, t4, wt); sB.x[0] = t4[0]; }
        sB.wn[0] = w_norm_b;
        sB.wp[0] = w_post_b;
        sB.rs[0] = res_in;
        Prologue prB{};
        prB.kind = kAddThenRms;
        prB.eps = p.eps;
        prB.x_out = p.x;                                  // (workgroup 0 writes x1: the LM head reads it after the last layer)
        prB.nwg = __builtin_bit_cast(int, 1.0f);
        stage_finish<kXI8, NT>(prB, lds, HID, sB);
        resid = sB.x[0];
    }
    __syncthreads();
    // down: 8 rows of 8192 columns per workgroup, a row per wave pair, two per lane
#pragma unroll
    for (int k = 0; k < 2; k++) lc[k] = q4k_load(p.wdown + (size_t)(8 * w + (tid >> 7) + 4 * k) * kRowBytesF + (size_t)sbc * 144, g);
    X.load(lds, HID, sb, g);
    {
        float2 s2[4];
#pragma unroll
        for (int k = 0; k < 4; k++) s2[k] = wave_half_sums(q4k_group_dot<kXI8>(lb[k], g, X));
        if (lane == 0) {
            // half-waves 2 wave, 2 wave + 1: rows hw and hw + 16 of this workgroup's 32
            st_agent(p.ff + 32 * w + 2 * wave, as_u32(gelu_mul_f32(s2[0].x, s2[2].x)));
            st_agent(p.ff + 32 * w + 2 * wave + 1, as_u32(gelu_mul_f32(s2[0].y, s2[2].y)));
            st_agent(p.ff + 32 * w + 16 + 2 * wave, as_u32(gelu_mul_f32(s2[1].x, s2[3].x)));
            st_agent(p.ff + 32 * w + 16 + 2 * wave + 1, as_u32(gelu_mul_f32(s2[1].y, s2[3].y)));
        }
    }
    __syncthreads();

    // ---- phase C: y = Wdown . ff
    Q4kLane ld_{};
    {
        StageRegs sC;
        {
            float4 t4[FFN / 4 / NT];
            poll_vec<FFN / 4 / NT>(p.ff, tid, t4, wt);
#pragma unroll
            for (int k = 0; k < FFN / 4 / NT; k++) sC.x[k] = t4[k];
        }
        // q | k | v of the next layer: 2560 rows, 10 per workgroup, one per half-wave of the first five waves
        if (!p.last && wave < 5) {
            const int rr = 10 * w + hw;
            const uint8_t *base = rr < QROWS ? p.wq + (size_t)rr * kRowBytesH
                                  : rr < QROWS + KVROWS ? p.wk + (size_t)(rr - QROWS) * kRowBytesH
                                                        : p.wv + (size_t)(rr - QROWS - KVROWS) * kRowBytesH;
            ld_ = q4k_load(base + (size_t)sb * 144, g);
        }
        Prologue prC{};
        prC.kind = kPlain;
        stage_finish<kXI8, NT>(prC, lds, FFN, sC);
    }
    __syncthreads();
    {
        XGroup<kXI8> XC;
        XC.load(lds, FFN, sbc, g);
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const float s = wave_sum(q4k_group_dot<kXI8>(lc[k], g, XC));
            if (lane == 0) red2[wave][k] = s;
        }
    }
    __syncthreads();
    if (tid < 8) {
        // row r = (wave pair) + 4 k
        const int k = tid >> 2, wp2 = 2 * (tid & 3);
        const float y = red2[wp2][k] + red2[wp2 + 1][k];
        if (p.last) p.y_out[8 * w + tid] = y;
        else st_agent(p.y + 8 * w + tid, as_u32(y));
    }
    if (p.last) return;
    __syncthreads();   // the staged vector and red2 are free again

    // ---- phase D: x2 = x1 + rms(y) w_post;  q | k | v = W . (rms(x2) w_attn')
    {
        StageRegs sD;
        { float4 t4[1]; poll_vec<1>(p.y, tid, t4, wt); sD.x[0] = t4[0]; }
        sD.wn[0] = w_norm_d;
        sD.wp[0] = w_post_d;
        sD.rs[0] = resid;
        Prologue prD{};
        prD.kind = kAddThenRms;
        prD.eps = p.eps;
        prD.x_out = p.x;                                  // the residual stream the next launch starts from
        prD.nwg = __builtin_bit_cast(int, 1.0f);
        stage_finish<kXI8, NT>(prD, lds, HID, sD);
    }
    __syncthreads();
    X.load(lds, HID, sb, g);
    {
        const float v = wave < 5 ? q4k_group_dot<kXI8>(ld_, g, X) : 0.f;
        const float2 s2 = wave_half_sums(v);
        if (wave < 5 && lane == 0) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int r = 10 * w + 2 * wave + h;
                const float val = h ? s2.y : s2.x;
                if (r < QROWS) p.q_out[r] = val;
                else if (r < QROWS + KVROWS) p.k_out[r - QROWS] = val;
                else p.v_out[r - QROWS - KVROWS] = val;
            }
        }
    }
}

__global__ void chain_fill_kernel(uint32_t *buf, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) buf[i] = SENT;
}

}  // namespace

size_t decode_chain_lds_bytes() { return xs_bytes<kXI8>(FFN); }

// every workgroup of the launch must be resident at once: the waits assume that all producers run
bool decode_chain_fits_device()
{
    int dev = 0, cus = 0, per_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return false;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, decode_chain_kernel, NT, decode_chain_lds_bytes()) != hipSuccess) return false;
    return (long)cus * per_cu >= NWG;
}

int decode_chain_launch(const ChainParams &p, hipStream_t st)
{
    hipLaunchKernelGGL(decode_chain_kernel, dim3(NWG), dim3(NT), decode_chain_lds_bytes(), st, p);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "decode chain launch");
}

int decode_chain_fill(uint32_t *buf, int n, hipStream_t st)
{
    hipLaunchKernelGGL(chain_fill_kernel, dim3((n + 255) / 256), dim3(256), 0, st, buf, n);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "decode chain fill launch");
}

}  // namespace ksh
