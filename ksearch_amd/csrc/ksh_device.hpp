// Device-side helpers shared by the gfx950 kernels: wave64 reductions over DPP,
// half conversion, unaligned little-endian loads and Q4_K scale unpacking.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdint>

namespace ksh {

// Phase timestamps, compiled in only with -DKSH_STAMPS (the timeline build of the library; the product build has
// none).  A wave reads the chip-wide 100 MHz real-time counter at its phase boundaries into registers
// (KSH_STAMP(slot)) and writes the lot when it is done (KSH_STAMP_FLUSH: waits for the wave's own memory operations
// to be acknowledged, takes the last slot, stores the record) -- a store in the middle of the kernel would be a
// second kind of memory operation in flight, and the exact counts the kernels wait on would turn into waits for
// everything.  Records are indexed by (tag, wave in the launch), a tag per kernel shape, so the buffer holds the
// last launch of each shape; the counter is the same for every wave of the chip, so records of different kernels
// share one time axis.  Each translation unit that stamps defines the buffer with KSH_STAMP_BUFFER and an
// extern "C" reader with KSH_STAMP_READER(name).
constexpr int kStampSlots = 8, kStampWaves = 4096, kStampTags = 8;
#ifdef KSH_STAMPS
#define KSH_STAMP_BUFFER static __device__ unsigned long long g_stamps[ksh::kStampTags * ksh::kStampWaves * ksh::kStampSlots];
#define KSH_STAMP_BEGIN unsigned long long ksh_st_[ksh::kStampSlots] = {}; ksh_st_[0] = wall_clock64();
#define KSH_STAMP(slot)                                                                                                   \
    do {                                                                                                                  \
        __builtin_amdgcn_sched_barrier(0); /* nothing is scheduled across the reading of the counter */                   \
        ksh_st_[slot] = wall_clock64();                                                                                   \
        __builtin_amdgcn_sched_barrier(0);                                                                                \
    } while (0)
// pins "value v is in its register" in front of the next timestamp (a load's result is otherwise waited for wherever
// the compiler first needs it)
#define KSH_STAMP_USE(v) asm volatile("" ::"v"(v))
#define KSH_STAMP_FLUSH(tag, wave_in_launch, last_slot)                                                                   \
    do {                                                                                                                  \
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                                  \
        ksh_st_[last_slot] = wall_clock64();                                                                              \
        if ((threadIdx.x & 63) == 0 && (int)(wave_in_launch) < ksh::kStampWaves) {                                         \
            unsigned long long *rec_ = g_stamps + ((size_t)(tag) * ksh::kStampWaves + (size_t)(wave_in_launch)) * ksh::kStampSlots; \
            for (int i_ = 0; i_ < ksh::kStampSlots; i_++) rec_[i_] = ksh_st_[i_];                                          \
        }                                                                                                                 \
    } while (0)
// copies the records out (and clears them): dst holds n counters, n <= tags * waves * slots
#define KSH_STAMP_READER(name)                                                                                            \
    extern "C" int name(unsigned long long *dst, size_t n)                                                                \
    {                                                                                                                     \
        const size_t all = (size_t)ksh::kStampTags * ksh::kStampWaves * ksh::kStampSlots;                                  \
        if (!dst || n > all) return 1;                                                                                    \
        if (hipDeviceSynchronize() != hipSuccess) return 1;                                                               \
        if (hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_stamps), n * 8, 0, hipMemcpyDeviceToHost) != hipSuccess) return 1;       \
        void *p = nullptr;                                                                                                \
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_stamps)) != hipSuccess) return 1;                                        \
        return hipMemset(p, 0, all * 8) != hipSuccess;                                                                    \
    }
#else
#define KSH_STAMP_BUFFER
#define KSH_STAMP_BEGIN
#define KSH_STAMP(slot) do {} while (0)
#define KSH_STAMP_USE(v) do {} while (0)
#define KSH_STAMP_FLUSH(tag, wave_in_launch, last_slot) do {} while (0)
#define KSH_STAMP_READER(name)
#endif

// Loads and stores that say "global memory" themselves.  A pointer that went
// through an opaque statement (or a select the compiler cannot see through) is
// otherwise accessed with flat instructions, which count against the LDS
// counter as well and turn every later wait into a wait for everything.
#define KSH_GLOBAL __attribute__((address_space(1)))
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint4 ldg_u4(const void *p, size_t i)
{
    const u32x4_t v = ((const KSH_GLOBAL u32x4_t *)p)[i];
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float4 ldg_f4(const float *p, size_t i)
{
    const f32x4_t v = ((const KSH_GLOBAL f32x4_t *)p)[i];
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float2 ldg_f2(const float *p, size_t i)
{
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = ((const KSH_GLOBAL f32x2_t *)p)[i];
    return make_float2(v.x, v.y);
}
__device__ __forceinline__ void stg_f4(float *p, size_t i, float4 v)
{
    f32x4_t w;
    w.x = v.x; w.y = v.y; w.z = v.z; w.w = v.w;
    ((KSH_GLOBAL f32x4_t *)p)[i] = w;
}
__device__ __forceinline__ void stg_f32(float *p, size_t i, float v) { ((KSH_GLOBAL float *)p)[i] = v; }

constexpr int kWave = 64;

// A zero the compiler cannot see through, in a vector register.  Added to the index of a load whose address is the
// same in every lane, it keeps the load a vector load.  Left alone such a load becomes a scalar load, and scalar
// loads return out of order: the first wait for ANY of them -- the kernel arguments included -- then waits for all,
// which puts a memory round trip for a small record in front of everything issued behind that wait.
__device__ __forceinline__ int opaque_zero_v()
{
    int z = 0;
    asm volatile("" : "+v"(z));
    return z;
}

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// IEEE half bits -> f32 (exact, subnormals included)
__device__ __forceinline__ float half_bits_to_f32(uint32_t h16)
{
    return __half2float(__ushort_as_half((unsigned short)h16));
}

// f32 -> half bits, round-to-nearest-even (what Metal's half() does)
__device__ __forceinline__ uint32_t f32_to_half_bits(float f)
{
    return (uint32_t)__half_as_ushort(__float2half_rn(f));
}

// byte K of a dword as f32 in one instruction (v_cvt_f32_ubyteK).  Written as
// inline asm because, given the C expression, the optimizer first folds the
// caller's nibble mask into a per-element bit-field extract, which costs an
// extra instruction per weight.
template <int K>
__device__ __forceinline__ float ubyte_f32(uint32_t w)
{
    float f;
    if (K == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(w));
    if (K == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(w));
    if (K == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(w));
    if (K == 3) asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(w));
    return f;
}

// ---- DPP butterflies.  A DPP row is 16 lanes; quad_perm / row_half_mirror /
// row_mirror combine lanes inside a row without touching LDS.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v)
{
    return as_f32((uint32_t)__builtin_amdgcn_update_dpp(0, (int)as_u32(v), CTRL, 0xF, 0xF, true));
}

// sum over each 16-lane row, result in every lane of the row
__device__ __forceinline__ float row16_sum(float v)
{
    v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);  // row_half_mirror
    v += dpp_f32<0x140>(v);  // row_mirror
    return v;
}

// sum over the whole wave64, result wave-uniform
// A value about to be split into hi = f16(x) and lo = f16(x - hi): pinned to a register first.  Where x is a product
// (or sum) the compiler sees, it folds the conversion of hi into a mixed-precision fma that rounds the exact product
// once in one use and converts the rounded f32 in another; at a rounding tie the two differ by an f16 ulp and the
// parts then belong to different values.
__device__ __forceinline__ float pinned(float x)
{
    asm volatile("" : "+v"(x));
    return x;
}

__device__ __forceinline__ float wave_sum(float v)
{
    v = row16_sum(v);
    float a = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 0));
    float b = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 16));
    float c = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 32));
    float d = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 48));
    return (a + b) + (c + d);
}

// sums over lanes [0,32) and [32,64): lo half's total in .x, hi half's in .y
__device__ __forceinline__ float2 wave_half_sums(float v)
{
    v = row16_sum(v);
    float a = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 0));
    float b = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 16));
    float c = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 32));
    float d = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 48));
    return make_float2(a + b, c + d);
}

__device__ __forceinline__ float wave_max(float v)
{
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    v = fmaxf(v, dpp_f32<0x140>(v));
    float a = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 0));
    float b = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 16));
    float c = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 32));
    float d = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// ---- Q4_K scales.  `sy, sz, sw` are the three dwords holding the 12 scale
// bytes (bytes 4..15 of the block).  Returns for 64-element group g (0..3) the
// (scale, min) of its low-nibble sub-block 2g in .x/.y and of its high-nibble
// sub-block 2g+1 in .z/.w, all as small integers.  Same bit algebra as
// get_scale_min_k4 (crates/ksearch_gguf/src/gguf_impl.rs:563-573) in its
// 16-bit-pair form (crates/ksearch_codegen/src/render.rs:486-489).
__device__ __forceinline__ uint4 q4k_group_scales(uint32_t sy, uint32_t sz, uint32_t sw, int g)
{
    const int sh = (g & 1) * 16;
    const uint32_t a = (sy >> sh) & 0xFFFFu;  // bytes 2iq, 2iq+1
    const uint32_t b = (sz >> sh) & 0xFFFFu;  // bytes 4+2iq, 5+2iq
    const uint32_t c = (sw >> sh) & 0xFFFFu;  // bytes 8+2iq, 9+2iq
    uint32_t scp, mnp;
    if (g < 2) {
        scp = a & 0x3F3Fu;
        mnp = b & 0x3F3Fu;
    } else {
        scp = (c & 0x0F0Fu) | ((a & 0xC0C0u) >> 2);
        mnp = ((c >> 4) & 0x0F0Fu) | ((b & 0xC0C0u) >> 2);
    }
    return make_uint4(scp & 0xFFu, mnp & 0xFFu, scp >> 8, mnp >> 8);
}

}  // namespace ksh
