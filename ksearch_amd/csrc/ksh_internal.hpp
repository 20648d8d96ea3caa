// Shared internals of libksearch_hip: error plumbing, handle structs and the
// per-kind binder table.  Nothing here is part of the C ABI.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>

#include "../../include/ksearch_hip.h"

namespace ksh {

int set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int hip_fail(hipError_t e, const char *what);

#define KSH_HIP(expr)                                            \
    do {                                                         \
        hipError_t _e = (expr);                                  \
        if (_e != hipSuccess) return ::ksh::hip_fail(_e, #expr); \
    } while (0)

constexpr int kMaxIn = 8;
constexpr int kMaxOut = 4;

// device pointers with the caller's byte offsets already applied
struct LaunchArgs {
    const void *in[kMaxIn];
    void *out[kMaxOut];
};

}  // namespace ksh

struct ksh_buf {
    void *ptr = nullptr;
    size_t bytes = 0;
    std::atomic<int> rc{1};
    ksh_buf *parent = nullptr;   // a view: ptr lies inside the parent's allocation, which the view keeps alive
};

struct ksh_kernel {
    ksh_kernel_desc desc{};
    ksh_kernel_info info{};
    // bytes each binding must provide from its offset on (0 = not checked)
    size_t in_bytes[ksh::kMaxIn] = {};
    size_t out_bytes[ksh::kMaxOut] = {};
    // alignment each binding's device address must have
    uint32_t in_align[ksh::kMaxIn] = {};
    uint32_t out_align[ksh::kMaxOut] = {};
    int variant = 0;
    // device scratch the runtime allocates for the handle after a successful bind
    size_t scratch_bytes = 0;
    void *scratch = nullptr;
    int (*launch)(const ksh_kernel &, const ksh::LaunchArgs &, hipStream_t) = nullptr;
    // a handle with half activations at the boundary (half_boundary.hip): the f32 handle it wraps, which bindings are
    // half, and where their f32 staging lies in `scratch`
    const ksh_kernel *inner = nullptr;
    uint32_t half_in = 0, half_out = 0;
    size_t stage_in[ksh::kMaxIn] = {}, stage_out[ksh::kMaxOut] = {};
};

namespace ksh {
// what entry points outside the runtime's translation unit need of a context
hipStream_t ctx_stream(ksh_ctx *ctx);
int ctx_device(ksh_ctx *ctx);   // the ordinal of the device the context's stream belongs to
// a buffer object over bytes [off, off + bytes) of `parent` (retained until the view is released); nullptr + error when out of range
ksh_buf *buffer_view(ksh_buf *parent, size_t off, size_t bytes);
void ctx_mark_pending(ksh_ctx *ctx);
// half activations at the boundary: whether the kind takes them, and the wrapping of its bound f32 handle
bool half_boundary_kind(const ksh_kernel_desc &d);
int bind_half_boundary(ksh_kernel &k, const ksh_kernel &inner);
// resolves the device address of the static partial-result array of ksh_softcap_argmax_static for the current
// device (called when a context is created, with the context's device current; the entry point then uses the
// address kept for the context's device)
int argmax_static_setup();
// the end of a decode step (glue.hip): argmax over the logits, position update, the next token's embedding row
struct DecodeTail {
    const float *pv; const uint32_t *pi; int nparts;       // filled in by launch_decode_tail
    float *tok, *history; int max_hist;
    float *meta; const float *rope; float *rope_cur; int hd;
    const uint8_t *embd; int dtype; int64_t n_rows; int n; float scale; float *x_out;
};
int launch_decode_tail(const ksh_kernel &k_argmax, const float *logits, DecodeTail t, hipStream_t st);
}  // namespace ksh

// a pool's identity for whoever caches things per pool (HIP graphs captured over its buffers): unlike its address,
// never handed out twice
extern "C" uint64_t ksh_kvpool_uid(const ksh_kvpool *p);

// hands a buffer's reference over to a model, which releases it when it is destroyed (the GGUF loader's uploads)
extern "C" void ksh_gemma4_adopt(ksh_gemma4 *m, ksh_buf *b);

namespace ksh {

// block geometry: crates/ksearch_ir/src/lib.rs:52-74, gguf_impl.rs:50-64
inline bool block_spec(int dtype, size_t &elems, size_t &bytes)
{
    switch (dtype) {
    case KSH_F32: elems = 1; bytes = 4; return true;
    case KSH_F16: case KSH_BF16: elems = 1; bytes = 2; return true;
    case KSH_Q40: elems = 32; bytes = 18; return true;
    case KSH_Q4K: elems = 256; bytes = 144; return true;
    case KSH_Q5K: elems = 256; bytes = 176; return true;
    case KSH_Q6K: case KSH_Q6K_ROWS: elems = 256; bytes = 210; return true;
    }
    return false;
}

inline size_t packed_bytes(int dtype, size_t n)
{
    size_t e, b;
    if (!block_spec(dtype, e, b) || n % e) return 0;
    return n / e * b;
}

inline bool sched_is_zero(const ksh_sched &s)
{
    return s.tg == 0 && s.vec == 0 && s.unroll == 0 && s.nsg == 0 && s.nr0 == 0 && s.k_split == 0 &&
           s.lds_tile == 0;
}

// per-kind binders: validate the descriptor, pick a template instance, fill
// info / sizes / launch.  Return non-zero (with the error set) to refuse.
int bind_matvec(ksh_kernel &k);
int bind_matvec_q4k(ksh_kernel &k);
int bind_matvec_q6k(ksh_kernel &k);
int bind_matvec_q4k_family(ksh_kernel &k);
int bind_matvec_qkv(ksh_kernel &k);
int bind_matvec_gate_up_gelu(ksh_kernel &k);
int bind_matvec_batch(ksh_kernel &k);
int bind_round_prep(ksh_kernel &k);
int bind_matvec_round(ksh_kernel &k);
int bind_dequant(ksh_kernel &k);
int bind_repack_rows(ksh_kernel &k);
int bind_quantize_k(ksh_kernel &k);
int bind_quantize_q40(ksh_kernel &k);
int bind_sdpa(ksh_kernel &k);
bool sdpa_lanes_supports(int64_t n_q, int64_t n_kv, int64_t hd);
int bind_sdpa_lanes(ksh_kernel &k, int nwg, int n_slots);
int bind_attend_decode(ksh_kernel &k);          // NAIVE, MWG_PART, MWG_REDUCE, SLOTS
int bind_rmsnorm(ksh_kernel &k);       // RMSNORM, RMSNORM_ADD_THEN_RMSNORM
int bind_per_head_qkv_q40(ksh_kernel &k);
int bind_glue(ksh_kernel &k);          // COPY_SCALE_INDEXED, GELU_MUL, COPY_SLICE
int bind_softcap_argmax(ksh_kernel &k);
int bind_ple_ops(ksh_kernel &k);       // RMSNORM_PER_HEAD, ADD_SCALE, MATVEC_GELU_MUL
int bind_read_floor(ksh_kernel &k);

int plan_dims(const ksh_kernel_desc &d);   // how many leading dims take part in a plan's key
// candidate schedules per kind (BEAM)
int matvec_candidates(const ksh_kernel_desc &d, ksh_sched *out, int cap);

inline void set_name(ksh_kernel &k, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(k.info.name, sizeof(k.info.name), fmt, ap);
    va_end(ap);
}

inline void set_launch(ksh_kernel &k, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t lds)
{
    k.info.grid[0] = gx; k.info.grid[1] = gy; k.info.grid[2] = gz;
    k.info.block[0] = bx; k.info.block[1] = 1; k.info.block[2] = 1;
    k.info.lds_bytes = lds;
}

}  // namespace ksh
