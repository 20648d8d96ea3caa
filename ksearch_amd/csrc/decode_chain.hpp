// The decode chain (decode_chain.hip): launch parameters and the host-side entry points the decode loop uses.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace ksh {

constexpr int kChainWorkgroups = 256;     // one per compute unit: all of them must be resident at once
constexpr int kChainHidden = 2048, kChainFfn = 8192;
constexpr uint32_t kChainSentinel = 0xFFFFFFFFu;   // "not written yet" in a handed-over vector (a NaN no GEMV produces)

struct ChainParams {
    // o-projection: the attention output f32[2048], or attn_parts > 0 unmerged partitions {o[heads][parts][hd], (m, l)[heads][parts]}
    const uint8_t *wo;
    const float *attn;
    int attn_parts, hd_log2;
    // feed-forward
    const uint8_t *wgate, *wup, *wdown;
    const float *post_attn_norm, *ffn_norm;
    float *x;              // the residual stream: read at the start, rewritten by workgroup 0
    // the next layer's q | k | v (not in the last layer's launch, which stores down's output instead)
    const uint8_t *wq, *wk, *wv;
    const float *post_ffw_norm, *attn_norm_next;
    float *q_out, *k_out, *v_out;
    float *y_out;
    int last;
    float eps;
    // hand-over vectors of this launch (o[2048], ff[8192], y[2048]) and of the other set, which this launch resets
    uint32_t *o, *ff, *y, *o_other, *ff_other, *y_other;
    int *err;
    int spin_limit;
};

size_t decode_chain_lds_bytes();
bool decode_chain_fits_device();   // all kChainWorkgroups workgroups resident at once
int decode_chain_launch(const ChainParams &p, hipStream_t st);
int decode_chain_fill(uint32_t *buf, int n, hipStream_t st);   // every word the sentinel

}  // namespace ksh
