// Kinds that are declared in the C ABI but whose kernels are not built yet:
// binding them is an error, never a fallback.
#include "ksh_internal.hpp"

namespace ksh {
int bind_matvec_batch(ksh_kernel &) { return set_error("matvec_batch (Q4_K prefill GEMM) is not built yet"); }
int bind_quantize_k(ksh_kernel &) { return set_error("quantize_k is not built yet"); }
int bind_sdpa(ksh_kernel &) { return set_error("sdpa kernels are not built yet"); }
}  // namespace ksh

extern "C" {
int ksh_gemma_create(ksh_ctx *, const ksh_gemma_cfg *, const ksh_gemma_layer *, ksh_buf *, ksh_buf *, ksh_gemma **)
{
    return ksh::set_error("the decode loop is not built yet");
}
void ksh_gemma_destroy(ksh_gemma *) {}
int ksh_gemma_reset(ksh_gemma *) { return ksh::set_error("the decode loop is not built yet"); }
int ksh_gemma_forward_token(ksh_gemma *, uint32_t, int, uint32_t *) { return ksh::set_error("the decode loop is not built yet"); }
int ksh_gemma_generate(ksh_gemma *, const uint32_t *, int, int, int, uint32_t *, double *, double *)
{
    return ksh::set_error("the decode loop is not built yet");
}
ksh_buf *ksh_gemma_logits(ksh_gemma *) { return nullptr; }
ksh_buf *ksh_gemma_hidden(ksh_gemma *) { return nullptr; }
ksh_buf *ksh_gemma_kv(ksh_gemma *, int, int) { return nullptr; }
int ksh_gemma_pos(ksh_gemma *) { return -1; }
int ksh_gemma_launches_per_token(ksh_gemma *) { return -1; }
}
