// Kinds that are declared in the C ABI but whose kernels are not built yet:
// binding them is an error, never a fallback.
#include "ksh_internal.hpp"

namespace ksh {
int bind_matvec_batch(ksh_kernel &) { return set_error("matvec_batch (Q4_K prefill GEMM) is not built yet"); }
}  // namespace ksh

