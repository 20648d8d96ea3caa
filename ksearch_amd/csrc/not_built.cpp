// Kinds that are declared in the C ABI but whose kernels are not built yet:
// binding them is an error, never a fallback.
#include "ksh_internal.hpp"

namespace ksh {
}  // namespace ksh

