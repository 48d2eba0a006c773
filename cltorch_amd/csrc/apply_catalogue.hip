// Ahead-of-time kernels of the operator catalogue (THCL_CATALOGUE_OPS): every layout family
// of the apply engine for the unary math functions, pow / tpow / cpow, clamp, atan2,
// element-wise max / min, the comparisons and maskedFill.  The host side (planning, launch)
// is apply.hip's; this file only instantiates kernels, so that the two operator tables
// compile side by side.
#include <hip/hip_runtime.h>

#include "apply_kernels.h"

namespace {
THCL_CATALOGUE_OPS(THCL_DEFINE_OP_STRUCT)
}  // namespace

#define X(name, nt, stmt) THCL_DEFINE_APPLY_KERNELS(thcl_k_##name, Op_##name, nt)
THCL_CATALOGUE_OPS(X)
#undef X

namespace {
const ThclKernelSet kCatalogue[OP_COUNT - OP_FIXED_COUNT] = {THCL_CATALOGUE_OPS(THCL_KERNEL_SET_ENTRY)};
}  // namespace

const ThclKernelSet *thcl_catalogue_kernel_sets() { return kCatalogue; }
