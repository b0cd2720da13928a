// MXFP4-weight instantiations of the grouped GEMM kernel.
#include "gemm_kernel.hpp"

namespace gptoss {
GPTOSS_GEMM_INSTANTIATE(true)
GPTOSS_GEMM_SET_ATTRS(gemm_set_attrs_mxfp4, true)
}  // namespace gptoss
