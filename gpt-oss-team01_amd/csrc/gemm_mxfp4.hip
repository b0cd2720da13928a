// MXFP4-weight instantiations of the grouped GEMM kernel.
#include "gemm_kernel.hpp"

namespace gptoss {
GPTOSS_GEMM_INSTANTIATE(true)
}  // namespace gptoss
