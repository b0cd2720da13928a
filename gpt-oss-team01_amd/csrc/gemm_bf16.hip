// bf16-weight instantiations of the grouped GEMM kernel.
#include "gemm_kernel.hpp"

namespace gptoss {
GPTOSS_GEMM_INSTANTIATE(false)
}  // namespace gptoss
