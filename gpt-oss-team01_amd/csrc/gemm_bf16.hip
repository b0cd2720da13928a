// bf16-weight instantiations of the grouped GEMM kernel.
#include "gemm_kernel.hpp"

namespace gptoss {
GPTOSS_GEMM_INSTANTIATE(false)
GPTOSS_GEMM_SET_ATTRS(gemm_set_attrs_bf16, false)
int gemm_col_tiles(int N) { return (N + BN - 1) / BN; }
}  // namespace gptoss
