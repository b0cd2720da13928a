// Diagnostic: the issue rate of the matrix instructions the expert GEMMs could use, measured with
// operands that never leave the registers (no loads, no LDS).  It is what the choice between the
// bf16 MFMA and the scaled f8f6f4 MFMA for MXFP4 experts rests on: the scaled instruction takes
// 4-bit weights unexpanded only if the other operand is 8 bits or narrower.
#include "common.hpp"

namespace gptoss {

typedef int i32x8 __attribute__((ext_vector_type(8)));

// KIND 0: v_mfma_f32_32x32x16_bf16; 1: v_mfma_scale_f32_32x32x64_f8f6f4 with fp8 (e4m3) x fp4
// operands; 2: fp4 x fp4; 3: fp8 x fp8.  Four independent accumulators per wave.
template <int KIND>
__global__ __launch_bounds__(512, 2) void mfma_rate_kernel(int iters, float *sink) {
  constexpr int NACC = 4;
  f32x16 acc[NACC];
#pragma unroll
  for (int i = 0; i < NACC; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[i][r] = 0.f;
  i32x8 a8 = {(int)threadIdx.x, 1, 2, 3, 4, 5, 6, 7}, b8 = {5, (int)threadIdx.x * 3, 7, 9, 1, 2, 3, 4};
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < NACC; i++) {
      if (KIND == 0) {
        const u32x4 av = {(uint32_t)a8[0], 1u, 2u, 3u}, bv = {(uint32_t)b8[0], 2u, 3u, 4u};
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(bv), as_bf16x8(av), acc[i], 0, 0, 0);
      } else if (KIND == 1) {
        acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, acc[i], 0, 4, 0, 127, 0, 127);
      } else if (KIND == 2) {
        acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, acc[i], 4, 4, 0, 127, 0, 127);
      } else {
        acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, acc[i], 0, 0, 0, 127, 0, 127);
      }
    }
    b8[0] += 1;
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NACC; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) s += acc[i][r];
  if (s == 12345.f) sink[0] = s;  // keeps the loop alive; never true in practice
}

}  // namespace gptoss

using namespace gptoss;

extern "C" int gptoss_diag_mfma_rate(int kind, int workgroups, int iters, float *sink, double *flop, void *stream) {
  GPTOSS_REQUIRE(sink && flop, GPTOSS_ERR_NULL, "diag_mfma_rate: null pointer");
  GPTOSS_REQUIRE(kind >= 0 && kind <= 3 && workgroups > 0 && iters > 0, GPTOSS_ERR_DIM,
                 "diag_mfma_rate: kind %d outside 0..3, or non-positive workgroups / iters", kind);
  hipStream_t s = (hipStream_t)stream;
  switch (kind) {
    case 0: mfma_rate_kernel<0><<<workgroups, 512, 0, s>>>(iters, sink); break;
    case 1: mfma_rate_kernel<1><<<workgroups, 512, 0, s>>>(iters, sink); break;
    case 2: mfma_rate_kernel<2><<<workgroups, 512, 0, s>>>(iters, sink); break;
    default: mfma_rate_kernel<3><<<workgroups, 512, 0, s>>>(iters, sink); break;
  }
  GPTOSS_LAUNCH_CHECK("mfma_rate_kernel");
  // 8 waves x 4 accumulators x iters instructions of 2 * 32 * 32 * k flop
  *flop = (double)workgroups * 8 * 4 * (double)iters * 2.0 * 32 * 32 * (kind == 0 ? 16.0 : 64.0);
  return GPTOSS_OK;
}
