// Host side of the grouped/dense GEMMs (kernel dispatch), the weighted combine kernel and the
// weight repacking kernels.  The GEMM kernel itself is in gemm_kernel.hpp.
#include <stdlib.h>

#include <mutex>

#include "common.hpp"
#include "gemm.hpp"

namespace gptoss {

// Weighted combine: out[b,:] (+)= sum over the token's k experts, in ascending expert order (the
// order of the reference CPU loop, run.cpp:642-704), of w * y2[row of that pair].  Products and
// sums are rounded separately, as that loop rounds them.
template <int VPT>  // float4 chunks per thread: rows of at most 1024 * VPT floats (0: any length, a loop)
__global__ __launch_bounds__(256) void combine_kernel(const float *__restrict__ y2,
                                                      const float *__restrict__ topk_w,
                                                      const int *__restrict__ inv_perm,
                                                      float *__restrict__ out, int H, int k,
                                                      int accumulate) {
  const int b = blockIdx.x;
  int rows[8];
  float w[8];
#pragma unroll
  for (int s = 0; s < 8; s++) {
    rows[s] = (s < k) ? inv_perm[(size_t)b * k + s] : 0x7fffffff;
    w[s] = (s < k) ? topk_w[(size_t)b * k + s] : 0.f;
  }
  // sorted position grows with expert id, so ordering by row orders by expert
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j + 1 < 8 - i; j++)
      if (rows[j] > rows[j + 1]) {
        int tr = rows[j]; rows[j] = rows[j + 1]; rows[j + 1] = tr;
        float tw = w[j]; w[j] = w[j + 1]; w[j + 1] = tw;
      }
  auto chunk = [&](int h) {
    f32x4 agg = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 8; s++) {
      if (s < k) {
        f32x4 v = *reinterpret_cast<const f32x4 *>(y2 + (size_t)rows[s] * H + h);
#pragma unroll
        for (int q = 0; q < 4; q++) agg[q] = __fadd_rn(agg[q], __fmul_rn(v[q], w[s]));
      }
    }
    f32x4 *op = reinterpret_cast<f32x4 *>(out + (size_t)b * H + h);
    if (accumulate) {
      f32x4 prev = *op;
#pragma unroll
      for (int q = 0; q < 4; q++) agg[q] = __fadd_rn(prev[q], agg[q]);
    }
    *op = agg;
  };
  if constexpr (VPT > 0) {
    // unrolled: the loads of every chunk are in flight before the first sum needs one
#pragma unroll
    for (int i = 0; i < VPT; i++) {
      const int h = (threadIdx.x + 256 * i) * 4;
      if (h < H) chunk(h);
    }
  } else {
    for (int h = threadIdx.x * 4; h < H; h += 256 * 4) chunk(h);
  }
}

// The same combine followed by the RMSNorm of the updated row (the next block's input norm), for
// rows of at most 1024 * VPT floats: every thread keeps its elements in registers between the two
// steps.  Element-to-thread mapping, the double-precision sum of squares and the scaling are those
// of rmsnorm_rows_kernel (glue.hip), so the result equals running the two kernels one after the
// other bit for bit.
template <int VPT>
__global__ __launch_bounds__(256) void combine_norm_kernel(const float *__restrict__ y2,
                                                           const float *__restrict__ topk_w,
                                                           const int *__restrict__ inv_perm,
                                                           float *__restrict__ out, int H, int k,
                                                           const float *__restrict__ norm_w,
                                                           bf16_t *__restrict__ t_bf16) {
  __shared__ double red[4];
  const int b = blockIdx.x;
  int rows[8];
  float w[8];
#pragma unroll
  for (int s = 0; s < 8; s++) {
    rows[s] = (s < k) ? inv_perm[(size_t)b * k + s] : 0x7fffffff;
    w[s] = (s < k) ? topk_w[(size_t)b * k + s] : 0.f;
  }
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j + 1 < 8 - i; j++)
      if (rows[j] > rows[j + 1]) {
        int tr = rows[j]; rows[j] = rows[j + 1]; rows[j + 1] = tr;
        float tw = w[j]; w[j] = w[j + 1]; w[j + 1] = tw;
      }
  f32x4 v[VPT];
  double ss = 0.0;
#pragma unroll
  for (int i = 0; i < VPT; i++) {
    const int h = (threadIdx.x + 256 * i) * 4;
    v[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (h < H) {
      f32x4 agg = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 8; s++) {
        if (s < k) {
          const f32x4 y = *reinterpret_cast<const f32x4 *>(y2 + (size_t)rows[s] * H + h);
#pragma unroll
          for (int q = 0; q < 4; q++) agg[q] = __fadd_rn(agg[q], __fmul_rn(y[q], w[s]));
        }
      }
      f32x4 *op = reinterpret_cast<f32x4 *>(out + (size_t)b * H + h);
      const f32x4 prev = *op;
#pragma unroll
      for (int q = 0; q < 4; q++) v[i][q] = __fadd_rn(prev[q], agg[q]);
      *op = v[i];
#pragma unroll
      for (int q = 0; q < 4; q++) ss += (double)__fmul_rn(v[i][q], v[i][q]);
    }
  }
  for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  ss = red[0] + red[1] + red[2] + red[3];
  ss /= H;
  ss += 1e-5f;
  const double inv = (double)(1.0f / sqrtf((float)ss));
#pragma unroll
  for (int i = 0; i < VPT; i++) {
    const int h = (threadIdx.x + 256 * i) * 4;
    if (h < H) {
      const f32x4 nw = *reinterpret_cast<const f32x4 *>(norm_w + h);
      f32x4 o;
#pragma unroll
      for (int q = 0; q < 4; q++) o[q] = (float)((double)nw[q] * (inv * (double)v[i][q]));
      *reinterpret_cast<u32x2 *>(t_bf16 + (size_t)b * H + h) =
          u32x2{pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
    }
  }
}

// Repack row-major [n_out, n_in] matrices into fragment order:
//   dst[((nb*KS + ks)*64 + lane)*8 + j] = W[row(nb*32 + lane%32)][ks*16 + (lane/32)*8 + j]
// With GLU pairing, virtual row v of a 32-row block maps to pair (v/32)*16 + v%16, gate for the
// first 16 virtual rows and up for the second 16.
template <typename SRC>
__global__ __launch_bounds__(256) void pack_weight_kernel(const SRC *__restrict__ src,
                                                          bf16_t *__restrict__ dst, int n_out,
                                                          int n_in, int glu) {
  const int ksteps = n_in / 16;
  const size_t frags_per_mat = (size_t)(n_out / 32) * ksteps;
  const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;  // one (fragment, lane) per thread
  const size_t frag = gid >> 6;
  const int lane = (int)(gid & 63);
  const int mat = blockIdx.y;
  if (frag >= frags_per_mat) return;
  const int nb = (int)(frag / ksteps), ks = (int)(frag - (size_t)nb * ksteps);
  int v = nb * 32 + (lane & 31);
  int row = v;
  if (glu) row = 2 * ((v >> 5) * 16 + (v & 15)) + ((v >> 4) & 1);
  const SRC *sp = src + ((size_t)mat * n_out + row) * n_in + ks * 16 + (lane >> 5) * 8;
  uint32_t o[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    if constexpr (sizeof(SRC) == 4) {
      o[j] = pack_bf16x2((float)sp[2 * j], (float)sp[2 * j + 1]);
    } else {
      o[j] = (uint32_t)sp[2 * j] | ((uint32_t)sp[2 * j + 1] << 16);
    }
  }
  u32x4 *dp = reinterpret_cast<u32x4 *>(dst + ((size_t)mat * frags_per_mat + frag) * 512 + lane * 8);
  *dp = u32x4{o[0], o[1], o[2], o[3]};
}

// MXFP4 repack: blocks [n_out, n_in/2] (low nibble = even element) and e8m0 scales [n_out, n_in/32]
// -> per (32-column block, 64-k slab): 64 lanes x 16 bytes of codes, then 32 x 2 scale bytes.
__global__ __launch_bounds__(256) void pack_mxfp4_kernel(const unsigned char *__restrict__ blocks,
                                                         const unsigned char *__restrict__ scales,
                                                         unsigned char *__restrict__ dst, int n_out,
                                                         int n_in, int glu) {
  const int nslab = n_in / 64;
  const size_t items = (size_t)(n_out / 32) * nslab;          // (column block, slab)
  const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;  // one (item, lane) per thread
  const size_t item = gid >> 6;
  const int lane = (int)(gid & 63);
  const int mat = blockIdx.y;
  if (item >= items) return;
  const int nb = (int)(item / nslab), slab = (int)(item - (size_t)nb * nslab);
  int v = nb * 32 + (lane & 31);
  int row = v;
  if (glu) row = 2 * ((v >> 5) * 16 + (v & 15)) + ((v >> 4) & 1);
  const size_t mat_bytes = (size_t)n_out * n_in / 2 + (size_t)n_out * n_in / 32;
  const unsigned char *brow = blocks + ((size_t)mat * n_out + row) * (n_in / 2);
  const unsigned char *srow = scales + ((size_t)mat * n_out + row) * (n_in / 32);
  unsigned char *md = dst + (size_t)mat * mat_bytes;
  uint32_t w[4];
#pragma unroll
  for (int kk = 0; kk < 4; kk++) {
    const int k0 = (slab * 4 + kk) * 16 + (lane >> 5) * 8;  // the lane's 8 consecutive k
    w[kk] = *reinterpret_cast<const uint32_t *>(brow + k0 / 2);  // nibble j = element k0+j
  }
  *reinterpret_cast<u32x4 *>(md + (item * 64 + lane) * 16) = u32x4{w[0], w[1], w[2], w[3]};
  if (lane < 32) {
    unsigned char *sd = md + (size_t)n_out * n_in / 2 + (item * 32 + lane) * 2;
    sd[0] = srow[slab * 2];
    sd[1] = srow[slab * 2 + 1];
  }
}

// Host-side dispatcher used by the MoE layer and the engine.  rows_per_tile selects the kernel.
template <int MBMAX, bool GATHER, int EPI, bool FP4>
int launch_gemm(const GemmParams &p, int max_tiles, hipStream_t s);  // gemm_bf16.hip, gemm_mxfp4.hip

template <bool GATHER, int EPI>
static int dispatch_rows(const GemmParams &p, int rows_per_tile, int max_tiles, hipStream_t s) {
  const bool q = p.w_mxfp4 != 0;
  switch (rows_per_tile) {
    case 32: return q ? launch_gemm<1, GATHER, EPI, true>(p, max_tiles, s) : launch_gemm<1, GATHER, EPI, false>(p, max_tiles, s);
    case 64: return q ? launch_gemm<2, GATHER, EPI, true>(p, max_tiles, s) : launch_gemm<2, GATHER, EPI, false>(p, max_tiles, s);
    case 96:
      return q ? launch_gemm<3, GATHER, EPI, true>(p, max_tiles, s) : launch_gemm<3, GATHER, EPI, false>(p, max_tiles, s);
    case 128: return q ? launch_gemm<4, GATHER, EPI, true>(p, max_tiles, s) : launch_gemm<4, GATHER, EPI, false>(p, max_tiles, s);
    case 160: return q ? launch_gemm<5, GATHER, EPI, true>(p, max_tiles, s) : launch_gemm<5, GATHER, EPI, false>(p, max_tiles, s);
  }
  return fail(GPTOSS_ERR_DIM, "run_gemm: unsupported rows_per_tile %d", rows_per_tile);
}

hipError_t gemm_set_attrs_bf16();   // gemm_bf16.hip
hipError_t gemm_set_attrs_mxfp4();  // gemm_mxfp4.hip


// Raises the dynamic-LDS limit of every GEMM kernel on the calling thread's current device, the
// first time that device launches one.
static int gemm_prepare_device() {
  constexpr int MAX_DEV = 64;
  static std::mutex mu;
  static bool done[MAX_DEV];
  int dev = 0;
  GPTOSS_HIP(hipGetDevice(&dev));
  GPTOSS_REQUIRE(dev >= 0 && dev < MAX_DEV, GPTOSS_ERR_STATE, "run_gemm: device ordinal %d outside 0..%d", dev, MAX_DEV - 1);
  std::lock_guard<std::mutex> lock(mu);
  if (!done[dev]) {
    GPTOSS_HIP(gemm_set_attrs_bf16());
    GPTOSS_HIP(gemm_set_attrs_mxfp4());
    done[dev] = true;
  }
  return GPTOSS_OK;
}

int run_gemm(const GemmParams &p, bool gather, int epi, int rows_per_tile, int max_tiles,
             hipStream_t s) {
  // output and operand offsets inside the kernels are 32-bit element counts
  const long long max_rows = p.tiles ? (long long)max_tiles * rows_per_tile : p.dense_rows;
  GPTOSS_REQUIRE(max_rows * p.N < (1ll << 32) && max_rows * p.K < (1ll << 32), GPTOSS_ERR_DIM,
                 "run_gemm: rows x columns must stay below 2^32 elements (rows<=%lld N=%d K=%d)", max_rows, p.N, p.K);
  if (rows_per_tile == 256) return run_gemm_tall(p, gather, epi, max_tiles, max_rows, s);
  int prc = gemm_prepare_device();
  if (prc != GPTOSS_OK) return prc;
  if (gather && epi == EPI_SWIGLU) return dispatch_rows<true, EPI_SWIGLU>(p, rows_per_tile, max_tiles, s);
  if (!gather && epi == EPI_F32) return dispatch_rows<false, EPI_F32>(p, rows_per_tile, max_tiles, s);
  if (!gather && epi == EPI_ARGMAX && p.tiles == nullptr && p.amax_val && p.amax_idx)
    return dispatch_rows<false, EPI_ARGMAX>(p, rows_per_tile, max_tiles, s);
  return fail(GPTOSS_ERR_DIM, "run_gemm: unsupported combination (gather=%d epi=%d)", (int)gather, epi);
}

// rows from which a dense fp32-output GEMM uses the 256-row kernel of gemm_tall.hip
static int dense_tall_min_rows() {
  static const int v = [] {
    const char *e = getenv("GPTOSS_DENSE_TALL_MIN_ROWS");
    const int n = e ? atoi(e) : 0;
    return n > 0 ? n : 2048;
  }();
  return v;
}

// rows from which the classifier's arg-max GEMM uses it (measured, vocabulary 201088 x 2880: 256 rows
// 360 -> 295 us, 512 rows 716 -> 556, 1024 rows 1194 -> 986-1007, 2048 rows 2319 -> 1859)
static int argmax_tall_min_rows() {
  static const int v = [] {
    const char *e = getenv("GPTOSS_ARGMAX_TALL_MIN_ROWS");
    const int n = e ? atoi(e) : 0;
    return n > 0 ? n : 256;
  }();
  return v;
}

// C[B, N] = A[B, K] . W[N, K]^T (+ bias): the dense GEMMs of a step (QKV and output projections,
// classifier), with the kernel and row tile chosen from the batch size.
int dense_gemm(const bf16_t *A, const bf16_t *W, const float *bias, void *out, int epi, int B, int N,
               int K, hipStream_t s, float *amax_val, int *amax_idx, int *amax_tiles) {
  GemmParams g{};
  g.amax_val = amax_val;
  g.amax_idx = amax_idx;
  g.A = A;
  g.W = W;
  g.bias = bias;
  g.out = out;
  g.tiles = nullptr;
  g.dense_rows = B;
  g.N = N;
  g.K = K;
  g.n_col_tiles = gemm_col_tiles(N);
  // Row tile.  Up to 96 rows: the smallest size that holds every row, so the weights are requested
  // once.  A prompt pass (thousands of rows): 160 rows, every weight fragment feeds five MFMAs.  In
  // between the launch is a handful of rounds of work items on 256 CUs, and an item of MB 32-row
  // blocks takes (0.39 + 0.115 MB) us per 64-k slab (measured at 1024 rows: 0.50 / 0.64 / 0.76 /
  // 0.85 us for 32 / 64 / 96 / 128 rows), so the tile that needs the least rounds x slab time wins:
  // 96 rows for the QKV projection of 1024 rows (220 items, one round), 64 for the output
  // projection (192 items instead of 132: 48 -> 41 us).
  static const int sizes[5] = {32, 64, 96, 128, 160};
  int rpt = 160;
  if (B <= 96) {
    for (int i = 0; i < 5; i++)
      if (B <= sizes[i]) {
        rpt = sizes[i];
        break;
      }
  } else if (B < 2048 && g.n_col_tiles >= 64) {
    rpt = 128;  // the unembedding: hundreds of column tiles, measured best at 1024 rows
  } else if (B < 2048) {
    double best = 0.0;
    for (int mb = 1; mb <= 5; mb++) {
      const long long items = (long long)cdiv(B, 32 * mb) * g.n_col_tiles;
      const double cost = (double)((items + 255) / 256) * (0.39 + 0.115 * mb);
      if (mb == 1 || cost <= best) {  // ties go to the larger tile: fewer re-reads of the weights
        best = cost;
        rpt = 32 * mb;
      }
    }
  }
  if (B >= (epi == EPI_ARGMAX ? argmax_tall_min_rows() : dense_tall_min_rows()) && gemm_tall_applies(g, false, epi) &&
      gemm_tall_shape_ok(N, K, B))
    rpt = 256;
  if (epi == EPI_ARGMAX) {
    GPTOSS_REQUIRE(amax_tiles, GPTOSS_ERR_NULL, "dense_gemm: the arg-max form reports its pairs per row");
    *amax_tiles = rpt == 256 ? 2 * g.n_col_tiles : g.n_col_tiles;
  }
  return run_gemm(g, false, epi, rpt, cdiv(B, rpt), s);
}

int run_combine(const float *y2, const float *topk_w, const int *inv_perm, float *out, int B, int H,
                int k, int accumulate, const float *norm_w, bf16_t *norm_out, hipStream_t s) {
  if (B == 0) return GPTOSS_OK;
  // out += combine, then norm_out = RMSNorm(out) * norm_w in the same kernel, when asked for
  if (norm_w && norm_out && accumulate && H % 4 == 0 && H <= 4096 && aligned(norm_w, 16) && aligned(norm_out, 8)) {
    TraceScope ts("combine_rmsnorm", s);
    if (H <= 1024) combine_norm_kernel<1><<<B, 256, 0, s>>>(y2, topk_w, inv_perm, out, H, k, norm_w, norm_out);
    else if (H <= 2048) combine_norm_kernel<2><<<B, 256, 0, s>>>(y2, topk_w, inv_perm, out, H, k, norm_w, norm_out);
    else if (H <= 3072) combine_norm_kernel<3><<<B, 256, 0, s>>>(y2, topk_w, inv_perm, out, H, k, norm_w, norm_out);
    else combine_norm_kernel<4><<<B, 256, 0, s>>>(y2, topk_w, inv_perm, out, H, k, norm_w, norm_out);
    GPTOSS_LAUNCH_CHECK("combine_norm_kernel");
    return GPTOSS_OK;
  }
  {
    TraceScope ts("combine", s);
    if (H <= 3072 && H > 2048) combine_kernel<3><<<B, 256, 0, s>>>(y2, topk_w, inv_perm, out, H, k, accumulate);
    else if (H <= 1024) combine_kernel<1><<<B, 256, 0, s>>>(y2, topk_w, inv_perm, out, H, k, accumulate);
    else combine_kernel<0><<<B, 256, 0, s>>>(y2, topk_w, inv_perm, out, H, k, accumulate);
  }
  GPTOSS_LAUNCH_CHECK("combine_kernel");
  return GPTOSS_OK;
}

}  // namespace gptoss

using namespace gptoss;

extern "C" size_t gptoss_packed_weight_bytes(int n_mat, int n_out, int n_in) {
  if (n_mat <= 0 || n_out <= 0 || n_in <= 0) return 0;
  return (size_t)n_mat * n_out * n_in * sizeof(bf16_t);
}

extern "C" int gptoss_pack_weight(const void *src, void *dst, int n_mat, int n_out, int n_in,
                                  int flags, void *stream) {
  GPTOSS_REQUIRE(src && dst, GPTOSS_ERR_NULL, "pack_weight: null pointer");
  const int glu = (flags & GPTOSS_PACK_GLU) ? 1 : 0;
  GPTOSS_REQUIRE(n_mat >= 1 && n_out > 0 && n_in > 0 && n_out % 32 == 0 && n_in % 64 == 0, GPTOSS_ERR_DIM,
                 "pack_weight: need n_out %% 32 == 0 and n_in %% 64 == 0 (n_out=%d n_in=%d)", n_out, n_in);
  GPTOSS_REQUIRE(aligned(src, 16) && aligned(dst, 16), GPTOSS_ERR_ALIGN,
                 "pack_weight: pointers must be 16-byte aligned");
  size_t threads = (size_t)(n_out / 32) * (n_in / 16) * 64;
  dim3 grid((unsigned)((threads + 255) / 256), n_mat);
  hipStream_t s = (hipStream_t)stream;
  if (flags & GPTOSS_PACK_SRC_FP32)
    pack_weight_kernel<float><<<grid, 256, 0, s>>>((const float *)src, (bf16_t *)dst, n_out, n_in, glu);
  else
    pack_weight_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t *)src, (bf16_t *)dst, n_out, n_in, glu);
  GPTOSS_LAUNCH_CHECK("pack_weight_kernel");
  return GPTOSS_OK;
}

extern "C" size_t gptoss_packed_mxfp4_bytes(int n_mat, int n_out, int n_in) {
  if (n_mat <= 0 || n_out <= 0 || n_in <= 0) return 0;
  return (size_t)n_mat * ((size_t)n_out * n_in / 2 + (size_t)n_out * n_in / 32);
}

extern "C" int gptoss_pack_mxfp4(const void *blocks, const void *scales, void *dst, int n_mat,
                                 int n_out, int n_in, int flags, void *stream) {
  GPTOSS_REQUIRE(blocks && scales && dst, GPTOSS_ERR_NULL, "pack_mxfp4: null pointer");
  const int glu = (flags & GPTOSS_PACK_GLU) ? 1 : 0;
  GPTOSS_REQUIRE(n_mat >= 1 && n_out > 0 && n_in > 0 && n_out % 32 == 0 && n_in % 64 == 0, GPTOSS_ERR_DIM,
                 "pack_mxfp4: need n_out %% 32 == 0 and n_in %% 64 == 0 (n_out=%d n_in=%d)", n_out, n_in);
  GPTOSS_REQUIRE(aligned(blocks, 4) && aligned(dst, 16), GPTOSS_ERR_ALIGN,
                 "pack_mxfp4: blocks must be 4-byte and dst 16-byte aligned");
  size_t threads = (size_t)(n_out / 32) * (n_in / 64) * 64;
  dim3 grid((unsigned)((threads + 255) / 256), n_mat);
  pack_mxfp4_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const unsigned char *)blocks,
                                                          (const unsigned char *)scales,
                                                          (unsigned char *)dst, n_out, n_in, glu);
  GPTOSS_LAUNCH_CHECK("pack_mxfp4_kernel");
  return GPTOSS_OK;
}
