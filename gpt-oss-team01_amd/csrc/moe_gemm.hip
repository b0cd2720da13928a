// Grouped (per-expert) and dense bf16 GEMMs for gfx950 built on v_mfma_f32_32x32x16_bf16.
//
//   C[rows, N] = A[rows, K] . W[N, K]^T      rows = the tokens routed to one expert (or a slice
//                                            of a dense batch), W = that expert's matrix
//
// Shape of the problem at decode time: a few hundred rows per expert against 25 M weights per
// expert, i.e. every weight is used by ~128 rows and the kernel is bound by streaming W from
// HBM.  The design follows from that:
//   * W is stored in MFMA-fragment order (gptoss_pack_weight): the 1 KB a wave needs for one
//     32-column x 16-k operand is contiguous, so each wave streams its own columns with
//     perfectly coalesced 128-bit loads straight into registers (no LDS hop, no reuse needed:
//     a workgroup covers all rows of its tile, up to 256, so W is read once);
//   * the activations (shared by the 4 waves) go through a double-buffered, padded LDS tile; the
//     token gather of the reference's pack step is folded into that load;
//   * a workgroup = 256 virtual columns x up to 256 rows; each wave owns 64 columns as two
//     B fragments and reuses every A fragment it reads from LDS for two MFMAs;
//   * work items come from the device-built tile list (expert,row0,rows), mapped so that the
//     workgroups of one XCD walk consecutive column tiles of the same expert (A stays in that
//     XCD's L2);
//   * epilogues: +bias -> fp32, or +bias -> clamped SwiGLU -> bf16 with gate and up of a pair in
//     the same lane (arranged by the packing order, so no cross-lane traffic).
#include <type_traits>

#include "common.hpp"
#include "gemm.hpp"

namespace gptoss {

constexpr int GEMM_THREADS = 256;
constexpr int BK = 64;            // k per LDS slab (4 MFMA k-steps)
constexpr int LDS_ROW = BK + 8;   // padded row length in bf16 elements (144 B)
constexpr int BN = 256;           // virtual columns per workgroup (4 waves x 64)

// One (row tile, column tile) work item with a compile-time number of 32-row blocks, so every
// loop below is fully unrolled and every global load is unconditional (the wait counters the
// compiler derives stay exact and the prefetches stay in flight across iterations).
template <int MB, bool GATHER, int EPI>
__device__ __forceinline__ void gemm_tile(const GemmParams &p, bf16_t *lds, int lds_stage, int mat,
                                          int row0, int rows, int ct) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int K = p.K, N = p.N;
  const int n0_raw = ct * BN + wave * 64;
  const bool wave_active = n0_raw < N;
  const int n0 = wave_active ? n0_raw : N - 64;  // idle waves of the last column tile redo a valid one
  const int nslab = K / BK;
  const int ksteps = K / 16;

  // ---- A: each thread moves one 16-byte chunk per 32-row block and slab -----------------------
  const int a_row = tid >> 3, a_kc = tid & 7;
  uint32_t a_off[MB];
#pragma unroll
  for (int i = 0; i < MB; i++) {
    int r = a_row + 32 * i;
    int src = 0;
    if (r < rows) {
      if (GATHER) src = p.row_ids[row0 + r] / p.top_k;
      else src = row0 + r;
    } else if (!GATHER) {
      src = row0;
    }
    a_off[i] = (uint32_t)src * (uint32_t)K + a_kc * 8;
  }
  u32x4 areg[MB];
  auto load_a = [&](int s) {
#pragma unroll
    for (int i = 0; i < MB; i++) areg[i] = *reinterpret_cast<const u32x4 *>(p.A + a_off[i] + s * BK);
  };
  bf16_t *a_dst = lds + a_row * LDS_ROW + a_kc * 8;
  auto store_a = [&](int stage) {
#pragma unroll
    for (int i = 0; i < MB; i++)
      *reinterpret_cast<u32x4 *>(a_dst + stage * lds_stage + 32 * i * LDS_ROW) = areg[i];
  };

  // ---- B: two fragment streams per wave, three slabs in the register ring ---------------------
  const bf16_t *wbase = p.W + (size_t)mat * N * K + ((size_t)(n0 >> 5) * ksteps * 64 + lane) * 8;
  const size_t frag_stride = (size_t)ksteps * 512;  // elements between adjacent 32-column blocks
  u32x4 breg[3][2][4];
  auto load_b = [&](int s, auto ring) {
    constexpr int R = decltype(ring)::value;
#pragma unroll
    for (int f = 0; f < 2; f++)
#pragma unroll
      for (int kk = 0; kk < 4; kk++)
        breg[R][f][kk] = *reinterpret_cast<const u32x4 *>(wbase + f * frag_stride +
                                                          (size_t)(s * 4 + kk) * 512);
  };

  f32x16 acc[MB][2];
#pragma unroll
  for (int i = 0; i < MB; i++)
#pragma unroll
    for (int f = 0; f < 2; f++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][f][r] = 0.f;

  const bf16_t *a_src = lds + (lane & 31) * LDS_ROW + (lane >> 5) * 8;
  auto compute = [&](int stage, auto ring) {
    constexpr int R = decltype(ring)::value;
    const bf16_t *base = a_src + stage * lds_stage;
#pragma unroll
    for (int kk = 0; kk < 4; kk++) {
      bf16x8 b0 = as_bf16x8(breg[R][0][kk]), b1 = as_bf16x8(breg[R][1][kk]);
#pragma unroll
      for (int i = 0; i < MB; i++) {
        bf16x8 a = as_bf16x8(*reinterpret_cast<const u32x4 *>(base + i * 32 * LDS_ROW + kk * 16));
        acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b0, acc[i][0], 0, 0, 0);
        acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b1, acc[i][1], 0, 0, 0);
      }
    }
  };

  using R0 = std::integral_constant<int, 0>;
  using R1 = std::integral_constant<int, 1>;
  using R2 = std::integral_constant<int, 2>;
  const int last = nslab - 1;

  load_b(0, R0{});
  load_b(min(1, last), R1{});
  load_a(0);
  store_a(0);
  load_a(min(1, last));
  __syncthreads();

  // slab s: prefetch B and A of slab s+2 (clamped at the end: a harmless re-read), multiply slab
  // s, publish A of slab s+1 to the other LDS stage.
  auto body = [&](int s, auto ring, auto ring_next2) {
    load_b(min(s + 2, last), ring_next2);
    compute(s & 1, ring);
    store_a((s + 1) & 1);
    load_a(min(s + 2, last));
    __syncthreads();
  };
  int s = 0;
  for (; s + 3 <= nslab; s += 3) {
    body(s, R0{}, R2{});
    body(s + 1, R1{}, R0{});
    body(s + 2, R2{}, R1{});
  }
  if (s < nslab) {
    body(s, R0{}, R2{});
    if (s + 1 < nslab) body(s + 1, R1{}, R0{});
  }

  if (!wave_active) return;

  // ---- epilogue ------------------------------------------------------------------------------
  const int c = lane & 31, rsub = (lane >> 5) * 4;
  if (EPI == EPI_SWIGLU) {
    const int half_n = N >> 1;
    const int j = (n0 >> 1) + c;  // pair index: gate = row 2j, up = row 2j+1 of the .bin matrix
    float bg = 0.f, bu = 0.f;
    if (p.bias) {
      bg = p.bias[(size_t)mat * N + 2 * j];
      bu = p.bias[(size_t)mat * N + 2 * j + 1];
    }
    bf16_t *o = reinterpret_cast<bf16_t *>(p.out);
    const float L = p.limit;
#pragma unroll
    for (int i = 0; i < MB; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int row = i * 32 + (r >> 2) * 8 + rsub + (r & 3);
        if (row < rows) {
          float g = acc[i][0][r] + bg, u = acc[i][1][r] + bu;
          g = fminf(g, L);
          u = fminf(fmaxf(u, -L), L);
          float v = g * (1.0f / (1.0f + expf(-1.702f * g)));
          v *= (u + 1.0f);
          o[(size_t)(row0 + row) * half_n + j] = f32_to_bf16(v);
        }
      }
    }
  } else {
#pragma unroll
    for (int f = 0; f < 2; f++) {
      const int col = n0 + f * 32 + c;
      float bv = p.bias ? p.bias[(size_t)mat * N + col] : 0.f;
#pragma unroll
      for (int i = 0; i < MB; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          int row = i * 32 + (r >> 2) * 8 + rsub + (r & 3);
          if (row < rows) {
            float v = acc[i][f][r] + bv;
            if (EPI == EPI_F32)
              reinterpret_cast<float *>(p.out)[(size_t)(row0 + row) * N + col] = v;
            else
              reinterpret_cast<bf16_t *>(p.out)[(size_t)(row0 + row) * N + col] = f32_to_bf16(v);
          }
        }
      }
    }
  }
}

template <int MBMAX, bool GATHER, int EPI>
__global__ __launch_bounds__(GEMM_THREADS) void grouped_gemm_kernel(GemmParams p) {
  constexpr int BM = MBMAX * 32;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);  // [2][BM][LDS_ROW]
  constexpr int STAGE = BM * LDS_ROW;

  // ---- which (row tile, column tile) is this workgroup's: workgroups are dealt round-robin to
  // the 8 XCDs, so XCD x takes the x-th contiguous eighth of the work list -----------------------
  const int n_tiles = p.tiles ? p.tiles[0] : (p.dense_rows + BM - 1) / BM;
  const int total = n_tiles * p.n_col_tiles;
  const int chunk = (total + 7) >> 3;
  const int slot = blockIdx.x >> 3;
  if (slot >= chunk) return;
  const int work = (blockIdx.x & 7) * chunk + slot;
  if (work >= total) return;
  const int tile = work / p.n_col_tiles, ct = work - tile * p.n_col_tiles;
  int mat, row0, rows;
  if (p.tiles) {
    mat = p.tiles[1 + 3 * tile];
    row0 = p.tiles[2 + 3 * tile];
    rows = p.tiles[3 + 3 * tile];
  } else {
    mat = 0;
    row0 = tile * BM;
    rows = min(BM, p.dense_rows - row0);
  }
  const int mb = (rows + 31) >> 5;
  if (MBMAX >= 8 && mb > 6) {
    if (mb == 8) gemm_tile<(MBMAX >= 8 ? 8 : MBMAX), GATHER, EPI>(p, lds, STAGE, mat, row0, rows, ct);
    else gemm_tile<(MBMAX >= 8 ? 7 : MBMAX), GATHER, EPI>(p, lds, STAGE, mat, row0, rows, ct);
  } else if (MBMAX >= 8 && mb > 4) {
    if (mb == 6) gemm_tile<(MBMAX >= 8 ? 6 : MBMAX), GATHER, EPI>(p, lds, STAGE, mat, row0, rows, ct);
    else gemm_tile<(MBMAX >= 8 ? 5 : MBMAX), GATHER, EPI>(p, lds, STAGE, mat, row0, rows, ct);
  } else if (MBMAX >= 4 && mb > 2) {
    if (mb == 4) gemm_tile<(MBMAX >= 4 ? 4 : MBMAX), GATHER, EPI>(p, lds, STAGE, mat, row0, rows, ct);
    else gemm_tile<(MBMAX >= 4 ? 3 : MBMAX), GATHER, EPI>(p, lds, STAGE, mat, row0, rows, ct);
  } else if (MBMAX >= 2 && mb == 2) {
    gemm_tile<(MBMAX >= 2 ? 2 : MBMAX), GATHER, EPI>(p, lds, STAGE, mat, row0, rows, ct);
  } else {
    gemm_tile<1, GATHER, EPI>(p, lds, STAGE, mat, row0, rows, ct);
  }
}

// Weighted combine: out[b,:] (+)= sum over the token's k experts, in ascending expert order (the
// order of the reference CPU loop, run.cpp:642-704), of w * y2[row of that pair].  Products and
// sums are rounded separately, as that loop rounds them.
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
  for (int h = threadIdx.x * 4; h < H; h += 256 * 4) {
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
  }
}

// Repack row-major [n_out, n_in] matrices into fragment order:
//   dst[((nb*KS + ks)*64 + lane)*8 + j] = W[row(nb*32 + lane%32)][ks*16 + (lane/32)*8 + j]
// With GLU pairing, virtual row v of a 64-row wave tile maps to pair (v/64)*32 + v%32, gate for
// the first 32 virtual rows and up for the second 32.
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
  if (glu) row = 2 * ((v >> 6) * 32 + (v & 31)) + ((v >> 5) & 1);
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

template <int MB, bool GATHER, int EPI>
static int launch_gemm(const GemmParams &p, int max_tiles, hipStream_t s) {
  static bool attr_done = false;
  size_t smem = (size_t)2 * MB * 32 * LDS_ROW * sizeof(bf16_t);
  auto kern = grouped_gemm_kernel<MB, GATHER, EPI>;
  if (!attr_done) {
    GPTOSS_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    attr_done = true;
  }
  int total = max_tiles * p.n_col_tiles;
  int grid = ((total + 7) / 8) * 8;
  if (grid == 0) return GPTOSS_OK;
  {
    TraceScope ts(GATHER ? "gemm1_gather_swiglu" : (EPI == EPI_F32 ? "gemm_f32" : (EPI == EPI_BF16 ? "gemm_bf16" : "gemm_swiglu")), s);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(GEMM_THREADS), smem, s, p);
  }
  GPTOSS_LAUNCH_CHECK("grouped_gemm_kernel");
  return GPTOSS_OK;
}

// Host-side dispatcher used by the MoE layer and the engine.  rows_per_tile selects MB.
int run_gemm(const GemmParams &p, bool gather, int epi, int rows_per_tile, int max_tiles,
             hipStream_t s) {
#define GPTOSS_GEMM_CASE(MBV)                                                                  \
  if (rows_per_tile == MBV * 32) {                                                             \
    if (gather && epi == EPI_SWIGLU) return launch_gemm<MBV, true, EPI_SWIGLU>(p, max_tiles, s); \
    if (!gather && epi == EPI_F32) return launch_gemm<MBV, false, EPI_F32>(p, max_tiles, s);    \
    if (!gather && epi == EPI_BF16) return launch_gemm<MBV, false, EPI_BF16>(p, max_tiles, s);  \
    if (!gather && epi == EPI_SWIGLU) return launch_gemm<MBV, false, EPI_SWIGLU>(p, max_tiles, s); \
  }
  GPTOSS_GEMM_CASE(1)
  GPTOSS_GEMM_CASE(2)
  GPTOSS_GEMM_CASE(4)
  GPTOSS_GEMM_CASE(8)
#undef GPTOSS_GEMM_CASE
  return fail(GPTOSS_ERR_DIM, "run_gemm: unsupported combination (rows_per_tile=%d gather=%d epi=%d)",
              rows_per_tile, (int)gather, epi);
}

int run_combine(const float *y2, const float *topk_w, const int *inv_perm, float *out, int B, int H,
                int k, int accumulate, hipStream_t s) {
  if (B == 0) return GPTOSS_OK;
  {
    TraceScope ts("combine", s);
    combine_kernel<<<B, 256, 0, s>>>(y2, topk_w, inv_perm, out, H, k, accumulate);
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
  GPTOSS_REQUIRE(n_mat >= 1 && n_out > 0 && n_in > 0 && n_out % (glu ? 64 : 32) == 0 && n_in % 64 == 0,
                 GPTOSS_ERR_DIM, "pack_weight: need n_out %% %d == 0 and n_in %% 64 == 0 (n_out=%d n_in=%d)",
                 glu ? 64 : 32, n_out, n_in);
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
