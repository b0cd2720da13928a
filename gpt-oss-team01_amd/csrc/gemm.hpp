// Internal interface of the grouped/dense GEMM kernels (moe_gemm.hip).
#pragma once
#include "common.hpp"

namespace gptoss {

enum { EPI_F32 = 0, EPI_SWIGLU = 1, EPI_BF16 = 2, EPI_ARGMAX = 3 };

// Row tiles of ONE expert are grouped into blocks of up to MOE_TILE_BLOCK consecutive tiles by the
// grouping kernel; a block never spans two experts, so every tile of a block multiplies the same
// weights.
constexpr int MOE_TILE_BLOCK = 8;
constexpr int XCD_BOUNDS_INTS = 16;  // ints reserved for the cut positions in front of the block table

struct GemmParams {
  const bf16_t *A;     // activations, row-major [*, K]
  const int *row_ids;  // gather: sorted pair ids (row of A = id / top_k); else unused
  int top_k;
  const bf16_t *W;     // packed weights, per-matrix stride N*K (or MXFP4 bytes when w_mxfp4)
  int w_mxfp4;         // W holds gptoss_pack_mxfp4 output
  const float *bias;   // [n_mat, N] or nullptr
  void *out;           // EPI_F32: float [*, N]; EPI_SWIGLU: bf16 [*, N/2]; EPI_BF16: bf16 [*, N]
  float *amax_val;     // EPI_ARGMAX (dense only): per (row, column tile) the largest value ...
  int *amax_idx;       // ... and the lowest column that holds it, [rows, n_col_tiles] (the 256-row
                       // kernel: per (row, 128-column half of a tile), [rows, 2 n_col_tiles])
  const int *tiles;    // {n_tiles, (mat,row0,rows)*} or nullptr for a dense problem
  const int *xcd_bounds;  // 9 positions in the tile list (tile << 16 | 16-bit fraction) that cut the
                          // work into 8 parts of equal estimated cost, or nullptr: equal item counts.
                          // From index XCD_BOUNDS_INTS on: one int per row tile, the block it belongs
                          // to (first tile << 8 | tiles in the block; see MOE_TILE_BLOCK)
  int tile_block;      // grouped problems, > 1: the row tiles of a block are walked together, column
                       // tile by column tile (needs xcd_bounds); 0 or 1 = every row tile on its own
  int dense_rows;      // rows of the dense problem when tiles == nullptr
  int N, K;
  int n_col_tiles;     // gemm_col_tiles(N)
  float limit;         // SwiGLU clamp
};

// rows_per_tile in {32,64,96,128,160}, or 256 where gemm_tall_applies(); max_tiles bounds the number of
// (mat,row-tile) items.
int run_gemm(const GemmParams &p, bool gather, int epi, int rows_per_tile, int max_tiles,
             hipStream_t s);
// gemm_tall.hip: tiles of 256 x 256 with both operands through LDS, for launches of thousands of rows,
// bound by the matrix cores (bf16 weights; gather + SwiGLU, plain fp32 output, or the row arg-max).  max_rows bounds
// the rows of A that the launch can address.
bool gemm_tall_applies(const GemmParams &p, bool gather, int epi);
// what the 256-row kernels need of a problem besides its form: whole 64-k chunks, at least 8 stages
// of 32 k, whole 32-column blocks, and every row of A within a 32-bit byte offset
inline bool gemm_tall_shape_ok(int N, int K, long long max_rows) {
  return K % 64 == 0 && K >= 256 && N % 32 == 0 && max_rows * K * 2 < (1ll << 32);
}
int run_gemm_tall(const GemmParams &p, bool gather, int epi, int max_tiles, long long max_rows, hipStream_t s);
// norm_w / norm_out (optional, accumulate only): also write RMSNorm(out) * norm_w as bf16.  Returns
// with only the combine done when the fused form does not apply (H > 4096 or misaligned); the
// caller checks with combine_norm_applies().
int run_combine(const float *y2, const float *topk_w, const int *inv_perm, float *out, int B, int H,
                int k, int accumulate, const float *norm_w, bf16_t *norm_out, hipStream_t s);
inline bool combine_norm_applies(int H, const float *norm_w, const bf16_t *norm_out) {
  return norm_w && norm_out && H % 4 == 0 && H <= 4096 && aligned(norm_w, 16) && aligned(norm_out, 8);
}
// The norm in front of the MoE block, for the block to run itself: x += residual (residual may be
// null), t = RMSNorm(x) * weight written to the block's input buffer.
struct MoePreNorm {
  float *x;
  const float *residual;
  const float *weight;
};
// The MoE block with the RMSNorm of the updated residual stream fused into its last kernel
// (moe_layer.cpp); out is accumulated into.  With `pre`, t is an output of the call as well: the norm
// that produces it runs inside the router kernel (or in a kernel of its own where that kernel's
// limits do not allow it).
int moe_forward_norm(const gptoss_moe_weights *w, const void *t, int B, float *out, void *workspace,
                     size_t workspace_bytes, hipStream_t s, int mxfp4, const float *norm_w, bf16_t *norm_out,
                     const MoePreNorm *pre = nullptr);
// moe_route.hip: residual add + RMSNorm + router GEMM + gating in one launch
bool norm_router_applies(int B, int H, int E, const float *x, const float *residual, const float *weight,
                         const void *t_out);
int run_norm_router(float *x, const float *residual, const float *weight, void *t_out, const void *w_router,
                    const float *b_router, float *logits, int B, int H, int E, int k, float *topk_w, int *topk_i,
                    hipStream_t s);
int moe_rows_per_tile(int B, int k, int E, bool mxfp4);
// dense C = A . W^T (+ bias) with the epilogue `epi`; EPI_ARGMAX fills amax_val / amax_idx [B, *amax_tiles]
// EPI_ARGMAX: *amax_tiles (required) receives the number of (value, column) pairs written per row,
// at most gemm_argmax_tiles(N), for run_argmax_tiles to finish
int dense_gemm(const bf16_t *A, const bf16_t *W, const float *bias, void *out, int epi, int B, int N, int K,
               hipStream_t s, float *amax_val = nullptr, int *amax_idx = nullptr, int *amax_tiles = nullptr);
int gemm_col_tiles(int N);  // column tiles of one workgroup's width
inline int gemm_argmax_tiles(int N) { return 2 * gemm_col_tiles(N); }  // pairs per row to allocate for EPI_ARGMAX
// moe_route.hip
int run_router(const void *t, const void *w_router, const float *b_router, float *logits, int B,
               int H, int E, int k, float *topk_w, int *topk_i, hipStream_t s);
int run_topk_softmax(const float *logits, int B, int E, int k, float *topk_w, int *topk_i, hipStream_t s);
// xcd_bounds (optional, XCD_BOUNDS_INTS + max_tiles ints): see GemmParams; tile_cost0_x2 = twice the fixed part of a tile's
// cost in units of one 32-row block of arithmetic (cost = fixed + number of 32-row blocks);
// sort_scratch (optional, group_sort_scratch_ints(B, k, E) ints): lets batches of 8192 pairs and more
// be sorted by many workgroups
int run_group(int B, int E, int k, float *topk_w, int *topk_i, int *expert_offsets,
              int *sorted_pair_ids, int *inv_perm, int *tiles, int rows_per_tile, int *xcd_bounds,
              int tile_cost0_x2, hipStream_t s, int *sort_scratch = nullptr);
inline size_t group_sort_scratch_ints(int B, int k, int E) { return (size_t)cdiv(B * k, 1024) * E; }

}  // namespace gptoss
