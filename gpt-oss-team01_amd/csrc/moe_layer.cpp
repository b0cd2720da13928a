// Host side of the MoE block: workspace layout and the launch sequence
// router GEMM -> top-k/softmax -> stable grouping + tile list -> grouped GEMM1 (+gather, +SwiGLU)
// -> grouped GEMM2 -> ordered weighted combine.  Nothing here synchronises or allocates.
#include <math.h>
#include <stdlib.h>

#include <algorithm>

#include "common.hpp"
#include "gemm.hpp"
#include "glue.hpp"

namespace gptoss {

struct MoeWorkspace {
  float *logits, *topk_w;
  int *topk_i, *expert_offsets, *sorted_pair_ids, *inv_perm, *tiles, *xcd_bounds, *sort_scratch;
  bf16_t *act;
  float *y2;
  size_t bytes;
};

static MoeWorkspace carve(void *base, int B, int E, int k, int H, int I) {
  MoeWorkspace w;
  size_t off = 0;
  auto take = [&](size_t n) {
    size_t o = off;
    off += align_up(n, 256);
    return reinterpret_cast<unsigned char *>(base) + o;
  };
  const size_t P = (size_t)B * k;
  w.logits = (float *)take((size_t)B * E * 4);
  w.topk_w = (float *)take(P * 4);
  w.topk_i = (int *)take(P * 4);
  w.expert_offsets = (int *)take((size_t)(E + 1) * 4);
  w.sorted_pair_ids = (int *)take(P * 4);
  w.inv_perm = (int *)take(P * 4);
  w.tiles = (int *)take((1 + 3 * (P / 32 + E)) * 4);
  w.xcd_bounds = (int *)take((XCD_BOUNDS_INTS + P / 32 + E) * 4);
  w.sort_scratch = (int *)take(group_sort_scratch_ints(B, k, E) * 4);
  w.act = (bf16_t *)take(P * I * 2);
  w.y2 = (float *)take(P * H * 4);
  w.bytes = off;
  return w;
}

// Row-tile size for B*k pairs over E experts.
// bf16 weights (32, 64, 128 or 160 rows): the smallest tile that holds an average expert's rows
// plus 2.5 standard deviations of a uniform routing, so that nearly every expert is a single tile
// and its weights are streamed exactly once; the kernel is bound by that stream.
// MXFP4 weights (32 or 64 rows): tiles of at most 64 rows, whose kernels run two workgroups per
// CU within 128 registers; an expert's few row tiles are walked column tile by column tile
// (tile_block), so its weights still come from HBM once.  The 96-row kernel does not fit that
// budget (it spills 12-97 registers, and every reload in its slab loop waits for the loads in
// flight): 384 / 512 tokens on 32 experts, where 96 rows would hold a whole expert, GEMM1 108 /
// 119 us and GEMM2 141 / 150 us with it against 91 / 115 and 56 / 78 us with 64-row tiles.
static int env_int(const char *name, int dflt) {
  const char *e = getenv(name);
  const int n = e ? atoi(e) : 0;
  return n > 0 ? n : dflt;
}
// average rows per expert from which a bf16 MoE block uses the 256-row kernels of gemm_tall.hip
int moe_tall_min_rows() {
  static const int v = env_int("GPTOSS_MOE_TALL_MIN_ROWS", 512);
  return v;
}

int moe_rows_per_tile(int B, int k, int E, bool mxfp4) {
  double avg = (double)B * k / E;
  double need = avg + 2.5 * sqrt(avg);

  if (need <= 32) return 32;
  if (need <= 64) return 64;
  if (mxfp4) return 64;
  if (need <= 128) return 128;
  return 160;
}

// Fixed part of a work item's cost, in half units of one 32-row block of arithmetic, used to cut
// the work list into 8 equally expensive parts.  With bf16 weights an item is dominated by
// streaming its 1.5 MB of W whatever its row count (16 + blocks); with MXFP4 weights, a quarter of
// the bytes, the arithmetic weighs more (5 + blocks).  Both constants are the measured optimum on a
// Zipf-skewed routing; a uniform routing is indifferent to them.
constexpr int MOE_TILE_COST0_X2_BF16 = 32;
constexpr int MOE_TILE_COST0_X2_MXFP4 = 10;

static int check_moe(const gptoss_moe_weights *w, const void *t, int B, float *out, void *ws,
                     size_t ws_bytes) {
  GPTOSS_REQUIRE(w && t && out, GPTOSS_ERR_NULL, "moe_forward: null pointer");
  GPTOSS_REQUIRE(w->w_router && w->w1 && w->w2, GPTOSS_ERR_NULL, "moe_forward: null weight pointer");
  const int E = w->n_experts, k = w->top_k, H = w->hidden, I = w->intermediate;
  GPTOSS_REQUIRE(B >= 0 && E >= 1 && E <= 256 && k >= 1 && k <= 8 && k <= E, GPTOSS_ERR_DIM,
                 "moe_forward: need 1 <= k <= min(8,E), E <= 256 (B=%d E=%d k=%d)", B, E, k);
  GPTOSS_REQUIRE(aligned(t, 16), GPTOSS_ERR_ALIGN, "moe_forward: t must be 16-byte aligned");
  GPTOSS_REQUIRE(H > 0 && I > 0 && H % 64 == 0 && I % 64 == 0, GPTOSS_ERR_DIM,
                 "moe_forward: need hidden %% 64 == 0 and intermediate %% 64 == 0 (H=%d I=%d)", H, I);
  GPTOSS_REQUIRE((long long)B * k * (long long)(H > I ? H : I) < (1ll << 31), GPTOSS_ERR_DIM,
                 "moe_forward: B*k*max(H,I) must stay below 2^31");
  GPTOSS_REQUIRE(aligned(t, 16) && aligned(out, 16) && aligned(w->w1, 16) && aligned(w->w2, 16) &&
                     aligned(w->w_router, 16),
                 GPTOSS_ERR_ALIGN, "moe_forward: pointers must be 16-byte aligned");
  GPTOSS_REQUIRE(ws != nullptr && aligned(ws, 256), GPTOSS_ERR_WORKSPACE,
                 "moe_forward: workspace missing or not 256-byte aligned");
  size_t need = gptoss_moe_workspace_bytes(B, E, k, H, I);
  GPTOSS_REQUIRE(ws_bytes >= need, GPTOSS_ERR_WORKSPACE,
                 "moe_forward: workspace has %zu bytes, needs %zu", ws_bytes, need);
  return GPTOSS_OK;
}

}  // namespace gptoss

using namespace gptoss;

extern "C" size_t gptoss_moe_workspace_bytes(int B, int E, int k, int H, int I) {
  if (B < 0 || E <= 0 || k <= 0 || H <= 0 || I <= 0) return 0;
  return carve(nullptr, B, E, k, H, I).bytes;
}

extern "C" int gptoss_moe_workspace_views(void *workspace, int B, int E, int k, int H, int I,
                                          float **logits, float **topk_w, int **topk_i,
                                          int **expert_offsets, int **sorted_pair_ids,
                                          int **inv_perm) {
  GPTOSS_REQUIRE(workspace, GPTOSS_ERR_NULL, "moe_workspace_views: null workspace");
  GPTOSS_REQUIRE(B >= 0 && E > 0 && k > 0 && H > 0 && I > 0, GPTOSS_ERR_DIM,
                 "moe_workspace_views: bad dimensions");
  MoeWorkspace w = carve(workspace, B, E, k, H, I);
  if (logits) *logits = w.logits;
  if (topk_w) *topk_w = w.topk_w;
  if (topk_i) *topk_i = w.topk_i;
  if (expert_offsets) *expert_offsets = w.expert_offsets;
  if (sorted_pair_ids) *sorted_pair_ids = w.sorted_pair_ids;
  if (inv_perm) *inv_perm = w.inv_perm;
  return GPTOSS_OK;
}

static int moe_forward_impl(const gptoss_moe_weights *w, const void *t, int B, float *out,
                            int accumulate, void *workspace, size_t workspace_bytes, void *stream,
                            int mxfp4, const float *norm_w = nullptr, bf16_t *norm_out = nullptr,
                            const MoePreNorm *pre = nullptr) {
  int rc = check_moe(w, t, B, out, workspace, workspace_bytes);
  if (rc != GPTOSS_OK) return rc;
  if (B == 0) return GPTOSS_OK;
  const int E = w->n_experts, k = w->top_k, H = w->hidden, I = w->intermediate;
  hipStream_t s = (hipStream_t)stream;
  MoeWorkspace ws = carve(workspace, B, E, k, H, I);
  int rpt = moe_rows_per_tile(B, k, E, mxfp4 != 0);
  // a prompt pass, hundreds of rows per expert: bound by the matrix cores, not by streaming W
  // (the kernels address a row of A by a 32-bit byte offset: batches beyond that stay on the streaming kernels)
  const long long tall_rows = ((long long)B * k / 256 + E) * 256;
  if (!mxfp4 && (long long)B * k >= (long long)moe_tall_min_rows() * E && gemm_tall_shape_ok(2 * I, H, tall_rows) &&
      gemm_tall_shape_ok(H, I, tall_rows))
    rpt = 256;
  const int max_tiles = gptoss_moe_max_tiles(B, k, E, rpt);
  // Each expert's row tiles are walked in blocks of up to MOE_TILE_BLOCK, column tile by column
  // tile, so the workgroups of an XCD share a column tile of the expert's weights among the block's
  // row tiles instead of streaming it once per row tile.  With one tile per expert (a decode step
  // under uniform routing) the order is the plain one; a skewed routing (Zipf 0.6-1.1 over 32
  // experts, seven of them above 160 rows) runs the layer 7 % faster, prompt passes 2-4 %.
  const int tile_block = MOE_TILE_BLOCK;

  // router GEMM with the gating of its own 16 tokens fused in, then the stable grouping
  // (with `pre`, the residual add and RMSNorm that produce t run in the same launch)
  if (pre && norm_router_applies(B, H, E, pre->x, pre->residual, pre->weight, t))
    rc = run_norm_router(pre->x, pre->residual, pre->weight, const_cast<void *>(t), w->w_router, w->b_router,
                         ws.logits, B, H, E, k, ws.topk_w, ws.topk_i, s);
  else {
    if (pre) {
      rc = run_rmsnorm(pre->x, pre->residual, pre->weight, (bf16_t *)const_cast<void *>(t), nullptr, B, H, s);
      if (rc != GPTOSS_OK) return rc;
    }
    rc = run_router(t, w->w_router, w->b_router, ws.logits, B, H, E, k, ws.topk_w, ws.topk_i, s);
  }
  if (rc != GPTOSS_OK) return rc;
  rc = run_group(B, E, k, ws.topk_w, ws.topk_i, ws.expert_offsets, ws.sorted_pair_ids, ws.inv_perm,
                 ws.tiles, rpt, ws.xcd_bounds, mxfp4 ? MOE_TILE_COST0_X2_MXFP4 : MOE_TILE_COST0_X2_BF16, s,
                 ws.sort_scratch);
  const int *bounds = max_tiles < 32768 ? ws.xcd_bounds : nullptr;
  if (rc != GPTOSS_OK) return rc;

  GemmParams g1{};
  g1.A = (const bf16_t *)t;
  g1.row_ids = ws.sorted_pair_ids;
  g1.top_k = k;
  g1.W = (const bf16_t *)w->w1;
  g1.w_mxfp4 = mxfp4;
  g1.bias = w->b1;
  g1.out = ws.act;
  g1.tiles = ws.tiles;
  g1.tile_block = tile_block;
  g1.xcd_bounds = bounds;
  g1.N = 2 * I;
  g1.K = H;
  g1.n_col_tiles = gemm_col_tiles(2 * I);
  g1.limit = w->swiglu_limit;
  rc = run_gemm(g1, true, EPI_SWIGLU, rpt, max_tiles, s);
  if (rc != GPTOSS_OK) return rc;

  GemmParams g2{};
  g2.A = ws.act;
  g2.W = (const bf16_t *)w->w2;
  g2.w_mxfp4 = mxfp4;
  g2.bias = w->b2;
  g2.out = ws.y2;
  g2.tiles = ws.tiles;
  g2.tile_block = tile_block;
  g2.xcd_bounds = bounds;
  g2.N = H;
  g2.K = I;
  g2.n_col_tiles = gemm_col_tiles(H);
  rc = run_gemm(g2, false, EPI_F32, rpt, max_tiles, s);
  if (rc != GPTOSS_OK) return rc;

  return run_combine(ws.y2, ws.topk_w, ws.inv_perm, out, B, H, k, accumulate, norm_w, norm_out, s);
}

int gptoss::moe_forward_norm(const gptoss_moe_weights *w, const void *t, int B, float *out, void *workspace,
                             size_t workspace_bytes, hipStream_t s, int mxfp4, const float *norm_w,
                             bf16_t *norm_out, const MoePreNorm *pre) {
  return moe_forward_impl(w, t, B, out, 1, workspace, workspace_bytes, s, mxfp4, norm_w, norm_out, pre);
}

extern "C" int gptoss_moe_forward(const gptoss_moe_weights *w, const void *t, int B, float *out,
                                  int accumulate, void *workspace, size_t workspace_bytes,
                                  void *stream) {
  return moe_forward_impl(w, t, B, out, accumulate, workspace, workspace_bytes, stream, 0);
}

extern "C" int gptoss_moe_forward_mxfp4(const gptoss_moe_weights *w, const void *t, int B, float *out,
                                        int accumulate, void *workspace, size_t workspace_bytes,
                                        void *stream) {
  return moe_forward_impl(w, t, B, out, accumulate, workspace, workspace_bytes, stream, 1);
}
