// C ABI of the glue ops around the two hot ops of a decode step: thin, validating wrappers over
// the kernels of glue.hip and the dense GEMM dispatch, for a host that keeps the reference's own
// forward loop (getp-csrc/src/model.cpp:6-151) and binds it op by op.
#include "common.hpp"
#include "gemm.hpp"
#include "glue.hpp"

using namespace gptoss;

extern "C" int gptoss_embedding(const void *table, const int *tokens, float *x, int B, int H, int V, void *stream) {
  GPTOSS_REQUIRE(table && tokens && x, GPTOSS_ERR_NULL, "embedding: null pointer");
  GPTOSS_REQUIRE(B >= 0 && H > 0 && V > 0, GPTOSS_ERR_DIM, "embedding: bad dimensions (B=%d H=%d V=%d)", B, H, V);
  if (B == 0) return GPTOSS_OK;
  return run_embedding((const bf16_t *)table, tokens, x, B, H, V, (hipStream_t)stream);
}

extern "C" int gptoss_rmsnorm(float *x, const float *residual, const float *weight, void *t_bf16, int B, int H,
                              void *stream) {
  GPTOSS_REQUIRE(x && weight && t_bf16, GPTOSS_ERR_NULL, "rmsnorm: null pointer");
  GPTOSS_REQUIRE(B >= 0 && H > 0, GPTOSS_ERR_DIM, "rmsnorm: bad dimensions (B=%d H=%d)", B, H);
  if (B == 0) return GPTOSS_OK;
  return run_rmsnorm(x, residual, weight, (bf16_t *)t_bf16, nullptr, B, H, (hipStream_t)stream);
}

static int check_dense(const void *a, const void *w, int B, int N, int K, const char *who) {
  GPTOSS_REQUIRE(a && w, GPTOSS_ERR_NULL, "%s: null pointer", who);
  GPTOSS_REQUIRE(B >= 0 && N > 0 && K > 0 && N % 32 == 0 && K % 64 == 0, GPTOSS_ERR_DIM,
                 "%s: need N %% 32 == 0 and K %% 64 == 0 (B=%d N=%d K=%d)", who, B, N, K);
  GPTOSS_REQUIRE(aligned(a, 16) && aligned(w, 16), GPTOSS_ERR_ALIGN, "%s: pointers must be 16-byte aligned", who);
  return GPTOSS_OK;
}

extern "C" int gptoss_dense_gemm(const void *a, const void *w_packed, const float *bias, float *out, int B, int N,
                                 int K, void *stream) {
  int rc = check_dense(a, w_packed, B, N, K, "dense_gemm");
  if (rc != GPTOSS_OK) return rc;
  GPTOSS_REQUIRE(out && aligned(out, 16), GPTOSS_ERR_NULL, "dense_gemm: out is NULL or not 16-byte aligned");
  if (B == 0) return GPTOSS_OK;
  return dense_gemm((const bf16_t *)a, (const bf16_t *)w_packed, bias, out, EPI_F32, B, N, K, (hipStream_t)stream);
}

extern "C" size_t gptoss_classifier_argmax_workspace_bytes(int B, int V) {
  if (B <= 0 || V <= 0) return 0;
  return 2 * align_up((size_t)B * gemm_argmax_tiles(V) * sizeof(float), 256);
}

extern "C" int gptoss_classifier_argmax(const void *a, const void *w_packed, int *next_ids, int B, int V, int K,
                                        void *workspace, size_t workspace_bytes, void *stream) {
  int rc = check_dense(a, w_packed, B, V, K, "classifier_argmax");
  if (rc != GPTOSS_OK) return rc;
  GPTOSS_REQUIRE(next_ids, GPTOSS_ERR_NULL, "classifier_argmax: null pointer");
  if (B == 0) return GPTOSS_OK;
  const size_t half = align_up((size_t)B * gemm_argmax_tiles(V) * sizeof(float), 256);
  GPTOSS_REQUIRE(workspace && aligned(workspace, 256) && workspace_bytes >= 2 * half, GPTOSS_ERR_WORKSPACE,
                 "classifier_argmax: workspace missing, misaligned or smaller than %zu bytes", 2 * half);
  float *val = (float *)workspace;
  int *idx = (int *)((unsigned char *)workspace + half);
  int pairs = 0;
  rc = dense_gemm((const bf16_t *)a, (const bf16_t *)w_packed, nullptr, nullptr, EPI_ARGMAX, B, V, K,
                  (hipStream_t)stream, val, idx, &pairs);
  if (rc != GPTOSS_OK) return rc;
  return run_argmax_tiles(val, idx, next_ids, B, pairs, (hipStream_t)stream);
}

extern "C" int gptoss_argmax(const float *logits, int *ids, int B, int V, void *stream) {
  GPTOSS_REQUIRE(logits && ids, GPTOSS_ERR_NULL, "argmax: null pointer");
  GPTOSS_REQUIRE(B >= 0 && V > 0, GPTOSS_ERR_DIM, "argmax: bad dimensions (B=%d V=%d)", B, V);
  GPTOSS_REQUIRE(aligned(logits, 16) && V % 4 == 0, GPTOSS_ERR_ALIGN, "argmax: logits must be 16-byte aligned, V %% 4 == 0");
  if (B == 0) return GPTOSS_OK;
  return run_argmax(logits, ids, B, V, (hipStream_t)stream);
}

extern "C" int gptoss_rope_kv_store(const float *qkv, float *q_out, void *kv_cache, const float *cos_t,
                                    const float *sin_t, const int *lens, int B, int n_q, int n_kv, int head_dim,
                                    int capacity, void *stream) {
  GPTOSS_REQUIRE(qkv && q_out && kv_cache && cos_t && sin_t && lens, GPTOSS_ERR_NULL, "rope_kv_store: null pointer");
  GPTOSS_REQUIRE(B >= 0 && n_q > 0 && n_kv > 0 && (head_dim == 32 || head_dim == 64) && capacity > 0 &&
                     capacity % 64 == 0,
                 GPTOSS_ERR_DIM, "rope_kv_store: need head_dim in {32,64} and capacity %% 64 == 0 (D=%d capacity=%d)",
                 head_dim, capacity);
  GPTOSS_REQUIRE(aligned(qkv, 16) && aligned(q_out, 16) && aligned(kv_cache, 16) && aligned(cos_t, 16) &&
                     aligned(sin_t, 16),
                 GPTOSS_ERR_ALIGN, "rope_kv_store: pointers must be 16-byte aligned");
  if (B == 0) return GPTOSS_OK;
  return run_rope_store_lens(qkv, q_out, (bf16_t *)kv_cache, cos_t, sin_t, B, n_q, n_kv, head_dim, capacity, lens,
                             (hipStream_t)stream);
}
