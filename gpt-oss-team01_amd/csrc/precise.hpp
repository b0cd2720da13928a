// Internal interface of the fp32-faithful kernels (precise.hip).
#pragma once
#include "common.hpp"

namespace gptoss {

// out[r,:] = W[m(r)] . x[r / x_row_div,:] + bias[m(r)]; W is [n_mat][n_out, n_in] row-major fp32
int precise_matmul(float *out, const float *x, const float *w, const float *bias, const int *mat_ids,
                   int rows, int n_in, int n_out, int x_row_div, hipStream_t s);
int precise_embedding(const float *table, const int *tokens, float *x, int B, int H, int V, hipStream_t s);
int precise_rope_store(const float *qkv, float *q_out, float *kc, float *vc, const float *cos_t,
                       const float *sin_t, int B, int n_q, int n_kv, int D, int S, int pos, hipStream_t s);
int precise_attn(const float *q, const float *kc, const float *vc, const float *sinks, float *att,
                 float *out, int B, int n_q, int n_kv, int D, int S, int pos, int window, hipStream_t s);
int precise_swiglu(const float *mlp1, float *act, int rows, int I, float limit, hipStream_t s);
int precise_moe_agg(const float *mlp2, const float *topk_w, const int *topk_i, float *x, int B, int H,
                    int k, hipStream_t s);
int precise_add(float *x, const float *y, size_t n, hipStream_t s);

}  // namespace gptoss
