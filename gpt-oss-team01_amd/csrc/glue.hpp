// Internal interface of the glue kernels (glue.hip).
#pragma once
#include "common.hpp"

namespace gptoss {

int run_embedding(const bf16_t *table, const int *tokens, float *x, int B, int H, int V, hipStream_t s);
// x (+= residual) -> t_bf16 (and t_f32 when not null); residual may be null
int run_rmsnorm(float *x, const float *residual, const float *weight, bf16_t *t_bf16, float *t_f32,
                int B, int H, hipStream_t s);
int run_rope_store(const float *qkv, float *q_out, bf16_t *kv, const float *cos_t,
                   const float *sin_t, int B, int n_q, int n_kv, int D, int cap, int pos,
                   hipStream_t s);
// rows = sequences * T: row r is position pos0 + r % T of sequence r / T; K/V of positions below
// store_from are not stored; q_out may be null
int run_rope_store_rows(const float *qkv, float *q_out, bf16_t *kv, const float *cos_t,
                        const float *sin_t, int rows, int T, int n_q, int n_kv, int D, int cap, int pos0,
                        int store_from, hipStream_t s);
// row r at position lens[r] - 1 of sequence r (or seq_map[r]: several rows may then belong to one
// sequence, at different positions)
int run_rope_store_lens(const float *qkv, float *q_out, bf16_t *kv, const float *cos_t,
                        const float *sin_t, int B, int n_q, int n_kv, int D, int cap, const int *lens,
                        hipStream_t s, const int *seq_map = nullptr);
// attn_decode.hip: gptoss_attn_decode with row b reading the cache of sequence seq_map[b] (device
// array) up to lens[b]
int attn_decode_mapped(const float *q, const void *kv_cache, const int *lens, const float *sinks, void *out, int B,
                       int n_q, int n_kv, int head_dim, int capacity, int window, int max_len, void *workspace,
                       size_t workspace_bytes, void *stream, const int *seq_map);
// dst[i, :] = src[idx[i], :]
int run_gather_rows_idx(const float *src, float *dst, const int *idx, int rows, int n, hipStream_t s);
// dst[i, :] = src[i * stride + offset, :]
int run_gather_rows(const float *src, float *dst, int rows, int n, int stride, int offset, hipStream_t s);
int run_argmax(const float *logits, int *ids, int B, int V, hipStream_t s);
int run_argmax_tiles(const float *val, const int *idx, int *ids, int B, int n_tiles, hipStream_t s);
int run_f32_to_bf16(const float *src, bf16_t *dst, size_t n, hipStream_t s);
// fp32 [n_blocks * 32] -> e2m1 codes [n_blocks, 16] + e8m0 scales [n_blocks]; *not_exact is set when a
// value has no exact MXFP4 representation
int run_requant_mxfp4(const float *src, size_t n_blocks, unsigned char *blocks, unsigned char *scales,
                      int *not_exact, hipStream_t s);
int run_synth_mxfp4(unsigned char *blocks, unsigned char *scales, size_t n_blocks, uint64_t seed, int e_hi,
                    hipStream_t s);
int run_synth_bf16(bf16_t *dst, size_t n, uint64_t seed, float mean, float std, hipStream_t s);
int run_synth_f32(float *dst, size_t n, uint64_t seed, float mean, float std, hipStream_t s);

}  // namespace gptoss
