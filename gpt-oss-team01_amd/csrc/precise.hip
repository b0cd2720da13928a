// fp32-faithful decode kernels (GPTOSS_ENGINE_PRECISE): the arithmetic of the reference CPU model
// (run.cpp:304-337 rmsnorm/softmax, :339-352 matmul, :501-717 forward) on the GPU — fp32 weights
// and activations, every dot product a sum of fp32 products accumulated in double, the fp32 KV
// cache, products and sums rounded separately (no fused multiply-add).  Only the order of the
// double-precision additions inside one dot product differs from the CPU loop (a 64-lane tree
// instead of a sequential sum, differences of ~1e-16 relative before the rounding to float) and
// expf is the device library's.  This mode exists to reproduce the reference's greedy token ids
// exactly; it makes no attempt at speed.
#include "common.hpp"
#include "precise.hpp"

namespace gptoss {

__device__ __forceinline__ double wave_sum(double v) {
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

// out[r, i] = float(sum_j double(w[m(r)][i, j] * x[xr(r), j])) + bias[m(r)][i]      (run.cpp:339-352)
// One wave per output element.  m(r) = mat_ids ? mat_ids[r] : 0, xr(r) = r / x_row_div.
__global__ __launch_bounds__(256) void precise_matmul_kernel(float *__restrict__ out,
                                                             const float *__restrict__ x,
                                                             const float *__restrict__ w,
                                                             const float *__restrict__ bias,
                                                             const int *__restrict__ mat_ids,
                                                             int n_in, int n_out, int x_row_div) {
  const int r = blockIdx.y;
  const int i = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (i >= n_out) return;
  const int m = mat_ids ? mat_ids[r] : 0;
  const float *wr = w + ((size_t)m * n_out + i) * n_in;
  const float *xr = x + (size_t)(r / x_row_div) * n_in;
  double val = 0.0;
  for (int j = lane; j < n_in; j += 64) val += (double)__fmul_rn(wr[j], xr[j]);
  val = wave_sum(val);
  if (lane == 0) {
    float o = (float)val;
    if (bias) o = __fadd_rn(o, bias[(size_t)m * n_out + i]);
    out[(size_t)r * n_out + i] = o;
  }
}

__global__ __launch_bounds__(256) void precise_embedding_kernel(const float *__restrict__ table,
                                                                const int *__restrict__ tokens,
                                                                float *__restrict__ x, int H, int V) {
  const int b = blockIdx.x;
  int tok = tokens[b];
  tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);
  for (int h = threadIdx.x; h < H; h += 256) x[(size_t)b * H + h] = table[(size_t)tok * H + h];
}

// q (rotated) -> q_out; k (rotated), v -> fp32 cache [B, S, kv_dim] at position pos (run.cpp:480-499)
__global__ __launch_bounds__(256) void precise_rope_store_kernel(const float *__restrict__ qkv,
                                                                 float *__restrict__ q_out,
                                                                 float *__restrict__ kc,
                                                                 float *__restrict__ vc,
                                                                 const float *__restrict__ cos_t,
                                                                 const float *__restrict__ sin_t, int n_q,
                                                                 int n_kv, int D, int S, int pos) {
  const int b = blockIdx.x;
  const int half = D >> 1;
  const int q_dim = n_q * D, kv_dim = n_kv * D;
  const float *row = qkv + (size_t)b * (q_dim + 2 * kv_dim);
  const float *cs = cos_t + (size_t)pos * half, *sn = sin_t + (size_t)pos * half;
  float *kdst = kc + ((size_t)b * S + pos) * kv_dim, *vdst = vc + ((size_t)b * S + pos) * kv_dim;
  for (int p = threadIdx.x; p < (n_q + n_kv) * half; p += 256) {
    const int h = p / half, j = p - h * half;
    const float x1 = row[h * D + j], x2 = row[h * D + half + j];
    const float c = cs[j], s = sn[j];
    const float o1 = __fsub_rn(__fmul_rn(x1, c), __fmul_rn(x2, s));
    const float o2 = __fadd_rn(__fmul_rn(x2, c), __fmul_rn(x1, s));
    if (h < n_q) {
      q_out[(size_t)b * q_dim + h * D + j] = o1;
      q_out[(size_t)b * q_dim + h * D + half + j] = o2;
    } else {
      kdst[(h - n_q) * D + j] = o1;
      kdst[(h - n_q) * D + half + j] = o2;
    }
  }
  for (int p = threadIdx.x; p < kv_dim; p += 256) vdst[p] = row[q_dim + kv_dim + p];
}

// One workgroup per (sequence, q head): scores over positions 0..pos with the sliding-window mask,
// the sink as one more logit, softmax with a double maximum and sum, weighted sum of V accumulated
// in float in position order (run.cpp:562-607).  att: scratch [B, n_q, S + 2].
__global__ __launch_bounds__(256) void precise_attn_kernel(const float *__restrict__ q,
                                                           const float *__restrict__ kc,
                                                           const float *__restrict__ vc,
                                                           const float *__restrict__ sinks,
                                                           float *__restrict__ att_all,
                                                           float *__restrict__ out, int n_q, int n_kv,
                                                           int D, int S, int pos, int window) {
  __shared__ double red[4];
  __shared__ double sh_max, sh_sum;
  const int h = blockIdx.x, b = blockIdx.y;
  const int kv_dim = n_kv * D, g = h / (n_q / n_kv);
  const float *qh = q + ((size_t)b * n_q + h) * D;
  float *att = att_all + ((size_t)b * n_q + h) * (S + 2);
  const int n = pos + 2;
  const float inv_div = sqrtf((float)D);
  for (int t = threadIdx.x; t <= pos; t += 256) {
    const float *k = kc + ((size_t)b * S + t) * kv_dim + g * D;
    double score = 0.0;
    for (int i = 0; i < D; i++) score += (double)__fmul_rn(qh[i], k[i]);
    score /= (double)inv_div;
    if (window > 0 && pos - t >= window) score += (double)(-INFINITY);
    att[t] = (float)score;
  }
  if (threadIdx.x == 0) att[pos + 1] = sinks[h];
  __syncthreads();
  // maximum (exact in any order)
  double mx = -INFINITY;
  for (int t = threadIdx.x; t < n; t += 256) mx = fmax(mx, (double)att[t]);
  for (int m = 32; m >= 1; m >>= 1) mx = fmax(mx, __shfl_xor(mx, m, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0) sh_max = fmax(fmax(red[0], red[1]), fmax(red[2], red[3]));
  __syncthreads();
  const double max_val = sh_max;
  double sum = 0.0;
  for (int t = threadIdx.x; t < n; t += 256) {
    const float e = expf((float)((double)att[t] - max_val));
    att[t] = e;
    sum += (double)e;
  }
  sum = wave_sum(sum);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
  __syncthreads();
  if (threadIdx.x == 0) sh_sum = (red[0] + red[1]) + (red[2] + red[3]);
  __syncthreads();
  const double total = sh_sum;
  for (int t = threadIdx.x; t < n; t += 256) att[t] = (float)((double)att[t] / total);
  __syncthreads();
  for (int i = threadIdx.x; i < D; i += 256) {
    float acc = 0.f;
    for (int t = 0; t <= pos; t++) {
      const float v = vc[((size_t)b * S + t) * kv_dim + g * D + i];
      acc = __fadd_rn(acc, __fmul_rn(att[t], v));
    }
    out[((size_t)b * n_q + h) * D + i] = acc;
  }
}

// clamped SwiGLU of interleaved (gate, up) rows (run.cpp:664-686)
__global__ __launch_bounds__(256) void precise_swiglu_kernel(const float *__restrict__ mlp1,
                                                             float *__restrict__ act, int I, float limit,
                                                             size_t total) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const size_t r = idx / I;
  const int j = (int)(idx - r * I);
  float val = mlp1[r * 2 * I + 2 * j], up = mlp1[r * 2 * I + 2 * j + 1];
  if (val > limit) val = limit;
  if (up > limit) up = limit;
  if (up < -limit) up = -limit;
  val = __fmul_rn(val, 1.0f / __fadd_rn(1.0f, expf(__fmul_rn(-1.702f, val))));
  val = __fmul_rn(val, __fadd_rn(up, 1.0f));
  act[idx] = val;
}

// x[b,:] += sum over the token's experts, in ascending expert order, of mlp2 row * weight
// (the order of the expert loop, run.cpp:642-709)
__global__ __launch_bounds__(256) void precise_moe_agg_kernel(const float *__restrict__ mlp2,
                                                              const float *__restrict__ topk_w,
                                                              const int *__restrict__ topk_i,
                                                              float *__restrict__ x, int H, int k) {
  const int b = blockIdx.x;
  int order[8];
  for (int s = 0; s < k; s++) order[s] = s;
  for (int a = 0; a < k; a++)
    for (int c = a + 1; c < k; c++)
      if (topk_i[b * k + order[c]] < topk_i[b * k + order[a]]) {
        int t = order[a];
        order[a] = order[c];
        order[c] = t;
      }
  for (int h = threadIdx.x; h < H; h += 256) {
    float agg = 0.f;
    for (int s = 0; s < k; s++) {
      const int slot = order[s];
      agg = __fadd_rn(agg, __fmul_rn(mlp2[((size_t)b * k + slot) * H + h], topk_w[b * k + slot]));
    }
    x[(size_t)b * H + h] = __fadd_rn(x[(size_t)b * H + h], agg);
  }
}

__global__ __launch_bounds__(256) void precise_add_kernel(float *__restrict__ x,
                                                          const float *__restrict__ y, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[i] = __fadd_rn(x[i], y[i]);
}

int precise_matmul(float *out, const float *x, const float *w, const float *bias, const int *mat_ids,
                   int rows, int n_in, int n_out, int x_row_div, hipStream_t s) {
  if (rows == 0) return GPTOSS_OK;
  dim3 grid(cdiv(n_out, 4), rows);
  precise_matmul_kernel<<<grid, 256, 0, s>>>(out, x, w, bias, mat_ids, n_in, n_out, x_row_div);
  GPTOSS_LAUNCH_CHECK("precise_matmul_kernel");
  return GPTOSS_OK;
}

int precise_embedding(const float *table, const int *tokens, float *x, int B, int H, int V, hipStream_t s) {
  precise_embedding_kernel<<<B, 256, 0, s>>>(table, tokens, x, H, V);
  GPTOSS_LAUNCH_CHECK("precise_embedding_kernel");
  return GPTOSS_OK;
}

int precise_rope_store(const float *qkv, float *q_out, float *kc, float *vc, const float *cos_t,
                       const float *sin_t, int B, int n_q, int n_kv, int D, int S, int pos, hipStream_t s) {
  precise_rope_store_kernel<<<B, 256, 0, s>>>(qkv, q_out, kc, vc, cos_t, sin_t, n_q, n_kv, D, S, pos);
  GPTOSS_LAUNCH_CHECK("precise_rope_store_kernel");
  return GPTOSS_OK;
}

int precise_attn(const float *q, const float *kc, const float *vc, const float *sinks, float *att,
                 float *out, int B, int n_q, int n_kv, int D, int S, int pos, int window, hipStream_t s) {
  dim3 grid(n_q, B);
  precise_attn_kernel<<<grid, 256, 0, s>>>(q, kc, vc, sinks, att, out, n_q, n_kv, D, S, pos, window);
  GPTOSS_LAUNCH_CHECK("precise_attn_kernel");
  return GPTOSS_OK;
}

int precise_swiglu(const float *mlp1, float *act, int rows, int I, float limit, hipStream_t s) {
  const size_t total = (size_t)rows * I;
  if (total == 0) return GPTOSS_OK;
  precise_swiglu_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(mlp1, act, I, limit, total);
  GPTOSS_LAUNCH_CHECK("precise_swiglu_kernel");
  return GPTOSS_OK;
}

int precise_moe_agg(const float *mlp2, const float *topk_w, const int *topk_i, float *x, int B, int H,
                    int k, hipStream_t s) {
  precise_moe_agg_kernel<<<B, 256, 0, s>>>(mlp2, topk_w, topk_i, x, H, k);
  GPTOSS_LAUNCH_CHECK("precise_moe_agg_kernel");
  return GPTOSS_OK;
}

int precise_add(float *x, const float *y, size_t n, hipStream_t s) {
  if (n == 0) return GPTOSS_OK;
  precise_add_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(x, y, n);
  GPTOSS_LAUNCH_CHECK("precise_add_kernel");
  return GPTOSS_OK;
}

}  // namespace gptoss
