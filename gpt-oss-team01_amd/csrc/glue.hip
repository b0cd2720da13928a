// Small memory-bound kernels around the two hot ops of a decode step: embedding gather, RMSNorm
// (optionally fused with the residual add), q/k/v split + rotary embedding + KV-cache store, row
// arg-max, dtype conversion and on-device synthetic weight generation.
#include "common.hpp"
#include "glue.hpp"

namespace gptoss {

// x[b,:] = embedding[token[b],:]   (bf16 table -> fp32 residual stream)
// reference: embedding_lookup_kernel, layer_hip_batch.cpp:199-214
__global__ __launch_bounds__(256) void embedding_kernel(const bf16_t *__restrict__ table,
                                                        const int *__restrict__ tokens,
                                                        float *__restrict__ x, int H, int V) {
  const int b = blockIdx.x;
  int tok = tokens[b];
  tok = min(max(tok, 0), V - 1);
  const bf16_t *row = table + (size_t)tok * H;
  float *xr = x + (size_t)b * H;
  if (H % 8 == 0 && reinterpret_cast<uintptr_t>(table) % 16 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
    // eight values per lane and step: one 16-byte load, two 16-byte stores
    for (int h = threadIdx.x * 8; h < H; h += 256 * 8) {
      const u32x4 v = *reinterpret_cast<const u32x4 *>(row + h);
      *reinterpret_cast<f32x4 *>(xr + h) = f32x4{__uint_as_float(v[0] << 16), __uint_as_float(v[0] & 0xffff0000u),
                                                 __uint_as_float(v[1] << 16), __uint_as_float(v[1] & 0xffff0000u)};
      *reinterpret_cast<f32x4 *>(xr + h + 4) = f32x4{__uint_as_float(v[2] << 16), __uint_as_float(v[2] & 0xffff0000u),
                                                     __uint_as_float(v[3] << 16), __uint_as_float(v[3] & 0xffff0000u)};
    }
    return;
  }
  for (int h = threadIdx.x; h < H; h += 256) xr[h] = bf16_to_f32(row[h]);
}

// RMSNorm with the arithmetic of run.cpp:304-317: sum of squares accumulated in double from
// float products, eps added after the mean, 1/sqrtf in float, scale applied in double and
// rounded once.  If residual != nullptr, x += residual first (in place), as
// residual_rmsnorm_bf16_kernel does (layer_hip_batch.cpp:94-155).
// Outputs: t_bf16 (always) and t_f32 (optional full-precision copy).
__global__ __launch_bounds__(256) void rmsnorm_kernel(float *__restrict__ x,
                                                      const float *__restrict__ residual,
                                                      const float *__restrict__ weight,
                                                      bf16_t *__restrict__ t_bf16,
                                                      float *__restrict__ t_f32, int H) {
  __shared__ double red[4];
  const int b = blockIdx.x;
  float *xr = x + (size_t)b * H;
  double ss = 0.0;
  for (int h = threadIdx.x; h < H; h += 256) {
    float v = xr[h];
    if (residual) {
      v = __fadd_rn(v, residual[(size_t)b * H + h]);
      xr[h] = v;
    }
    ss += (double)__fmul_rn(v, v);
  }
  for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  ss = red[0] + red[1] + red[2] + red[3];
  ss /= H;
  ss += 1e-5f;
  const double inv = (double)(1.0f / sqrtf((float)ss));
  for (int h = threadIdx.x; h < H; h += 256) {
    float o = (float)((double)weight[h] * (inv * (double)xr[h]));
    t_bf16[(size_t)b * H + h] = f32_to_bf16(o);
    if (t_f32) t_f32[(size_t)b * H + h] = o;
  }
}

// The same for rows of at most 256 * 4 * VPT floats: every thread keeps its 4 * VPT elements in
// registers between the two passes and moves them 16 bytes at a time.
template <int VPT>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(float *__restrict__ x,
                                                           const float *__restrict__ residual,
                                                           const float *__restrict__ weight,
                                                           bf16_t *__restrict__ t_bf16,
                                                           float *__restrict__ t_f32, int H) {
  __shared__ double red[4];
  const size_t row = (size_t)blockIdx.x * H;
  f32x4 v[VPT];
  double ss = 0.0;
#pragma unroll
  for (int i = 0; i < VPT; i++) {
    const int h = (threadIdx.x + 256 * i) * 4;
    v[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (h < H) {
      v[i] = *reinterpret_cast<const f32x4 *>(x + row + h);
      if (residual) {
        const f32x4 r = *reinterpret_cast<const f32x4 *>(residual + row + h);
#pragma unroll
        for (int q = 0; q < 4; q++) v[i][q] = __fadd_rn(v[i][q], r[q]);
        *reinterpret_cast<f32x4 *>(x + row + h) = v[i];
      }
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
      const f32x4 w = *reinterpret_cast<const f32x4 *>(weight + h);
      f32x4 o;
#pragma unroll
      for (int q = 0; q < 4; q++) o[q] = (float)((double)w[q] * (inv * (double)v[i][q]));
      *reinterpret_cast<u32x2 *>(t_bf16 + row + h) = u32x2{pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
      if (t_f32) *reinterpret_cast<f32x4 *>(t_f32 + row + h) = o;
    }
  }
}

// Split the fused qkv row, rotate q and k (half-split pairs i, i+D/2; run.cpp:480-499), write q
// (fp32) and store k, v as bf16 into this layer's cache slot pos % cap.
// reference: qkv_split_rope_store_kernel, layer_hip_batch.cpp:686-776
// Q_ONCE: q is stored with the non-temporal hint (a compile-time choice: the compiler merges a plain
// and a hinted store of the same value under a run-time condition into one plain store).
template <bool Q_ONCE>
__global__ __launch_bounds__(256) void rope_store_kernel(const float *__restrict__ qkv,
                                                         float *__restrict__ q_out,
                                                         bf16_t *__restrict__ kv,
                                                         const float *__restrict__ cos_t,
                                                         const float *__restrict__ sin_t, int n_q,
                                                         int n_kv, int D, int cap, int pos0, int T,
                                                         int store_from, const int *__restrict__ lens,
                                                         const int *__restrict__ seq_map) {
  // row r of the batch is position pos0 + r % T of sequence r / T (T = 1: one lock-step position),
  // or, with lens, the last position (lens[r] - 1) of sequence r
  // seq_map (optional): the cache of the r / T-th sequence of the batch is that of sequence seq_map[r / T]
  const int r = blockIdx.x;
  const int bi = r / T;
  const int b = seq_map ? seq_map[bi] : bi;
  const int pos = lens ? lens[r] - 1 : pos0 + (r - bi * T);
  if (pos < 0) {  // an empty sequence (lens[r] == 0): nothing to rotate or store, its q row is zero
    if (q_out != nullptr)
      for (int p = threadIdx.x; p < n_q * D; p += 256) q_out[(size_t)r * n_q * D + p] = 0.f;
    return;
  }
  const int half = D >> 1;
  const int q_dim = n_q * D, kv_dim = n_kv * D;
  const float *row = qkv + (size_t)r * (q_dim + 2 * kv_dim);
  const float *cs = cos_t + (size_t)pos * half, *sn = sin_t + (size_t)pos * half;
  const int slot = pos % cap;
  // four rotation pairs per thread and step: 16-byte loads and stores (half % 4 == 0 for D in {32, 64})
  const int quads = half >> 2;
  auto rotate = [&](const float *x, int j4, f32x4 &lo, f32x4 &hi) {
    const f32x4 x1 = *reinterpret_cast<const f32x4 *>(x + j4), x2 = *reinterpret_cast<const f32x4 *>(x + half + j4);
    const f32x4 c = *reinterpret_cast<const f32x4 *>(cs + j4), s = *reinterpret_cast<const f32x4 *>(sn + j4);
#pragma unroll
    for (int q = 0; q < 4; q++) {
      lo[q] = __fsub_rn(__fmul_rn(x1[q], c[q]), __fmul_rn(x2[q], s[q]));
      hi[q] = __fadd_rn(__fmul_rn(x2[q], c[q]), __fmul_rn(x1[q], s[q]));
    }
  };
  if (q_out != nullptr) {
    for (int p = threadIdx.x; p < n_q * quads; p += 256) {
      const int h = p / quads, j4 = (p - h * quads) * 4;
      f32x4 lo, hi;
      rotate(row + h * D, j4, lo, hi);
      // One position per sequence: q is read once, by the attention call that follows.  Stored with
      // the non-temporal hint it does not wait in L2 as dirty lines that are then written back in the
      // middle of that call's K/V stream (full-context attention of a 1024-sequence step at 190
      // positions 92.7 -> 89.0 us).  The rows of a prompt pass keep the plain store: their attention
      // reads q through L2 (3.00 against 3.08 ms per pass of 8192 rows).
      f32x4 *q_lo = reinterpret_cast<f32x4 *>(q_out + (size_t)r * q_dim + h * D + j4);
      f32x4 *q_hi = reinterpret_cast<f32x4 *>(q_out + (size_t)r * q_dim + h * D + half + j4);
      if (Q_ONCE) {
        __builtin_nontemporal_store(lo, q_lo);
        __builtin_nontemporal_store(hi, q_hi);
      } else {
        *q_lo = lo;
        *q_hi = hi;
      }
    }
  }
  if (pos < store_from) return;  // a ring cache keeps only the last positions of a prefill
  for (int p = threadIdx.x; p < n_kv * quads; p += 256) {
    const int g = p / quads, j4 = (p - g * quads) * 4;
    f32x4 lo, hi;
    rotate(row + q_dim + g * D, j4, lo, hi);
    bf16_t *krow = kv + kv_block_off(b, g, n_kv, cap, D, slot) + kv_k_elem(slot, 0, D);
    *reinterpret_cast<u32x2 *>(krow + j4) = u32x2{pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3])};
    *reinterpret_cast<u32x2 *>(krow + half + j4) = u32x2{pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3])};
  }
  for (int p = threadIdx.x; p < kv_dim; p += 256) {
    int g = p / D, d = p - g * D;
    kv[kv_block_off(b, g, n_kv, cap, D, slot) + kv_v_elem(slot, d, D)] = f32_to_bf16(row[q_dim + kv_dim + p]);
  }
}

// ids[b] = arg max over logits[b,:], lowest index among equal maxima (run.cpp:739-750).
// reference: max_kernel_gpu_v2, layer_hip_batch.cpp:1542-1597
__global__ __launch_bounds__(1024) void argmax_kernel(const float *__restrict__ logits,
                                                      int *__restrict__ ids, int V) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const int b = blockIdx.x;
  const float *row = logits + (size_t)b * V;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x * 4; i < V; i += 1024 * 4) {
    if (i + 3 < V) {
      f32x4 v = *reinterpret_cast<const f32x4 *>(row + i);
#pragma unroll
      for (int q = 0; q < 4; q++)
        if (v[q] > bv || bi == 0x7fffffff) { bv = v[q]; bi = i + q; }
    } else {
      for (int q = 0; q < 4 && i + q < V; q++)
        if (row[i + q] > bv || bi == 0x7fffffff) { bv = row[i + q]; bi = i + q; }
    }
  }
  for (int m = 32; m >= 1; m >>= 1) {
    float ov = __shfl_xor(bv, m, 64);
    int oi = __shfl_xor(bi, m, 64);
    if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
  }
  if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = bv; si[threadIdx.x >> 6] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 16; w++)
      if (si[w] != 0x7fffffff && (bi == 0x7fffffff || sv[w] > bv || (sv[w] == bv && si[w] < bi))) {
        bv = sv[w];
        bi = si[w];
      }
    ids[b] = (bi == 0x7fffffff) ? 0 : bi;
  }
}

__global__ __launch_bounds__(256) void f32_to_bf16_kernel(const float *__restrict__ src,
                                                          bf16_t *__restrict__ dst, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    dst[i] = f32_to_bf16(src[i]);
}

// N(mean, std) from a counter-based generator (splitmix64 of seed+index, Box-Muller), rounded to
// bf16 or kept fp32.  Used to build random-init models of sizes whose fp32 file would not fit.
__device__ __forceinline__ uint64_t splitmix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ float normal_at(uint64_t seed, uint64_t i) {
  uint64_t r = splitmix64(seed * 0xD1342543DE82EF95ull + i);
  float u1 = ((uint32_t)(r >> 40) + 1.0f) * (1.0f / 16777217.0f);  // (0,1]
  float u2 = (uint32_t)(r & 0xffffffu) * (1.0f / 16777216.0f);
  return sqrtf(-2.0f * __logf(u1)) * __cosf(6.2831853071795865f * u2);
}

__global__ __launch_bounds__(256) void synth_normal_bf16_kernel(bf16_t *__restrict__ dst, size_t n,
                                                                uint64_t seed, float mean, float std) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    dst[i] = f32_to_bf16(mean + std * normal_at(seed, i));
}

__global__ __launch_bounds__(256) void synth_normal_f32_kernel(float *__restrict__ dst, size_t n,
                                                               uint64_t seed, float mean, float std) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    dst[i] = bf16_to_f32(f32_to_bf16(mean + std * normal_at(seed, i)));
}

// fp32 -> MXFP4, exact or not at all.  One thread per block of 32 consecutive inputs of a row:
// the scale is the smallest power of two that brings the block's largest magnitude to at most 6
// (any block that has an exact e2m1 representation under some scale also has one under this,
// the finest, scale); every value must then equal sign * {0,.5,1,1.5,2,3,4,6} * scale, otherwise
// *not_exact is set.  blocks [n_blocks, 16]: byte j = elements 2j (low nibble), 2j+1 (high nibble);
// scales [n_blocks] e8m0 (the checkpoint layout, export_model_bin/gpt-oss-20b/export_model_bin.py:66-123).
__global__ __launch_bounds__(256) void requant_mxfp4_kernel(const float *__restrict__ src, size_t n_blocks,
                                                            unsigned char *__restrict__ blocks,
                                                            unsigned char *__restrict__ scales,
                                                            int *__restrict__ not_exact) {
  for (size_t b = (size_t)blockIdx.x * 256 + threadIdx.x; b < n_blocks; b += (size_t)gridDim.x * 256) {
    const f32x4 *sp = reinterpret_cast<const f32x4 *>(src + b * 32);
    float v[32];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const f32x4 q = sp[i];
      v[4 * i] = q[0], v[4 * i + 1] = q[1], v[4 * i + 2] = q[2], v[4 * i + 3] = q[3];
    }
    float mx = 0.f;
#pragma unroll
    for (int i = 0; i < 32; i++) mx = fmaxf(mx, fabsf(v[i]));
    int e = 0;  // scale = 2^e
    if (mx > 0.f) {
      int ex;
      const float m = frexpf(mx, &ex);  // mx = m * 2^ex, m in [0.5, 1)
      // mx / 2^e <= 6 = 0.75 * 2^3  <=>  e >= ex - 3 when m <= 0.75, else e >= ex - 2
      e = (m <= 0.75f) ? ex - 3 : ex - 2;
    }
    bool bad = !(mx < INFINITY) || e < -120 || e > 120;
    const float inv = ldexpf(1.0f, -e);
    uint32_t packed[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 32; i++) {
      const float a = fabsf(v[i]) * inv;  // exact: a power-of-two factor
      // codes 0..7 = 0, .5, 1, 1.5, 2, 3, 4, 6
      int code = (a <= 2.0f) ? (int)(a * 2.0f) : (a <= 4.0f ? (int)a + 2 : 7);
      const float back = (code <= 4) ? 0.5f * code : (code == 5 ? 3.0f : (code == 6 ? 4.0f : 6.0f));
      bad = bad || back != a;
      code |= (__float_as_uint(v[i]) >> 31) << 3;
      packed[i >> 3] |= (uint32_t)code << (4 * (i & 7));
    }
    *reinterpret_cast<u32x4 *>(blocks + b * 16) = u32x4{packed[0], packed[1], packed[2], packed[3]};
    scales[b] = (unsigned char)(e + 127);
    if (bad) *not_exact = 1;
  }
}

// random MXFP4 weights: codes uniform over the 16 values, scale exponents uniform in [e_hi - 8, e_hi]
__global__ __launch_bounds__(256) void synth_mxfp4_kernel(unsigned char *__restrict__ blocks,
                                                          unsigned char *__restrict__ scales,
                                                          size_t n_blocks, uint64_t seed, int e_hi) {
  for (size_t b = (size_t)blockIdx.x * 256 + threadIdx.x; b < n_blocks; b += (size_t)gridDim.x * 256) {
    const uint64_t r0 = splitmix64(seed * 0xD1342543DE82EF95ull + 3 * b);
    const uint64_t r1 = splitmix64(seed * 0xD1342543DE82EF95ull + 3 * b + 1);
    const uint64_t r2 = splitmix64(seed * 0xD1342543DE82EF95ull + 3 * b + 2);
    *reinterpret_cast<u32x4 *>(blocks + b * 16) =
        u32x4{(uint32_t)r0, (uint32_t)(r0 >> 32), (uint32_t)r1, (uint32_t)(r1 >> 32)};
    scales[b] = (unsigned char)(127 + e_hi - (int)(r2 % 9));
  }
}

static inline int grid_for(size_t n) {
  size_t g = (n + 255) / 256;
  return (int)(g > 65536 ? 65536 : (g == 0 ? 1 : g));
}

int run_embedding(const bf16_t *table, const int *tokens, float *x, int B, int H, int V, hipStream_t s) {
  TraceScope ts("embedding", s);
  embedding_kernel<<<B, 256, 0, s>>>(table, tokens, x, H, V);
  GPTOSS_LAUNCH_CHECK("embedding_kernel");
  return GPTOSS_OK;
}

int run_rmsnorm(float *x, const float *residual, const float *weight, bf16_t *t_bf16, float *t_f32,
                int B, int H, hipStream_t s) {
  TraceScope ts(residual ? "residual_rmsnorm" : "rmsnorm", s);
  const bool vec = H % 4 == 0 && aligned(x, 16) && aligned(weight, 16) && aligned(t_bf16, 8) &&
                   (!residual || aligned(residual, 16)) && (!t_f32 || aligned(t_f32, 16));
  if (vec && H <= 1024) rmsnorm_rows_kernel<1><<<B, 256, 0, s>>>(x, residual, weight, t_bf16, t_f32, H);
  else if (vec && H <= 2048) rmsnorm_rows_kernel<2><<<B, 256, 0, s>>>(x, residual, weight, t_bf16, t_f32, H);
  else if (vec && H <= 3072) rmsnorm_rows_kernel<3><<<B, 256, 0, s>>>(x, residual, weight, t_bf16, t_f32, H);
  else if (vec && H <= 4096) rmsnorm_rows_kernel<4><<<B, 256, 0, s>>>(x, residual, weight, t_bf16, t_f32, H);
  else rmsnorm_kernel<<<B, 256, 0, s>>>(x, residual, weight, t_bf16, t_f32, H);
  GPTOSS_LAUNCH_CHECK("rmsnorm_kernel");
  return GPTOSS_OK;
}

// dst[i, :] = src[(i * stride + offset), :], n floats per row (n % 4 == 0)
__global__ __launch_bounds__(256) void gather_rows_kernel(const float *__restrict__ src,
                                                          float *__restrict__ dst, int n, int stride,
                                                          int offset) {
  const float *sp = src + ((size_t)blockIdx.x * stride + offset) * n;
  float *dp = dst + (size_t)blockIdx.x * n;
  for (int i = threadIdx.x * 4; i < n; i += 256 * 4)
    *reinterpret_cast<f32x4 *>(dp + i) = *reinterpret_cast<const f32x4 *>(sp + i);
}

// dst[i, :] = src[idx[i], :], n floats per row (n % 4 == 0)
__global__ __launch_bounds__(256) void gather_rows_idx_kernel(const float *__restrict__ src,
                                                              float *__restrict__ dst,
                                                              const int *__restrict__ idx, int n) {
  const float *sp = src + (size_t)idx[blockIdx.x] * n;
  float *dp = dst + (size_t)blockIdx.x * n;
  for (int i = threadIdx.x * 4; i < n; i += 256 * 4)
    *reinterpret_cast<f32x4 *>(dp + i) = *reinterpret_cast<const f32x4 *>(sp + i);
}

int run_gather_rows_idx(const float *src, float *dst, const int *idx, int rows, int n, hipStream_t s) {
  TraceScope ts("gather_rows", s);
  gather_rows_idx_kernel<<<rows, 256, 0, s>>>(src, dst, idx, n);
  GPTOSS_LAUNCH_CHECK("gather_rows_idx_kernel");
  return GPTOSS_OK;
}

int run_gather_rows(const float *src, float *dst, int rows, int n, int stride, int offset, hipStream_t s) {
  TraceScope ts("gather_rows", s);
  gather_rows_kernel<<<rows, 256, 0, s>>>(src, dst, n, stride, offset);
  GPTOSS_LAUNCH_CHECK("gather_rows_kernel");
  return GPTOSS_OK;
}

int run_rope_store(const float *qkv, float *q_out, bf16_t *kv, const float *cos_t,
                   const float *sin_t, int B, int n_q, int n_kv, int D, int cap, int pos,
                   hipStream_t s) {
  return run_rope_store_rows(qkv, q_out, kv, cos_t, sin_t, B, 1, n_q, n_kv, D, cap, pos, 0, s);
}

int run_rope_store_lens(const float *qkv, float *q_out, bf16_t *kv, const float *cos_t,
                        const float *sin_t, int B, int n_q, int n_kv, int D, int cap, const int *lens,
                        hipStream_t s, const int *seq_map) {
  TraceScope ts("rope_store", s);
  rope_store_kernel<true><<<B, 256, 0, s>>>(qkv, q_out, kv, cos_t, sin_t, n_q, n_kv, D, cap, 0, 1, 0, lens, seq_map);
  GPTOSS_LAUNCH_CHECK("rope_store_kernel");
  return GPTOSS_OK;
}

int run_rope_store_rows(const float *qkv, float *q_out, bf16_t *kv, const float *cos_t,
                        const float *sin_t, int rows, int T, int n_q, int n_kv, int D, int cap, int pos0,
                        int store_from, hipStream_t s) {
  TraceScope ts("rope_store", s);
  if (T == 1)
    rope_store_kernel<true><<<rows, 256, 0, s>>>(qkv, q_out, kv, cos_t, sin_t, n_q, n_kv, D, cap, pos0, T, store_from,
                                                 nullptr, nullptr);
  else
    rope_store_kernel<false><<<rows, 256, 0, s>>>(qkv, q_out, kv, cos_t, sin_t, n_q, n_kv, D, cap, pos0, T, store_from,
                                                  nullptr, nullptr);
  GPTOSS_LAUNCH_CHECK("rope_store_kernel");
  return GPTOSS_OK;
}

// ids[b] = column of the largest per-tile maximum, lowest column among equal ones: the second
// stage of the arg-max that the classifier GEMM's epilogue starts.
__global__ __launch_bounds__(256) void argmax_tiles_kernel(const float *__restrict__ val,
                                                           const int *__restrict__ idx,
                                                           int *__restrict__ ids, int n_tiles) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const int b = blockIdx.x;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int t = threadIdx.x; t < n_tiles; t += 256) {
    const float v = val[(size_t)b * n_tiles + t];
    const int i = idx[(size_t)b * n_tiles + t];
    if (v > bv || (v == bv && i < bi)) {
      bv = v;
      bi = i;
    }
  }
  for (int m = 32; m >= 1; m >>= 1) {
    const float ov = __shfl_xor(bv, m, 64);
    const int oi = __shfl_xor(bi, m, 64);
    if (ov > bv || (ov == bv && oi < bi)) {
      bv = ov;
      bi = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    sv[threadIdx.x >> 6] = bv;
    si[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; w++)
      if (sv[w] > bv || (sv[w] == bv && si[w] < bi)) {
        bv = sv[w];
        bi = si[w];
      }
    ids[b] = bi == 0x7fffffff ? 0 : bi;
  }
}

int run_argmax_tiles(const float *val, const int *idx, int *ids, int B, int n_tiles, hipStream_t s) {
  TraceScope ts("argmax_tiles", s);
  argmax_tiles_kernel<<<B, 256, 0, s>>>(val, idx, ids, n_tiles);
  GPTOSS_LAUNCH_CHECK("argmax_tiles_kernel");
  return GPTOSS_OK;
}

int run_argmax(const float *logits, int *ids, int B, int V, hipStream_t s) {
  TraceScope ts("argmax", s);
  argmax_kernel<<<B, 1024, 0, s>>>(logits, ids, V);
  GPTOSS_LAUNCH_CHECK("argmax_kernel");
  return GPTOSS_OK;
}

int run_f32_to_bf16(const float *src, bf16_t *dst, size_t n, hipStream_t s) {
  f32_to_bf16_kernel<<<grid_for(n), 256, 0, s>>>(src, dst, n);
  GPTOSS_LAUNCH_CHECK("f32_to_bf16_kernel");
  return GPTOSS_OK;
}

int run_requant_mxfp4(const float *src, size_t n_blocks, unsigned char *blocks, unsigned char *scales,
                      int *not_exact, hipStream_t s) {
  requant_mxfp4_kernel<<<grid_for(n_blocks), 256, 0, s>>>(src, n_blocks, blocks, scales, not_exact);
  GPTOSS_LAUNCH_CHECK("requant_mxfp4_kernel");
  return GPTOSS_OK;
}

int run_synth_mxfp4(unsigned char *blocks, unsigned char *scales, size_t n_blocks, uint64_t seed, int e_hi,
                    hipStream_t s) {
  synth_mxfp4_kernel<<<grid_for(n_blocks), 256, 0, s>>>(blocks, scales, n_blocks, seed, e_hi);
  GPTOSS_LAUNCH_CHECK("synth_mxfp4_kernel");
  return GPTOSS_OK;
}

int run_synth_bf16(bf16_t *dst, size_t n, uint64_t seed, float mean, float std, hipStream_t s) {
  synth_normal_bf16_kernel<<<grid_for(n), 256, 0, s>>>(dst, n, seed, mean, std);
  GPTOSS_LAUNCH_CHECK("synth_normal_bf16_kernel");
  return GPTOSS_OK;
}

int run_synth_f32(float *dst, size_t n, uint64_t seed, float mean, float std, hipStream_t s) {
  synth_normal_f32_kernel<<<grid_for(n), 256, 0, s>>>(dst, n, seed, mean, std);
  GPTOSS_LAUNCH_CHECK("synth_normal_f32_kernel");
  return GPTOSS_OK;
}

}  // namespace gptoss
