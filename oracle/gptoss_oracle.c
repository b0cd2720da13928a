/*
 * CPU oracle for the GPT-OSS decode hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the reference's CPU model (run.cpp) and of the
 * integer semantics of its MoE grouping kernel.  It exists to check the HIP kernels; nothing
 * in the shipped library links, loads or calls it.  Only tests/, __graft_entry__.smoke() and
 * the cpu_baseline leg of bench.py may use it.
 *
 * Every function cites the reference lines it follows.  How each one is pinned (against the
 * compiled reference CPU code in oracle/_ref, against closed forms, invariants and brute
 * force) is listed next to it; tests/test_oracle_*.py run those pins.
 *
 *   orc_rmsnorm, orc_softmax, orc_matmul   run.cpp:304-352     pinned: numpy float64 closed forms
 *   orc_topk_softmax                       run.cpp:371-402,636-638; layer_hip_batch.cpp:1120-1127
 *                                                              pinned: argsort on distinct values,
 *                                                              explicit tie vectors, sum-to-one
 *   orc_group                              kernel.cpp:504-542  pinned: stable argsort, bincount,
 *                                                              bijection, brute force
 *   orc_swiglu                             run.cpp:669-686     pinned: closed form + clamp cases
 *   orc_moe_layer                          run.cpp:625-704     pinned: dense one-hot formulation
 *                                                              in float64, and via orc_forward
 *   orc_attn_decode                        run.cpp:562-607     pinned: naive softmax with the sink
 *                                                              as an extra logit, SDPA when
 *                                                              sink=-inf, len=1 closed form
 *   orc_rope_tables                        run.cpp:404-478     pinned: cos^2+sin^2, bit-equality
 *                                                              with the compiled reference
 *   orc_forward, orc_generate              run.cpp:501-717,922-947; getp_run_submit.cpp:60-96
 *                                                              pinned: logits and greedy ids
 *                                                              bit-identical to the compiled
 *                                                              reference (oracle/_ref) and to the
 *                                                              committed golden ids
 *   orc_mxfp4_dequant                      export_model_bin.py:66-123 (gpt-oss-20b)
 *                                                              pinned: brute force over all
 *                                                              16 codes x 256 scales vs ldexp
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#ifndef M_PI
#define M_PI 3.14159265358979323846
#endif

/* ---- header of the flat .bin checkpoint: run.cpp:25-45 (15 four-byte fields) ---- */
typedef struct {
  int vocab_size, hidden_dim, n_experts, experts_per_token, intermediate_dim, n_layers;
  int head_dim, n_attn_heads, n_kv_heads, seq_len, initial_context_length;
  float rope_theta, rope_scaling_factor;
  int sliding_window;
  float swiglu_limit;
} OrcConfig;

/* rounding points of the reference GPU dataflow (model.cpp:28-131, alloc.cpp:205-228) */
enum {
  ORC_STAGE_NORM = 1,    /* rmsnorm outputs -> bf16 */
  ORC_STAGE_KV = 2,      /* K (after RoPE) and V -> bf16 in the cache */
  ORC_STAGE_ATTN = 4,    /* attention output -> bf16 */
  ORC_STAGE_SWIGLU = 8,  /* SwiGLU output -> bf16 */
  ORC_STAGE_Q = 16,      /* q (after RoPE) -> bf16 (only the MFMA attention kernel does this) */
  ORC_STAGE_FLOAT_ACC = 32 /* float instead of double accumulators in matmul */
};

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* round-to-nearest-even fp32 -> bf16 -> fp32 */
static inline float bf16_round(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return f; /* NaN */
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  memcpy(&f, &u, 4);
  return f;
}

void orc_bf16_round(float *x, long long n) {
  for (long long i = 0; i < n; i++) x[i] = bf16_round(x[i]);
}

/* run.cpp:304-317 */
void orc_rmsnorm(float *o, const float *x, const float *weight, int size) {
  double ss = 0.0f;
  for (int j = 0; j < size; j++) ss += x[j] * x[j];
  ss /= size;
  ss += 1e-5f;
  ss = 1.0f / sqrtf(ss);
  for (int j = 0; j < size; j++) o[j] = weight[j] * (ss * x[j]);
}

/* run.cpp:319-337 */
void orc_softmax(float *x, int size) {
  double max_val = x[0];
  for (int i = 1; i < size; i++)
    if (x[i] > max_val) max_val = x[i];
  double sum = 0.0f;
  for (int i = 0; i < size; i++) {
    x[i] = expf(x[i] - max_val);
    sum += x[i];
  }
  for (int i = 0; i < size; i++) x[i] /= sum;
}

/* run.cpp:339-352: W (d,n) @ x (n,) -> xout (d,), double accumulator, OpenMP over rows */
void orc_matmul(float *xout, const float *x, const float *w, int n, int d) {
  int i;
#pragma omp parallel for private(i)
  for (i = 0; i < d; i++) {
    double val = 0.0f;
    const float *wr = w + 1ll * i * n;
    for (int j = 0; j < n; j++) val += wr[j] * x[j];
    xout[i] = val;
  }
}

static void matmul_serial(float *xout, const float *x, const float *w, int n, int d,
                          int float_acc) {
  for (int i = 0; i < d; i++) {
    const float *wr = w + 1ll * i * n;
    if (float_acc) {
      float val = 0.0f;
      for (int j = 0; j < n; j++) val += wr[j] * x[j];
      xout[i] = val;
    } else {
      double val = 0.0f;
      for (int j = 0; j < n; j++) val += wr[j] * x[j];
      xout[i] = val;
    }
  }
}

/*
 * Top-k in descending order followed by softmax over the k picked values.
 * run.cpp:371-402 sorts (value,index) pairs descending with qsort and keeps the first k;
 * run.cpp:636-638 softmaxes them.  qsort leaves the order of equal values open, so ties are
 * fixed here to "lowest expert id first", the order the reference GPU kernel's strict-'>'
 * scan produces for its first pick (layer_hip_batch.cpp:1120-1127).
 */
void orc_topk_softmax(const float *logits, int B, int E, int k, float *topk_v, int *topk_i) {
  unsigned char *used = (unsigned char *)malloc(E);
  for (int b = 0; b < B; b++) {
    const float *r = logits + 1ll * b * E;
    memset(used, 0, E);
    for (int s = 0; s < k; s++) {
      int best = -1;
      for (int e = 0; e < E; e++) {
        if (used[e]) continue;
        if (best < 0 || r[e] > r[best]) best = e;
      }
      used[best] = 1;
      topk_i[1ll * b * k + s] = best;
      topk_v[1ll * b * k + s] = r[best];
    }
    orc_softmax(topk_v + 1ll * b * k, k);
  }
  free(used);
}

/*
 * Expert grouping (counting sort of the B*k (token,slot) pairs by expert id).
 * kernel.cpp:504-542: histogram, exclusive prefix -> expert_offsets[E+1], then scatter of pair
 * ids (pair = token*k + slot) into sorted_pair_ids.  The reference scatters through an LDS
 * atomic cursor so its order inside one expert is not defined; the canonical order here is the
 * one its loop gives when run in thread order: ascending pair id (a stable sort).
 * inv[pair] = position of that pair in sorted_pair_ids.
 */
void orc_group(const int *topk_i, int B, int k, int E, int *expert_offsets, int *sorted_pair_ids,
               int *inv) {
  int P = B * k;
  int *cursor = (int *)calloc(E, sizeof(int));
  for (int e = 0; e <= E; e++) expert_offsets[e] = 0;
  for (int p = 0; p < P; p++) {
    int e = topk_i[p];
    if (0 <= e && e < E) expert_offsets[e + 1]++;
  }
  for (int e = 0; e < E; e++) expert_offsets[e + 1] += expert_offsets[e];
  for (int p = 0; p < P; p++) {
    int e = topk_i[p];
    if (0 <= e && e < E) {
      int pos = expert_offsets[e] + cursor[e]++;
      sorted_pair_ids[pos] = p;
      if (inv) inv[p] = pos;
    }
  }
  free(cursor);
}

/* run.cpp:664-686: interleaved (gate,up) -> clamped SwiGLU, alpha 1.702, up+1 */
void orc_swiglu(const float *mlp1_out, float *out, int I, float limit) {
  const float alpha = 1.702f;
  for (int i = 0; i < I; i++) {
    float val = mlp1_out[2 * i];
    float up_val = mlp1_out[2 * i + 1];
    if (val > limit) val = limit;
    if (up_val > limit) up_val = limit;
    if (up_val < -limit) up_val = -limit;
    val *= (1.0f / (1.0f + expf(-alpha * val)));
    val *= (up_val + 1.0f);
    out[i] = val;
  }
}

/*
 * One MoE block for B independent tokens: run.cpp:625-704.
 *   t        [B,H]      normalised activations (inputs of the router and the experts)
 *   w_router [E,H], b_router [E]; w1 [E,2I,H] rows interleaved gate/up, b1 [E,2I];
 *   w2 [E,H,I], b2 [E,H]         (the .bin layouts, run.cpp:66-76)
 *   out      [B,H]      e_agg (the residual add is left to the caller)
 * Optional outputs (may be NULL): logits [B,E], topk_v [B,k], topk_i [B,k].
 * stage: ORC_STAGE_SWIGLU rounds the SwiGLU output to bf16 as the GPU dataflow does;
 *        ORC_STAGE_FLOAT_ACC uses float accumulators.
 * Tokens are independent, so OpenMP runs over tokens here (the reference parallelises the rows
 * of each matmul instead; the arithmetic per output element is the same).
 */
void orc_moe_layer(const float *t, const float *w_router, const float *b_router, const float *w1,
                   const float *b1, const float *w2, const float *b2, int B, int H, int I, int E,
                   int k, float limit, int stage, float *out, float *logits_out, float *topk_v_out,
                   int *topk_i_out) {
  int facc = (stage & ORC_STAGE_FLOAT_ACC) != 0;
#pragma omp parallel
  {
    float *score = (float *)malloc(sizeof(float) * E);
    float *tv = (float *)malloc(sizeof(float) * k);
    int *ti = (int *)malloc(sizeof(int) * k);
    float *mlp1 = (float *)malloc(sizeof(float) * 2 * I);
    float *act = (float *)malloc(sizeof(float) * I);
    float *tb2 = (float *)malloc(sizeof(float) * H);
#pragma omp for schedule(dynamic, 1)
    for (int b = 0; b < B; b++) {
      const float *tt = t + 1ll * b * H;
      float *agg = out + 1ll * b * H;
      matmul_serial(score, tt, w_router, H, E, facc);
      for (int i = 0; i < E; i++) score[i] += b_router[i];
      if (logits_out) memcpy(logits_out + 1ll * b * E, score, sizeof(float) * E);
      orc_topk_softmax(score, 1, E, k, tv, ti);
      if (topk_v_out) memcpy(topk_v_out + 1ll * b * k, tv, sizeof(float) * k);
      if (topk_i_out) memcpy(topk_i_out + 1ll * b * k, ti, sizeof(int) * k);
      memset(agg, 0, sizeof(float) * H);
      for (int e = 0; e < E; e++) {
        float expert_w = 0;
        int in_topk = 0;
        for (int idx = 0; idx < k; idx++) {
          if (ti[idx] == e) {
            in_topk = 1;
            expert_w = tv[idx];
            break;
          }
        }
        if (!in_topk) continue;
        matmul_serial(mlp1, tt, w1 + 1ll * e * (2 * I) * H, H, 2 * I, facc);
        for (int i = 0; i < 2 * I; i++) mlp1[i] += b1[1ll * e * 2 * I + i];
        orc_swiglu(mlp1, act, I, limit);
        if (stage & ORC_STAGE_SWIGLU)
          for (int i = 0; i < I; i++) act[i] = bf16_round(act[i]);
        matmul_serial(tb2, act, w2 + 1ll * e * H * I, I, H, facc);
        for (int i = 0; i < H; i++) tb2[i] += b2[1ll * e * H + i];
        for (int i = 0; i < H; i++) agg[i] += tb2[i] * expert_w;
      }
    }
    free(score); free(tv); free(ti); free(mlp1); free(act); free(tb2);
  }
}

/*
 * Single-query attention with sinks and an optional sliding window: run.cpp:562-607.
 *   q     [B, n_q, D]   (already rotated)
 *   K, V  [B, S, n_kv, D]  position-major cache (no ring indexing: slot == position)
 *   lens  [B]           number of cached positions per sequence (pos+1)
 *   window > 0 keeps positions t with (len-1) - t < window  (mask of run.cpp:160-162);
 *   sinks [n_q]         extra logit per head that only feeds the softmax denominator
 *   out   [B, n_q, D]
 */
void orc_attn_decode(const float *q, const float *K, const float *V, const int *lens,
                     const float *sinks, int B, int S, int n_q, int n_kv, int D, int window,
                     float *out) {
  int kv_mul = n_q / n_kv;
  long long kv_dim = 1ll * n_kv * D;
#pragma omp parallel
  {
    float *att = (float *)malloc(sizeof(float) * (S + 2));
#pragma omp for collapse(2) schedule(dynamic, 1)
    for (int b = 0; b < B; b++) {
      for (int h = 0; h < n_q; h++) {
        int pos = lens[b] - 1;
        const float *qh = q + (1ll * b * n_q + h) * D;
        const float *Kb = K + 1ll * b * S * kv_dim;
        const float *Vb = V + 1ll * b * S * kv_dim;
        for (int t = 0; t <= pos; t++) {
          const float *kk = Kb + t * kv_dim + (h / kv_mul) * D;
          double score = 0.0f;
          for (int i = 0; i < D; i++) score += qh[i] * kk[i];
          score /= sqrtf(D);
          if (window > 0 && pos - t >= window) score += -INFINITY;
          att[t] = score;
        }
        att[pos + 1] = sinks[h];
        orc_softmax(att, pos + 2);
        float *tb = out + (1ll * b * n_q + h) * D;
        memset(tb, 0, D * sizeof(float));
        for (int t = 0; t <= pos; t++) {
          const float *vv = Vb + t * kv_dim + (h / kv_mul) * D;
          float a = att[t];
          for (int i = 0; i < D; i++) tb[i] += a * vv[i];
        }
      }
    }
    free(att);
  }
}

/* run.cpp:404-453 */
static void concentration_and_inv_freq(float base, int head_dim, float scaling_factor,
                                       float initial_context_length, float ntk_beta,
                                       float ntk_alpha, float *concentration_out,
                                       float *inv_freq_out) {
  int d_half = head_dim / 2;
  float *freq = (float *)malloc(d_half * sizeof(float));
  for (int i = 0; i < d_half; i++) freq[i] = powf(base, ((float)(2 * i)) / (float)head_dim);
  float concentration;
  if (scaling_factor > 1.0f) {
    concentration = 0.1f * logf(scaling_factor) + 1.0f;
    float low = d_half * logf(initial_context_length / (ntk_beta * 2.0f * M_PI)) / logf(base);
    float high = d_half * logf(initial_context_length / (ntk_alpha * 2.0f * M_PI)) / logf(base);
    for (int i = 0; i < d_half; i++) {
      float interpolation = 1.0f / (scaling_factor * freq[i]);
      float extrapolation = 1.0f / freq[i];
      float ramp = ((float)i - low) / (high - low);
      if (ramp < 0) ramp = 0;
      if (ramp > 1) ramp = 1;
      float mask = 1.0f - ramp;
      inv_freq_out[i] = interpolation * (1.0f - mask) + extrapolation * mask;
    }
  } else {
    concentration = 1.0f;
    for (int i = 0; i < d_half; i++) inv_freq_out[i] = 1.0f / freq[i];
  }
  *concentration_out = concentration;
  free(freq);
}

/* run.cpp:455-478 for every pos in [0,n_pos): cos/sin tables [n_pos, head_dim/2],
 * ntk_beta=32, ntk_alpha=1 as at run.cpp:550-551 */
void orc_rope_tables(const OrcConfig *p, int n_pos, float *cos_out, float *sin_out) {
  int d_half = p->head_dim / 2;
  float concentration;
  float *inv_freq = (float *)malloc(d_half * sizeof(float));
  concentration_and_inv_freq(p->rope_theta, p->head_dim, p->rope_scaling_factor,
                             p->initial_context_length, 32.0f, 1.0f, &concentration, inv_freq);
  for (int pos = 0; pos < n_pos; pos++) {
    for (int j = 0; j < d_half; j++) {
      float val = (float)pos * inv_freq[j];
      cos_out[1ll * pos * d_half + j] = cosf(val) * concentration;
      sin_out[1ll * pos * d_half + j] = sinf(val) * concentration;
    }
  }
  free(inv_freq);
}

/* run.cpp:480-499 */
static void apply_rotary(float *x, const float *c, const float *s, int n_heads, int head_dim) {
  int half = head_dim / 2;
  for (int h = 0; h < n_heads; h++) {
    for (int i = 0; i < half; i++) {
      float x1 = x[h * head_dim + i];
      float x2 = x[h * head_dim + half + i];
      float o1 = x1 * c[i] - x2 * s[i];
      float o2 = x2 * c[i] + x1 * s[i];
      x[h * head_dim + i] = o1;
      x[h * head_dim + half + i] = o2;
    }
  }
}

/* ---- whole model: weights in the order of run.cpp:194-233 ---- */
typedef struct {
  OrcConfig cfg;
  const float *emb, *unemb, *rms_attn, *rms_ffn, *rms_out, *w_qkv, *b_qkv, *w_o, *b_o, *sinks;
  const float *w_router, *b_router, *w_mlp1, *b_mlp1, *w_mlp2, *b_mlp2;
  /* run state for ONE sequence (run.cpp:83-108) */
  float *x, *t, *tb, *tb2, *score, *topk_v, *mlp1, *act, *e_agg, *qkv, *att, *logits;
  int *topk_i;
  float *key_cache, *value_cache; /* [L, seq_len, kv_dim] */
  float *cos_t, *sin_t;           /* [seq_len, D/2] */
  int stage;
  float min_router_gap; /* smallest (k-th - (k+1)-th) router score seen by orc_forward */
  float last_router_gap; /* the same over the layers of the last orc_forward call only */
} OrcModel;

long long orc_weight_floats(const OrcConfig *c) {
  long long H = c->hidden_dim, V = c->vocab_size, L = c->n_layers, E = c->n_experts;
  long long D = c->head_dim, nq = c->n_attn_heads, nkv = c->n_kv_heads, I = c->intermediate_dim;
  long long qkv = D * (nq + 2 * nkv);
  return 2 * V * H + 2 * L * H + H + L * qkv * H + L * qkv + L * nq * D * H + L * H + L * nq +
         L * E * H + L * E + L * E * 2 * I * H + L * E * 2 * I + L * E * H * I + L * E * H;
}

/* weights = pointer just past the 60-byte header; layout run.cpp:194-233 */
OrcModel *orc_model_create(const OrcConfig *cfg, const float *weights, int stage) {
  OrcModel *m = (OrcModel *)calloc(1, sizeof(OrcModel));
  m->cfg = *cfg;
  m->stage = stage;
  m->min_router_gap = INFINITY;
  const OrcConfig *c = cfg;
  long long H = c->hidden_dim, V = c->vocab_size, L = c->n_layers, E = c->n_experts;
  long long D = c->head_dim, nq = c->n_attn_heads, nkv = c->n_kv_heads, I = c->intermediate_dim;
  long long qkv = D * (nq + 2 * nkv);
  const float *p = weights;
  m->emb = p; p += V * H;
  m->unemb = p; p += V * H;
  m->rms_attn = p; p += L * H;
  m->rms_ffn = p; p += L * H;
  m->rms_out = p; p += H;
  m->w_qkv = p; p += L * qkv * H;
  m->b_qkv = p; p += L * qkv;
  m->w_o = p; p += L * nq * D * H;
  m->b_o = p; p += L * H;
  m->sinks = p; p += L * nq;
  m->w_router = p; p += L * H * E;
  m->b_router = p; p += L * E;
  m->w_mlp1 = p; p += L * E * 2 * I * H;
  m->b_mlp1 = p; p += L * E * 2 * I;
  m->w_mlp2 = p; p += L * E * H * I;
  m->b_mlp2 = p; p += L * E * H;
  long long kv_dim = D * nkv, S = c->seq_len;
  m->x = (float *)calloc(H, 4);
  m->t = (float *)calloc(H, 4);
  m->tb = (float *)calloc(D * nq, 4);
  m->tb2 = (float *)calloc(H, 4);
  m->score = (float *)calloc(E, 4);
  m->topk_v = (float *)calloc(c->experts_per_token, 4);
  m->topk_i = (int *)calloc(c->experts_per_token, 4);
  m->mlp1 = (float *)calloc(2 * I, 4);
  m->act = (float *)calloc(I, 4);
  m->e_agg = (float *)calloc(H, 4);
  m->qkv = (float *)calloc(qkv, 4);
  m->att = (float *)calloc(nq * (S + 2), 4);
  m->logits = (float *)calloc(V, 4);
  m->key_cache = (float *)calloc(L * S * kv_dim, 4);
  m->value_cache = (float *)calloc(L * S * kv_dim, 4);
  m->cos_t = (float *)calloc(S * (D / 2), 4);
  m->sin_t = (float *)calloc(S * (D / 2), 4);
  orc_rope_tables(c, (int)S, m->cos_t, m->sin_t);
  return m;
}

void orc_model_destroy(OrcModel *m) {
  if (!m) return;
  free(m->x); free(m->t); free(m->tb); free(m->tb2); free(m->score); free(m->topk_v);
  free(m->topk_i); free(m->mlp1); free(m->act); free(m->e_agg); free(m->qkv); free(m->att);
  free(m->logits); free(m->key_cache); free(m->value_cache); free(m->cos_t); free(m->sin_t);
  free(m);
}

float *orc_model_logits(OrcModel *m) { return m->logits; }
float *orc_model_x(OrcModel *m) { return m->x; }
float orc_model_min_router_gap(OrcModel *m) { return m->min_router_gap; }
float orc_model_last_router_gap(OrcModel *m) { return m->last_router_gap; }

static void round_vec(float *x, long long n) {
  for (long long i = 0; i < n; i++) x[i] = bf16_round(x[i]);
}

static void mm(OrcModel *m, float *xout, const float *x, const float *w, int n, int d) {
  if (m->stage & ORC_STAGE_FLOAT_ACC) {
    int i;
#pragma omp parallel for private(i)
    for (i = 0; i < d; i++) {
      float val = 0.0f;
      const float *wr = w + 1ll * i * n;
      for (int j = 0; j < n; j++) val += wr[j] * x[j];
      xout[i] = val;
    }
  } else {
    orc_matmul(xout, x, w, n, d);
  }
}

/* run.cpp:501-717.  Returns the logits of `token` at position `pos` for this model's single
 * sequence state. */
float *orc_forward(OrcModel *m, int token, int pos) {
  const OrcConfig *p = &m->cfg;
  float *x = m->x;
  int head_dim = p->head_dim, hidden_dim = p->hidden_dim;
  int kv_dim = p->head_dim * p->n_kv_heads;
  int kv_mul = p->n_attn_heads / p->n_kv_heads;
  int I = p->intermediate_dim, E = p->n_experts, k = p->experts_per_token;
  int qkv_dim = (p->n_attn_heads + 2 * p->n_kv_heads) * head_dim;
  int S = p->seq_len;
  int stage = m->stage;

  m->last_router_gap = INFINITY;
  memcpy(x, m->emb + 1ll * token * hidden_dim, hidden_dim * sizeof(float));

  for (long long l = 0; l < p->n_layers; l++) {
    orc_rmsnorm(m->t, x, m->rms_attn + l * hidden_dim, hidden_dim);
    if (stage & ORC_STAGE_NORM) round_vec(m->t, hidden_dim);

    long long loff = l * S * kv_dim;
    float *kc = m->key_cache + loff + 1ll * pos * kv_dim;
    float *vc = m->value_cache + loff + 1ll * pos * kv_dim;

    mm(m, m->qkv, m->t, m->w_qkv + l * hidden_dim * qkv_dim, hidden_dim, qkv_dim);
    for (int i = 0; i < qkv_dim; i++) m->qkv[i] += m->b_qkv[l * qkv_dim + i];
    float *q = m->qkv;
    memcpy(kc, m->qkv + head_dim * p->n_attn_heads, kv_dim * sizeof(float));
    memcpy(vc, m->qkv + head_dim * p->n_attn_heads + kv_dim, kv_dim * sizeof(float));

    const float *cs = m->cos_t + 1ll * pos * (head_dim / 2);
    const float *sn = m->sin_t + 1ll * pos * (head_dim / 2);
    apply_rotary(q, cs, sn, p->n_attn_heads, head_dim);
    apply_rotary(kc, cs, sn, p->n_kv_heads, head_dim);
    if (stage & ORC_STAGE_KV) {
      round_vec(kc, kv_dim);
      round_vec(vc, kv_dim);
    }
    if (stage & ORC_STAGE_Q) round_vec(q, head_dim * p->n_attn_heads);

    int h;
#pragma omp parallel for private(h)
    for (h = 0; h < p->n_attn_heads; h++) {
      const float *qh = q + h * head_dim;
      float *att = m->att + 1ll * h * (S + 2);
      for (int t = 0; t <= pos; t++) {
        const float *kk = m->key_cache + loff + 1ll * t * kv_dim + (h / kv_mul) * head_dim;
        double score = 0.0f;
        for (int i = 0; i < head_dim; i++) score += qh[i] * kk[i];
        score /= sqrtf(head_dim);
        /* mask of run.cpp:157-164 applied on even layers, run.cpp:582-584 */
        if (p->sliding_window > 0 && (l % 2 == 0) && pos - t >= p->sliding_window)
          score += -INFINITY;
        att[t] = score;
      }
      att[pos + 1] = m->sinks[l * p->n_attn_heads + h];
      orc_softmax(att, pos + 2);
      float *tb = m->tb + h * head_dim;
      memset(tb, 0, head_dim * sizeof(float));
      for (int t = 0; t <= pos; t++) {
        const float *vv = m->value_cache + loff + 1ll * t * kv_dim + (h / kv_mul) * head_dim;
        float a = att[t];
        for (int i = 0; i < head_dim; i++) tb[i] += a * vv[i];
      }
    }
    if (stage & ORC_STAGE_ATTN) round_vec(m->tb, head_dim * p->n_attn_heads);

    mm(m, m->tb2, m->tb, m->w_o + l * (head_dim * p->n_attn_heads) * hidden_dim,
       head_dim * p->n_attn_heads, hidden_dim);
    for (int i = 0; i < hidden_dim; i++) m->tb2[i] += m->b_o[l * hidden_dim + i];
    for (int i = 0; i < hidden_dim; i++) x[i] += m->tb2[i];

    orc_rmsnorm(m->t, x, m->rms_ffn + l * hidden_dim, hidden_dim);
    if (stage & ORC_STAGE_NORM) round_vec(m->t, hidden_dim);

    /* MoE: run.cpp:625-704 */
    mm(m, m->score, m->t, m->w_router + l * hidden_dim * E, hidden_dim, E);
    for (int i = 0; i < E; i++) m->score[i] += m->b_router[l * E + i];
    orc_topk_softmax(m->score, 1, E, k, m->topk_v, m->topk_i);
    if (k < E) {
      float kth = m->score[m->topk_i[k - 1]], next = -INFINITY;
      for (int i = 0; i < E; i++) {
        int picked = 0;
        for (int j = 0; j < k; j++) picked |= (m->topk_i[j] == i);
        if (!picked && m->score[i] > next) next = m->score[i];
      }
      if (kth - next < m->min_router_gap) m->min_router_gap = kth - next;
      if (kth - next < m->last_router_gap) m->last_router_gap = kth - next;
    }
    memset(m->e_agg, 0, hidden_dim * sizeof(float));
    for (int e = 0; e < E; e++) {
      float expert_w = 0;
      int in_topk = 0;
      for (int idx = 0; idx < k; idx++) {
        if (m->topk_i[idx] == e) {
          in_topk = 1;
          expert_w = m->topk_v[idx];
          break;
        }
      }
      if (!in_topk) continue;
      mm(m, m->mlp1, m->t, m->w_mlp1 + (l * E + e) * (2ll * I) * hidden_dim, hidden_dim, 2 * I);
      for (int i = 0; i < 2 * I; i++) m->mlp1[i] += m->b_mlp1[(l * E + e) * (2ll * I) + i];
      orc_swiglu(m->mlp1, m->act, I, p->swiglu_limit);
      if (stage & ORC_STAGE_SWIGLU) round_vec(m->act, I);
      mm(m, m->tb2, m->act, m->w_mlp2 + (l * E + e) * 1ll * hidden_dim * I, I, hidden_dim);
      for (int i = 0; i < hidden_dim; i++) m->tb2[i] += m->b_mlp2[(l * E + e) * hidden_dim + i];
      for (int i = 0; i < hidden_dim; i++) m->e_agg[i] += m->tb2[i] * expert_w;
    }
    for (int i = 0; i < hidden_dim; i++) x[i] += m->e_agg[i];
  }
  orc_rmsnorm(x, x, m->rms_out, hidden_dim);
  if (stage & ORC_STAGE_NORM) {
    /* the GPU path rounds the final norm into a separate bf16 buffer (model.cpp:140-141) */
    float *xr = m->t;
    for (int i = 0; i < hidden_dim; i++) xr[i] = bf16_round(x[i]);
    mm(m, m->logits, xr, m->unemb, hidden_dim, p->vocab_size);
  } else {
    mm(m, m->logits, x, m->unemb, hidden_dim, p->vocab_size);
  }
  return m->logits;
}

/* run.cpp:739-750 */
int orc_argmax(const float *v, int n) {
  int max_i = 0;
  float max_p = v[0];
  for (int i = 1; i < n; i++) {
    if (v[i] > max_p) {
      max_i = i;
      max_p = v[i];
    }
  }
  return max_i;
}

/*
 * Greedy generation for a batch of token-id prompts with the semantics of the getp decode loop
 * (getp_run_submit.cpp:60-96; per sequence it is the loop of run.cpp:922-947):
 * positions 0..max_seq_len-2 are run; while pos < n_prompt-1 the next prompt token is forced;
 * afterwards the arg-max is stored at out[pos-(n_prompt-1)] and fed back; ids 199999 and 200002
 * stop the sequence after being stored; out[generated_len+1] = -1.
 *   prompts [n_req, prompt_stride] with n_prompt[r] valid ids each
 *   out     [n_req, max_seq_len+1]
 *   margins (optional) [n_req, max_seq_len+1]: top1-top2 logit gap of every sampled position
 *   min_router_gap (optional): smallest gap between the k-th and (k+1)-th router score met
 * Returns the number of generated tokens counted the way the harness counts them.
 */
long long orc_generate(const OrcConfig *cfg, const float *weights, int stage, const int *prompts,
                       const int *n_prompt, int prompt_stride, int n_req, int max_seq_len,
                       int *out, float *margins, float *min_router_gap) {
  long long total = 0;
  if (min_router_gap) *min_router_gap = INFINITY;
  for (int r = 0; r < n_req; r++) {
    OrcModel *m = orc_model_create(cfg, weights, stage);
    const int *pt = prompts + 1ll * r * prompt_stride;
    int *o = out + 1ll * r * (max_seq_len + 1);
    int np = n_prompt[r];
    int token = pt[0];
    int cur = 0;
    for (int pos = 0; pos < max_seq_len - 1; pos++) {
      float *logits = orc_forward(m, token, pos);
      int next = orc_argmax(logits, cfg->vocab_size);
      if (cur < np - 1) {
        next = pt[cur + 1];
      } else {
        o[cur - (np - 1)] = next;
        if (margins) {
          float best = logits[next], second = -INFINITY;
          for (int i = 0; i < cfg->vocab_size; i++)
            if (i != next && logits[i] > second) second = logits[i];
          margins[1ll * r * (max_seq_len + 1) + cur - (np - 1)] = best - second;
        }
      }
      token = next;
      cur++;
      if (next == 199999 || next == 200002) break;
    }
    int generated_len = cur - np;
    if (generated_len < 0) generated_len = 0;
    o[generated_len + 1] = -1;
    total += generated_len + 1;
    if (min_router_gap && m->min_router_gap < *min_router_gap) *min_router_gap = m->min_router_gap;
    orc_model_destroy(m);
  }
  return total;
}

/*
 * MXFP4 block dequantisation: export_model_bin/gpt-oss-20b/export_model_bin.py:66-123.
 * blocks: n_blocks x 16 bytes, each byte = two e2m1 codes (low nibble = even element, high
 * nibble = odd element); scales: one e8m0 byte per block; value = LUT[code] * 2^(scale-127).
 * out: n_blocks x 32 floats.
 */
void orc_mxfp4_dequant(const uint8_t *blocks, const uint8_t *scales, long long n_blocks,
                       float *out) {
  static const float lut[16] = {+0.0f, +0.5f, +1.0f, +1.5f, +2.0f, +3.0f, +4.0f, +6.0f,
                                -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
  for (long long b = 0; b < n_blocks; b++) {
    int ex = (int)scales[b] - 127;
    for (int j = 0; j < 16; j++) {
      uint8_t byte = blocks[b * 16 + j];
      out[b * 32 + 2 * j] = ldexpf(lut[byte & 0x0f], ex);
      out[b * 32 + 2 * j + 1] = ldexpf(lut[byte >> 4], ex);
    }
  }
}
