// Single-GPU decode engine: device weights in kernel layout, run state, one decode step (the op
// order of the reference's forward_gpu_20b_batched, getp-csrc/src/model.cpp:6-151; all sequences
// at one position, or each at its own), a prompt pass that runs many positions of a sequence
// through the same kernels at once, and greedy generation: the reference's lock-step batches
// (getp-csrc/submit/getp_run_submit.cpp:13-96) or, by default, the same requests over a fixed set
// of slots that are refilled as sequences end.
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <system_error>
#include <thread>
#include <vector>

#include "common.hpp"
#include "gemm.hpp"
#include "glue.hpp"
#include "precise.hpp"

#ifndef M_PI
#define M_PI 3.14159265358979323846
#endif

namespace gptoss {

struct LayerWeights {
  float *attn_norm, *mlp_norm;    // fp32 [H]
  bf16_t *w_qkv;                  // packed [(nq+2nkv)D, H]
  float *b_qkv;
  bf16_t *w_o;                    // packed [H, nq*D]
  float *b_o;
  float *sinks;                   // [nq]
  bf16_t *w_router;               // [E,H] row-major
  float *b_router;
  bf16_t *w1;                     // packed GLU [E][2I,H] (bf16, or MXFP4 bytes with GPTOSS_ENGINE_MXFP4_EXPERTS)
  float *b1;
  bf16_t *w2;                     // packed [E][H,I]     (likewise)
  float *b2;
  bf16_t *kv_cache;               // K and V of the layer, block layout of common.hpp
  int cache_cap;
  int window;                     // 0 = full attention
};

}  // namespace gptoss

using namespace gptoss;

struct gptoss_engine {
  gptoss_config cfg;
  int max_batch, max_seq, flags;
  hipStream_t stream;
  std::vector<void *> allocs;
  // weights
  bf16_t *embedding;   // [V,H]
  bf16_t *unembedding; // packed [V,H]
  float *final_norm;
  std::vector<LayerWeights> layers;
  float *cos_t, *sin_t;  // [max_seq, D/2]
  // run state
  int *d_tokens, *d_next, *d_lens;
  int *h_tokens, *h_next, *h_lens;  // pinned
  float *x, *qkv, *q, *tb2, *logits;  // logits == nullptr unless GPTOSS_ENGINE_LOGITS
  float *amax_val;                     // [B, column tiles of the classifier]: fused arg-max partials
  int *amax_idx;
  bf16_t *t, *attn_out;
  void *moe_ws, *attn_ws;
  size_t moe_ws_bytes, attn_ws_bytes;
  size_t device_bytes;
  // prompt processing (many positions of a sequence at once): activations for up to pf.rows rows,
  // and a linear K/V scratch for the sliding-window layers when a prompt is longer than their ring
  struct Prefill {
    int rows;  // 0: not available
    int *tokens;          // [rows] followed by seq_map [rows], lens [rows], sample [max_batch]: one upload
    int *seq_map, *lens;  // cache slot (and, for a step over arbitrary rows, cached positions) of every row
    int *sample;          // rows whose next id is wanted
    int *h_rows;          // pinned host image of tokens .. sample
    float *x, *qkv, *q, *tb2;
    bf16_t *t, *attn_out, *kv_scratch;
    size_t scratch_tokens;  // positions (summed over sequences) the scratch holds
    void *moe_ws, *attn_ws;
    size_t moe_ws_bytes, attn_ws_bytes;
  } pf;
  // fp32-faithful mode (GPTOSS_ENGINE_PRECISE): the .bin payload as it is, fp32 KV caches and
  // fp32 intermediates
  struct Precise {
    float *payload;  // whole fp32 payload, tensor offsets below in floats
    size_t emb, unemb, attn_norm, mlp_norm, fin, w_qkv, b_qkv, w_o, b_o, sinks, w_router, b_router, w1, b1, w2, b2;
    float *kc, *vc;  // [L, B, max_seq, kv_dim]
    float *t, *attn, *att, *router, *topk_w, *mlp1, *act, *mlp2;
    int *topk_i;
  } pr;
};

namespace {

// Host -> device staging of the fp32 payload: two pinned host buffers and two device buffers.
// Chunk i is copied by the host into pinned[i % 2] (several threads), sent with an asynchronous
// copy on its own stream, and converted/packed by a kernel on the engine's stream; the copy of chunk
// i+1 and the host's work on chunk i+2 overlap that kernel.  Events order the reuse of either
// buffer; the host only ever waits for the copy issued two chunks earlier.  Replaces the host-side
// transposes and synchronous uploads of getp-csrc/src/alloc.cpp:27-35,112-127.
struct Stager {
  hipStream_t copy = nullptr;
  float *pinned[2] = {nullptr, nullptr}, *dev[2] = {nullptr, nullptr};
  hipEvent_t h2d_done[2] = {nullptr, nullptr}, consumed[2] = {nullptr, nullptr};
  size_t elems = 0;   // floats per buffer
  unsigned next = 0;
};

// plain copy by a few threads: one thread reaches a fraction of what the host memory can deliver
static void host_copy(float *dst, const float *src, size_t n) {
  constexpr int T = 6;
  if (n < ((size_t)1 << 20)) {
    memcpy(dst, src, n * sizeof(float));
    return;
  }
  std::thread th[T - 1];
  const size_t per = (n + T - 1) / T;
  int started = 0;
  for (int i = 1; i < T; i++) {
    const size_t lo = std::min(n, per * i), hi = std::min(n, per * (i + 1));
    try {
      th[i - 1] = std::thread([=] { memcpy(dst + lo, src + lo, (hi - lo) * sizeof(float)); });
      started = i;
    } catch (const std::system_error &) {
      break;  // no more threads to be had (a thread or pid limit): this thread copies the rest
    }
  }
  memcpy(dst, src, std::min(n, per) * sizeof(float));
  const size_t rest = std::min(n, per * (size_t)(started + 1));
  if (rest < n) memcpy(dst + rest, src + rest, (n - rest) * sizeof(float));
  for (int i = 1; i <= started; i++) th[i - 1].join();
}

struct Builder {
  gptoss_engine *e;
  int rc = GPTOSS_OK;
  Stager st;                      // fp32 payload on its way to the device (host weights only)
  bf16_t *stage_bf16 = nullptr;   // synthetic weights before packing
  size_t stage_elems = 0;
  // MXFP4 expert storage: unpacked codes and scales of one staging chunk, and the flag the
  // requantisation kernel raises when a value has no exact MXFP4 representation
  unsigned char *q_blocks = nullptr, *q_scales = nullptr;
  int *q_not_exact = nullptr;

  template <typename T>
  T *alloc(size_t n) {
    if (rc != GPTOSS_OK) return nullptr;
    void *p = nullptr;
    size_t bytes = align_up(n * sizeof(T), 256);
    hipError_t err = hipMalloc(&p, bytes);
    if (err != hipSuccess) {
      rc = fail(GPTOSS_ERR_HIP, "engine: hipMalloc of %zu bytes failed: %s", bytes, hipGetErrorString(err));
      return nullptr;
    }
    e->allocs.push_back(p);
    e->device_bytes += bytes;
    return (T *)p;
  }

  bool ok() const { return rc == GPTOSS_OK; }
  void check(int r) { if (rc == GPTOSS_OK && r != GPTOSS_OK) rc = r; }
  void hip(hipError_t err, const char *what) {
    if (rc == GPTOSS_OK && err != hipSuccess) rc = fail(GPTOSS_ERR_HIP, "engine: %s: %s", what, hipGetErrorString(err));
  }

  void stager_create(size_t elems) {
    st.elems = elems;
    hip(hipStreamCreate(&st.copy), "hipStreamCreate");
    for (int i = 0; i < 2 && ok(); i++) {
      hip(hipHostMalloc((void **)&st.pinned[i], elems * sizeof(float), hipHostMallocDefault), "staging hipHostMalloc");
      hip(hipMalloc((void **)&st.dev[i], elems * sizeof(float)), "staging hipMalloc");
      hip(hipEventCreateWithFlags(&st.h2d_done[i], hipEventDisableTiming), "hipEventCreate");
      hip(hipEventCreateWithFlags(&st.consumed[i], hipEventDisableTiming), "hipEventCreate");
    }
  }
  void stager_destroy() {
    if (st.copy) (void)hipStreamSynchronize(st.copy);
    for (int i = 0; i < 2; i++) {
      if (st.pinned[i]) (void)hipHostFree(st.pinned[i]);
      if (st.dev[i]) (void)hipFree(st.dev[i]);
      if (st.h2d_done[i]) (void)hipEventDestroy(st.h2d_done[i]);
      if (st.consumed[i]) (void)hipEventDestroy(st.consumed[i]);
    }
    if (st.copy) (void)hipStreamDestroy(st.copy);
    st = Stager();
  }
  // n floats of the payload -> a device buffer the engine's stream may read once this returns (the
  // wait is enqueued, not performed); release(slot) after the kernels that read it are enqueued
  const float *stage_in(const float *host, size_t n, int *slot) {
    const int sl = (int)(st.next++ & 1);
    *slot = sl;
    if (!ok()) return nullptr;
    // pinned[sl] is free once the copy that last read it has finished (an event never recorded is complete)
    hip(hipEventSynchronize(st.h2d_done[sl]), "hipEventSynchronize");
    if (!ok()) return nullptr;
    host_copy(st.pinned[sl], host, n);
    // dev[sl] is free once the kernels that last read it have finished
    hip(hipStreamWaitEvent(st.copy, st.consumed[sl], 0), "hipStreamWaitEvent");
    hip(hipMemcpyAsync(st.dev[sl], st.pinned[sl], n * sizeof(float), hipMemcpyHostToDevice, st.copy), "H2D");
    hip(hipEventRecord(st.h2d_done[sl], st.copy), "hipEventRecord");
    hip(hipStreamWaitEvent(e->stream, st.h2d_done[sl], 0), "hipStreamWaitEvent");
    return st.dev[sl];
  }
  void release(int slot) { hip(hipEventRecord(st.consumed[slot], e->stream), "hipEventRecord"); }

  // fp32 host tensor -> fp32 device tensor
  float *upload_f32(const float *host, size_t n, uint64_t seed, float mean, float std) {
    float *d = alloc<float>(n);
    if (!ok()) return nullptr;
    if (!host) {
      check(run_synth_f32(d, n, seed, mean, std, e->stream));
      return d;
    }
    for (size_t o = 0; o < n && ok(); o += st.elems) {
      const size_t c = std::min(st.elems, n - o);
      int slot;
      const float *src = stage_in(host + o, c, &slot);
      if (!ok()) break;
      hip(hipMemcpyAsync(d + o, src, c * sizeof(float), hipMemcpyDeviceToDevice, e->stream), "D2D");
      release(slot);
    }
    return d;
  }

  // fp32 host matrices -> bf16 device matrices, row-major (pack == false) or fragment order
  bf16_t *upload_matrices(const float *host, int n_mat, int n_out, int n_in, bool pack, int pack_flags,
                          uint64_t seed, float std) {
    size_t per = (size_t)n_out * n_in;
    bf16_t *dst = alloc<bf16_t>(per * n_mat);
    if (!ok()) return nullptr;
    if (per > stage_elems) {
      rc = fail(GPTOSS_ERR_DIM, "engine: a %d x %d matrix exceeds the staging buffer", n_out, n_in);
      return nullptr;
    }
    int group = (int)std::max<size_t>(1, stage_elems / per);
    for (int m0 = 0; m0 < n_mat && ok(); m0 += group) {
      int nm = std::min(group, n_mat - m0);
      size_t n = per * nm;
      if (host) {
        int slot;
        const float *src = stage_in(host + per * m0, n, &slot);
        if (!ok()) break;
        if (pack) check(gptoss_pack_weight(src, dst + per * m0, nm, n_out, n_in, pack_flags | GPTOSS_PACK_SRC_FP32, e->stream));
        else check(run_f32_to_bf16(src, dst + per * m0, n, e->stream));
        release(slot);
      } else {
        // one stream, in order: the staging buffer is rewritten only after the kernel that read it
        check(run_synth_bf16(stage_bf16, n, seed + 7919ull * (uint64_t)m0, 0.f, std, e->stream));
        if (!ok()) break;
        if (pack) check(gptoss_pack_weight(stage_bf16, dst + per * m0, nm, n_out, n_in, pack_flags, e->stream));
        else hip(hipMemcpyAsync(dst + per * m0, stage_bf16, n * sizeof(bf16_t), hipMemcpyDeviceToDevice, e->stream), "D2D");
      }
    }
    return dst;
  }

  // fp32 host matrices (exactly MXFP4-representable) or random MXFP4 weights -> packed MXFP4
  bf16_t *upload_matrices_mxfp4(const float *host, int n_mat, int n_out, int n_in, int pack_flags,
                                uint64_t seed) {
    const size_t per = (size_t)n_out * n_in;
    const size_t mat_bytes = per / 2 + per / 32;
    unsigned char *dst = alloc<unsigned char>(mat_bytes * n_mat);
    if (!ok()) return nullptr;
    if (per > stage_elems) {
      rc = fail(GPTOSS_ERR_DIM, "engine: a %d x %d matrix exceeds the staging buffer", n_out, n_in);
      return nullptr;
    }
    const int group = (int)std::max<size_t>(1, stage_elems / per);
    for (int m0 = 0; m0 < n_mat && ok(); m0 += group) {
      const int nm = std::min(group, n_mat - m0);
      const size_t n_blocks = per * nm / 32;
      if (host) {
        int slot;
        const float *src = stage_in(host + per * m0, per * nm, &slot);
        if (!ok()) break;
        check(run_requant_mxfp4(src, n_blocks, q_blocks, q_scales, q_not_exact, e->stream));
        release(slot);
      } else {
        // scale exponents -13..-5: weights of the order of 0.02, as the bf16 synthetic weights
        check(run_synth_mxfp4(q_blocks, q_scales, n_blocks, seed + 7919ull * (uint64_t)m0, -5, e->stream));
      }
      if (!ok()) break;
      check(gptoss_pack_mxfp4(q_blocks, q_scales, dst + mat_bytes * m0, nm, n_out, n_in, pack_flags, e->stream));
    }
    return reinterpret_cast<bf16_t *>(dst);
  }
};

// cos/sin tables with the float arithmetic of run.cpp:404-478 (ntk_beta 32, ntk_alpha 1)
void rope_tables(const gptoss_config &c, int n_pos, std::vector<float> &cs, std::vector<float> &sn) {
  const int d_half = c.head_dim / 2;
  std::vector<float> inv_freq(d_half);
  const float base = c.rope_theta, scaling_factor = c.rope_scaling_factor;
  const float initial_context_length = (float)c.initial_context_length;
  const float ntk_beta = 32.0f, ntk_alpha = 1.0f;
  float concentration;
  std::vector<float> freq(d_half);
  for (int i = 0; i < d_half; i++) freq[i] = powf(base, ((float)(2 * i)) / (float)c.head_dim);
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
      inv_freq[i] = interpolation * (1.0f - mask) + extrapolation * mask;
    }
  } else {
    concentration = 1.0f;
    for (int i = 0; i < d_half; i++) inv_freq[i] = 1.0f / freq[i];
  }
  cs.resize((size_t)n_pos * d_half);
  sn.resize((size_t)n_pos * d_half);
  for (int pos = 0; pos < n_pos; pos++)
    for (int j = 0; j < d_half; j++) {
      float val = (float)pos * inv_freq[j];
      cs[(size_t)pos * d_half + j] = cosf(val) * concentration;
      sn[(size_t)pos * d_half + j] = sinf(val) * concentration;
    }
}

// most rows (sequences x positions) one prompt-processing pass works on
constexpr long long PREFILL_ROWS = 8192;

void destroy(gptoss_engine *e) {
  if (!e) return;
  for (void *p : e->allocs) (void)hipFree(p);
  if (e->h_tokens) (void)hipHostFree(e->h_tokens);
  if (e->h_next) (void)hipHostFree(e->h_next);
  if (e->pf.h_rows) (void)hipHostFree(e->pf.h_rows);
  if (e->h_lens) (void)hipHostFree(e->h_lens);
  if (e->stream) (void)hipStreamDestroy(e->stream);
  delete e;
}

}  // namespace

// ---- fp32-faithful mode ------------------------------------------------------------------------
static int create_precise(gptoss_engine *e, Builder &b, const float *host_weights) {
  const gptoss_config &c = e->cfg;
  const size_t H = c.hidden_dim, V = c.vocab_size, L = c.n_layers, E = c.n_experts, k = c.experts_per_token;
  const size_t D = c.head_dim, nq = c.n_attn_heads, nkv = c.n_kv_heads, I = c.intermediate_dim;
  const size_t qkv_dim = (nq + 2 * nkv) * D, B = e->max_batch, S = e->max_seq;
  gptoss_engine::Precise &pr = e->pr;
  // tensor order of the .bin payload (reference run.cpp:194-233)
  size_t off = 0;
  auto take = [&](size_t n) {
    size_t o = off;
    off += n;
    return o;
  };
  pr.emb = take(V * H);
  pr.unemb = take(V * H);
  pr.attn_norm = take(L * H);
  pr.mlp_norm = take(L * H);
  pr.fin = take(H);
  pr.w_qkv = take(L * qkv_dim * H);
  pr.b_qkv = take(L * qkv_dim);
  pr.w_o = take(L * H * nq * D);
  pr.b_o = take(L * H);
  pr.sinks = take(L * nq);
  pr.w_router = take(L * E * H);
  pr.b_router = take(L * E);
  pr.w1 = take(L * E * 2 * I * H);
  pr.b1 = take(L * E * 2 * I);
  pr.w2 = take(L * E * H * I);
  pr.b2 = take(L * E * H);
  pr.payload = b.alloc<float>(off);
  if (b.ok()) b.hip(hipMemcpy(pr.payload, host_weights, off * sizeof(float), hipMemcpyHostToDevice), "H2D");
  const size_t kv_dim = nkv * D;
  pr.kc = b.alloc<float>(L * B * S * kv_dim);
  pr.vc = b.alloc<float>(L * B * S * kv_dim);
  std::vector<float> cs, sn;
  rope_tables(c, (int)S, cs, sn);
  e->cos_t = b.alloc<float>(cs.size());
  e->sin_t = b.alloc<float>(sn.size());
  if (b.ok()) {
    b.hip(hipMemcpy(e->cos_t, cs.data(), cs.size() * 4, hipMemcpyHostToDevice), "H2D");
    b.hip(hipMemcpy(e->sin_t, sn.data(), sn.size() * 4, hipMemcpyHostToDevice), "H2D");
  }
  e->d_tokens = b.alloc<int>(B);
  e->d_next = b.alloc<int>(B);
  e->d_lens = nullptr;
  e->x = b.alloc<float>(B * H);
  e->t = b.alloc<bf16_t>(B * H);  // written by the norm kernel, unused
  pr.t = b.alloc<float>(B * H);
  e->qkv = b.alloc<float>(B * qkv_dim);
  e->q = b.alloc<float>(B * nq * D);
  pr.attn = b.alloc<float>(B * nq * D);
  pr.att = b.alloc<float>(B * nq * (S + 2));
  e->tb2 = b.alloc<float>(B * H);
  pr.router = b.alloc<float>(B * E);
  pr.topk_w = b.alloc<float>(B * k);
  pr.topk_i = b.alloc<int>(B * k);
  pr.mlp1 = b.alloc<float>(B * k * 2 * I);
  pr.act = b.alloc<float>(B * k * I);
  pr.mlp2 = b.alloc<float>(B * k * H);
  e->logits = b.alloc<float>(B * V);
  if (b.ok()) b.hip(hipStreamSynchronize(e->stream), "sync");
  return b.rc;
}

// one lock-step position with the arithmetic of the reference CPU forward (run.cpp:501-717)
static int precise_step(gptoss_engine *e, int pos, int B) {
  const gptoss_config &c = e->cfg;
  const int H = c.hidden_dim, V = c.vocab_size, L = c.n_layers, E = c.n_experts, k = c.experts_per_token;
  const int D = c.head_dim, nq = c.n_attn_heads, nkv = c.n_kv_heads, I = c.intermediate_dim;
  const int qkv_dim = (nq + 2 * nkv) * D, S = e->max_seq;
  const size_t kv_dim = (size_t)nkv * D;
  hipStream_t s = e->stream;
  const gptoss_engine::Precise &pr = e->pr;
  const float *W = pr.payload;
  int rc;
#define STEP(call)                   \
  do {                               \
    rc = (call);                     \
    if (rc != GPTOSS_OK) return rc;  \
  } while (0)
  STEP(precise_embedding(W + pr.emb, e->d_tokens, e->x, B, H, V, s));
  for (int l = 0; l < L; l++) {
    STEP(run_rmsnorm(e->x, nullptr, W + pr.attn_norm + (size_t)l * H, e->t, pr.t, B, H, s));
    STEP(precise_matmul(e->qkv, pr.t, W + pr.w_qkv + (size_t)l * qkv_dim * H, W + pr.b_qkv + (size_t)l * qkv_dim,
                        nullptr, B, H, qkv_dim, 1, s));
    float *kc = pr.kc + (size_t)l * e->max_batch * S * kv_dim, *vc = pr.vc + (size_t)l * e->max_batch * S * kv_dim;
    STEP(precise_rope_store(e->qkv, e->q, kc, vc, e->cos_t, e->sin_t, B, nq, nkv, D, S, pos, s));
    const int window = (c.sliding_window > 0 && l % 2 == 0) ? c.sliding_window : 0;
    STEP(precise_attn(e->q, kc, vc, W + pr.sinks + (size_t)l * nq, pr.att, pr.attn, B, nq, nkv, D, S, pos,
                      window, s));
    STEP(precise_matmul(e->tb2, pr.attn, W + pr.w_o + (size_t)l * H * nq * D, W + pr.b_o + (size_t)l * H, nullptr,
                        B, nq * D, H, 1, s));
    STEP(precise_add(e->x, e->tb2, (size_t)B * H, s));
    STEP(run_rmsnorm(e->x, nullptr, W + pr.mlp_norm + (size_t)l * H, e->t, pr.t, B, H, s));
    STEP(precise_matmul(pr.router, pr.t, W + pr.w_router + (size_t)l * E * H, W + pr.b_router + (size_t)l * E,
                        nullptr, B, H, E, 1, s));
    STEP(run_topk_softmax(pr.router, B, E, k, pr.topk_w, pr.topk_i, s));
    // one row per (token, slot): the slot's expert selects the matrix
    STEP(precise_matmul(pr.mlp1, pr.t, W + pr.w1 + (size_t)l * E * 2 * I * H, W + pr.b1 + (size_t)l * E * 2 * I,
                        pr.topk_i, B * k, H, 2 * I, k, s));
    STEP(precise_swiglu(pr.mlp1, pr.act, B * k, I, c.swiglu_limit, s));
    STEP(precise_matmul(pr.mlp2, pr.act, W + pr.w2 + (size_t)l * E * H * I, W + pr.b2 + (size_t)l * E * H,
                        pr.topk_i, B * k, I, H, 1, s));
    STEP(precise_moe_agg(pr.mlp2, pr.topk_w, pr.topk_i, e->x, B, H, k, s));
  }
  STEP(run_rmsnorm(e->x, nullptr, W + pr.fin, e->t, pr.t, B, H, s));
  STEP(precise_matmul(e->logits, pr.t, W + pr.unemb, nullptr, nullptr, B, H, V, 1, s));
#undef STEP
  return GPTOSS_OK;
}

extern "C" int gptoss_engine_create(const gptoss_config *cfg, const float *host_weights, int max_batch,
                                    int max_seq, int flags, uint64_t seed, gptoss_engine **out) {
  GPTOSS_REQUIRE(cfg && out, GPTOSS_ERR_NULL, "engine_create: null pointer");
  *out = nullptr;
  const bool synthetic = (flags & GPTOSS_ENGINE_SYNTHETIC) != 0;
  GPTOSS_REQUIRE(synthetic || host_weights, GPTOSS_ERR_NULL, "engine_create: host_weights is NULL");
  const bool precise = (flags & GPTOSS_ENGINE_PRECISE) != 0;
  GPTOSS_REQUIRE(!(precise && (flags & GPTOSS_ENGINE_MXFP4_EXPERTS)), GPTOSS_ERR_STATE,
                 "engine_create: GPTOSS_ENGINE_PRECISE keeps fp32 weights (not GPTOSS_ENGINE_MXFP4_EXPERTS)");
  GPTOSS_REQUIRE(!(precise && synthetic), GPTOSS_ERR_STATE,
                 "engine_create: GPTOSS_ENGINE_PRECISE needs host weights (not GPTOSS_ENGINE_SYNTHETIC)");
  const gptoss_config &c = *cfg;
  const int H = c.hidden_dim, V = c.vocab_size, L = c.n_layers, E = c.n_experts, k = c.experts_per_token;
  const int D = c.head_dim, nq = c.n_attn_heads, nkv = c.n_kv_heads, I = c.intermediate_dim;
  GPTOSS_REQUIRE(H > 0 && V > 0 && L > 0 && E > 0 && k > 0 && D > 0 && nq > 0 && nkv > 0 && I > 0,
                 GPTOSS_ERR_DIM, "engine_create: non-positive model dimension");
  const int qkv_dim = (nq + 2 * nkv) * D;
  GPTOSS_REQUIRE(H % 64 == 0 && I % 64 == 0 && qkv_dim % 64 == 0 && (nq * D) % 64 == 0 && V % 64 == 0,
                 GPTOSS_ERR_DIM,
                 "engine_create: hidden, intermediate, (n_q+2n_kv)*head_dim, n_q*head_dim and vocab must be "
                 "multiples of 64 (H=%d I=%d qkv=%d V=%d)", H, I, qkv_dim, V);
  GPTOSS_REQUIRE((D == 32 || D == 64) && nq % nkv == 0 && nq / nkv <= 16, GPTOSS_ERR_DIM,
                 "engine_create: head_dim must be 32 or 64 and n_q/n_kv <= 16");
  GPTOSS_REQUIRE(E <= 256 && k <= 8 && k <= E, GPTOSS_ERR_DIM, "engine_create: need E <= 256, k <= min(8,E)");
  GPTOSS_REQUIRE(max_batch >= 1 && max_seq >= 1 && max_seq <= c.seq_len, GPTOSS_ERR_DIM,
                 "engine_create: need max_batch >= 1 and 1 <= max_seq <= seq_len (%d)", c.seq_len);
  GPTOSS_REQUIRE(c.sliding_window >= 0, GPTOSS_ERR_DIM, "engine_create: negative sliding window");
  // the GEMM kernels address their operands and results with 32-bit element offsets
  {
    const long long widest = std::max<long long>({qkv_dim, H, 2ll * I, (flags & (GPTOSS_ENGINE_LOGITS | GPTOSS_ENGINE_PRECISE)) ? V : 0});
    GPTOSS_REQUIRE((long long)max_batch * widest < (1ll << 32), GPTOSS_ERR_DIM,
                   "engine_create: max_batch x the widest activation row (%lld elements%s) must stay below 2^32 "
                   "(max_batch=%d)", widest, widest == V ? ", the logits of GPTOSS_ENGINE_LOGITS" : "", max_batch);
  }

  gptoss_engine *e = new gptoss_engine();
  e->cfg = c;
  e->max_batch = max_batch;
  e->max_seq = max_seq;
  e->flags = flags;
  e->device_bytes = 0;
  e->h_tokens = e->h_next = e->h_lens = nullptr;
  e->stream = nullptr;
  e->pf.rows = 0;
  e->pf.h_rows = nullptr;
  Builder b;
  b.e = e;
  b.hip(hipStreamCreate(&e->stream), "hipStreamCreate");
  b.hip(hipHostMalloc((void **)&e->h_tokens, sizeof(int) * max_batch, hipHostMallocDefault), "hipHostMalloc");
  b.hip(hipHostMalloc((void **)&e->h_next, sizeof(int) * max_batch, hipHostMallocDefault), "hipHostMalloc");
  b.hip(hipHostMalloc((void **)&e->h_lens, sizeof(int) * max_batch, hipHostMallocDefault), "hipHostMalloc");
  if (precise) {
    int rc = create_precise(e, b, host_weights);
    if (rc != GPTOSS_OK) {
      destroy(e);
      return rc;
    }
    *out = e;
    return GPTOSS_OK;
  }

  // staging: large enough for one expert's gate/up matrix, one qkv matrix and a slice of the
  // (un)embedding table
  size_t biggest = std::max({(size_t)2 * I * H, (size_t)qkv_dim * H, (size_t)H * nq * D, (size_t)E * H});
  b.stage_elems = std::max<size_t>(biggest, (size_t)32 << 20);
  if (!synthetic) b.stager_create(b.stage_elems);
  else b.hip(hipMalloc((void **)&b.stage_bf16, b.stage_elems * sizeof(bf16_t)), "staging hipMalloc");
  const bool mxfp4 = (flags & GPTOSS_ENGINE_MXFP4_EXPERTS) != 0;
  if (mxfp4) {
    b.hip(hipMalloc((void **)&b.q_blocks, b.stage_elems / 2), "staging hipMalloc");
    b.hip(hipMalloc((void **)&b.q_scales, b.stage_elems / 32), "staging hipMalloc");
    b.hip(hipMalloc((void **)&b.q_not_exact, sizeof(int)), "staging hipMalloc");
    if (b.ok()) b.hip(hipMemsetAsync(b.q_not_exact, 0, sizeof(int), e->stream), "memset");
  }

  // walk the .bin payload in file order (reference run.cpp:194-233)
  const float *p = host_weights;
  auto take = [&](size_t n) -> const float * {
    if (synthetic) return nullptr;
    const float *r = p;
    p += n;
    return r;
  };
  uint64_t sd = seed * 1000003ull + 17;
  auto next_seed = [&]() { return sd += 0x9E3779B97F4A7C15ull; };
  const float STD = 0.02f;

  // embedding rows are gathered, not multiplied: row-major bf16.  Upload in row slices.
  {
    const float *emb = take((size_t)V * H);
    const float *unemb = take((size_t)V * H);
    int rows_per = (int)std::max<size_t>(64, (b.stage_elems / H) / 64 * 64);
    e->embedding = b.alloc<bf16_t>((size_t)V * H);
    e->unembedding = b.alloc<bf16_t>((size_t)V * H);
    for (int pass = 0; pass < 2 && b.ok(); pass++) {
      const float *src = pass == 0 ? emb : unemb;
      bf16_t *dst = pass == 0 ? e->embedding : e->unembedding;
      for (int r0 = 0; r0 < V && b.ok(); r0 += rows_per) {
        int nr = std::min(rows_per, V - r0);
        size_t n = (size_t)nr * H;
        if (src) {
          int slot;
          const float *sp = b.stage_in(src + (size_t)r0 * H, n, &slot);
          if (!b.ok()) break;
          // fragment order is blocked by 32 output rows, so a slice of rows packs independently
          if (pass == 0) b.check(run_f32_to_bf16(sp, dst + (size_t)r0 * H, n, e->stream));
          else b.check(gptoss_pack_weight(sp, dst + (size_t)r0 * H, 1, nr, H, GPTOSS_PACK_SRC_FP32, e->stream));
          b.release(slot);
        } else {
          b.check(run_synth_bf16(b.stage_bf16, n, next_seed(), 0.f, STD, e->stream));
          if (!b.ok()) break;
          if (pass == 0) b.hip(hipMemcpyAsync(dst + (size_t)r0 * H, b.stage_bf16, n * sizeof(bf16_t), hipMemcpyDeviceToDevice, e->stream), "D2D");
          else b.check(gptoss_pack_weight(b.stage_bf16, dst + (size_t)r0 * H, 1, nr, H, 0, e->stream));
        }
      }
    }
  }
  const float *attn_norm = take((size_t)L * H), *mlp_norm = take((size_t)L * H), *fin = take(H);
  const float *w_qkv = take((size_t)L * qkv_dim * H), *b_qkv = take((size_t)L * qkv_dim);
  const float *w_o = take((size_t)L * H * nq * D), *b_o = take((size_t)L * H);
  const float *sinks = take((size_t)L * nq);
  const float *w_router = take((size_t)L * E * H), *b_router = take((size_t)L * E);
  const float *w1 = take((size_t)L * E * 2 * I * H), *b1 = take((size_t)L * E * 2 * I);
  const float *w2 = take((size_t)L * E * H * I), *b2 = take((size_t)L * E * H);
  auto at = [&](const float *base, size_t per, int l) -> const float * { return base ? base + per * l : nullptr; };

  e->final_norm = b.upload_f32(fin, H, next_seed(), 1.f, STD);
  e->layers.resize(L);
  const int W = c.sliding_window;
  const int cap_full = (int)align_up((size_t)max_seq, 64);
  for (int l = 0; l < L && b.ok(); l++) {
    LayerWeights &w = e->layers[l];
    w.attn_norm = b.upload_f32(at(attn_norm, H, l), H, next_seed(), 1.f, STD);
    w.mlp_norm = b.upload_f32(at(mlp_norm, H, l), H, next_seed(), 1.f, STD);
    w.w_qkv = b.upload_matrices(at(w_qkv, (size_t)qkv_dim * H, l), 1, qkv_dim, H, true, 0, next_seed(), STD);
    w.b_qkv = b.upload_f32(at(b_qkv, qkv_dim, l), qkv_dim, next_seed(), 0.f, STD);
    w.w_o = b.upload_matrices(at(w_o, (size_t)H * nq * D, l), 1, H, nq * D, true, 0, next_seed(), STD);
    w.b_o = b.upload_f32(at(b_o, H, l), H, next_seed(), 0.f, STD);
    w.sinks = b.upload_f32(at(sinks, nq, l), nq, next_seed(), 0.f, STD);
    w.w_router = b.upload_matrices(at(w_router, (size_t)E * H, l), 1, E, H, false, 0, next_seed(), STD);
    w.b_router = b.upload_f32(at(b_router, E, l), E, next_seed(), 0.f, STD);
    w.w1 = mxfp4 ? b.upload_matrices_mxfp4(at(w1, (size_t)E * 2 * I * H, l), E, 2 * I, H, GPTOSS_PACK_GLU, next_seed())
                 : b.upload_matrices(at(w1, (size_t)E * 2 * I * H, l), E, 2 * I, H, true, GPTOSS_PACK_GLU, next_seed(), STD);
    w.b1 = b.upload_f32(at(b1, (size_t)E * 2 * I, l), (size_t)E * 2 * I, next_seed(), 0.f, STD);
    w.w2 = mxfp4 ? b.upload_matrices_mxfp4(at(w2, (size_t)E * H * I, l), E, H, I, 0, next_seed())
                 : b.upload_matrices(at(w2, (size_t)E * H * I, l), E, H, I, true, 0, next_seed(), STD);
    w.b2 = b.upload_f32(at(b2, (size_t)E * H, l), (size_t)E * H, next_seed(), 0.f, STD);
    // even layers keep only the sliding window (ring buffer), odd layers the whole context
    // (reference run.cpp:582, getp-csrc/src/alloc.cpp:245-250)
    const bool windowed = W > 0 && (l % 2 == 0);
    w.window = windowed ? W : 0;
    w.cache_cap = windowed ? std::min(cap_full, (int)align_up((size_t)W, 64)) : cap_full;
    size_t cache_elems = (size_t)max_batch * nkv * kv_plane_elems(w.cache_cap, D);
    w.kv_cache = b.alloc<bf16_t>(cache_elems);
    if (b.ok()) b.hip(hipMemsetAsync(w.kv_cache, 0, cache_elems * sizeof(bf16_t), e->stream), "memset");
  }
  if (mxfp4 && b.ok()) {
    int not_exact = 0;
    b.hip(hipMemcpy(&not_exact, b.q_not_exact, sizeof(int), hipMemcpyDeviceToHost), "D2H");
    if (b.ok() && not_exact)
      b.rc = fail(GPTOSS_ERR_STATE, "engine_create: GPTOSS_ENGINE_MXFP4_EXPERTS needs expert weights that are exactly "
                                    "representable in MXFP4 (e2m1 codes, one power-of-two scale per 32 inputs)");
  }
  // the staging buffers are freed below: everything that reads them must have finished
  b.hip(hipStreamSynchronize(e->stream), "sync");
  b.stager_destroy();
  if (b.stage_bf16) (void)hipFree(b.stage_bf16);
  if (b.q_blocks) (void)hipFree(b.q_blocks);
  if (b.q_scales) (void)hipFree(b.q_scales);
  if (b.q_not_exact) (void)hipFree(b.q_not_exact);

  // rotary tables
  {
    std::vector<float> cs, sn;
    rope_tables(c, max_seq, cs, sn);
    e->cos_t = b.alloc<float>(cs.size());
    e->sin_t = b.alloc<float>(sn.size());
    if (b.ok()) {
      b.hip(hipMemcpy(e->cos_t, cs.data(), cs.size() * 4, hipMemcpyHostToDevice), "H2D");
      b.hip(hipMemcpy(e->sin_t, sn.data(), sn.size() * 4, hipMemcpyHostToDevice), "H2D");
    }
  }
  // run state
  const int B = max_batch;
  e->d_tokens = b.alloc<int>(B);
  e->d_next = b.alloc<int>(B);
  e->d_lens = b.alloc<int>(B);
  e->x = b.alloc<float>((size_t)B * H);
  e->t = b.alloc<bf16_t>((size_t)B * H);
  e->qkv = b.alloc<float>((size_t)B * qkv_dim);
  e->q = b.alloc<float>((size_t)B * nq * D);
  e->attn_out = b.alloc<bf16_t>((size_t)B * nq * D);
  e->tb2 = b.alloc<float>((size_t)B * H);
  e->logits = nullptr;
  e->amax_val = nullptr;
  e->amax_idx = nullptr;
  if (flags & GPTOSS_ENGINE_LOGITS) {
    e->logits = b.alloc<float>((size_t)B * V);
  } else {
    e->amax_val = b.alloc<float>((size_t)B * gemm_argmax_tiles(V));
    e->amax_idx = b.alloc<int>((size_t)B * gemm_argmax_tiles(V));
  }
  e->moe_ws_bytes = gptoss_moe_workspace_bytes(B, E, k, H, I);
  e->moe_ws = b.alloc<unsigned char>(e->moe_ws_bytes);
  e->attn_ws_bytes = std::max<size_t>(256, gptoss_attn_workspace_bytes(B, nq, nkv, D, max_seq));
  e->attn_ws = b.alloc<unsigned char>(e->attn_ws_bytes);
  if (!(flags & GPTOSS_ENGINE_NO_PREFILL)) {
    gptoss_engine::Prefill &pf = e->pf;
    const int R = (int)std::min<long long>((long long)max_batch * max_seq, PREFILL_ROWS);
    pf.tokens = b.alloc<int>((size_t)3 * R + max_batch);
    pf.seq_map = pf.tokens + R;
    pf.lens = pf.seq_map + R;
    pf.sample = pf.lens + R;
    b.hip(hipHostMalloc((void **)&pf.h_rows, sizeof(int) * ((size_t)3 * R + max_batch), hipHostMallocDefault),
          "hipHostMalloc");
    pf.x = b.alloc<float>((size_t)R * H);
    pf.t = b.alloc<bf16_t>((size_t)R * H);
    pf.qkv = b.alloc<float>((size_t)R * qkv_dim);
    pf.q = b.alloc<float>((size_t)R * nq * D);
    pf.attn_out = b.alloc<bf16_t>((size_t)R * nq * D);
    pf.tb2 = b.alloc<float>((size_t)R * H);
    pf.moe_ws_bytes = gptoss_moe_workspace_bytes(R, E, k, H, I);
    pf.moe_ws = b.alloc<unsigned char>(pf.moe_ws_bytes);
    // rows of one launch: B sequences x T positions with B*T <= R and T <= max_seq
    pf.attn_ws_bytes = gptoss_attn_prefill_workspace_bytes(1, R, nq, nkv, D, std::min(R, max_seq));
    pf.attn_ws = b.alloc<unsigned char>(pf.attn_ws_bytes);
    pf.kv_scratch = nullptr;
    pf.scratch_tokens = 0;
    if (W > 0 && max_seq > (int)align_up((size_t)W, 64)) {
      pf.scratch_tokens = (size_t)R + (size_t)64 * max_batch;
      pf.kv_scratch = b.alloc<bf16_t>(pf.scratch_tokens * nkv * D * 2);
      // slots past a prompt's end are masked, but must hold finite values
      if (b.ok()) {
        b.hip(hipMemsetAsync(pf.kv_scratch, 0, pf.scratch_tokens * nkv * D * 2 * sizeof(bf16_t), e->stream), "memset");
      }
    }
    if (b.ok()) pf.rows = R;
  }
  if (b.ok()) b.hip(hipStreamSynchronize(e->stream), "sync");
  if (!b.ok()) {
    destroy(e);
    return b.rc;
  }
  *out = e;
  return GPTOSS_OK;
}

extern "C" void gptoss_engine_destroy(gptoss_engine *e) { destroy(e); }

// One decode step.  host_pos == nullptr: every sequence is at position pos (lock step); else
// sequence i is at its own position host_pos[i] and pos is their maximum.
static int step_impl(gptoss_engine *e, const int *host_tokens, int pos, const int *host_pos, int B,
                     int *host_next) {
  const gptoss_config &c = e->cfg;
  const int H = c.hidden_dim, V = c.vocab_size, L = c.n_layers, E = c.n_experts, k = c.experts_per_token;
  const int D = c.head_dim, nq = c.n_attn_heads, nkv = c.n_kv_heads, I = c.intermediate_dim;
  const int qkv_dim = (nq + 2 * nkv) * D;
  hipStream_t s = e->stream;
  int rc;
#define STEP(call)                   \
  do {                               \
    rc = (call);                     \
    if (rc != GPTOSS_OK) return rc;  \
  } while (0)

  memcpy(e->h_tokens, host_tokens, sizeof(int) * B);
  GPTOSS_HIP(hipMemcpyAsync(e->d_tokens, e->h_tokens, sizeof(int) * B, hipMemcpyHostToDevice, s));
  if (e->flags & GPTOSS_ENGINE_PRECISE) {
    STEP(precise_step(e, pos, B));
    STEP(run_argmax(e->logits, e->d_next, B, V, s));
    GPTOSS_HIP(hipMemcpyAsync(e->h_next, e->d_next, sizeof(int) * B, hipMemcpyDeviceToHost, s));
    GPTOSS_HIP(hipStreamSynchronize(s));
    memcpy(host_next, e->h_next, sizeof(int) * B);
    return GPTOSS_OK;
  }
  if (host_pos) {
    for (int i = 0; i < B; i++) e->h_lens[i] = host_pos[i] + 1;
    GPTOSS_HIP(hipMemcpyAsync(e->d_lens, e->h_lens, sizeof(int) * B, hipMemcpyHostToDevice, s));
  }
  STEP(run_embedding(e->embedding, e->d_tokens, e->x, B, H, V, s));
  for (int l = 0; l < L; l++) {
    const LayerWeights &w = e->layers[l];
    if (l == 0) STEP(run_rmsnorm(e->x, nullptr, w.attn_norm, e->t, nullptr, B, H, s));
    STEP(dense_gemm(e->t, w.w_qkv, w.b_qkv, e->qkv, EPI_F32, B, qkv_dim, H, s));
    if (host_pos)
      STEP(run_rope_store_lens(e->qkv, e->q, w.kv_cache, e->cos_t, e->sin_t, B, nq, nkv, D,
                               w.cache_cap, e->d_lens, s));
    else
      STEP(run_rope_store(e->qkv, e->q, w.kv_cache, e->cos_t, e->sin_t, B, nq, nkv, D,
                          w.cache_cap, pos, s));
    // lock step: every sequence has pos + 1 positions, which the call takes from max_len
    STEP(gptoss_attn_decode(e->q, w.kv_cache, host_pos ? e->d_lens : nullptr, w.sinks, e->attn_out, B, nq, nkv, D,
                            w.cache_cap, w.window, pos + 1, e->attn_ws, e->attn_ws_bytes, s));
    STEP(dense_gemm(e->attn_out, w.w_o, w.b_o, e->tb2, EPI_F32, B, H, nq * D, s));
    // x += attention branch, then the ffn norm (model.cpp:66)
    const MoePreNorm pre{e->x, e->tb2, w.mlp_norm};   // runs inside the block's router kernel
    gptoss_moe_weights mw;
    mw.n_experts = E;
    mw.top_k = k;
    mw.hidden = H;
    mw.intermediate = I;
    mw.swiglu_limit = c.swiglu_limit;
    mw.w_router = w.w_router;
    mw.b_router = w.b_router;
    mw.w1 = w.w1;
    mw.b1 = w.b1;
    mw.w2 = w.w2;
    mw.b2 = w.b2;
    // x += MoE branch (the combine kernel adds into the residual stream, model.cpp:121-131), and
    // the next layer's attention norm (or the final norm) of the updated rows in the same kernel
    const float *nw = (l + 1 < L) ? e->layers[l + 1].attn_norm : e->final_norm;
    const int q4 = (e->flags & GPTOSS_ENGINE_MXFP4_EXPERTS) ? 1 : 0;
    const bool fused = combine_norm_applies(H, nw, e->t);
    STEP(moe_forward_norm(&mw, e->t, B, e->x, e->moe_ws, e->moe_ws_bytes, s, q4, fused ? nw : nullptr,
                          fused ? e->t : nullptr, &pre));
    if (!fused) STEP(run_rmsnorm(e->x, nullptr, nw, e->t, nullptr, B, H, s));
  }
  if (e->logits) {
    STEP(dense_gemm(e->t, e->unembedding, nullptr, e->logits, EPI_F32, B, V, H, s));
    STEP(run_argmax(e->logits, e->d_next, B, V, s));
  } else {
    // the classifier keeps only (max, column) per row and column tile; a small second stage picks
    // the row's arg-max (lowest column among equal maxima, run.cpp:739-750)
    int pairs = 0;
    STEP(dense_gemm(e->t, e->unembedding, nullptr, nullptr, EPI_ARGMAX, B, V, H, s, e->amax_val, e->amax_idx, &pairs));
    STEP(run_argmax_tiles(e->amax_val, e->amax_idx, e->d_next, B, pairs, s));
  }
  GPTOSS_HIP(hipMemcpyAsync(e->h_next, e->d_next, sizeof(int) * B, hipMemcpyDeviceToHost, s));
  GPTOSS_HIP(hipStreamSynchronize(s));
  memcpy(host_next, e->h_next, sizeof(int) * B);
#undef STEP
  return GPTOSS_OK;
}

extern "C" int gptoss_engine_step(gptoss_engine *e, const int *host_tokens, int pos, int B, int *host_next) {
  GPTOSS_REQUIRE(e && host_tokens && host_next, GPTOSS_ERR_NULL, "engine_step: null pointer");
  GPTOSS_REQUIRE(B >= 1 && B <= e->max_batch, GPTOSS_ERR_DIM, "engine_step: batch %d outside 1..%d", B, e->max_batch);
  GPTOSS_REQUIRE(pos >= 0 && pos < e->max_seq, GPTOSS_ERR_STATE, "engine_step: position %d outside 0..%d", pos, e->max_seq - 1);
  return step_impl(e, host_tokens, pos, nullptr, B, host_next);
}

extern "C" int gptoss_engine_step_ragged(gptoss_engine *e, const int *host_tokens, const int *host_pos, int B,
                                         int *host_next) {
  GPTOSS_REQUIRE(e && host_tokens && host_pos && host_next, GPTOSS_ERR_NULL, "engine_step_ragged: null pointer");
  GPTOSS_REQUIRE(B >= 1 && B <= e->max_batch, GPTOSS_ERR_DIM, "engine_step_ragged: batch %d outside 1..%d", B,
                 e->max_batch);
  GPTOSS_REQUIRE(!(e->flags & GPTOSS_ENGINE_PRECISE), GPTOSS_ERR_STATE,
                 "engine_step_ragged: not available with GPTOSS_ENGINE_PRECISE");
  int max_pos = 0;
  for (int i = 0; i < B; i++) {
    GPTOSS_REQUIRE(host_pos[i] >= 0 && host_pos[i] < e->max_seq, GPTOSS_ERR_STATE,
                   "engine_step_ragged: sequence %d at position %d outside 0..%d", i, host_pos[i], e->max_seq - 1);
    max_pos = std::max(max_pos, host_pos[i]);
  }
  return step_impl(e, host_tokens, max_pos, host_pos, B, host_next);
}

// Positions 0..T-1 of sequences seq0..seq0+Bc-1 in one pass (Bc*T <= pf.rows): same kernels and the
// same per-row arithmetic as T lock-step steps, so the caches and the arg-max after the last
// position are those the lock-step loop would have produced (bit for bit as long as no sliding
// window ring has wrapped; after that the window layers sum their scores in another order).
static int prefill_chunk(gptoss_engine *e, const int *host_tokens, int seq0, int Bc, int T) {
  const gptoss_config &c = e->cfg;
  const int H = c.hidden_dim, V = c.vocab_size, L = c.n_layers, E = c.n_experts, k = c.experts_per_token;
  const int D = c.head_dim, nq = c.n_attn_heads, nkv = c.n_kv_heads, I = c.intermediate_dim;
  const int qkv_dim = (nq + 2 * nkv) * D;
  const int rows = Bc * T;
  gptoss_engine::Prefill &pf = e->pf;
  hipStream_t s = e->stream;
  int rc;
#define STEP(call)                   \
  do {                               \
    rc = (call);                     \
    if (rc != GPTOSS_OK) return rc;  \
  } while (0)
  GPTOSS_HIP(hipMemcpyAsync(pf.tokens, host_tokens, sizeof(int) * rows, hipMemcpyHostToDevice, s));
  STEP(run_embedding(e->embedding, pf.tokens, pf.x, rows, H, V, s));
  for (int l = 0; l < L; l++) {
    const LayerWeights &w = e->layers[l];
    if (l == 0) STEP(run_rmsnorm(pf.x, nullptr, w.attn_norm, pf.t, nullptr, rows, H, s));
    STEP(dense_gemm(pf.t, w.w_qkv, w.b_qkv, pf.qkv, EPI_F32, rows, qkv_dim, H, s));
    bf16_t *kv = w.kv_cache + (size_t)nkv * kv_plane_elems(w.cache_cap, D) * seq0;
    if (T > w.cache_cap) {
      // a sliding-window ring shorter than the prompt: attention reads a linear copy of the
      // prompt's K/V, the ring receives the positions it would hold after T lock-step steps
      const int cap_t = (int)align_up((size_t)T, 64);
      STEP(run_rope_store_rows(pf.qkv, pf.q, pf.kv_scratch, e->cos_t, e->sin_t, rows, T, nq, nkv, D,
                               cap_t, 0, 0, s));
      STEP(run_rope_store_rows(pf.qkv, nullptr, kv, e->cos_t, e->sin_t, rows, T, nq, nkv, D, w.cache_cap, 0,
                               T - w.cache_cap, s));
      STEP(gptoss_attn_prefill(pf.q, pf.kv_scratch, w.sinks, pf.attn_out, Bc, T, 0, nq, nkv, D, cap_t,
                               w.window, pf.attn_ws, pf.attn_ws_bytes, s));
    } else {
      STEP(run_rope_store_rows(pf.qkv, pf.q, kv, e->cos_t, e->sin_t, rows, T, nq, nkv, D, w.cache_cap, 0, 0, s));
      STEP(gptoss_attn_prefill(pf.q, kv, w.sinks, pf.attn_out, Bc, T, 0, nq, nkv, D, w.cache_cap, w.window,
                               pf.attn_ws, pf.attn_ws_bytes, s));
    }
    STEP(dense_gemm(pf.attn_out, w.w_o, w.b_o, pf.tb2, EPI_F32, rows, H, nq * D, s));
    const MoePreNorm pre{pf.x, pf.tb2, w.mlp_norm};   // runs inside the block's router kernel
    gptoss_moe_weights mw;
    mw.n_experts = E;
    mw.top_k = k;
    mw.hidden = H;
    mw.intermediate = I;
    mw.swiglu_limit = c.swiglu_limit;
    mw.w_router = w.w_router;
    mw.b_router = w.b_router;
    mw.w1 = w.w1;
    mw.b1 = w.b1;
    mw.w2 = w.w2;
    mw.b2 = w.b2;
    const float *nw = (l + 1 < L) ? e->layers[l + 1].attn_norm : nullptr;  // the last rows are normed below
    const int q4 = (e->flags & GPTOSS_ENGINE_MXFP4_EXPERTS) ? 1 : 0;
    const bool fused = nw && combine_norm_applies(H, nw, pf.t);
    STEP(moe_forward_norm(&mw, pf.t, rows, pf.x, pf.moe_ws, pf.moe_ws_bytes, s, q4, fused ? nw : nullptr,
                          fused ? pf.t : nullptr, &pre));
    if (nw && !fused) STEP(run_rmsnorm(pf.x, nullptr, nw, pf.t, nullptr, rows, H, s));
  }
  // only the last position of every sequence goes through the final norm and the classifier
  STEP(run_gather_rows(pf.x, e->x, Bc, H, T, T - 1, s));
  STEP(run_rmsnorm(e->x, nullptr, e->final_norm, e->t, nullptr, Bc, H, s));
  if (e->logits) {
    STEP(dense_gemm(e->t, e->unembedding, nullptr, e->logits + (size_t)seq0 * V, EPI_F32, Bc, V, H, s));
    STEP(run_argmax(e->logits + (size_t)seq0 * V, e->d_next + seq0, Bc, V, s));
  } else {
    int pairs = 0;
    STEP(dense_gemm(e->t, e->unembedding, nullptr, nullptr, EPI_ARGMAX, Bc, V, H, s, e->amax_val, e->amax_idx, &pairs));
    STEP(run_argmax_tiles(e->amax_val, e->amax_idx, e->d_next + seq0, Bc, pairs, s));
  }
#undef STEP
  return GPTOSS_OK;
}

extern "C" int gptoss_engine_prefill(gptoss_engine *e, const int *host_tokens, int B, int T, int *host_next) {
  GPTOSS_REQUIRE(e && host_tokens && host_next, GPTOSS_ERR_NULL, "engine_prefill: null pointer");
  GPTOSS_REQUIRE(!(e->flags & GPTOSS_ENGINE_PRECISE) && e->pf.rows > 0, GPTOSS_ERR_STATE,
                 "engine_prefill: not available (GPTOSS_ENGINE_PRECISE or GPTOSS_ENGINE_NO_PREFILL)");
  GPTOSS_REQUIRE(B >= 1 && B <= e->max_batch, GPTOSS_ERR_DIM, "engine_prefill: batch %d outside 1..%d", B, e->max_batch);
  GPTOSS_REQUIRE(T >= 1 && T <= e->max_seq && T <= e->pf.rows, GPTOSS_ERR_DIM,
                 "engine_prefill: %d positions outside 1..%d", T, std::min(e->max_seq, e->pf.rows));
  const int per = std::max(1, e->pf.rows / T);  // sequences per pass
  for (int s0 = 0; s0 < B; s0 += per) {
    const int bc = std::min(per, B - s0);
    int rc = prefill_chunk(e, host_tokens + (size_t)s0 * T, s0, bc, T);
    if (rc != GPTOSS_OK) return rc;
    // the token staging buffer and the activations are reused by the next pass
    GPTOSS_HIP(hipStreamSynchronize(e->stream));
  }
  GPTOSS_HIP(hipMemcpyAsync(e->h_next, e->d_next, sizeof(int) * B, hipMemcpyDeviceToHost, e->stream));
  GPTOSS_HIP(hipStreamSynchronize(e->stream));
  memcpy(host_next, e->h_next, sizeof(int) * B);
  return GPTOSS_OK;
}

// One step over n arbitrary rows: row i feeds token tok[i] at position pos[i] of the sequence in
// cache slot slot[i].  Rows of one sequence must be consecutive positions in ascending order (a
// stretch of its prompt): every row's K/V is stored before any row attends, and row i attends to
// the positions up to its own.  On the sliding-window layers that is only correct while such a
// stretch stays inside the ring's first lap (all its positions below the ring's capacity): the
// caller sees to that.  The rows share every weight pass of the step, so the prompt of a request
// that has just been admitted costs a few more rows in the GEMMs of a step that runs anyway.
// host_next[j] = arg-max after row sample[j] (n_sample <= max_batch rows).
static int step_rows(gptoss_engine *e, int n, const int *tok, const int *slot, const int *pos, int n_sample,
                     const int *sample, int *host_next) {
  const gptoss_config &c = e->cfg;
  const int H = c.hidden_dim, V = c.vocab_size, L = c.n_layers, E = c.n_experts, k = c.experts_per_token;
  const int D = c.head_dim, nq = c.n_attn_heads, nkv = c.n_kv_heads, I = c.intermediate_dim;
  const int qkv_dim = (nq + 2 * nkv) * D;
  gptoss_engine::Prefill &pf = e->pf;
  GPTOSS_REQUIRE(n >= 1 && n <= pf.rows && n_sample >= 1 && n_sample <= e->max_batch, GPTOSS_ERR_DIM,
                 "step_rows: %d rows (at most %d), %d sampled (at most %d)", n, pf.rows, n_sample, e->max_batch);
  hipStream_t s = e->stream;
  int rc;
#define STEP(call)                   \
  do {                               \
    rc = (call);                     \
    if (rc != GPTOSS_OK) return rc;  \
  } while (0)
  const size_t R = pf.rows;
  int max_len = 1;
  for (int i = 0; i < n; i++) {
    pf.h_rows[i] = tok[i];
    pf.h_rows[R + i] = slot[i];
    pf.h_rows[2 * R + i] = pos[i] + 1;
    max_len = std::max(max_len, pos[i] + 1);
  }
  for (int j = 0; j < n_sample; j++) pf.h_rows[3 * R + j] = sample[j];
  // one copy when the rows are few enough that the gaps between the four arrays do not matter
  if ((size_t)n * 8 >= R) {
    GPTOSS_HIP(hipMemcpyAsync(pf.tokens, pf.h_rows, sizeof(int) * (3 * R + n_sample), hipMemcpyHostToDevice, s));
  } else {
    GPTOSS_HIP(hipMemcpyAsync(pf.tokens, pf.h_rows, sizeof(int) * n, hipMemcpyHostToDevice, s));
    GPTOSS_HIP(hipMemcpyAsync(pf.seq_map, pf.h_rows + R, sizeof(int) * n, hipMemcpyHostToDevice, s));
    GPTOSS_HIP(hipMemcpyAsync(pf.lens, pf.h_rows + 2 * R, sizeof(int) * n, hipMemcpyHostToDevice, s));
    GPTOSS_HIP(hipMemcpyAsync(pf.sample, pf.h_rows + 3 * R, sizeof(int) * n_sample, hipMemcpyHostToDevice, s));
  }
  STEP(run_embedding(e->embedding, pf.tokens, pf.x, n, H, V, s));
  for (int l = 0; l < L; l++) {
    const LayerWeights &w = e->layers[l];
    if (l == 0) STEP(run_rmsnorm(pf.x, nullptr, w.attn_norm, pf.t, nullptr, n, H, s));
    STEP(dense_gemm(pf.t, w.w_qkv, w.b_qkv, pf.qkv, EPI_F32, n, qkv_dim, H, s));
    STEP(run_rope_store_lens(pf.qkv, pf.q, w.kv_cache, e->cos_t, e->sin_t, n, nq, nkv, D, w.cache_cap, pf.lens, s,
                             pf.seq_map));
    STEP(attn_decode_mapped(pf.q, w.kv_cache, pf.lens, w.sinks, pf.attn_out, n, nq, nkv, D, w.cache_cap, w.window,
                            max_len, pf.attn_ws, pf.attn_ws_bytes, s, pf.seq_map));
    STEP(dense_gemm(pf.attn_out, w.w_o, w.b_o, pf.tb2, EPI_F32, n, H, nq * D, s));
    const MoePreNorm pre{pf.x, pf.tb2, w.mlp_norm};   // runs inside the block's router kernel
    gptoss_moe_weights mw;
    mw.n_experts = E;
    mw.top_k = k;
    mw.hidden = H;
    mw.intermediate = I;
    mw.swiglu_limit = c.swiglu_limit;
    mw.w_router = w.w_router;
    mw.b_router = w.b_router;
    mw.w1 = w.w1;
    mw.b1 = w.b1;
    mw.w2 = w.w2;
    mw.b2 = w.b2;
    const float *nw = (l + 1 < L) ? e->layers[l + 1].attn_norm : nullptr;  // the sampled rows are normed below
    const int q4 = (e->flags & GPTOSS_ENGINE_MXFP4_EXPERTS) ? 1 : 0;
    const bool fused = nw && combine_norm_applies(H, nw, pf.t);
    STEP(moe_forward_norm(&mw, pf.t, n, pf.x, pf.moe_ws, pf.moe_ws_bytes, s, q4, fused ? nw : nullptr,
                          fused ? pf.t : nullptr, &pre));
    if (nw && !fused) STEP(run_rmsnorm(pf.x, nullptr, nw, pf.t, nullptr, n, H, s));
  }
  STEP(run_gather_rows_idx(pf.x, e->x, pf.sample, n_sample, H, s));
  STEP(run_rmsnorm(e->x, nullptr, e->final_norm, e->t, nullptr, n_sample, H, s));
  if (e->logits) {
    // the logits are kept per cache slot: one classifier row at a time
    for (int j = 0; j < n_sample; j++) {
      float *lg = e->logits + (size_t)slot[sample[j]] * V;
      STEP(dense_gemm(e->t + (size_t)j * H, e->unembedding, nullptr, lg, EPI_F32, 1, V, H, s));
      STEP(run_argmax(lg, e->d_next + j, 1, V, s));
    }
  } else {
    int pairs = 0;
    STEP(dense_gemm(e->t, e->unembedding, nullptr, nullptr, EPI_ARGMAX, n_sample, V, H, s, e->amax_val, e->amax_idx, &pairs));
    STEP(run_argmax_tiles(e->amax_val, e->amax_idx, e->d_next, n_sample, pairs, s));
  }
  GPTOSS_HIP(hipMemcpyAsync(e->h_next, e->d_next, sizeof(int) * n_sample, hipMemcpyDeviceToHost, s));
  GPTOSS_HIP(hipStreamSynchronize(s));
  memcpy(host_next, e->h_next, sizeof(int) * n_sample);
#undef STEP
  return GPTOSS_OK;
}

extern "C" int gptoss_engine_step_rows(gptoss_engine *e, int n_rows, const int *host_tokens, const int *host_slots,
                                       const int *host_pos, int n_sample, const int *host_sample, int *host_next) {
  GPTOSS_REQUIRE(e && host_tokens && host_slots && host_pos && host_sample && host_next, GPTOSS_ERR_NULL,
                 "engine_step_rows: null pointer");
  GPTOSS_REQUIRE(!(e->flags & GPTOSS_ENGINE_PRECISE) && e->pf.rows > 0, GPTOSS_ERR_STATE,
                 "engine_step_rows: not available (GPTOSS_ENGINE_PRECISE or GPTOSS_ENGINE_NO_PREFILL)");
  GPTOSS_REQUIRE(n_rows >= 1 && n_rows <= e->pf.rows && n_sample >= 1 && n_sample <= e->max_batch, GPTOSS_ERR_DIM,
                 "engine_step_rows: %d rows outside 1..%d or %d sampled rows outside 1..%d", n_rows, e->pf.rows,
                 n_sample, e->max_batch);
  int ring_cap = e->max_seq + 1;
  for (const LayerWeights &w : e->layers)
    if (w.window > 0) ring_cap = std::min(ring_cap, w.cache_cap);
  for (int i = 0; i < n_rows; i++) {
    GPTOSS_REQUIRE(host_slots[i] >= 0 && host_slots[i] < e->max_batch && host_pos[i] >= 0 && host_pos[i] < e->max_seq,
                   GPTOSS_ERR_STATE, "engine_step_rows: row %d names slot %d, position %d (slots 0..%d, positions 0..%d)",
                   i, host_slots[i], host_pos[i], e->max_batch - 1, e->max_seq - 1);
    // several rows of one sequence: consecutive, ascending, and inside the first lap of the window rings
    if (i > 0 && host_slots[i] == host_slots[i - 1])
      GPTOSS_REQUIRE(host_pos[i] == host_pos[i - 1] + 1 && host_pos[i] < ring_cap, GPTOSS_ERR_STATE,
                     "engine_step_rows: rows %d and %d of slot %d must be consecutive positions below %d (got %d, %d)",
                     i - 1, i, host_slots[i], ring_cap, host_pos[i - 1], host_pos[i]);
  }
  for (int j = 0; j < n_sample; j++)
    GPTOSS_REQUIRE(host_sample[j] >= 0 && host_sample[j] < n_rows, GPTOSS_ERR_DIM,
                   "engine_step_rows: sampled row %d outside 0..%d", host_sample[j], n_rows - 1);
  return step_rows(e, n_rows, host_tokens, host_slots, host_pos, n_sample, host_sample, host_next);
}

// The reference's schedule: requests in batches of max_batch, every batch in lock step until its
// last sequence ends (getp_run_submit.cpp:13-87).
static int generate_lockstep(gptoss_engine *e, const int *host_prompts, const int *host_n_prompt,
                             int prompt_stride, int n_req, int max_seq_len, int *host_out,
                             long long *n_generated) {
  long long total = 0;
  // requests are served in batches of max_batch, all sequences of a batch in lock step
  // (getp_run_submit.cpp:13-87)
  for (int r0 = 0; r0 < n_req; r0 += e->max_batch) {
    const int B = std::min(e->max_batch, n_req - r0);
    std::vector<int> cur_tok(B), cur_pos(B, 0), next(B);
    std::vector<char> active(B, 1);
    int active_count = B;
    for (int i = 0; i < B; i++) cur_tok[i] = host_prompts[(size_t)(r0 + i) * prompt_stride];
    // The prompt positions every sequence of the batch has in common go through one prefill pass
    // instead of one lock-step step each (the reference feeds prompts token by token,
    // getp_run_submit.cpp:60-72).  The pass stops before a prompt's own stop token, which ends
    // that sequence in the lock-step loop, and before the last position the loop may visit.
    int first_pos = 0;
    if (e->pf.rows > 0 && !(e->flags & GPTOSS_ENGINE_PRECISE)) {
      int T = std::min(max_seq_len - 1, e->pf.rows);
      for (int i = 0; i < B; i++) {
        const int *pt = host_prompts + (size_t)(r0 + i) * prompt_stride;
        const int np = host_n_prompt[r0 + i];
        T = std::min(T, np);
        for (int j = 1; j < T; j++)
          if (pt[j] == 199999 || pt[j] == 200002) T = j;
      }
      if (T >= 2) {
        std::vector<int> toks((size_t)B * T);
        for (int i = 0; i < B; i++)
          memcpy(&toks[(size_t)i * T], host_prompts + (size_t)(r0 + i) * prompt_stride, sizeof(int) * T);
        int rc = gptoss_engine_prefill(e, toks.data(), B, T, next.data());
        if (rc != GPTOSS_OK) return rc;
        first_pos = T;
        for (int i = 0; i < B; i++) cur_pos[i] = T - 1;  // the loop body below finishes position T-1
      }
    }
    for (int pos = first_pos > 0 ? first_pos - 1 : 0; pos < max_seq_len - 1 && active_count > 0; pos++) {
      if (pos >= first_pos) {
        int rc = gptoss_engine_step(e, cur_tok.data(), pos, B, next.data());
        if (rc != GPTOSS_OK) return rc;
      }
      for (int i = 0; i < B; i++) {
        if (!active[i]) continue;
        const int *pt = host_prompts + (size_t)(r0 + i) * prompt_stride;
        const int np = host_n_prompt[r0 + i];
        int *o = host_out + (size_t)(r0 + i) * (max_seq_len + 1);
        int nt = next[i];
        if (cur_pos[i] < np - 1) nt = pt[cur_pos[i] + 1];
        else o[cur_pos[i] - (np - 1)] = nt;
        if (nt == 199999 || nt == 200002) {
          active[i] = 0;
          active_count--;
        }
        cur_tok[i] = nt;
        cur_pos[i]++;
      }
    }
    for (int i = 0; i < B; i++) {
      int generated_len = cur_pos[i] - host_n_prompt[r0 + i];
      if (generated_len < 0) generated_len = 0;
      host_out[(size_t)(r0 + i) * (max_seq_len + 1) + generated_len + 1] = -1;
      total += generated_len + 1;
    }
  }
  if (n_generated) *n_generated = total;
  return GPTOSS_OK;
}

// Continuous batching: max_batch slots; a slot whose sequence ended (stop id or its length limit)
// takes the next waiting request at once, while the other slots carry on at their own positions.
// Every request sees the arithmetic it would see alone, so its output is the one the lock-step
// schedule gives; only the order of the work changes.  host_max_len (optional) limits request r
// to host_max_len[r] positions in all (prompt included) instead of max_seq_len.
//
// Prompts are not forced one token per step (getp_run_submit.cpp:67-72 does that).  The positions
// the first max_batch requests share go through one prompt pass; after that every step is a step
// over rows (step_rows): one row for each sequence that is decoding, and for a request that has
// just been admitted all the prompt positions it has left, as consecutive rows of the same step.
// Those rows ride along in the weight passes the step makes anyway, so a prompt costs its slot
// one step instead of one step per token.  On the sliding-window layers the rows of one step must
// stay inside the first lap of the ring, so prompt positions from the ring's capacity on are
// forced one per step as before; and a step never has more rows than the prompt buffers hold.
static int generate_continuous(gptoss_engine *e, const int *host_prompts, const int *host_n_prompt,
                               int prompt_stride, int n_req, int max_seq_len, const int *host_max_len,
                               int *host_out, long long *n_generated) {
  long long total = 0;
  const int B = std::min(e->max_batch, n_req);
  if (B == 0) {
    if (n_generated) *n_generated = 0;
    return GPTOSS_OK;
  }
  std::vector<int> req(B, -1), cur_tok(B, 0), cur_pos(B, 0), next(B), prefix(B, 0);
  int next_req = 0, active_count = 0;
  const bool rows_path = e->pf.rows > 0;
  int ring_cap = e->max_seq + 1;  // positions a stretch of rows may reach on the window layers
  for (const LayerWeights &w : e->layers)
    if (w.window > 0) ring_cap = std::min(ring_cap, w.cache_cap);
  auto limit = [&](int r) { return host_max_len ? std::min(host_max_len[r], max_seq_len) : max_seq_len; };
  // prompt positions of request r that may be run without looking at a result: a prompt's own stop
  // token ends the sequence when it is fed, and the loop visits limit - 1 positions at most
  auto forced_prefix = [&](int r) {
    const int *pt = host_prompts + (size_t)r * prompt_stride;
    int T = std::min(host_n_prompt[r], limit(r) - 1);
    for (int j = 1; j < T; j++)
      if (pt[j] == 199999 || pt[j] == 200002) T = j;
    return T;
  };
  auto finish = [&](int i) {
    const int r = req[i];
    int generated_len = cur_pos[i] - host_n_prompt[r];
    if (generated_len < 0) generated_len = 0;
    host_out[(size_t)r * (max_seq_len + 1) + generated_len + 1] = -1;
    total += generated_len + 1;
    req[i] = -1;
    active_count--;
  };
  auto admit = [&](int i) {
    // requests that may not even take one step are closed as the lock-step loop closes them
    while (next_req < n_req) {
      const int r = next_req++;
      req[i] = r;
      cur_tok[i] = host_prompts[(size_t)r * prompt_stride];
      cur_pos[i] = 0;
      active_count++;
      if (limit(r) - 1 > 0) {
        prefix[i] = forced_prefix(r);
        return;
      }
      finish(i);
    }
    cur_tok[i] = 0;
    cur_pos[i] = 0;
  };
  // what the loop of getp_run_submit.cpp:60-96 does with the id the forward call of position
  // cur_pos returned
  auto advance = [&](int i, int next_id) {
    const int r = req[i];
    const int *pt = host_prompts + (size_t)r * prompt_stride;
    const int np = host_n_prompt[r];
    int *o = host_out + (size_t)r * (max_seq_len + 1);
    int nt = next_id;
    if (cur_pos[i] < np - 1) nt = pt[cur_pos[i] + 1];
    else o[cur_pos[i] - (np - 1)] = nt;
    cur_tok[i] = nt;
    cur_pos[i]++;
    if (nt == 199999 || nt == 200002 || cur_pos[i] >= limit(r) - 1) {
      finish(i);
      admit(i);
    }
  };
  for (int i = 0; i < B; i++) admit(i);

  // the prompt positions the first B requests share go through one prompt pass
  bool first_wave = rows_path;
  for (int i = 0; i < B; i++) first_wave = first_wave && req[i] == i;
  if (first_wave) {
    int T = e->pf.rows;
    for (int i = 0; i < B; i++) T = std::min(T, prefix[i]);
    if (T >= 2) {
      std::vector<int> toks((size_t)B * T);
      for (int i = 0; i < B; i++)
        memcpy(&toks[(size_t)i * T], host_prompts + (size_t)i * prompt_stride, sizeof(int) * T);
      int rc = gptoss_engine_prefill(e, toks.data(), B, T, next.data());
      if (rc != GPTOSS_OK) return rc;
      for (int i = 0; i < B; i++) cur_pos[i] = T - 1;  // advance() finishes position T-1
      for (int i = 0; i < B; i++) advance(i, next[i]);
    }
  }
  if (!rows_path) {
    while (active_count > 0) {
      int rc = gptoss_engine_step_ragged(e, cur_tok.data(), cur_pos.data(), B, next.data());
      if (rc != GPTOSS_OK) return rc;
      for (int i = 0; i < B; i++)
        if (req[i] >= 0) advance(i, next[i]);
    }
    if (n_generated) *n_generated = total;
    return GPTOSS_OK;
  }
  std::vector<int> r_tok, r_slot, r_pos, sample, owner, count(B);
  while (active_count > 0) {
    // rows of this step: one per running sequence, plus what fits of the prompt stretches
    int extra = e->pf.rows - active_count;
    r_tok.clear();
    r_slot.clear();
    r_pos.clear();
    sample.clear();
    owner.clear();
    for (int i = 0; i < B; i++) {
      count[i] = 0;
      if (req[i] < 0) continue;
      // positions cur_pos .. stretch_end - 1 are prompt positions whose inputs are known
      const int stretch_end = std::min(prefix[i], ring_cap);
      int m = 1;
      if (cur_pos[i] + 1 < stretch_end) {
        m = std::min(stretch_end - cur_pos[i], 1 + std::max(0, extra));
        extra -= m - 1;
      }
      const int *pt = host_prompts + (size_t)req[i] * prompt_stride;
      for (int j = 0; j < m; j++) {
        r_tok.push_back(j == 0 ? cur_tok[i] : pt[cur_pos[i] + j]);
        r_slot.push_back(i);
        r_pos.push_back(cur_pos[i] + j);
      }
      count[i] = m;
      sample.push_back((int)r_tok.size() - 1);
      owner.push_back(i);
    }
    int rc = step_rows(e, (int)r_tok.size(), r_tok.data(), r_slot.data(), r_pos.data(), (int)sample.size(),
                       sample.data(), next.data());
    if (rc != GPTOSS_OK) return rc;
    for (size_t j = 0; j < owner.size(); j++) {
      const int i = owner[j];
      cur_pos[i] += count[i] - 1;  // advance() finishes the stretch's last position
      advance(i, next[j]);
    }
  }
  if (n_generated) *n_generated = total;
  return GPTOSS_OK;
}

extern "C" int gptoss_engine_generate_ragged(gptoss_engine *e, const int *host_prompts, const int *host_n_prompt,
                                             int prompt_stride, int n_req, int max_seq_len,
                                             const int *host_max_len, int *host_out, long long *n_generated) {
  GPTOSS_REQUIRE(e && host_prompts && host_n_prompt && host_out, GPTOSS_ERR_NULL, "engine_generate: null pointer");
  GPTOSS_REQUIRE(n_req >= 0 && prompt_stride >= 1 && max_seq_len >= 1 && max_seq_len <= e->max_seq + 1,
                 GPTOSS_ERR_DIM, "engine_generate: max_seq_len %d needs an engine with max_seq >= %d",
                 max_seq_len, max_seq_len - 1);
  for (int r = 0; r < n_req; r++)
    GPTOSS_REQUIRE(host_n_prompt[r] >= 1 && host_n_prompt[r] <= prompt_stride, GPTOSS_ERR_DIM,
                   "engine_generate: request %d has %d prompt tokens", r, host_n_prompt[r]);
  if (host_max_len)
    for (int r = 0; r < n_req; r++)
      GPTOSS_REQUIRE(host_max_len[r] >= 1, GPTOSS_ERR_DIM, "engine_generate: request %d has length limit %d", r,
                     host_max_len[r]);
  const bool reference_schedule = (e->flags & (GPTOSS_ENGINE_PRECISE | GPTOSS_ENGINE_NO_PREFILL)) != 0;
  if (reference_schedule) {
    GPTOSS_REQUIRE(!host_max_len, GPTOSS_ERR_STATE,
                   "engine_generate: per-request length limits need the continuous schedule "
                   "(not GPTOSS_ENGINE_PRECISE / GPTOSS_ENGINE_NO_PREFILL)");
    return generate_lockstep(e, host_prompts, host_n_prompt, prompt_stride, n_req, max_seq_len, host_out, n_generated);
  }
  return generate_continuous(e, host_prompts, host_n_prompt, prompt_stride, n_req, max_seq_len, host_max_len,
                             host_out, n_generated);
}

extern "C" int gptoss_engine_generate(gptoss_engine *e, const int *host_prompts, const int *host_n_prompt,
                                      int prompt_stride, int n_req, int max_seq_len, int *host_out,
                                      long long *n_generated) {
  return gptoss_engine_generate_ragged(e, host_prompts, host_n_prompt, prompt_stride, n_req, max_seq_len, nullptr,
                                       host_out, n_generated);
}

extern "C" int gptoss_rope_tables(const gptoss_config *cfg, int n_pos, float *host_cos, float *host_sin) {
  GPTOSS_REQUIRE(cfg && host_cos && host_sin, GPTOSS_ERR_NULL, "rope_tables: null pointer");
  GPTOSS_REQUIRE(n_pos > 0 && cfg->head_dim > 0 && cfg->head_dim % 2 == 0 && cfg->rope_theta > 0.f, GPTOSS_ERR_DIM,
                 "rope_tables: bad dimensions (n_pos=%d head_dim=%d)", n_pos, cfg->head_dim);
  std::vector<float> cs, sn;
  rope_tables(*cfg, n_pos, cs, sn);
  memcpy(host_cos, cs.data(), cs.size() * sizeof(float));
  memcpy(host_sin, sn.data(), sn.size() * sizeof(float));
  return GPTOSS_OK;
}

// Device view of one weight tensor in the layout the kernels read.
extern "C" int gptoss_engine_tensor_view(gptoss_engine *e, int tensor, int layer, void **ptr, size_t *bytes) {
  GPTOSS_REQUIRE(e && ptr && bytes, GPTOSS_ERR_NULL, "engine_tensor_view: null pointer");
  GPTOSS_REQUIRE(!(e->flags & GPTOSS_ENGINE_PRECISE), GPTOSS_ERR_STATE,
                 "engine_tensor_view: GPTOSS_ENGINE_PRECISE keeps the fp32 payload as it is");
  const gptoss_config &c = e->cfg;
  const size_t H = c.hidden_dim, V = c.vocab_size, E = c.n_experts, I = c.intermediate_dim;
  const size_t nq = c.n_attn_heads, nkv = c.n_kv_heads, D = c.head_dim, qkv_dim = (nq + 2 * nkv) * D;
  const bool per_layer = tensor >= GPTOSS_TENSOR_ATTN_NORM;
  GPTOSS_REQUIRE(tensor >= 0 && tensor <= GPTOSS_TENSOR_B2, GPTOSS_ERR_DIM, "engine_tensor_view: unknown tensor %d", tensor);
  GPTOSS_REQUIRE(!per_layer || (layer >= 0 && layer < c.n_layers), GPTOSS_ERR_DIM,
                 "engine_tensor_view: layer %d outside 0..%d", layer, c.n_layers - 1);
  const bool q4 = (e->flags & GPTOSS_ENGINE_MXFP4_EXPERTS) != 0;
  auto expert_bytes = [&](size_t n_out, size_t n_in) {
    return q4 ? gptoss_packed_mxfp4_bytes((int)E, (int)n_out, (int)n_in) : E * n_out * n_in * sizeof(bf16_t);
  };
  const LayerWeights *w = per_layer ? &e->layers[layer] : nullptr;
  switch (tensor) {
    case GPTOSS_TENSOR_EMBEDDING: *ptr = e->embedding; *bytes = V * H * 2; break;
    case GPTOSS_TENSOR_UNEMBEDDING: *ptr = e->unembedding; *bytes = V * H * 2; break;
    case GPTOSS_TENSOR_FINAL_NORM: *ptr = e->final_norm; *bytes = H * 4; break;
    case GPTOSS_TENSOR_ATTN_NORM: *ptr = w->attn_norm; *bytes = H * 4; break;
    case GPTOSS_TENSOR_MLP_NORM: *ptr = w->mlp_norm; *bytes = H * 4; break;
    case GPTOSS_TENSOR_W_QKV: *ptr = w->w_qkv; *bytes = qkv_dim * H * 2; break;
    case GPTOSS_TENSOR_B_QKV: *ptr = w->b_qkv; *bytes = qkv_dim * 4; break;
    case GPTOSS_TENSOR_W_O: *ptr = w->w_o; *bytes = H * nq * D * 2; break;
    case GPTOSS_TENSOR_B_O: *ptr = w->b_o; *bytes = H * 4; break;
    case GPTOSS_TENSOR_SINKS: *ptr = w->sinks; *bytes = nq * 4; break;
    case GPTOSS_TENSOR_W_ROUTER: *ptr = w->w_router; *bytes = E * H * 2; break;
    case GPTOSS_TENSOR_B_ROUTER: *ptr = w->b_router; *bytes = E * 4; break;
    case GPTOSS_TENSOR_W1: *ptr = w->w1; *bytes = expert_bytes(2 * I, H); break;
    case GPTOSS_TENSOR_B1: *ptr = w->b1; *bytes = E * 2 * I * 4; break;
    case GPTOSS_TENSOR_W2: *ptr = w->w2; *bytes = expert_bytes(H, I); break;
    default: *ptr = w->b2; *bytes = E * H * 4; break;
  }
  return GPTOSS_OK;
}

// Device views for tests and tracing: logits of the last step [B,V] and the residual stream.
extern "C" int gptoss_engine_debug_views(gptoss_engine *e, float **logits, float **x, size_t *device_bytes) {
  GPTOSS_REQUIRE(e, GPTOSS_ERR_NULL, "engine_debug_views: null engine");
  if (logits) *logits = e->logits;
  if (x) *x = e->x;
  if (device_bytes) *device_bytes = e->device_bytes;
  return GPTOSS_OK;
}
