/*
 * gptoss_mi355 -- C ABI of the MI355X (gfx950) GPT-OSS decode hot path.
 *
 * This is the boundary the reference's host code binds instead of the C++ op layer in
 * getp-csrc/include/{layer_hip_batch,kernel,flash_attn_hip}.hpp.  Conventions, all entry points:
 *   - plain pointers and sizes only; every data pointer is DEVICE memory unless its name starts
 *     with host_;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); calls enqueue work
 *     and return without synchronising, never allocate, and never abort;
 *   - return value: GPTOSS_OK or an error code; gptoss_last_error_string() gives the text of the
 *     calling thread's last error;
 *   - scratch memory comes from the caller: ask gptoss_*_workspace_bytes, pass a 256-byte aligned
 *     device buffer of at least that size.  One workspace may be reused by consecutive calls on
 *     the same stream; calls sharing a workspace on different streams race;
 *   - thread-compatible: distinct workspaces/streams may be driven from distinct host threads.
 *
 * Weight matrices are [n_out, n_in] with n_in contiguous, exactly as the flat .bin stores them
 * (reference run.cpp:54-80); the reference instead transposes every matrix to [n_in, n_out] while
 * loading (getp-csrc/src/alloc.cpp:27-35,112-127).  GEMM entry points take them in the packed
 * MFMA-fragment order produced by gptoss_pack_weight().
 */
#ifndef GPTOSS_MI355_H
#define GPTOSS_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  GPTOSS_OK = 0,
  GPTOSS_ERR_NULL = 1,      /* a required pointer is NULL */
  GPTOSS_ERR_DIM = 2,       /* unsupported or inconsistent dimension */
  GPTOSS_ERR_ALIGN = 3,     /* pointer not aligned as required */
  GPTOSS_ERR_WORKSPACE = 4, /* workspace missing or too small */
  GPTOSS_ERR_HIP = 5,       /* HIP runtime / launch error */
  GPTOSS_ERR_STATE = 6,     /* call not valid in the engine's current state */
  GPTOSS_ERR_IO = 7         /* checkpoint file problem */
};

/* Text of the last error raised on the calling thread ("" if none).  No reference counterpart:
 * the reference prints and aborts (getp-csrc/include/tensor.hpp:20-27). */
const char *gptoss_last_error_string(void);

/* ABI version of this header (major*100+minor). */
int gptoss_abi_version(void);

/* Kernel timing hook.  Replaces the reference's GpuTimer (getp-csrc/include/utils.hpp:13-39, a
 * hipEvent pair around each op, compiled in with -DTIME_GPU).  After gptoss_trace_set(start, stop,
 * n) with two arrays of n hipEvent_t created by the caller, every kernel launched by an entry point
 * called from this thread records start[i] / stop[i] around itself on its stream (i counts
 * launches since the call).  gptoss_trace_set(NULL, NULL, 0) disarms.  gptoss_trace_name(i) is the
 * label of launch i.  The caller synchronises before reading the events. */
int gptoss_trace_set(void *const *start_events, void *const *stop_events, int n);
int gptoss_trace_count(void);
const char *gptoss_trace_name(int i);

/* ------------------------------------------------------------------ weight layout ---------- */

/* Flags for gptoss_pack_weight. */
enum {
  GPTOSS_PACK_SRC_FP32 = 1, /* source elements are fp32 (the .bin payload); default bf16 */
  GPTOSS_PACK_GLU = 2       /* rows are interleaved (gate,up) pairs (run.cpp:664-667): reorder them
                               so a wave holds the gates of 16 pairs in lanes 0-15 and their ups in
                               lanes 16-31 of its result columns */
};

/* Bytes of n_mat packed [n_out,n_in] matrices (bf16). */
size_t gptoss_packed_weight_bytes(int n_mat, int n_out, int n_in);

/* Repack n_mat row-major [n_out,n_in] matrices (device, bf16 or fp32) into MFMA-fragment order.
 * Replaces the host-side transposes of getp-csrc/src/alloc.cpp:27-35,52-59,79-88,112-127,155-170.
 * Needs n_out % 32 == 0 and n_in % 64 == 0. */
int gptoss_pack_weight(const void *src, void *dst, int n_mat, int n_out, int n_in, int flags,
                       void *stream);

/* ------------------------------------------------------------------ MoE routing ------------ */

/* logits[B,E] = t[B,H] . w_router[E,H]^T + b_router[E]     (bf16 x bf16 -> fp32)
 * Replaces router_gemm_batched_quantize (getp-csrc/src/layer_hip_batch.cpp:1006-1044).
 * t bf16 [B,H]; w_router bf16 [E,H] row-major (unpacked); b_router fp32 [E] or NULL.
 * Needs H % 32 == 0 and 1 <= E <= 256. */
int gptoss_router_gemm(const void *t, const void *w_router, const float *b_router, float *logits,
                       int B, int H, int E, void *stream);

/* Upper bound of the number of (expert,row0,rows) entries gptoss_moe_route can write for B tokens. */
int gptoss_moe_max_tiles(int B, int k, int E, int rows_per_tile);

/* Top-k gating and expert grouping from router logits.  Replaces
 *   topk_softmax_batched        (layer_hip_batch.cpp:1087-1203): top-k, descending, lowest expert
 *                               id first among equal logits; softmax over the k picked values;
 *   moe_build_offsets           (kernel.cpp:504-542,851-865): counting sort of the B*k pairs
 *                               (pair = token*k + slot) by expert, STABLE (ascending pair id inside
 *                               an expert);
 *   moe_get_max_rows_per_expert (kernel.cpp:709-719,916-925): replaced by a device-side tile list,
 *                               no host read-back.
 * Outputs (device): topk_w fp32 [B,k], topk_i int32 [B,k], expert_offsets int32 [E+1],
 * sorted_pair_ids int32 [B*k], inv_perm int32 [B*k] (inv_perm[pair] = its row in the sorted
 * order), tiles int32 [1 + 3*gptoss_moe_max_tiles()] = {n_tiles, (expert,row0,rows)...} cutting
 * every expert's rows into tiles of rows_per_tile (may be NULL with rows_per_tile 0).
 * Needs 1 <= k <= 8, k <= E <= 256, rows_per_tile 0 or a multiple of 32 up to 256. */
int gptoss_moe_route(const float *logits, int B, int E, int k, float *topk_w, int *topk_i,
                     int *expert_offsets, int *sorted_pair_ids, int *inv_perm, int *tiles,
                     int rows_per_tile, void *stream);

/* ------------------------------------------------------------------ MoE layer -------------- */

typedef struct {
  int n_experts;         /* E */
  int top_k;             /* k */
  int hidden;            /* H */
  int intermediate;      /* I */
  float swiglu_limit;    /* clamp, 7.0 */
  const void *w_router;  /* bf16 [E,H] row-major */
  const float *b_router; /* fp32 [E] */
  const void *w1;        /* experts' gate/up matrices [E,2I,H], packed with GPTOSS_PACK_GLU;
                            for the MXFP4 entry point: gptoss_pack_mxfp4 output */
  const float *b1;       /* fp32 [E,2I], interleaved (gate,up) as in the .bin */
  const void *w2;        /* experts' down matrices [E,H,I], packed */
  const float *b2;       /* fp32 [E,H] */
} gptoss_moe_weights;

size_t gptoss_moe_workspace_bytes(int B, int E, int k, int H, int I);

/* One MoE block for B tokens:  out[B,H] (+)= sum_slot w[b,slot] * FFN_expert(b,slot)(t[b]).
 * Replaces the sequence router_gemm_batched_quantize .. moe_scatter_aggregate_hip_120b (+ the
 * residual add_vector_batched when accumulate != 0) of forward_gpu_20b_batched
 * (getp-csrc/src/model.cpp:74-131): router GEMM, top-k softmax, stable grouping, grouped GEMM1
 * with the token gather folded into its operand load and clamped SwiGLU folded into its epilogue
 * (kernel.cpp:560-573,636-685,927-952), grouped GEMM2 (kernel.cpp:1061-1089) and a deterministic
 * per-token weighted combine in ascending expert order, the order of the CPU loop run.cpp:642-704
 * (replaces the atomicAdd scatter, kernel.cpp:748-768).
 * t bf16 [B,H]; out fp32 [B,H].  Needs H % 64 == 0, I % 64 == 0, k <= min(8,E), E <= 256,
 * B*k*max(H,I) < 2^31. */
int gptoss_moe_forward(const gptoss_moe_weights *w, const void *t, int B, float *out,
                       int accumulate, void *workspace, size_t workspace_bytes, void *stream);

/* Views into a workspace after gptoss_moe_forward (for tests and tracing): device pointers to
 * logits fp32 [B,E], topk_w [B,k], topk_i [B,k], expert_offsets [E+1], sorted_pair_ids [B*k],
 * inv_perm [B*k].  Any output pointer may be NULL. */
int gptoss_moe_workspace_views(void *workspace, int B, int E, int k, int H, int I, float **logits,
                               float **topk_w, int **topk_i, int **expert_offsets,
                               int **sorted_pair_ids, int **inv_perm);

/* MXFP4 expert weights (OCP MX: e2m1 codes, low nibble = even element, one e8m0 scale per 32
 * elements along n_in; format of export_model_bin/gpt-oss-20b/export_model_bin.py:66-123).  The
 * reference dequantises offline to bf16 and has no FP4 kernel. */
size_t gptoss_packed_mxfp4_bytes(int n_mat, int n_out, int n_in);
/* blocks uint8 [n_mat,n_out,n_in/2], scales uint8 [n_mat,n_out,n_in/32] -> packed. */
int gptoss_pack_mxfp4(const void *blocks, const void *scales, void *dst, int n_mat, int n_out,
                      int n_in, int flags, void *stream);
/* Same contract as gptoss_moe_forward with w->w1 / w->w2 in gptoss_pack_mxfp4 order. */
int gptoss_moe_forward_mxfp4(const gptoss_moe_weights *w, const void *t, int B, float *out,
                             int accumulate, void *workspace, size_t workspace_bytes,
                             void *stream);

/* ------------------------------------------------------------------ decode attention ------- */

/* The KV cache of a layer is ONE array holding K and V (the reference keeps two tensors per layer,
 * getp-csrc/src/alloc.cpp:239-262): per sequence and kv head, blocks of 64 token slots, each the
 * K rows of its slots followed by their V in MFMA operand order, so that a wave streams one
 * contiguous 16 KB unit per 64 slots.  The layout is internal: size the array with
 * gptoss_kv_cache_bytes and fill it with gptoss_kv_cache_write.  `capacity` = token slots per
 * sequence (multiple of 64); position p lives in slot p % capacity, so a cache with capacity ==
 * window is the ring buffer the reference keeps for its sliding-window layers
 * (getp-csrc/src/alloc.cpp:245-250).  Sequences are the outermost dimension: the cache of the
 * first n sequences is the first gptoss_kv_cache_bytes(n, ...) bytes. */
size_t gptoss_kv_cache_bytes(int B, int n_kv, int head_dim, int capacity); /* K and V together */

/* Store n_tok consecutive positions [pos0, pos0+n_tok) of every sequence.  k_rows/v_rows bf16
 * [B, n_tok, n_kv, head_dim] (K already rotated).  Bulk form of the cache write in
 * qkv_split_rope_store_kernel (layer_hip_batch.cpp:686-776). */
int gptoss_kv_cache_write(void *kv_cache, const void *k_rows, const void *v_rows, int B, int n_kv,
                          int head_dim, int capacity, int pos0, int n_tok, void *stream);

size_t gptoss_attn_workspace_bytes(int B, int n_q, int n_kv, int head_dim, int max_len);

/* Single-query attention with sinks and optional sliding window over the bf16 KV cache.
 * Replaces single_query_attn_flash_batched_quantize (getp-csrc/src/flash_attn_hip.cpp:847-923).
 *   q fp32 [B,n_q,D] (rotated); lens int32 [B] = cached positions per sequence (pos+1; the
 *   reference has one scalar pos for the whole batch), or NULL when every sequence has max_len
 *   positions (lock-step decoding: the kernels then need no load to learn a row's length); window > 0 keeps the last `window`
 *   positions; sinks fp32 [n_q] or NULL; out bf16 [B,n_q,D].
 *   max_len: upper bound of lens known to the host (sizes the split of long sequences).
 * Needs D in {32,64}, n_q % n_kv == 0, n_q/n_kv <= 16; q and kv_cache 16-byte aligned, out 8-byte
 * aligned (a 16-byte aligned out lets rows of at most 512 slots be written in one burst at the end
 * of the launch instead of row by row during it: same bits, up to 8 % less time).
 * A row's result does not depend on the other rows of the call, with one exception: a row that
 * spans more than 512 slots is summed in one of two orders, chosen by the call's B * n_kv (below
 * 512: chunks of 512 slots, merged by a second kernel; from 512 on: four interleaved streams merged
 * inside one workgroup).  Calls with equal B, n_kv give bit-identical rows; across the two forms
 * rows agree to fp32 rounding of the softmax sums. */
int gptoss_attn_decode(const float *q, const void *kv_cache, const int *lens, const float *sinks,
                       void *out, int B, int n_q, int n_kv, int head_dim, int capacity, int window,
                       int max_len, void *workspace, size_t workspace_bytes, void *stream);

/* gptoss_attn_decode for callers that cannot allocate or bring a workspace (code under HIP graph
 * capture, serving loops and harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments, arithmetic and results as gptoss_attn_decode; what that call keeps in its
 * workspace (the chunk partials of long sequences when few sequences are served, the row order
 * when many are) goes to a device array built into the library (64 MiB, held by every GPU the library
 * runs on until the process ends).  The call allocates nothing.  Refused with
 * GPTOSS_ERR_WORKSPACE when gptoss_attn_workspace_bytes(B, n_q, n_kv, head_dim, max_len) exceeds
 * gptoss_attn_decode_static_max_bytes() (e.g. 256 sequences x 64 heads x 64 up to 4096 positions
 * need 39 MiB).  Nothing in the array has to start at zero.  All calls on one GPU share the array:
 * calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not.  The
 * first call on a device looks the array's address up (make it outside a graph capture). */
size_t gptoss_attn_decode_static_max_bytes(void);
int gptoss_attn_decode_static(const float *q, const void *kv_cache, const int *lens, const float *sinks,
                              void *out, int B, int n_q, int n_kv, int head_dim, int capacity, int window,
                              int max_len, void *stream);

/* The same attention for T consecutive positions of every sequence at once (prompt processing):
 * q fp32 [B, T, n_q, D] and out bf16 [B, T, n_q, D]; row (b, t) attends to the cached positions up
 * to pos0 + t of sequence b, with the arithmetic gptoss_attn_decode uses for lens = pos0 + t + 1,
 * so its result is the one the T lock-step calls of the reference would give
 * (getp-csrc/submit/getp_run_submit.cpp:60-72 feeds prompts one position per step): bit for bit
 * for rows whose active positions span at most 512 cache slots; a longer row is summed block by
 * block in one pass where the decode call merges partial sums, which can move the last bit of a
 * few outputs.  With 32 or more positions per sequence (and at most 8 query heads per kv head) 16
 * consecutive rows of a sequence share one pass over its K/V blocks, so a prompt of 1024 positions
 * (the reference's cap, getp-csrc/src/alloc.cpp:1047) reads its cache 64 times, not 512.  The cache must
 * already hold positions [0, pos0 + T) of every sequence, all of them (a sliding-window ring
 * shorter than pos0 + T is refused: copy the prompt's K/V to a linear cache for this call). */
size_t gptoss_attn_prefill_workspace_bytes(int B, int T, int n_q, int n_kv, int head_dim, int max_len);
int gptoss_attn_prefill(const float *q, const void *kv_cache, const float *sinks, void *out, int B,
                        int T, int pos0, int n_q, int n_kv, int head_dim, int capacity, int window,
                        void *workspace, size_t workspace_bytes, void *stream);

/* The 60-byte header of the flat .bin (reference run.cpp:25-45), same field order. */
typedef struct {
  int vocab_size, hidden_dim, n_experts, experts_per_token, intermediate_dim, n_layers;
  int head_dim, n_attn_heads, n_kv_heads, seq_len, initial_context_length;
  float rope_theta, rope_scaling_factor;
  int sliding_window;
  float swiglu_limit;
} gptoss_config;

/* ------------------------------------------------------------------ glue ops ---------------- */
/* The small ops between the two hot ones, for a host that keeps the reference's forward loop
 * (getp-csrc/src/model.cpp:6-151) and binds it op by op; the engine below uses the same kernels. */

/* x[b,:] = table[tokens[b],:]  (bf16 [V,H] row-major -> fp32 [B,H]; ids are clamped to 0..V-1).
 * Replaces embedding_lookup_batched (getp-csrc/src/layer_hip_batch.cpp:199-242). */
int gptoss_embedding(const void *table, const int *tokens, float *x, int B, int H, int V, void *stream);

/* RMSNorm with the CPU model's arithmetic (run.cpp:304-317: double sum of squares, eps 1e-5 after
 * the mean): t = weight * x / sqrt(mean(x^2) + eps) as bf16 [B,H].  With residual != NULL,
 * x += residual first, in place.  Replaces rmsnorm_batched_quantize and
 * residual_rmsnorm_batched_quantize (layer_hip_batch.cpp:339-438, 94-197). */
int gptoss_rmsnorm(float *x, const float *residual, const float *weight, void *t_bf16, int B, int H,
                   void *stream);

/* out[B,N] = a[B,K] . w[N,K]^T + bias[N]   (bf16 x bf16 -> fp32; w in gptoss_pack_weight order; bias
 * may be NULL).  Replaces qkv_gemm_batched_v2_quantize, attn_out_project_batched_v2_quantize and
 * classifier_gemm_batched_v2_quantize (layer_hip_batch.cpp:644-683, 881-923, 1465-1501).
 * Needs N % 32 == 0, K % 64 == 0, B*max(N,K) < 2^32. */
int gptoss_dense_gemm(const void *a, const void *w_packed, const float *bias, float *out, int B, int N,
                      int K, void *stream);

/* next_ids[b] = arg max over v of a[b,:] . w[v,:]  (lowest v among equal maxima) without writing the
 * [B,V] logits: the classifier GEMM keeps (max, column) per row and 256-column tile (per 128-column
 * half of a tile from 256 rows on, where it runs on 256-row tiles), a second small kernel picks the
 * row's winner.  Replaces classifier_gemm_batched_v2_quantize + max_logits_batched
 * (layer_hip_batch.cpp:1465-1501, 1542-1630; model.cpp:144-148). */
size_t gptoss_classifier_argmax_workspace_bytes(int B, int V);
int gptoss_classifier_argmax(const void *a, const void *w_packed, int *next_ids, int B, int V, int K,
                             void *workspace, size_t workspace_bytes, void *stream);

/* ids[b] = arg max of logits[b,:], lowest index among equal maxima (run.cpp:739-750).  Replaces
 * max_logits_batched (layer_hip_batch.cpp:1542-1630).  Needs V % 4 == 0. */
int gptoss_argmax(const float *logits, int *ids, int B, int V, void *stream);

/* cos/sin tables [n_pos, head_dim/2] of the rotary embedding with YaRN scaling, the float arithmetic
 * of run.cpp:404-478, written to HOST arrays.  Replaces rope_precompute_cs
 * (getp-csrc/include/alloc.hpp:11-93). */
int gptoss_rope_tables(const gptoss_config *cfg, int n_pos, float *host_cos, float *host_sin);

/* Split the fused qkv rows [B,(n_q+2n_kv)*D] fp32, rotate q and k of sequence b for position
 * lens[b]-1 (half-split pairs, run.cpp:480-499), write q fp32 [B,n_q,D] and store k, v as bf16 into
 * slot (lens[b]-1) % capacity of the layer's cache.  cos_t / sin_t: DEVICE copies of the
 * gptoss_rope_tables arrays covering every position used.  A sequence with lens[b] == 0 is empty
 * (as for gptoss_attn_decode): nothing is stored for it and its q row is set to zero; negative
 * lengths are treated the same way.  Replaces qkv_split_rope_fused
 * (layer_hip_batch.cpp:686-816), with a position per sequence instead of one for the batch. */
int gptoss_rope_kv_store(const float *qkv, float *q_out, void *kv_cache, const float *cos_t,
                         const float *sin_t, const int *lens, int B, int n_q, int n_kv, int head_dim,
                         int capacity, void *stream);

/* ------------------------------------------------------------------ engine ------------------ */

typedef struct gptoss_engine gptoss_engine;

enum {
  GPTOSS_ENGINE_SYNTHETIC = 1, /* host_weights ignored: N(0,0.02) bf16 weights generated on device */
  GPTOSS_ENGINE_LOGITS = 4,    /* write the fp32 logits [B, vocab] of every step to memory (for
                                  gptoss_engine_debug_views); without it the classifier GEMM keeps only
                                  each row's arg-max, as max_logits_batched consumes them
                                  (getp-csrc/src/model.cpp:144-148) */
  GPTOSS_ENGINE_PRECISE = 2,   /* the reference CPU model's arithmetic (run.cpp:501-717) instead of the
                                  reference GPU path's bf16 staging: fp32 weights, activations and KV
                                  cache, double-accumulated dot products.  Reproduces the CPU model's
                                  greedy ids; slow, needs host_weights, 4x the weight memory */
  GPTOSS_ENGINE_NO_PREFILL = 8, /* the reference's schedule, exactly: no prompt-processing buffers,
                                  gptoss_engine_generate serves requests in batches of max_batch, each
                                  batch in lock step from position 0, prompts one position per step
                                  (getp-csrc/submit/getp_run_submit.cpp:13-87) */
  GPTOSS_ENGINE_MXFP4_EXPERTS = 16 /* keep the expert matrices in MXFP4 (0.53 bytes per weight instead of
                                  2).  GPT-OSS checkpoints are MXFP4 at the source and the .bin holds
                                  their dequantised values (export_model_bin/gpt-oss-20b/
                                  export_model_bin.py:66-123), so the fp32 payload converts back
                                  exactly and the kernels multiply the same bf16 operands: results are
                                  bit-identical to the bf16 storage.  Creation fails with
                                  GPTOSS_ERR_STATE if a value has no exact MXFP4 representation. */
};

/* Build device weights (bf16, packed) and run state for up to max_batch sequences of up to
 * max_seq positions.  host_weights = the fp32 payload of the .bin just past the header (host
 * memory, e.g. the mmap the reference's build_transformer makes).  Replaces our_init
 * (getp-csrc/src/alloc.cpp:1035-1073) for one GPU.  This call allocates and synchronises. */
int gptoss_engine_create(const gptoss_config *cfg, const float *host_weights, int max_batch,
                         int max_seq, int flags, uint64_t seed, gptoss_engine **out);

/* One lock-step decode step: feed host_tokens[B] at position pos, return the arg-max next ids
 * (lowest id wins ties) in host_next[B].  Replaces forward_gpu_20b_batched
 * (getp-csrc/src/model.cpp:6-151).  Synchronises once, to hand the ids back. */
int gptoss_engine_step(gptoss_engine *e, const int *host_tokens, int pos, int B, int *host_next);

/* The same step with every sequence at its own position host_pos[B] (a scheduler that refills
 * the slot of a finished sequence while the others carry on).  The reference keeps one scalar pos
 * for the whole batch (getp-csrc/submit/getp_run_submit.cpp:60); with equal positions this is
 * gptoss_engine_step.  Not available with GPTOSS_ENGINE_PRECISE. */
int gptoss_engine_step_ragged(gptoss_engine *e, const int *host_tokens, const int *host_pos, int B,
                              int *host_next);

/* One step over n_rows arbitrary rows: row i feeds host_tokens[i] at position host_pos[i] of the
 * sequence in cache slot host_slots[i] (0 <= slot < max_batch).  Slots that have no row take no
 * part in the step.  A slot may have several rows, a stretch of its prompt: they must be adjacent
 * in the arrays, at consecutive ascending positions, and (with sliding-window layers) all below
 * the window rings' capacity; every row's K/V is stored before any row attends and a row attends
 * to the positions up to its own, so the stretch is processed as the same number of single steps
 * would process it, inside one pass over the weights.  host_next[j] is the arg-max after row
 * host_sample[j] (n_sample <= max_batch; the classifier runs for those rows only).  This is the
 * step the continuous schedule of gptoss_engine_generate is made of; the reference has one
 * position for the whole batch and one row per sequence
 * (getp-csrc/src/model.cpp:6-151, submit/getp_run_submit.cpp:60-72).  n_rows <= 8192; not
 * available with GPTOSS_ENGINE_PRECISE or GPTOSS_ENGINE_NO_PREFILL. */
int gptoss_engine_step_rows(gptoss_engine *e, int n_rows, const int *host_tokens, const int *host_slots,
                            const int *host_pos, int n_sample, const int *host_sample, int *host_next);

/* Positions 0..T-1 of B sequences in one pass: host_tokens int32 [B, T]; fills the KV caches and
 * returns in host_next[B] the arg-max ids after position T-1, i.e. what T calls of
 * gptoss_engine_step with pos = 0..T-1 leave behind (identical ids and caches while no
 * sliding-window ring has wrapped and the prompt has at most 512 positions; beyond either limit
 * attention sums a row's scores in another order, so results are equal to rounding).  Decoding continues with
 * gptoss_engine_step at pos = T.  The reference has no such pass: it feeds prompts one position
 * per step (getp-csrc/submit/getp_run_submit.cpp:60-72).  Needs T <= max_seq and T <= 8192; not
 * available with GPTOSS_ENGINE_PRECISE or GPTOSS_ENGINE_NO_PREFILL. */
int gptoss_engine_prefill(gptoss_engine *e, const int *host_tokens, int B, int T, int *host_next);

/* Greedy generation with the reference's getp loop semantics
 * (getp-csrc/submit/getp_run_submit.cpp:60-96): prompts int32 [n_req, prompt_stride] with
 * n_prompt[r] ids each; out int32 [n_req, max_seq_len+1], terminated by -1; returns the harness's
 * generated-token count in *n_generated. */
/* Unless the engine was created with GPTOSS_ENGINE_PRECISE or GPTOSS_ENGINE_NO_PREFILL the
 * requests are scheduled continuously: max_batch slots, the prompt positions shared by the first
 * max_batch requests in one prompt pass, and a slot whose sequence ended (stop id or length limit)
 * takes the next waiting request at once.  A request admitted that way does not force its prompt
 * one token per step (getp-csrc/submit/getp_run_submit.cpp:67-72): the prompt positions it has
 * left run as consecutive rows of the next step, beside the one row of every sequence that is
 * decoding, so they share that step's passes over the weights (on sliding-window layers only
 * while they stay inside the ring's first lap; later prompt positions are forced as before).
 * Every request gets the arithmetic it would get alone, so the output is that of the reference's
 * batch-by-batch lock-step schedule. */
int gptoss_engine_generate(gptoss_engine *e, const int *host_prompts, const int *host_n_prompt,
                           int prompt_stride, int n_req, int max_seq_len, int *host_out,
                           long long *n_generated);

/* The same with a length limit per request: request r stops after max_len[r] positions in all
 * (prompt included; capped by max_seq_len), as if it had been run alone with max_seq_len =
 * max_len[r].  The reference has one limit for all requests (run.cpp `-n`); ragged limits are what
 * shows the continuous schedule: a batch no longer waits for its longest sequence.  max_len may be
 * NULL; a non-NULL max_len needs the continuous schedule. */
int gptoss_engine_generate_ragged(gptoss_engine *e, const int *host_prompts, const int *host_n_prompt,
                                  int prompt_stride, int n_req, int max_seq_len, const int *max_len,
                                  int *host_out, long long *n_generated);

void gptoss_engine_destroy(gptoss_engine *e);

/* Device views for tests and tracing (the counterpart of the reference's Tensor::printDebug,
 * getp-csrc/src/tensor.cpp:158-172): logits fp32 [B,vocab] and residual stream fp32 [B,hidden] of
 * the last step, and the bytes of device memory the engine holds.  Outputs may be NULL. */
int gptoss_engine_debug_views(gptoss_engine *e, float **logits, float **x, size_t *device_bytes);

/* Device view of one weight tensor as the engine holds it after loading: the counterpart of the
 * fields of the reference's OurTransformerWeights (getp-csrc/include/config.hpp:50-158), which its
 * loader fills tensor by tensor (getp-csrc/src/alloc.cpp:6-197).  Matrices are bf16: embedding and
 * router row-major, every other matrix in gptoss_pack_weight order (mlp1 with GPTOSS_PACK_GLU),
 * expert matrices in gptoss_pack_mxfp4 order under GPTOSS_ENGINE_MXFP4_EXPERTS; vectors are fp32.
 * `layer` is ignored for the three tensors the model has once. */
enum {
  GPTOSS_TENSOR_EMBEDDING = 0, GPTOSS_TENSOR_UNEMBEDDING, GPTOSS_TENSOR_FINAL_NORM,
  GPTOSS_TENSOR_ATTN_NORM, GPTOSS_TENSOR_MLP_NORM, GPTOSS_TENSOR_W_QKV, GPTOSS_TENSOR_B_QKV,
  GPTOSS_TENSOR_W_O, GPTOSS_TENSOR_B_O, GPTOSS_TENSOR_SINKS, GPTOSS_TENSOR_W_ROUTER,
  GPTOSS_TENSOR_B_ROUTER, GPTOSS_TENSOR_W1, GPTOSS_TENSOR_B1, GPTOSS_TENSOR_W2, GPTOSS_TENSOR_B2
};
int gptoss_engine_tensor_view(gptoss_engine *e, int tensor, int layer, void **ptr, size_t *bytes);

/* Diagnostic without a counterpart in the reference: launches `workgroups` workgroups of 8 waves
 * that each issue 4 * iters matrix instructions on operands held in registers (kind 0:
 * v_mfma_f32_32x32x16_bf16; 1 / 2 / 3: v_mfma_scale_f32_32x32x64_f8f6f4 on fp8 x fp4, fp4 x fp4,
 * fp8 x fp8 operands) and returns the flop the launch performs; the caller times it.  sink: 4
 * bytes of device memory.  `python bench.py --mfma-rates` reports the rates. */
int gptoss_diag_mfma_rate(int kind, int workgroups, int iters, float *sink, double *flop, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GPTOSS_MI355_H */
