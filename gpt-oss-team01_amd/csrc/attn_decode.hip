// Single-query (decode) attention over a bf16 KV cache for gfx950, with attention sinks, optional
// sliding window, per-sequence lengths and grouped-query sharing.
//
// The op is bound by streaming K and V once from HBM, so:
//   * one wave owns one (sequence, kv head, chunk of the context) and serves ALL query heads of
//     that kv head from a single pass over K and V (the reference re-reads KV once per q head);
//   * scores and outputs are computed on the matrix cores in transposed form so the softmax
//     probabilities leave the first MFMA already in the operand layout of the second one:
//         S^T[token, head] = K[token, :] . Q^T[:, head]        (v_mfma_f32_16x16x32_bf16)
//         O^T[d, head]    += V^T[d, token] . P^T[token, head]
//     q and p are split into bf16 hi+lo parts (two MFMAs each) so they keep ~16 mantissa bits;
//   * K and V of a (sequence, kv head) share one stream of 64-slot blocks (K rows of the block,
//     then its V in V^T operand order, common.hpp): a wave reads 16 KB contiguous per block with
//     128-bit loads, the four waves of a workgroup 64 KB; position p lives in slot p % capacity
//     (ring buffer for window layers);
//   * contexts of up to ATT_CHUNK slots are one wave's single pass;
//   * longer contexts, few sequences: cut into chunks (flash-decoding), one wave each: partial
//     (max, sum, O) per chunk go to the workspace and a small second kernel merges them with the
//     sink.  The chunk length is a constant, so a row's result is the same whatever else is in
//     the launch;
//   * longer contexts, many sequences (enough to fill the chip with one workgroup per sequence
//     and kv head): the four waves of a workgroup share one (sequence, kv head), wave w taking the
//     64-slot blocks w, w+4, ..., and merge their states with the sink in LDS.  Nothing but the
//     result is written: 20 MB of partials written next to a saturated K/V read stream cost
//     38 us of a 260 us launch (256 sequences of 512..4096 positions), their merge kernel 11 more.
//     Workgroups are dealt longest sequence first;
//   * several query rows may share one sequence's cache (rows_per_seq), each with its own length:
//     the T positions of a prompt are T such rows, which is all the prompt-pass attention is; two
//     consecutive rows of a sequence then share a wave (8 heads each in the 16 operand columns).
#include <stdlib.h>

#include <algorithm>
#include <mutex>
#include <type_traits>

#include "common.hpp"
#include "glue.hpp"

namespace gptoss {

constexpr int ATT_BLOCK = 64;   // slots per inner iteration
constexpr float NEG_BIG = -1.0e30f;

struct AttnParams {
  const float *q;      // [B, n_q, D]
  const bf16_t *kv;    // [B, n_kv, cap/64] blocks of K [64, D] + V [2, D/16, 64, 8]
  const int *lens;     // [B], or nullptr: row b has len_base + b % len_period positions (len_period 0: len_base)
  int len_base, len_period;
  const float *sinks;  // [n_q] or nullptr
  bf16_t *out;         // [B, n_q, D]
  float *part_o;       // [B, max_chunks, n_q, D]
  float *part_ml;      // [B, max_chunks, n_q, 2]
  int B, n_q, n_kv, G, cap, window, max_chunks, max_len;
  int rows_per_seq;    // query rows per cached sequence: row b reads the cache of sequence b / rows_per_seq
  float scale_log2e;   // log2(e) / sqrt(D)
  int only_single;     // chunked kernels: leave rows of more than one chunk to the workgroup-per-row kernel
  const int2 *order;   // workgroup-per-row kernel: (row, its length) by descending slot span (nullptr: row order)
  int2 *order_out;     // chunked kernels: when set, one extra workgroup (the last) writes that order
  int order_buckets;   // slot-span buckets (of 64 slots) the order distinguishes
  const int *seq_map;  // optional: row b of a call with one row per sequence reads the cache of sequence seq_map[b]
};

// Cached positions of query row b: the caller's array, or the rule a host that knows every length
// passes instead (lock-step decoding: one length; a prompt pass: position within the sequence), which
// saves the kernels a dependent load.
__device__ __forceinline__ int row_len(const AttnParams &p, int b) {
  return p.lens ? p.lens[b] : p.len_base + (p.len_period > 0 ? b % p.len_period : 0);
}

struct SeqRange {
  int s_begin, s_end;  // slot range to visit (s_begin is a multiple of 64)
  int t_lo, len;       // active positions are [t_lo, len)
  int chunk, nchunks;  // slots per work item, number of work items
};

// Slots per work item: a constant, so that a row's result does not depend on what else is in the
// launch (one lock-step position or many positions of a prefill).  512 keeps contexts of up to
// 512 positions in one work item (no partial results, no merge kernel), which is what a batch of
// a thousand sequences wants; a single long sequence still gets one work item per 512 slots and
// kv head.
constexpr int ATT_CHUNK = 512;

__device__ __forceinline__ SeqRange seq_range(int len, int cap, int window, int max_len) {
  SeqRange r;
  len = max(0, min(len, max_len));
  r.len = len;
  if (len <= cap) {
    r.t_lo = (window > 0) ? max(0, len - window) : 0;
    r.s_begin = r.t_lo & ~(ATT_BLOCK - 1);
    r.s_end = len;
  } else {  // ring has wrapped: every slot holds one of the last `cap` positions
    r.t_lo = (window > 0) ? max(len - window, len - cap) : len - cap;
    r.s_begin = 0;
    r.s_end = cap;
  }
  r.chunk = ATT_CHUNK;
  r.nchunks = max(1, (r.s_end - r.s_begin + r.chunk - 1) / r.chunk);
  return r;
}

// Rows by descending slot span, rows of a single chunk last: the order in which the
// workgroup-per-row kernel is dealt its rows, so that the longest start first and the launch ends
// on the shortest.  A counting sort over spans in units of 64 slots by one workgroup of 256
// threads; rows of equal span come in any order (the order only schedules, no result depends on
// it).  Each entry carries the row's length, which saves the consumer a dependent load.
constexpr int ATT_ORDER_BUCKETS = 2048;

__device__ __forceinline__ void attn_write_order(const AttnParams &p, int *hist /* [2*(ATT_ORDER_BUCKETS+1)] */) {
  const int tid = threadIdx.x;
  const int nbk = min(p.order_buckets, ATT_ORDER_BUCKETS) + 1;
  int *start = hist + ATT_ORDER_BUCKETS + 1;
  for (int i = tid; i < nbk; i += 256) hist[i] = 0;
  __syncthreads();
  auto key_of = [&](int len) {
    const SeqRange r = seq_range(len, p.cap, p.window, p.max_len);
    return r.nchunks > 1 ? min(nbk - 1, (r.s_end - r.s_begin + ATT_BLOCK - 1) / ATT_BLOCK) : 0;
  };
  for (int b = tid; b < p.B; b += 256) atomicAdd(&hist[key_of(row_len(p, b))], 1);
  __syncthreads();
  // start[k] = number of rows with a larger key; thread t owns `per` consecutive buckets from the top
  const int per = (nbk + 255) / 256;
  int local = 0;
  for (int i = 0; i < per; i++) {
    const int k = nbk - 1 - (tid * per + i);
    if (k >= 0) local += hist[k];
  }
  __shared__ int scan[256];
  scan[tid] = local;
  __syncthreads();
  for (int off = 1; off < 256; off <<= 1) {
    const int v = (tid >= off) ? scan[tid - off] : 0;
    __syncthreads();
    scan[tid] += v;
    __syncthreads();
  }
  int run = scan[tid] - local;   // rows in the buckets above this thread's
  for (int i = 0; i < per; i++) {
    const int k = nbk - 1 - (tid * per + i);
    if (k >= 0) {
      start[k] = run;
      run += hist[k];
    }
  }
  __syncthreads();
  for (int b = tid; b < p.B; b += 256) {
    const int len = row_len(p, b);
    const int pos = atomicAdd(&start[key_of(len)], 1);
    p.order_out[pos] = make_int2(b, len);
  }
}

// PAIR (prompt passes, at most 8 query heads per kv head, ring not wrapped): a wave serves two
// consecutive query rows of one sequence, row b in operand columns 0-7 and row b+1 in columns 8-15,
// from one pass over the K/V blocks either of them needs.  Columns are independent in both MFMAs
// and a block outside a row's own range is a no-op for its columns (scores -inf: max unchanged,
// rescale factor exactly 1, probabilities exactly 0), so each row's result equals that of the
// one-row kernel bit for bit.
//
// WG (many sequences, contexts of more than one chunk): the workgroup's four waves serve one
// (row, kv head); wave w walks the 64-slot blocks w, w+4, ... of the row's slot range and the four
// states are merged in LDS.
//
// The body serves the work of one workgroup index `vblock` of `vgrid`.  HOLD: the wave's output row
// (its G heads) goes to LDS at hold and its place in `out`, in units of D elements, to *hold_row;
// the caller writes it to memory later.
template <int D, bool PAIR, bool WG, bool HOLD = false>
__device__ __forceinline__ void attn_decode_body(const AttnParams &p, const int vblock, const int vgrid,
                                                 bf16_t *hold, int *hold_row) {
  static_assert(!(PAIR && WG), "a workgroup per row serves one row");
  constexpr int KS = D / 32;   // k-steps of the score MFMA
  constexpr int DB = D / 16;   // 16-row blocks of O^T
  constexpr int STRIDE = WG ? 4 * ATT_BLOCK : ATT_BLOCK;   // slots between two blocks of one wave
  // HOLD (the body sits in a loop): the thread index is made opaque per call, so that what is
  // derived from it is computed per row, as in a kernel of its own, instead of being kept in
  // registers across the loop
  int tid_here = threadIdx.x;
  if (HOLD) asm volatile("" : "+v"(tid_here));
  const int lane = tid_here & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid_here >> 6);
  if constexpr (!WG && !HOLD) {   // (the resident kernel writes the order before its loop)
    if (p.order_out && vblock == vgrid - 1) {   // the extra workgroup of a launch that precedes the rows kernel
      __shared__ int order_lds[2 * (ATT_ORDER_BUCKETS + 1)];
      attn_write_order(p, order_lds);
      return;
    }
  }
  const int item = WG ? vblock : vblock * 4 + wave;  // wave-uniform: everything derived from it stays scalar
  const int g = item % p.n_kv;
  const int rest = item / p.n_kv;
  // work units per kv head and chunk: rows, or pairs of rows formed inside each sequence
  // (rows_per_seq odd: the last row of a sequence is a pair of one)
  const int pairs_per_seq = (p.rows_per_seq + 1) >> 1;
  const int units = PAIR ? (p.B / p.rows_per_seq) * pairs_per_seq : p.B;
  const int unit = rest % units;
  const int pair_seq = unit / pairs_per_seq, pair_idx = unit - pair_seq * pairs_per_seq;
  int2 ordered = make_int2(unit, 0);
  if (WG && p.order) {
    ordered = p.order[unit];
    ordered.x = __builtin_amdgcn_readfirstlane(ordered.x);
    ordered.y = __builtin_amdgcn_readfirstlane(ordered.y);
  }
  const int b = PAIR ? pair_seq * p.rows_per_seq + 2 * pair_idx : ordered.x;
  // late chunks first: only long sequences have them, so the sparse part of the grid runs while
  // the chip is still filling and the grid ends on chunk 0, which every sequence has
  const int chunk_id = WG ? 0 : p.max_chunks - 1 - rest / units;
  if (chunk_id < 0) return;
  SeqRange r = seq_range((WG && p.order) ? ordered.y : __builtin_amdgcn_readfirstlane(row_len(p, b)), p.cap, p.window,
                         p.max_len);
  if (WG) {
    if (r.nchunks <= 1) return;   // the whole workgroup: such rows belong to the one-wave kernel
    r.chunk = r.s_end - r.s_begin;  // the workgroup walks the whole range
  }
  // the second row of a pair: the next row of the same sequence, when there is one
  const bool two = PAIR && 2 * pair_idx + 1 < p.rows_per_seq;
  const SeqRange r1 = two ? seq_range(__builtin_amdgcn_readfirstlane(row_len(p, b + 1)), p.cap, p.window, p.max_len) : r;
  const bool act0 = WG || (chunk_id < r.nchunks && !(p.only_single && r.nchunks > 1));
  const bool act1 = two && chunk_id < r1.nchunks && !(p.only_single && r1.nchunks > 1);
  if (!act0 && !act1) return;
  // position held by slot s is s + pos_base, or cap less when that would lie beyond the last one
  const int pos_base = (r.len > 0) ? ((r.len - 1) / p.cap) * p.cap : 0;
  auto slot_pos = [&](int s) {
    int pp = s + pos_base;
    return (pp > r.len - 1) ? pp - p.cap : pp;   // negative for a slot that was never written
  };
  // slot range of this chunk for each row ([0,0) for a row that has no such chunk), their active
  // parts [lo, hi) (PAIR: slot == position), and the union the wave walks
  const int c0_0 = r.s_begin + chunk_id * r.chunk, c0_1 = r1.s_begin + chunk_id * r1.chunk;
  const int hi0 = act0 ? min(r.s_end, c0_0 + r.chunk) : 0, hi1 = act1 ? min(r1.s_end, c0_1 + r1.chunk) : 0;
  const int lo0 = max(c0_0, r.t_lo), lo1 = max(c0_1, r1.t_lo);
  const int c0 = WG ? c0_0 + wave * ATT_BLOCK : !PAIR ? c0_0 : (act0 && act1) ? min(c0_0, c0_1) : act0 ? c0_0 : c0_1;
  const int c1 = !PAIR ? hi0 : max(hi0, hi1);
  const int n = lane & 15, c = lane >> 4;
  const int G = p.G;
  const bool second = PAIR && n >= 8;            // lane's operand column belongs to row b+1
  const int hn = PAIR ? (n & 7) : n;             // head within the kv group
  const bool col_live = hn < G && (!second || two);
  const int bn = (second && two) ? b + 1 : b;    // the column's query row
  const int head = g * G + min(hn, G - 1);
  // the head's sink logit is only needed by the epilogue; requested here, its latency is hidden
  // behind the whole pass instead of sitting between the last block and the output store
  const float sink_logit = p.sinks ? p.sinks[head] : -INFINITY;

  int seq = (p.rows_per_seq > 1) ? b / p.rows_per_seq : b;
  if (p.seq_map) seq = __builtin_amdgcn_readfirstlane(p.seq_map[seq]);
  const bf16_t *plane = p.kv + kv_block_off(seq, g, p.n_kv, p.cap, D, 0);
  // lane's K bytes of a block: slot tb*16 + n, d chunk c*KS*8 .. +KS*8; its V bytes: 8 elements per
  // operand fragment
  const size_t k_lane = (size_t)n * D + c * KS * 8;
  const size_t v_lane = (size_t)KV_BLOCK * D + (size_t)lane * 8;

  u32x4 kreg[2][4][KS], vreg[2][2][DB];
  // One row per (sequence, kv head): nothing reads a K/V block a second time in this launch, so it
  // is requested with the non-temporal hint and does not displace what the caches hold (256
  // sequences of 512..4096 positions 218 -> 197 us, the 1024 x 384 shape of a decode step 147 ->
  // 140 us).  Row pairs of a prompt pass share blocks through L2 and keep the plain load.
  auto fetch = [](const bf16_t *q) {
    if (PAIR) return *reinterpret_cast<const u32x4 *>(q);
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(q));
  };
  auto load_kv = [&](int blk, auto buf) {
    constexpr int R = decltype(buf)::value;
    const bf16_t *bb = plane + (size_t)(blk >> 6) * (2 * KV_BLOCK * D);   // blk is a multiple of 64
#pragma unroll
    for (int tb = 0; tb < 4; tb++)
#pragma unroll
      for (int s = 0; s < KS; s++)
        kreg[R][tb][s] = fetch(bb + (size_t)(tb * 16) * D + k_lane + s * 8);
#pragma unroll
    for (int grp = 0; grp < 2; grp++)
#pragma unroll
      for (int db = 0; db < DB; db++)
        vreg[R][grp][db] = fetch(bb + (size_t)(grp * DB + db) * 512 + v_lane);
  };

  // the first K/V block is requested before anything waits on q, so the cache stream of a work
  // item starts one memory latency earlier
  using R0 = std::integral_constant<int, 0>;
  using R1 = std::integral_constant<int, 1>;
  if (c1 > c0) load_kv(c0, R0{});

  // ---- Q^T operand, split into bf16 hi and lo parts -----------------------------------------
  bf16x8 qh[KS], ql[KS];
  {
    const float *qp = p.q + ((size_t)bn * p.n_q + head) * D + c * KS * 8;
#pragma unroll
    for (int s = 0; s < KS; s++) {
      uint32_t h[4], l[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        float x0 = col_live ? qp[s * 8 + 2 * j] : 0.f, x1 = col_live ? qp[s * 8 + 2 * j + 1] : 0.f;
        bf16_t h0 = f32_to_bf16(x0), h1 = f32_to_bf16(x1);
        h[j] = (uint32_t)h0 | ((uint32_t)h1 << 16);
        l[j] = pack_bf16x2(x0 - bf16_to_f32(h0), x1 - bf16_to_f32(h1));
      }
      qh[s] = as_bf16x8(u32x4{h[0], h[1], h[2], h[3]});
      ql[s] = as_bf16x8(u32x4{l[0], l[1], l[2], l[3]});
    }
  }

  f32x4 o[DB];
#pragma unroll
  for (int db = 0; db < DB; db++) o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = NEG_BIG, l_run = 0.f;

  const int lane_lo = second ? lo1 : lo0, lane_hi = second ? hi1 : hi0;  // PAIR: the column's active slots

  // EDGE = the block holds slots outside the active positions (first/last block of a range, or
  // any block of a wrapped ring): only that variant carries the masking code.
  auto process = [&](int blk, auto buf, auto edge_sel) {
    constexpr int R = decltype(buf)::value;
    constexpr bool EDGE = decltype(edge_sel)::value;
    // scores for 64 slots x 16 head columns
    f32x4 s4[4];
#pragma unroll
    for (int tb = 0; tb < 4; tb++) {
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KS; s++) {
        bf16x8 kf = as_bf16x8(kreg[R][tb][s]);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qh[s], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, ql[s], acc, 0, 0, 0);
      }
      s4[tb] = acc;
    }
    float bmax = NEG_BIG;
#pragma unroll
    for (int tb = 0; tb < 4; tb++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        float v = s4[tb][i] * p.scale_log2e;
        // keep the product a rounded value of its own in both variants of this block (the unmasked
        // one would otherwise fuse it into the subtraction below): a row's result must not depend
        // on which variant its partner row forces
        asm volatile("" : "+v"(v));
        if (EDGE) {
          const int slot = blk + tb * 16 + c * 4 + i;
          const bool ok = PAIR ? (slot >= lane_lo && slot < lane_hi) : (slot < c1 && slot_pos(slot) >= r.t_lo);
          v = ok ? v : -INFINITY;
        }
        s4[tb][i] = v;
        bmax = fmaxf(bmax, v);
      }
    bmax = fmaxf(bmax, __shfl_xor(bmax, 16, 64));
    bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
    const float m_new = fmaxf(m_run, bmax);
    const float alpha = exp2f(m_run - m_new);
    m_run = m_new;
    float psum = 0.f;
    bf16x8 ph[2], pl[2];
#pragma unroll
    for (int grp = 0; grp < 2; grp++) {
      uint32_t h[4], l[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        // operand k index (c, jj): jj<4 -> slot c*4+jj of the first 16, jj>=4 -> of the second 16
        float p0 = exp2f(s4[grp * 2 + (j >> 1)][(j & 1) * 2] - m_new);
        float p1 = exp2f(s4[grp * 2 + (j >> 1)][(j & 1) * 2 + 1] - m_new);
        psum += p0 + p1;
        // p is in [0,1]: truncation to bf16 plus the bf16 remainder keeps 16 mantissa bits
        uint32_t u0 = __float_as_uint(p0), u1 = __float_as_uint(p1);
        h[j] = (u0 >> 16) | (u1 & 0xffff0000u);
        float r0 = p0 - __uint_as_float(u0 & 0xffff0000u), r1 = p1 - __uint_as_float(u1 & 0xffff0000u);
        l[j] = (__float_as_uint(r0) >> 16) | (__float_as_uint(r1) & 0xffff0000u);
      }
      ph[grp] = as_bf16x8(u32x4{h[0], h[1], h[2], h[3]});
      pl[grp] = as_bf16x8(u32x4{l[0], l[1], l[2], l[3]});
    }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int db = 0; db < DB; db++) {
#pragma unroll
      for (int i = 0; i < 4; i++) o[db][i] *= alpha;
    }
#pragma unroll
    for (int grp = 0; grp < 2; grp++)
#pragma unroll
      for (int db = 0; db < DB; db++) {
        u32x4 vv = vreg[R][grp][db];
        if (EDGE) {
          // zero V of inactive slots: never-written cache memory may hold NaN bit patterns
#pragma unroll
          for (int w = 0; w < 4; w++) {
            const int s_lo = blk + grp * 32 + (w >> 1) * 16 + c * 4 + (w & 1) * 2;
            // PAIR: V rows are shared by the two rows' columns, a slot is kept if either row uses it
            auto used = [&](int sl) {
              return PAIR ? ((sl >= lo0 && sl < hi0) || (sl >= lo1 && sl < hi1)) : (sl < c1 && slot_pos(sl) >= r.t_lo);
            };
            const uint32_t keep = (used(s_lo) ? 0x0000ffffu : 0u) | (used(s_lo + 1) ? 0xffff0000u : 0u);
            vv[w] &= keep;
          }
        }
        bf16x8 vf = as_bf16x8(vv);
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, ph[grp], o[db], 0, 0, 0);
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pl[grp], o[db], 0, 0, 0);
      }
  };
  const bool wrapped = r.len > p.cap;
  // a wrapped ring no longer than the window (the engine's window layers) holds active positions
  // in every slot: nothing to mask
  const bool ring_all_active = wrapped && (p.window <= 0 || p.window >= p.cap);
  auto step = [&](int blk, auto buf) {
    // wave-uniform (r.t_lo is a position: comparable with a slot index only while the ring has not wrapped)
    const bool edge = PAIR ? !(two && blk >= lo0 && blk + ATT_BLOCK <= hi0 && blk >= lo1 && blk + ATT_BLOCK <= hi1)
                           : (blk + ATT_BLOCK > c1 || (!ring_all_active && (wrapped || blk < r.t_lo)));
    if (edge) process(blk, buf, std::true_type{});
    else process(blk, buf, std::false_type{});
  };

  if (c1 > c0) {
    // Every call of step() knows how many loads were requested after the block it consumes: one
    // block's worth in the steady state, none for the last block.  (With the request under a
    // condition of its own the wait counts have to assume it was skipped, and every block waits for
    // the one just requested.)
    int blk = c0;
    while (true) {
      if (blk + STRIDE >= c1) { step(blk, R0{}); break; }
      load_kv(blk + STRIDE, R1{});
      step(blk, R0{});
      blk += STRIDE;
      if (blk + STRIDE >= c1) { step(blk, R1{}); break; }
      load_kv(blk + STRIDE, R0{});
      step(blk, R1{});
      blk += STRIDE;
    }
  }

  // ---- per-head totals: sum the partial denominators of the 4 lanes that share a head --------
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if constexpr (WG) {
    // the four waves' states (a wave without a block holds the neutral one: max -1e30, sum 0, O 0)
    // meet in LDS and are merged with the sink in wave order, by the formula of attn_reduce_kernel
    __shared__ float lds_o[4 * 16 * D];
    __shared__ float lds_ml[4 * 16 * 2];
    if (col_live) {
#pragma unroll
      for (int db = 0; db < DB; db++)
        *reinterpret_cast<f32x4 *>(&lds_o[(wave * 16 + n) * D + db * 16 + c * 4]) = o[db];
      if (c == 0) {
        lds_ml[(wave * 16 + n) * 2] = m_run;
        lds_ml[(wave * 16 + n) * 2 + 1] = l_run;
      }
    }
    __syncthreads();
    constexpr int TPP = D / 4;  // threads per head
    const int hm = threadIdx.x / TPP, d4 = (threadIdx.x % TPP) * 4;
    if (hm >= G) return;
    const int hq = g * G + hm;
    const float sink2 = p.sinks ? p.sinks[hq] * 1.4426950408889634f : -INFINITY;
    float M = sink2;
#pragma unroll
    for (int w = 0; w < 4; w++) M = fmaxf(M, lds_ml[(w * 16 + hm) * 2]);
    float denom = exp2f(sink2 - M);
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; w++) {
      const float wgt = exp2f(lds_ml[(w * 16 + hm) * 2] - M);
      denom += lds_ml[(w * 16 + hm) * 2 + 1] * wgt;
      const f32x4 ow = *reinterpret_cast<const f32x4 *>(&lds_o[(w * 16 + hm) * D + d4]);
#pragma unroll
      for (int q = 0; q < 4; q++) acc[q] += ow[q] * wgt;
    }
    u32x2 pk = u32x2{pack_bf16x2(denom > 0.f ? acc[0] / denom : 0.f, denom > 0.f ? acc[1] / denom : 0.f),
                     pack_bf16x2(denom > 0.f ? acc[2] / denom : 0.f, denom > 0.f ? acc[3] / denom : 0.f)};
    *reinterpret_cast<u32x2 *>(p.out + ((size_t)b * p.n_q + hq) * D + d4) = pk;
    return;
  }
  if (!col_live) return;
  if (PAIR && !(second ? act1 : act0)) return;  // this row has no such chunk
  const int hq = g * G + hn;
  const int row_chunks = second ? r1.nchunks : r.nchunks;
  if (row_chunks == 1) {
    float sink2 = sink_logit * 1.4426950408889634f;  // lanes that get here have head == hq
    float M = fmaxf(m_run, sink2);
    float w = exp2f(m_run - M);
    float denom = l_run * w + exp2f(sink2 - M);
    float inv = (denom > 0.f) ? w / denom : 0.f;
    bf16_t *op = HOLD ? hold + hn * D : p.out + ((size_t)bn * p.n_q + hq) * D;
    if (HOLD && lane == 0) *hold_row = b * p.n_q + g * G;
#pragma unroll
    for (int db = 0; db < DB; db++) {
      u32x2 pk = u32x2{pack_bf16x2(o[db][0] * inv, o[db][1] * inv),
                       pack_bf16x2(o[db][2] * inv, o[db][3] * inv)};
      *reinterpret_cast<u32x2 *>(op + db * 16 + c * 4) = pk;
    }
  } else {
    const size_t slot = ((size_t)bn * p.max_chunks + chunk_id) * p.n_q + hq;
    float *po = p.part_o + slot * D;
#pragma unroll
    for (int db = 0; db < DB; db++) *reinterpret_cast<f32x4 *>(po + db * 16 + c * 4) = o[db];
    if (c == 0) {
      p.part_ml[slot * 2] = m_run;
      p.part_ml[slot * 2 + 1] = l_run;
    }
  }
}

template <int D, bool PAIR, bool WG = false>
__global__ __launch_bounds__(256, 2) void attn_decode_kernel(AttnParams p) {
  attn_decode_body<D, PAIR, WG>(p, blockIdx.x, gridDim.x, nullptr, nullptr);
}

// One row per wave and one query row per sequence, as a resident grid: a workgroup walks the
// indices blockIdx.x, blockIdx.x + gridDim.x, ... of the `vgrid` a plain launch would have, keeps
// the finished rows in LDS (ATT_HOLD_SLOTS of up to 16 heads) and writes them to memory when it has
// walked them all.  Output lines written back in the middle of the K/V stream slow its reads far
// beyond their share of the bytes: at 1024 sequences of 384 positions (8.4 MB of outputs against
// 805 MB of K/V) the call takes 125 us with its outputs stored to one small region and 140 us with
// them stored in place, row by row.
constexpr int ATT_HOLD_SLOTS = 16;
template <int D>
__global__ __launch_bounds__(256, 2) void attn_decode_resident_kernel(AttnParams p, int vgrid) {
  __shared__ __attribute__((aligned(16))) bf16_t hold[ATT_HOLD_SLOTS][16 * D];
  __shared__ int hold_row[ATT_HOLD_SLOTS];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  auto flush = [&]() {
    __syncthreads();
    const int chunks = p.G * D / 8;   // 16-byte pieces of one slot's G heads
    for (int idx = threadIdx.x; idx < ATT_HOLD_SLOTS * chunks; idx += 256) {
      const int slot = idx / chunks, ch = idx - slot * chunks;
      const int row = hold_row[slot];
      if (row >= 0)
        *reinterpret_cast<u32x4 *>(p.out + (size_t)row * D + ch * 8) = *reinterpret_cast<const u32x4 *>(&hold[slot][ch * 8]);
    }
    __syncthreads();
    if (threadIdx.x < ATT_HOLD_SLOTS) hold_row[threadIdx.x] = -1;
    __syncthreads();
  };
  // The last index of a launch that precedes the rows kernel writes the row order, not rows.  That
  // code stays outside the loop: inlined into it, it cost the loop 220-340 spilled vector registers
  // and the call took three times as long.
  int n_items = vgrid;
  if (p.order_out) {
    n_items = vgrid - 1;
    if (blockIdx.x == (vgrid - 1) % gridDim.x) {
      __shared__ int order_lds[2 * (ATT_ORDER_BUCKETS + 1)];
      attn_write_order(p, order_lds);
    }
  }
  if (threadIdx.x < ATT_HOLD_SLOTS) hold_row[threadIdx.x] = -1;
  __syncthreads();
  int it = 0;
  for (int vb = blockIdx.x; vb < n_items; vb += gridDim.x, it++) {
    if (it == ATT_HOLD_SLOTS / 4) {   // every slot may be taken: four rows per round of the loop
      flush();
      it = 0;
    }
    const int slot = it * 4 + wave;
    // The parameters are made opaque per round: what the body derives from them (and from the
    // thread index, see there) is then computed per row, as in a kernel of its own, instead of
    // ahead of the loop and kept in registers across it (49 against 65 spilled scalar registers;
    // 1024 sequences of 384 positions 130 against 132.5 us).
    AttnParams q = p;
    asm volatile("" : "+s"(q.q), "+s"(q.kv), "+s"(q.lens), "+s"(q.len_base), "+s"(q.len_period), "+s"(q.sinks), "+s"(q.out),
                 "+s"(q.part_o), "+s"(q.part_ml), "+s"(q.B), "+s"(q.n_q), "+s"(q.n_kv), "+s"(q.G), "+s"(q.cap));
    asm volatile("" : "+s"(q.window), "+s"(q.max_chunks), "+s"(q.max_len), "+s"(q.rows_per_seq), "+s"(q.scale_log2e),
                 "+s"(q.only_single), "+s"(q.order), "+s"(q.order_out), "+s"(q.order_buckets), "+s"(q.seq_map));
    int vb_here = vb, vgrid_here = vgrid;
    asm volatile("" : "+s"(vb_here), "+s"(vgrid_here));
    attn_decode_body<D, false, false, true>(q, vb_here, vgrid_here, hold[slot], &hold_row[slot]);
  }
  flush();
}

// Merge the chunk partials of one (sequence, q head) with the sink logit.  One thread owns four
// consecutive output elements; the chunk loop is unrolled in groups of ATT_RED_UNROLL whose loads
// are all requested before the first use.
constexpr int ATT_RED_UNROLL = 4;

template <int D>
__global__ __launch_bounds__(256) void attn_reduce_kernel(AttnParams p) {
  constexpr int TPP = D / 4;  // threads per (b, head)
  const int pair = blockIdx.x * (256 / TPP) + threadIdx.x / TPP;
  const int d4 = (threadIdx.x % TPP) * 4;
  if (pair >= p.B * p.n_q) return;
  const int b = pair / p.n_q, hq = pair - b * p.n_q;
  const SeqRange r = seq_range(row_len(p, b), p.cap, p.window, p.max_len);
  if (r.nchunks <= 1) return;  // already finished by the first kernel
  const float sink2 = p.sinks ? p.sinks[hq] * 1.4426950408889634f : -INFINITY;
  const size_t slot0 = (size_t)b * p.max_chunks * p.n_q + hq;
  const size_t slot_stride = p.n_q;
  float M = sink2;
  for (int c0 = 0; c0 < r.nchunks; c0 += ATT_RED_UNROLL) {
    float m[ATT_RED_UNROLL];
#pragma unroll
    for (int u = 0; u < ATT_RED_UNROLL; u++)
      m[u] = (c0 + u < r.nchunks) ? p.part_ml[(slot0 + (size_t)(c0 + u) * slot_stride) * 2] : -INFINITY;
#pragma unroll
    for (int u = 0; u < ATT_RED_UNROLL; u++) M = fmaxf(M, m[u]);
  }
  float denom = exp2f(sink2 - M);
  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int c0 = 0; c0 < r.nchunks; c0 += ATT_RED_UNROLL) {
    float m[ATT_RED_UNROLL], l[ATT_RED_UNROLL];
    f32x4 o[ATT_RED_UNROLL];
#pragma unroll
    for (int u = 0; u < ATT_RED_UNROLL; u++) {
      const bool ok = c0 + u < r.nchunks;
      const size_t slot = slot0 + (size_t)(ok ? c0 + u : 0) * slot_stride;
      m[u] = ok ? p.part_ml[slot * 2] : -INFINITY;
      l[u] = ok ? p.part_ml[slot * 2 + 1] : 0.f;
      o[u] = *reinterpret_cast<const f32x4 *>(p.part_o + slot * D + d4);
    }
    // chunks are merged in ascending order, so the result does not depend on the unroll width
#pragma unroll
    for (int u = 0; u < ATT_RED_UNROLL; u++) {
      if (c0 + u < r.nchunks) {
        const float w = exp2f(m[u] - M);
        denom += l[u] * w;
#pragma unroll
        for (int q = 0; q < 4; q++) acc[q] += o[u][q] * w;
      }
    }
  }
  u32x2 pk = u32x2{pack_bf16x2(denom > 0.f ? acc[0] / denom : 0.f, denom > 0.f ? acc[1] / denom : 0.f),
                   pack_bf16x2(denom > 0.f ? acc[2] / denom : 0.f, denom > 0.f ? acc[3] / denom : 0.f)};
  *reinterpret_cast<u32x2 *>(p.out + ((size_t)b * p.n_q + hq) * D + d4) = pk;
}

// Prompt attention for many positions of one sequence: a workgroup of 8 waves serves 16
// consecutive query rows of one (sequence, kv head), two rows per wave as in the PAIR form above,
// and walks the K/V blocks any of them needs ONCE: every block goes from global memory into LDS
// (two buffers, one barrier per block) and the eight waves take their operands from there.  The
// pair form reads a sequence's cache once per row pair, which is quadratic traffic for long
// prompts; here it is read once per 16 rows, and the pass is bound by the matrix instructions.
// Every row sees the arithmetic of the one-wave kernel over its own blocks in ascending order (a
// block outside a row's range is a no-op for its columns), so rows of up to ATT_CHUNK positions
// equal the decode call bit for bit; longer rows are summed in one pass instead of chunk by
// chunk.  Needs slot == position (no wrapped ring) and at most 8 query heads per kv head.
constexpr int TILE_WAVES = 8;
constexpr int TILE_ROWS = 2 * TILE_WAVES;

template <int D>
__global__ __launch_bounds__(TILE_WAVES * 64, 4) void attn_prefill_tile_kernel(AttnParams p) {
  constexpr int KS = D / 32;
  constexpr int DB = D / 16;
  constexpr int BLOCK_BYTES = 2 * KV_BLOCK * D * 2;        // K rows then V fragments of 64 slots
  constexpr int K_BYTES = KV_BLOCK * D * 2;
  constexpr int CHUNKS = BLOCK_BYTES / 16;                   // 16-byte pieces per block
  constexpr int PASSES = CHUNKS / (TILE_WAVES * 64);         // pieces per thread
  constexpr int ROW_CHUNKS = D / 8;                          // 16-byte pieces per K row
  static_assert(PASSES >= 1 && CHUNKS % (TILE_WAVES * 64) == 0, "block size against workgroup size");
  __shared__ __attribute__((aligned(16))) unsigned char lds[2][BLOCK_BYTES];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int T = p.rows_per_seq;
  const int groups = (T + TILE_ROWS - 1) / TILE_ROWS;
  const int n_seq = p.B / T;
  // late row groups first: they walk the most blocks
  const int g = blockIdx.x % p.n_kv;
  const int rest = blockIdx.x / p.n_kv;
  const int seq = rest % n_seq;
  const int rg = groups - 1 - rest / n_seq;
  const int t0 = rg * TILE_ROWS;                             // first row of the group within the sequence
  const int t_last = min(T, t0 + TILE_ROWS) - 1;
  // active positions of row t: [lo(t), hi(t)), hi(t) = len_base + t
  auto row_hi = [&](int t) { return min(p.len_base + t, p.max_len); };
  auto row_lo = [&](int t) { return p.window > 0 ? max(0, row_hi(t) - p.window) : 0; };
  const int blk_begin = row_lo(t0) & ~(ATT_BLOCK - 1);
  const int blk_end = row_hi(t_last);
  // this wave's two rows
  const int tw = t0 + 2 * wave;
  const bool have0 = tw < T, two = tw + 1 < T;
  const int lo0 = have0 ? row_lo(tw) : 0, hi0 = have0 ? row_hi(tw) : 0;
  const int lo1 = two ? row_lo(tw + 1) : 0, hi1 = two ? row_hi(tw + 1) : 0;
  const int b = seq * T + (have0 ? tw : 0);                  // query row of the first of them
  const int n = lane & 15, c = lane >> 4;
  const int G = p.G;
  const bool second = n >= 8;
  const int hn = n & 7;
  const bool col_live = have0 && hn < G && (!second || two);
  const int bn = (second && two) ? b + 1 : b;
  const int head = g * G + min(hn, G - 1);
  const float sink_logit = p.sinks ? p.sinks[head] : -INFINITY;

  const int cache_seq = p.seq_map ? __builtin_amdgcn_readfirstlane(p.seq_map[seq]) : seq;
  const unsigned char *plane =
      reinterpret_cast<const unsigned char *>(p.kv + kv_block_off(cache_seq, g, p.n_kv, p.cap, D, 0));
  // the workgroup's copy of a block: piece i of thread t is bytes (i * 512 + t) * 16; a K piece is
  // chunk j of row r and lands at chunk position j ^ swz(r) of its row, so that the 16 lanes of a
  // fragment read (16 rows, one chunk) hit 16 different 16-byte slots modulo 256 bytes
  auto swz = [](int r) { return D == 64 ? ((r >> 1) & 7) : ((r >> 2) & 3); };
  u32x4 stage[PASSES];
  auto load_block = [&](int blk) {
    const unsigned char *src = plane + (size_t)(blk >> 6) * BLOCK_BYTES;
#pragma unroll
    for (int i = 0; i < PASSES; i++)
      stage[i] = *reinterpret_cast<const u32x4 *>(src + (size_t)(i * TILE_WAVES * 64 + tid) * 16);
  };
  auto store_block = [&](int buf) {
    // the destination is recomputed at every block from a thread id the optimiser cannot see through:
    // hoisted out of the loop it costs a register that the 128-register budget of two workgroups per
    // CU does not have, and a spilled register's reload in the loop waits for the block in flight
    int t_opaque = tid;
    asm volatile("" : "+v"(t_opaque));
#pragma unroll
    for (int i = 0; i < PASSES; i++) {
      const int piece = i * TILE_WAVES * 64 + t_opaque;
      int dst = piece * 16;
      if (piece * 16 < K_BYTES) {
        const int r = piece / ROW_CHUNKS, j = piece % ROW_CHUNKS;
        dst = r * (D * 2) + ((j ^ swz(r)) << 4);
      }
      *reinterpret_cast<u32x4 *>(&lds[buf][dst]) = stage[i];
    }
  };
  if (blk_end > blk_begin) load_block(blk_begin);

  bf16x8 qh[KS], ql[KS];
  {
    const float *qp = p.q + ((size_t)bn * p.n_q + head) * D + c * KS * 8;
#pragma unroll
    for (int s = 0; s < KS; s++) {
      uint32_t h[4], l[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        float x0 = col_live ? qp[s * 8 + 2 * j] : 0.f, x1 = col_live ? qp[s * 8 + 2 * j + 1] : 0.f;
        bf16_t h0 = f32_to_bf16(x0), h1 = f32_to_bf16(x1);
        h[j] = (uint32_t)h0 | ((uint32_t)h1 << 16);
        l[j] = pack_bf16x2(x0 - bf16_to_f32(h0), x1 - bf16_to_f32(h1));
      }
      qh[s] = as_bf16x8(u32x4{h[0], h[1], h[2], h[3]});
      ql[s] = as_bf16x8(u32x4{l[0], l[1], l[2], l[3]});
    }
  }
  f32x4 o[DB];
#pragma unroll
  for (int db = 0; db < DB; db++) o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = NEG_BIG, l_run = 0.f;
  const int lane_lo = second ? lo1 : lo0, lane_hi = second ? hi1 : hi0;

  // one 64-slot block from LDS buffer `buf`: the arithmetic of the one-wave kernel's block step
  auto process = [&](int blk, int buf, auto edge_sel) {
    constexpr bool EDGE = decltype(edge_sel)::value;
    const unsigned char *kb = lds[buf];
    const unsigned char *vb = lds[buf] + K_BYTES;
    f32x4 s4[4];
#pragma unroll
    for (int tb = 0; tb < 4; tb++) {
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
      const int r = tb * 16 + n;
#pragma unroll
      for (int s = 0; s < KS; s++) {
        const bf16x8 kf = as_bf16x8(*reinterpret_cast<const u32x4 *>(kb + r * (D * 2) + (((c * KS + s) ^ swz(r)) << 4)));
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qh[s], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, ql[s], acc, 0, 0, 0);
      }
      s4[tb] = acc;
    }
    float bmax = NEG_BIG;
#pragma unroll
    for (int tb = 0; tb < 4; tb++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        float v = s4[tb][i] * p.scale_log2e;
        asm volatile("" : "+v"(v));   // a rounded product of its own, as in the one-wave kernel
        if (EDGE) {
          const int slot = blk + tb * 16 + c * 4 + i;
          v = (slot >= lane_lo && slot < lane_hi) ? v : -INFINITY;
        }
        s4[tb][i] = v;
        bmax = fmaxf(bmax, v);
      }
    bmax = fmaxf(bmax, __shfl_xor(bmax, 16, 64));
    bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
    const float m_new = fmaxf(m_run, bmax);
    const float alpha = exp2f(m_run - m_new);
    m_run = m_new;
    float psum = 0.f;
    bf16x8 ph[2], pl[2];
#pragma unroll
    for (int grp = 0; grp < 2; grp++) {
      uint32_t h[4], l[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        float p0 = exp2f(s4[grp * 2 + (j >> 1)][(j & 1) * 2] - m_new);
        float p1 = exp2f(s4[grp * 2 + (j >> 1)][(j & 1) * 2 + 1] - m_new);
        psum += p0 + p1;
        uint32_t u0 = __float_as_uint(p0), u1 = __float_as_uint(p1);
        h[j] = (u0 >> 16) | (u1 & 0xffff0000u);
        float r0 = p0 - __uint_as_float(u0 & 0xffff0000u), r1 = p1 - __uint_as_float(u1 & 0xffff0000u);
        l[j] = (__float_as_uint(r0) >> 16) | (__float_as_uint(r1) & 0xffff0000u);
      }
      ph[grp] = as_bf16x8(u32x4{h[0], h[1], h[2], h[3]});
      pl[grp] = as_bf16x8(u32x4{l[0], l[1], l[2], l[3]});
    }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int db = 0; db < DB; db++) {
#pragma unroll
      for (int i = 0; i < 4; i++) o[db][i] *= alpha;
    }
#pragma unroll
    for (int grp = 0; grp < 2; grp++)
#pragma unroll
      for (int db = 0; db < DB; db++) {
        u32x4 vv = *reinterpret_cast<const u32x4 *>(vb + (grp * DB + db) * 1024 + lane * 16);
        if (EDGE) {
#pragma unroll
          for (int w = 0; w < 4; w++) {
            const int s_lo = blk + grp * 32 + (w >> 1) * 16 + c * 4 + (w & 1) * 2;
            auto used = [&](int sl) { return (sl >= lo0 && sl < hi0) || (sl >= lo1 && sl < hi1); };
            const uint32_t keep = (used(s_lo) ? 0x0000ffffu : 0u) | (used(s_lo + 1) ? 0xffff0000u : 0u);
            vv[w] &= keep;
          }
        }
        bf16x8 vf = as_bf16x8(vv);
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, ph[grp], o[db], 0, 0, 0);
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pl[grp], o[db], 0, 0, 0);
      }
  };

  int buf = 0;
  for (int blk = blk_begin; blk < blk_end; blk += ATT_BLOCK, buf ^= 1) {
    store_block(buf);
    __syncthreads();   // block `blk` is complete in lds[buf]; every wave is done with the other buffer's previous use
    if (blk + ATT_BLOCK < blk_end) load_block(blk + ATT_BLOCK);
    // the wave's rows: first block that holds an active position of either row .. their last one
    const bool mine = (have0 && blk < hi0 && blk + ATT_BLOCK > lo0) || (two && blk < hi1 && blk + ATT_BLOCK > lo1);
    if (mine) {
      const bool edge = !(two && blk >= lo0 && blk + ATT_BLOCK <= hi0 && blk >= lo1 && blk + ATT_BLOCK <= hi1);
      if (edge) process(blk, buf, std::true_type{});
      else process(blk, buf, std::false_type{});
    }
  }

  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if (!col_live) return;
  const int hq = g * G + hn;
  const float sink2 = sink_logit * 1.4426950408889634f;
  const float M = fmaxf(m_run, sink2);
  const float w = exp2f(m_run - M);
  const float denom = l_run * w + exp2f(sink2 - M);
  const float inv = (denom > 0.f) ? w / denom : 0.f;
  bf16_t *op = p.out + ((size_t)bn * p.n_q + hq) * D;
#pragma unroll
  for (int db = 0; db < DB; db++) {
    u32x2 pk = u32x2{pack_bf16x2(o[db][0] * inv, o[db][1] * inv), pack_bf16x2(o[db][2] * inv, o[db][3] * inv)};
    *reinterpret_cast<u32x2 *>(op + db * 16 + c * 4) = pk;
  }
}

// Bulk cache write: rows [B, n_tok, n_kv, D] -> the block layout of common.hpp.
__global__ __launch_bounds__(256) void kv_cache_write_kernel(bf16_t *__restrict__ kv,
                                                             const bf16_t *__restrict__ k_rows,
                                                             const bf16_t *__restrict__ v_rows, int B,
                                                             int n_kv, int D, int cap, int pos0,
                                                             int n_tok) {
  const size_t total = (size_t)B * n_tok * n_kv * D;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
    int d = (int)(i % D);
    size_t r = i / D;
    int g = (int)(r % n_kv);
    r /= n_kv;
    int t = (int)(r % n_tok);
    int b = (int)(r / n_tok);
    int slot = (pos0 + t) % cap;
    const size_t base = kv_block_off(b, g, n_kv, cap, D, slot);
    kv[base + kv_k_elem(slot, d, D)] = k_rows[i];
    kv[base + kv_v_elem(slot, d, D)] = v_rows[i];
  }
}

// Positions per sequence from which a prompt pass takes the tiled kernel.  GPTOSS_ATTN_TILE_MIN_ROWS
// overrides it (tests run both forms on the same inputs).
static int attn_tile_min_rows() {
  static const int v = [] {
    const char *e = getenv("GPTOSS_ATTN_TILE_MIN_ROWS");
    const int n = e ? atoi(e) : 0;
    return n > 0 ? n : 32;
  }();
  return v;
}

struct AttnPlan {
  int max_chunks;
  bool wide;          // many sequences: rows of more than one chunk get a workgroup each, no partials
  size_t order_bytes, part_o_bytes, part_ml_bytes;
};

// Enough sequences that one workgroup per (sequence, kv head) fills the chip twice over: then long
// rows are served by the workgroup-per-row kernel.  A property of the launch shape alone, so a
// row's arithmetic depends on the number of sequences in the call but never on their contents.
static bool attn_wide(int n_seq, int n_kv) { return (long long)n_seq * n_kv >= 512; }

static AttnPlan attn_plan(int B, int rows_per_seq, int n_q, int n_kv, int D, int span) {
  AttnPlan pl;
  // most work items any row can have: a slot range can start up to 63 slots before the first
  // active position
  const int longest = span + ATT_BLOCK - 1;
  pl.max_chunks = (longest + ATT_CHUNK - 1) / ATT_CHUNK;
  if (pl.max_chunks < 1) pl.max_chunks = 1;
  pl.wide = pl.max_chunks > 1 && attn_wide(B / std::max(1, rows_per_seq), n_kv);
  pl.order_bytes = align_up((size_t)B * sizeof(int2), 256);
  const int stored_chunks = pl.wide ? 0 : pl.max_chunks;
  pl.part_o_bytes = align_up((size_t)B * stored_chunks * n_q * D * sizeof(float), 256);
  pl.part_ml_bytes = align_up((size_t)B * stored_chunks * n_q * 2 * sizeof(float), 256);
  return pl;
}

}  // namespace gptoss

using namespace gptoss;

extern "C" size_t gptoss_kv_cache_bytes(int B, int n_kv, int head_dim, int capacity) {
  if (B <= 0 || n_kv <= 0 || head_dim <= 0 || capacity <= 0 || capacity % KV_BLOCK) return 0;
  return (size_t)B * n_kv * kv_plane_elems(capacity, head_dim) * sizeof(bf16_t);
}

extern "C" int gptoss_kv_cache_write(void *kv_cache, const void *k_rows, const void *v_rows, int B, int n_kv,
                                     int head_dim, int capacity, int pos0, int n_tok, void *stream) {
  GPTOSS_REQUIRE(kv_cache && k_rows && v_rows, GPTOSS_ERR_NULL, "kv_cache_write: null pointer");
  GPTOSS_REQUIRE(B > 0 && n_kv > 0 && (head_dim == 32 || head_dim == 64) && capacity > 0 &&
                     capacity % 64 == 0 && pos0 >= 0 && n_tok >= 0 && n_tok <= capacity,
                 GPTOSS_ERR_DIM,
                 "kv_cache_write: need head_dim in {32,64}, capacity %% 64 == 0, n_tok <= capacity "
                 "(D=%d capacity=%d n_tok=%d)", head_dim, capacity, n_tok);
  if (n_tok == 0) return GPTOSS_OK;
  size_t total = (size_t)B * n_tok * n_kv * head_dim;
  int grid = (int)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256);
  kv_cache_write_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((bf16_t *)kv_cache, (const bf16_t *)k_rows,
                                                               (const bf16_t *)v_rows, B, n_kv, head_dim, capacity,
                                                               pos0, n_tok);
  GPTOSS_LAUNCH_CHECK("kv_cache_write_kernel");
  return GPTOSS_OK;
}

extern "C" size_t gptoss_attn_workspace_bytes(int B, int n_q, int n_kv, int head_dim, int max_len) {
  if (B <= 0 || n_q <= 0 || n_kv <= 0 || head_dim <= 0 || max_len <= 0) return 0;
  // the row order of the workgroup-per-row kernel, or the chunk partials of the chunked one: sized
  // for the larger of the two whatever window/capacity the call then has
  int max_chunks = (max_len + ATT_BLOCK - 1 + ATT_CHUNK - 1) / ATT_CHUNK;
  return align_up((size_t)B * sizeof(int2), 256) +
         align_up((size_t)B * max_chunks * n_q * head_dim * sizeof(float), 256) +
         align_up((size_t)B * max_chunks * n_q * 2 * sizeof(float), 256);
}

// Workgroups of attn_decode_resident_kernel<D> that the device holds at once (asked of the runtime
// once per device and head size).
template <int D>
static int attn_resident_wgs(int *out) {
  constexpr int MAX_DEV = 64;
  static std::mutex mu;
  static int wgs[MAX_DEV];
  int dev = 0;
  GPTOSS_HIP(hipGetDevice(&dev));
  GPTOSS_REQUIRE(dev >= 0 && dev < MAX_DEV, GPTOSS_ERR_STATE, "attn_decode: device ordinal %d outside 0..%d", dev, MAX_DEV - 1);
  std::lock_guard<std::mutex> lock(mu);
  if (wgs[dev] == 0) {
    int per_cu = 0, cus = 0;
    GPTOSS_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attn_decode_resident_kernel<D>, 256, 0));
    GPTOSS_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    wgs[dev] = std::max(1, per_cu) * std::max(1, cus);
  }
  *out = wgs[dev];
  return GPTOSS_OK;
}

// B query rows; row b reads the cache of sequence b / rows_per_seq up to its own lens[b]
// (lens == nullptr: row b has len_base + b % len_period positions)
static int attn_launch(const float *q, const void *kv_cache, const int *lens,
                       const float *sinks, void *out, int B, int rows_per_seq, int n_q, int n_kv,
                       int head_dim, int capacity, int window, int max_len, void *workspace,
                       size_t workspace_bytes, void *stream, int len_base = 0, int len_period = 0,
                       const int *seq_map = nullptr) {
  GPTOSS_REQUIRE(q && kv_cache && out, GPTOSS_ERR_NULL, "attn_decode: null pointer");
  if (!lens && len_base == 0) len_base = max_len;  // no lengths given: every row has max_len positions
  GPTOSS_REQUIRE(B > 0 && n_q > 0 && n_kv > 0 && n_q % n_kv == 0 && n_q / n_kv <= 16, GPTOSS_ERR_DIM,
                 "attn_decode: need n_q %% n_kv == 0 and n_q/n_kv <= 16 (n_q=%d n_kv=%d)", n_q, n_kv);
  GPTOSS_REQUIRE(head_dim == 32 || head_dim == 64, GPTOSS_ERR_DIM,
                 "attn_decode: head_dim must be 32 or 64 (got %d)", head_dim);
  GPTOSS_REQUIRE(capacity > 0 && capacity % 64 == 0 && window >= 0 && max_len > 0, GPTOSS_ERR_DIM,
                 "attn_decode: need capacity %% 64 == 0, window >= 0, max_len > 0 (capacity=%d)", capacity);
  GPTOSS_REQUIRE(max_len <= capacity || (window > 0 && window <= capacity), GPTOSS_ERR_DIM,
                 "attn_decode: the cache must hold every active position (capacity=%d window=%d max_len=%d)",
                 capacity, window, max_len);
  GPTOSS_REQUIRE(aligned(q, 16) && aligned(kv_cache, 16) && aligned(out, 8),
                 GPTOSS_ERR_ALIGN, "attn_decode: pointers must be 16-byte aligned");
  // longest slot range one sequence can visit: the whole ring once it may have wrapped
  int span = (max_len > capacity) ? capacity
                                  : ((window > 0 && window < max_len) ? window : max_len);
  AttnPlan pl = attn_plan(B, rows_per_seq, n_q, n_kv, head_dim, span);
  const size_t need = pl.order_bytes + pl.part_o_bytes + pl.part_ml_bytes;
  GPTOSS_REQUIRE(workspace && aligned(workspace, 256) && workspace_bytes >= need, GPTOSS_ERR_WORKSPACE,
                 "attn_decode: workspace missing, misaligned or smaller than %zu bytes", need);
  AttnParams p;
  p.q = q;
  p.kv = (const bf16_t *)kv_cache;
  p.lens = lens;
  p.len_base = len_base;
  p.len_period = len_period;
  p.sinks = sinks;
  p.out = (bf16_t *)out;
  int2 *order = (int2 *)workspace;
  p.part_o = (float *)((unsigned char *)workspace + pl.order_bytes);
  p.part_ml = (float *)((unsigned char *)workspace + pl.order_bytes + pl.part_o_bytes);
  p.B = B;
  p.rows_per_seq = rows_per_seq;
  p.n_q = n_q;
  p.n_kv = n_kv;
  p.G = n_q / n_kv;
  p.cap = capacity;
  p.window = window;
  p.max_chunks = pl.wide ? 1 : pl.max_chunks;
  p.max_len = max_len;
  p.scale_log2e = 1.4426950408889634f / sqrtf((float)head_dim);
  p.only_single = pl.wide ? 1 : 0;
  p.order = nullptr;
  p.order_out = pl.wide ? order : nullptr;
  p.order_buckets = (span + 2 * ATT_BLOCK - 1) / ATT_BLOCK;
  p.seq_map = seq_map;
  hipStream_t s = (hipStream_t)stream;
  // prompt passes put two consecutive rows of a sequence into one wave when the 16 operand columns
  // hold both rows' query heads and no ring can have wrapped (slot == position)
  const bool pair = rows_per_seq > 1 && B % rows_per_seq == 0 && p.G <= 8 && max_len <= capacity;
  if (pair && rows_per_seq >= attn_tile_min_rows()) {
    // many positions per sequence: 16 rows per workgroup share every K/V block through LDS
    const long long wgs = (long long)(B / rows_per_seq) * n_kv * ((rows_per_seq + TILE_ROWS - 1) / TILE_ROWS);
    GPTOSS_REQUIRE(wgs < (1ll << 31), GPTOSS_ERR_DIM, "attn_prefill: too many row groups (%lld)", wgs);
    TraceScope ts("attn_prefill_tiles", s);
    if (head_dim == 64) attn_prefill_tile_kernel<64><<<(int)wgs, TILE_WAVES * 64, 0, s>>>(p);
    else attn_prefill_tile_kernel<32><<<(int)wgs, TILE_WAVES * 64, 0, s>>>(p);
    GPTOSS_LAUNCH_CHECK("attn_prefill_tile_kernel");
    return GPTOSS_OK;
  }
  long long items = (long long)(pair ? (B / rows_per_seq) * ((rows_per_seq + 1) / 2) : B) * n_kv * p.max_chunks;
  int grid = (int)((items + 3) / 4) + (pl.wide ? 1 : 0);
  {
    TraceScope ts("attn_decode", s);
    // one row per sequence: a resident grid that keeps its output rows in LDS until the end (it
    // writes them 16 bytes at a time; an output that is only 8-byte aligned gets the plain launch)
    const bool hold_rows = !pair && aligned(out, 16);
    int resident = 0;
    if (hold_rows) {
      const int rc = head_dim == 64 ? attn_resident_wgs<64>(&resident) : attn_resident_wgs<32>(&resident);
      if (rc != GPTOSS_OK) return rc;
    }
    if (head_dim == 64) {
      if (pair) attn_decode_kernel<64, true><<<grid, 256, 0, s>>>(p);
      else if (hold_rows) attn_decode_resident_kernel<64><<<std::min(grid, resident), 256, 0, s>>>(p, grid);
      else attn_decode_kernel<64, false><<<grid, 256, 0, s>>>(p);
    } else {
      if (pair) attn_decode_kernel<32, true><<<grid, 256, 0, s>>>(p);
      else if (hold_rows) attn_decode_resident_kernel<32><<<std::min(grid, resident), 256, 0, s>>>(p, grid);
      else attn_decode_kernel<32, false><<<grid, 256, 0, s>>>(p);
    }
  }
  GPTOSS_LAUNCH_CHECK("attn_decode_kernel");
  if (pl.wide) {
    // rows of more than one chunk: a workgroup each, longest first (the order was written by the
    // extra workgroup of the launch above)
    p.order = order;
    p.order_out = nullptr;
    TraceScope ts("attn_decode_rows", s);
    const int wgrid = B * n_kv;
    if (head_dim == 64) attn_decode_kernel<64, false, true><<<wgrid, 256, 0, s>>>(p);
    else attn_decode_kernel<32, false, true><<<wgrid, 256, 0, s>>>(p);
    GPTOSS_LAUNCH_CHECK("attn_decode_kernel (workgroup per row)");
  } else if (pl.max_chunks > 1) {
    int per_block = 256 / (head_dim / 4);
    int rgrid = (B * n_q + per_block - 1) / per_block;
    TraceScope ts("attn_reduce", s);
    if (head_dim == 64) attn_reduce_kernel<64><<<rgrid, 256, 0, s>>>(p);
    else attn_reduce_kernel<32><<<rgrid, 256, 0, s>>>(p);
    GPTOSS_LAUNCH_CHECK("attn_reduce_kernel");
  }
  return GPTOSS_OK;
}

extern "C" int gptoss_attn_decode(const float *q, const void *kv_cache, const int *lens, const float *sinks,
                                  void *out, int B, int n_q, int n_kv, int head_dim, int capacity, int window,
                                  int max_len, void *workspace, size_t workspace_bytes, void *stream) {
  return attn_launch(q, kv_cache, lens, sinks, out, B, 1, n_q, n_kv, head_dim, capacity, window,
                     max_len, workspace, workspace_bytes, stream);
}

int gptoss::attn_decode_mapped(const float *q, const void *kv_cache, const int *lens, const float *sinks, void *out,
                               int B, int n_q, int n_kv, int head_dim, int capacity, int window, int max_len,
                               void *workspace, size_t workspace_bytes, void *stream, const int *seq_map) {
  return attn_launch(q, kv_cache, lens, sinks, out, B, 1, n_q, n_kv, head_dim, capacity, window, max_len, workspace,
                     workspace_bytes, stream, 0, 0, seq_map);
}

// ---- the same call without a caller workspace ---------------------------------------------------
// The chunk partials live in a device array that is part of the library image: every GPU the
// library is loaded on holds its own copy until the process ends.  In host code the array's name
// is only a handle; its device address is looked up once per device and kept.
constexpr size_t ATTN_STATIC_SCRATCH_BYTES = (size_t)64 << 20;
static __device__ __align__(256) unsigned char scratch[ATTN_STATIC_SCRATCH_BYTES];

constexpr int ATTN_MAX_DEVICES = 64;
static std::mutex g_scratch_mutex;
static void *g_scratch_ptr[ATTN_MAX_DEVICES];  // per device, nullptr until looked up there

// address of the calling thread's current device's copy of `scratch`
static int static_scratch(void **ptr) {
  int dev = -1;
  GPTOSS_HIP(hipGetDevice(&dev));
  GPTOSS_REQUIRE(dev >= 0 && dev < ATTN_MAX_DEVICES, GPTOSS_ERR_STATE,
                 "attn_decode_static: device ordinal %d outside 0..%d", dev, ATTN_MAX_DEVICES - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    GPTOSS_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    GPTOSS_REQUIRE(p && aligned(p, 256), GPTOSS_ERR_HIP, "attn_decode_static: no address for the scratch array");
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return GPTOSS_OK;
}

extern "C" size_t gptoss_attn_decode_static_max_bytes(void) { return ATTN_STATIC_SCRATCH_BYTES; }

extern "C" int gptoss_attn_decode_static(const float *q, const void *kv_cache, const int *lens,
                                         const float *sinks, void *out, int B, int n_q, int n_kv, int head_dim,
                                         int capacity, int window, int max_len, void *stream) {
  const size_t need = gptoss_attn_workspace_bytes(B, n_q, n_kv, head_dim, max_len);
  GPTOSS_REQUIRE(need > 0, GPTOSS_ERR_DIM, "attn_decode_static: non-positive dimension");
  GPTOSS_REQUIRE(need <= ATTN_STATIC_SCRATCH_BYTES, GPTOSS_ERR_WORKSPACE,
                 "attn_decode_static: B=%d n_q=%d head_dim=%d max_len=%d needs %zu bytes of chunk partials, the "
                 "built-in scratch holds %zu; use gptoss_attn_decode with a workspace", B, n_q, head_dim,
                 max_len, need, ATTN_STATIC_SCRATCH_BYTES);
  void *ptr = nullptr;
  int rc = static_scratch(&ptr);
  if (rc != GPTOSS_OK) return rc;
  // every partial a merge reads was written by this call's first kernel: nothing to clear
  return attn_launch(q, kv_cache, lens, sinks, out, B, 1, n_q, n_kv, head_dim, capacity, window, max_len, ptr,
                     ATTN_STATIC_SCRATCH_BYTES, stream);
}

extern "C" size_t gptoss_attn_prefill_workspace_bytes(int B, int T, int n_q, int n_kv, int head_dim,
                                                      int max_len) {
  if (B <= 0 || T <= 0) return 0;
  size_t rows = (size_t)B * T;
  if (rows > 0x7fffffff) return 0;
  return align_up(rows * sizeof(int), 256) + gptoss_attn_workspace_bytes((int)rows, n_q, n_kv, head_dim, max_len);
}

extern "C" int gptoss_attn_prefill(const float *q, const void *kv_cache, const float *sinks, void *out, int B, int T, int pos0, int n_q,
                                   int n_kv, int head_dim, int capacity, int window, void *workspace,
                                   size_t workspace_bytes, void *stream) {

  GPTOSS_REQUIRE(B > 0 && T > 0 && pos0 >= 0 && (long long)B * T < (1ll << 24), GPTOSS_ERR_DIM,
                 "attn_prefill: need B > 0, T > 0, pos0 >= 0 and B*T < 2^24 (B=%d T=%d)", B, T);
  GPTOSS_REQUIRE(window == 0 || pos0 + T <= capacity, GPTOSS_ERR_DIM,
                 "attn_prefill: a windowed cache must hold all %d positions (capacity=%d): rows of one "
                 "launch read the cache as it is after the last position was written", pos0 + T, capacity);
  const int rows = B * T;
  const size_t lens_bytes = align_up((size_t)rows * sizeof(int), 256);
  GPTOSS_REQUIRE(workspace && aligned(workspace, 256) && workspace_bytes > lens_bytes, GPTOSS_ERR_WORKSPACE,
                 "attn_prefill: workspace missing, misaligned or too small");
  // row (b, t) has pos0 + t + 1 positions: a rule the kernels evaluate, no array of lengths
  return attn_launch(q, kv_cache, nullptr, sinks, out, rows, T, n_q, n_kv, head_dim, capacity, window,
                     pos0 + T, (unsigned char *)workspace + lens_bytes, workspace_bytes - lens_bytes, stream,
                     pos0 + 1, T);
}
