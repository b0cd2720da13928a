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
//   * K is stored [sequence, kv head, slot, d]: a wave reads 16 slots x 128 B = 2 KB contiguous
//     per 128-bit load pair; V is stored in 32-slot blocks already in V^T operand order, 1 KB
//     contiguous per load; position p lives in slot p % capacity (ring buffer for window layers);
//   * long contexts are cut into chunks (flash-decoding): partial (max, sum, O) per chunk, merged
//     with the sink by a small second kernel; sequences that fit one chunk finish in the first.
#include <type_traits>

#include "common.hpp"
#include "glue.hpp"

namespace gptoss {

constexpr int ATT_BLOCK = 64;   // slots per inner iteration
constexpr float NEG_BIG = -1.0e30f;

struct AttnParams {
  const float *q;      // [B, n_q, D]
  const bf16_t *kc;    // [B, n_kv, cap, D]
  const bf16_t *vc;    // [B, n_kv, cap/32, D/16, 64, 8]
  const int *lens;     // [B]
  const float *sinks;  // [n_q] or nullptr
  bf16_t *out;         // [B, n_q, D]
  float *part_o;       // [B, max_chunks, n_q, D]
  float *part_ml;      // [B, max_chunks, n_q, 2]
  int *ticket;         // work counter (zero on entry) for the dynamically dealt tail, or nullptr
  int B, n_q, n_kv, G, cap, window, chunk, max_chunks, max_len;
  float scale_log2e;   // log2(e) / sqrt(D)
};

struct SeqRange {
  int s_begin, s_end;  // slot range to visit (s_begin is a multiple of 64)
  int t_lo, len;       // active positions are [t_lo, len)
  int nchunks;         // chunks the range is cut into (at most `chunk` slots each) ...
  int chunk;           // ... of this many slots: the range split evenly, rounded up to 64
};

__device__ __forceinline__ SeqRange seq_range(int len, int cap, int window, int chunk, int max_len) {
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
  const int span = r.s_end - r.s_begin;
  r.nchunks = max(1, (span + chunk - 1) / chunk);
  r.chunk = max(64, ((span + r.nchunks - 1) / r.nchunks + 63) & ~63);
  return r;
}

constexpr int ATT_THREADS = 512;     // one workgroup of 8 waves per CU (two waves per SIMD)
constexpr int ATT_WAVES = ATT_THREADS / 64;
constexpr int ATT_MAX_BATCH = 2048;  // sequences per launch (four LDS ints each)

// Persistent kernel.  Work item of a wave = (sequence, kv head, chunk of the sequence's slot range);
// a sequence's range is cut into equal chunks, so item sizes only differ between sequences.
// Every workgroup first builds the same item order in LDS from the sequence lengths: sequences
// sorted by chunk size, largest first (counting sort over 32-slot size classes), each contributing
// its chunks x kv heads.  Wave w takes item w of round 0, item n_waves-1-w of round 1, item w of
// round 2, ...: a snake over a list sorted by size gives every wave nearly the same number of
// slots.  Waves do not stream equally fast (the second wave of a SIMD gets less than the first,
// and CUs differ by some 10 %), so when there are at least three rounds the last full round and
// the remainder - the smallest items - are handed out through a counter instead, one atomic per
// item, requested a whole item before its result is needed.  A wave's K/V double buffer keeps running across its items: while the
// last block of an item is multiplied, the first block of the wave's next item is already on its
// way.
template <int D>
__global__ __launch_bounds__(ATT_THREADS, 1) void attn_decode_kernel(AttnParams p) {
  constexpr int KS = D / 32;   // k-steps of the score MFMA
  constexpr int DB = D / 16;   // 16-row blocks of O^T
  extern __shared__ int att_smem[];
  int *s_len = att_smem;             // [B]
  int *s_pfull = att_smem + p.B;     // [B+1] exclusive prefix of the chunk counts, sorted order
  int *s_plist = s_pfull + p.B + 1;  // [B] sequences ordered by chunk size, largest first
  int *s_bkt = s_plist + p.B;        // [B] size class | chunk count << 4
  __shared__ int s_wsum[ATT_WAVES];
  __shared__ int s_bucket[16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  // ---- item order --------------------------------------------------------------------------
  if (threadIdx.x < 16) s_bucket[threadIdx.x] = 0;
  __syncthreads();
  for (int b = threadIdx.x; b < p.B; b += ATT_THREADS) {
    const int len = p.lens[b];
    const SeqRange r = seq_range(len, p.cap, p.window, p.chunk, p.max_len);
    const int bucket = 15 - min(15, (r.chunk - 1) >> 5);  // 0 = largest chunks
    s_len[b] = len;
    s_bkt[b] = bucket | (r.nchunks << 4);
    atomicAdd(&s_bucket[bucket], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int k = 0; k < 16; k++) {  // bucket counts -> bucket start cursors
      int c = s_bucket[k];
      s_bucket[k] = acc;
      acc += c;
    }
  }
  __syncthreads();
  // scatter the sequences into their buckets; the order inside a bucket does not matter (every
  // item's result is independent of the item order)
  for (int b = threadIdx.x; b < p.B; b += ATT_THREADS) s_plist[atomicAdd(&s_bucket[s_bkt[b] & 15], 1)] = b;
  __syncthreads();
  // exclusive prefix of the chunk counts in sorted order
  int running = 0;
  for (int r0 = 0; r0 < p.B; r0 += ATT_THREADS) {
    const int rk = r0 + threadIdx.x;
    const int cnt = (rk < p.B) ? (s_bkt[s_plist[rk]] >> 4) : 0;
    int inc = cnt;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      int o = __shfl_up(inc, d, 64);
      if (lane >= d) inc += o;
    }
    if (lane == 63) s_wsum[wave] = inc;
    __syncthreads();
    int base = running;
    for (int w = 0; w < wave; w++) base += s_wsum[w];
    if (rk < p.B) s_pfull[rk] = base + inc - cnt;
    for (int w = 0; w < ATT_WAVES; w++) running += s_wsum[w];
    __syncthreads();
  }
  if (threadIdx.x == 0) s_pfull[p.B] = running;
  __syncthreads();
  const int n_items = s_pfull[p.B] * p.n_kv;
  const int n_waves = gridDim.x * ATT_WAVES;
  const int wave_id = blockIdx.x * ATT_WAVES + wave;
  // item of this wave in round k of the snake
  auto item_index = [&](int k) { return k * n_waves + ((k & 1) ? n_waves - 1 - wave_id : wave_id); };
  const int full_rounds = n_items / n_waves;
  const bool use_tickets = p.ticket != nullptr && full_rounds >= 3;
  const int static_rounds = use_tickets ? full_rounds - 1 : 0x3fffffff;
  const int pool_base = use_tickets ? static_rounds * n_waves : 0;
  const int n = lane & 15, c = lane >> 4;
  const int G = p.G;
  // lane's K bytes for slot block `blk`: slot blk + tb*16 + n, d chunk c*KS*8 .. +KS*8
  const size_t k_lane = (size_t)n * D + c * KS * 8;
  const size_t v_lane = (size_t)lane * 8;

  struct Item {
    int b, g, chunk_id, nchunks, len, t_lo, c0, c1;
    bool has;  // at least one slot block
  };
  auto decode = [&](int i) {
    Item it;
    const int pair = i / p.n_kv;
    it.g = i - pair * p.n_kv;
    int lo = 0, hi = p.B;  // largest rank with pfull[rank] <= pair
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (s_pfull[mid] <= pair) lo = mid;
      else hi = mid;
    }
    int b = s_plist[lo];
    int chunk_id = pair - s_pfull[lo];
    b = __builtin_amdgcn_readfirstlane(b);
    const SeqRange r = seq_range(__builtin_amdgcn_readfirstlane(s_len[b]), p.cap, p.window, p.chunk, p.max_len);
    it.b = b;
    it.chunk_id = __builtin_amdgcn_readfirstlane(chunk_id);
    it.nchunks = r.nchunks;
    it.len = r.len;
    it.t_lo = r.t_lo;
    it.c0 = r.s_begin + it.chunk_id * r.chunk;
    it.c1 = min(r.s_end, it.c0 + r.chunk);
    it.has = it.c1 > it.c0;
    return it;
  };

  int round = 0;
  int i = item_index(0);  // wave-uniform: everything derived from it stays scalar
  if (i >= n_items) return;
  Item cur = decode(i);

  u32x4 kreg[2][4][KS], vreg[2][2][DB];
  auto load_kv = [&](const Item &it, int blk, auto buf) {
    constexpr int R = decltype(buf)::value;
    const bf16_t *kbase = p.kc + ((size_t)(it.b * p.n_kv + it.g) * p.cap) * D;
    const bf16_t *vbase = p.vc + ((size_t)(it.b * p.n_kv + it.g) * p.cap) * D;
#pragma unroll
    for (int tb = 0; tb < 4; tb++)
#pragma unroll
      for (int s = 0; s < KS; s++)
        kreg[R][tb][s] = *reinterpret_cast<const u32x4 *>(kbase + (size_t)(blk + tb * 16) * D + k_lane + s * 8);
#pragma unroll
    for (int grp = 0; grp < 2; grp++)
#pragma unroll
      for (int db = 0; db < DB; db++)
        vreg[R][grp][db] = *reinterpret_cast<const u32x4 *>(
            vbase + ((size_t)((blk >> 5) + grp) * DB + db) * 512 + v_lane);
  };
  using R0 = std::integral_constant<int, 0>;
  using R1 = std::integral_constant<int, 1>;
  bool have_first = false;  // the first block of `cur` is already in (or on its way to) buffer 0

  while (true) {
    // the wave's next item: by position while the static rounds last, then by ticket.  The ticket
    // is requested now and only read when the last block of this item is reached.
    const bool ticket_next = round + 1 >= static_rounds;
    int ticket = 0;
    if (ticket_next && lane == 0) ticket = atomicAdd(p.ticket, 1);
    int i_next = 0;
    bool more = false, nxt_has = false, resolved = false;
    Item nxt = cur;
    auto resolve_next = [&]() {
      if (resolved) return;
      resolved = true;
      i_next = ticket_next ? pool_base + __builtin_amdgcn_readfirstlane(ticket) : item_index(round + 1);
      more = i_next < n_items;
      if (more) nxt = decode(i_next);
      nxt_has = more && nxt.has;
    };
    if (cur.has && !have_first) load_kv(cur, cur.c0, R0{});
    have_first = false;

    // position held by slot s is s + pos_base, or cap less when that would lie beyond the last one
    const int pos_base = (cur.len > 0) ? ((cur.len - 1) / p.cap) * p.cap : 0;
    auto slot_pos = [&](int s) {
      int pp = s + pos_base;
      return (pp > cur.len - 1) ? pp - p.cap : pp;   // negative for a slot that was never written
    };
    const int c1 = cur.c1;
    const int head = cur.g * G + min(n, G - 1);

    // ---- Q^T operand, split into bf16 hi and lo parts -----------------------------------------
    bf16x8 qh[KS], ql[KS];
    {
      const float *qp = p.q + ((size_t)cur.b * p.n_q + head) * D + c * KS * 8;
#pragma unroll
      for (int s = 0; s < KS; s++) {
        uint32_t h[4], l[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          float x0 = (n < G) ? qp[s * 8 + 2 * j] : 0.f, x1 = (n < G) ? qp[s * 8 + 2 * j + 1] : 0.f;
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
        for (int q4 = 0; q4 < 4; q4++) {
          float v = s4[tb][q4] * p.scale_log2e;
          if (EDGE) {
            const int slot = blk + tb * 16 + c * 4 + q4;
            const bool ok = slot < c1 && slot_pos(slot) >= cur.t_lo;
            v = ok ? v : -INFINITY;
          }
          s4[tb][q4] = v;
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
        for (int q4 = 0; q4 < 4; q4++) o[db][q4] *= alpha;
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
              const uint32_t keep = ((s_lo < c1 && slot_pos(s_lo) >= cur.t_lo) ? 0x0000ffffu : 0u) |
                                    ((s_lo + 1 < c1 && slot_pos(s_lo + 1) >= cur.t_lo) ? 0xffff0000u : 0u);
              vv[w] &= keep;
            }
          }
          bf16x8 vf = as_bf16x8(vv);
          o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, ph[grp], o[db], 0, 0, 0);
          o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pl[grp], o[db], 0, 0, 0);
        }
    };
    const bool wrapped = cur.len > p.cap;
    auto step = [&](int blk, auto buf) {
      const bool edge = wrapped || blk < cur.t_lo || blk + ATT_BLOCK > c1;  // wave-uniform
      if (edge) process(blk, buf, std::true_type{});
      else process(blk, buf, std::false_type{});
    };
    // the block requested while `blk` is multiplied: the item's next block, else the first block
    // of the wave's next item, else (nothing left to fetch) this item's last block again
    const int last_blk = max(cur.c0, ((c1 - 1) & ~(ATT_BLOCK - 1)));
    auto prefetch = [&](int blk, auto buf) {
      if (blk + ATT_BLOCK < c1) {
        load_kv(cur, blk + ATT_BLOCK, buf);
      } else {
        resolve_next();
        if (nxt_has) load_kv(nxt, nxt.c0, buf);
        else load_kv(cur, last_blk, buf);
      }
    };

    int parity = 0;  // buffer that received the last prefetch
    if (cur.has) {
      int blk = cur.c0;
      while (true) {
        prefetch(blk, R1{});
        step(blk, R0{});
        blk += ATT_BLOCK;
        if (blk >= c1) {
          parity = 1;
          break;
        }
        prefetch(blk, R0{});
        step(blk, R1{});
        blk += ATT_BLOCK;
        if (blk >= c1) {
          parity = 0;
          break;
        }
      }
      have_first = nxt_has;
    }
    resolve_next();

    // ---- per-head totals: sum the partial denominators of the 4 lanes that share a head --------
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (n < G) {
      const int hq = cur.g * G + n;
      if (cur.nchunks == 1) {
        float sink2 = p.sinks ? p.sinks[hq] * 1.4426950408889634f : -INFINITY;
        float M = fmaxf(m_run, sink2);
        float w = exp2f(m_run - M);
        float denom = l_run * w + exp2f(sink2 - M);
        float inv = (denom > 0.f) ? w / denom : 0.f;
        bf16_t *op = p.out + ((size_t)cur.b * p.n_q + hq) * D;
#pragma unroll
        for (int db = 0; db < DB; db++) {
          u32x2 pk = u32x2{pack_bf16x2(o[db][0] * inv, o[db][1] * inv),
                           pack_bf16x2(o[db][2] * inv, o[db][3] * inv)};
          *reinterpret_cast<u32x2 *>(op + db * 16 + c * 4) = pk;
        }
      } else {
        const size_t slot = ((size_t)cur.b * p.max_chunks + cur.chunk_id) * p.n_q + hq;
        float *po = p.part_o + slot * D;
#pragma unroll
        for (int db = 0; db < DB; db++) *reinterpret_cast<f32x4 *>(po + db * 16 + c * 4) = o[db];
        if (c == 0) {
          p.part_ml[slot * 2] = m_run;
          p.part_ml[slot * 2 + 1] = l_run;
        }
      }
    }
    if (!more) break;
    // the next item's loop starts from buffer 0
    if (have_first && parity == 1) {
#pragma unroll
      for (int tb = 0; tb < 4; tb++)
#pragma unroll
        for (int s = 0; s < KS; s++) kreg[0][tb][s] = kreg[1][tb][s];
#pragma unroll
      for (int grp = 0; grp < 2; grp++)
#pragma unroll
        for (int db = 0; db < DB; db++) vreg[0][grp][db] = vreg[1][grp][db];
    }
    cur = nxt;
    i = i_next;
    round++;
  }
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
  const SeqRange r = seq_range(p.lens[b], p.cap, p.window, p.chunk, p.max_len);
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

// Bulk cache write: rows [B, n_tok, n_kv, D] -> K [B, n_kv, cap, D], V in 32-slot operand blocks.
__global__ __launch_bounds__(256) void kv_cache_write_kernel(bf16_t *__restrict__ kc, bf16_t *__restrict__ vc,
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
    size_t base = ((size_t)(b * n_kv + g) * cap) * D;
    kc[base + (size_t)slot * D + d] = k_rows[i];
    int tt = slot & 31, within = tt & 15;
    int lane = (within >> 2) * 16 + (d & 15);
    int j = (tt >> 4) * 4 + (within & 3);
    vc[base + ((size_t)(slot >> 5) * (D / 16) + (d >> 4)) * 512 + lane * 8 + j] = v_rows[i];
  }
}

static int attn_chunk_tokens(int span) { return span > 1024 ? 512 : 256; }

struct AttnPlan {
  int chunk, max_chunks;
  size_t part_o_bytes, part_ml_bytes;
  static constexpr size_t ticket_bytes = 256;  // one counter per slice of ATT_MAX_BATCH sequences
};

static AttnPlan attn_plan(int B, int n_q, int D, int max_len) {
  AttnPlan pl;
  pl.chunk = attn_chunk_tokens(max_len);
  // a window range can start up to 63 slots before its first active position
  pl.max_chunks = (max_len + ATT_BLOCK - 1 + pl.chunk - 1) / pl.chunk;
  if (pl.max_chunks < 1) pl.max_chunks = 1;
  pl.part_o_bytes = align_up((size_t)B * pl.max_chunks * n_q * D * sizeof(float), 256);
  pl.part_ml_bytes = align_up((size_t)B * pl.max_chunks * n_q * 2 * sizeof(float), 256);
  return pl;
}

}  // namespace gptoss

using namespace gptoss;

extern "C" size_t gptoss_kv_cache_bytes(int B, int n_kv, int head_dim, int capacity) {
  if (B <= 0 || n_kv <= 0 || head_dim <= 0 || capacity <= 0) return 0;
  return (size_t)B * n_kv * capacity * head_dim * sizeof(bf16_t);
}

extern "C" int gptoss_kv_cache_write(void *k_cache, void *v_cache, const void *k_rows,
                                     const void *v_rows, int B, int n_kv, int head_dim,
                                     int capacity, int pos0, int n_tok, void *stream) {
  GPTOSS_REQUIRE(k_cache && v_cache && k_rows && v_rows, GPTOSS_ERR_NULL, "kv_cache_write: null pointer");
  GPTOSS_REQUIRE(B > 0 && n_kv > 0 && (head_dim == 32 || head_dim == 64) && capacity > 0 &&
                     capacity % 64 == 0 && pos0 >= 0 && n_tok >= 0 && n_tok <= capacity,
                 GPTOSS_ERR_DIM,
                 "kv_cache_write: need head_dim in {32,64}, capacity %% 64 == 0, n_tok <= capacity "
                 "(D=%d capacity=%d n_tok=%d)", head_dim, capacity, n_tok);
  if (n_tok == 0) return GPTOSS_OK;
  size_t total = (size_t)B * n_tok * n_kv * head_dim;
  int grid = (int)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256);
  kv_cache_write_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((bf16_t *)k_cache, (bf16_t *)v_cache,
                                                               (const bf16_t *)k_rows, (const bf16_t *)v_rows,
                                                               B, n_kv, head_dim, capacity, pos0, n_tok);
  GPTOSS_LAUNCH_CHECK("kv_cache_write_kernel");
  return GPTOSS_OK;
}

extern "C" size_t gptoss_attn_workspace_bytes(int B, int n_q, int n_kv, int head_dim, int max_len) {
  if (B <= 0 || n_q <= 0 || n_kv <= 0 || head_dim <= 0 || max_len <= 0) return 0;
  // sized for the smallest chunk length so that any window/capacity combination fits
  int max_chunks = (max_len + ATT_BLOCK - 1 + 255) / 256;
  return align_up((size_t)B * max_chunks * n_q * head_dim * sizeof(float), 256) +
         align_up((size_t)B * max_chunks * n_q * 2 * sizeof(float), 256) + AttnPlan::ticket_bytes;
}

extern "C" int gptoss_attn_decode(const float *q, const void *k_cache, const void *v_cache,
                                  const int *lens, const float *sinks, void *out, int B, int n_q,
                                  int n_kv, int head_dim, int capacity, int window, int max_len,
                                  void *workspace, size_t workspace_bytes, void *stream) {
  GPTOSS_REQUIRE(q && k_cache && v_cache && lens && out, GPTOSS_ERR_NULL, "attn_decode: null pointer");
  GPTOSS_REQUIRE(B > 0 && n_q > 0 && n_kv > 0 && n_q % n_kv == 0 && n_q / n_kv <= 16, GPTOSS_ERR_DIM,
                 "attn_decode: need n_q %% n_kv == 0 and n_q/n_kv <= 16 (n_q=%d n_kv=%d)", n_q, n_kv);
  GPTOSS_REQUIRE(head_dim == 32 || head_dim == 64, GPTOSS_ERR_DIM,
                 "attn_decode: head_dim must be 32 or 64 (got %d)", head_dim);
  GPTOSS_REQUIRE(capacity > 0 && capacity % 64 == 0 && window >= 0 && max_len > 0, GPTOSS_ERR_DIM,
                 "attn_decode: need capacity %% 64 == 0, window >= 0, max_len > 0 (capacity=%d)", capacity);
  GPTOSS_REQUIRE(max_len <= capacity || (window > 0 && window <= capacity), GPTOSS_ERR_DIM,
                 "attn_decode: the cache must hold every active position (capacity=%d window=%d max_len=%d)",
                 capacity, window, max_len);
  GPTOSS_REQUIRE(aligned(q, 16) && aligned(k_cache, 16) && aligned(v_cache, 16) && aligned(out, 8),
                 GPTOSS_ERR_ALIGN, "attn_decode: pointers must be 16-byte aligned");
  // longest slot range one sequence can visit: the whole ring once it may have wrapped
  int span = (max_len > capacity) ? capacity
                                  : ((window > 0 && window < max_len) ? window : max_len);
  AttnPlan pl = attn_plan(B, n_q, head_dim, span);
  GPTOSS_REQUIRE(workspace && aligned(workspace, 256) &&
                     workspace_bytes >= pl.part_o_bytes + pl.part_ml_bytes + pl.ticket_bytes,
                 GPTOSS_ERR_WORKSPACE, "attn_decode: workspace missing, misaligned or smaller than %zu bytes",
                 pl.part_o_bytes + pl.part_ml_bytes + pl.ticket_bytes);
  AttnParams p;
  p.q = q;
  p.kc = (const bf16_t *)k_cache;
  p.vc = (const bf16_t *)v_cache;
  p.lens = lens;
  p.sinks = sinks;
  p.out = (bf16_t *)out;
  p.part_o = (float *)workspace;
  p.part_ml = (float *)((unsigned char *)workspace + pl.part_o_bytes);
  p.ticket = (int *)((unsigned char *)workspace + pl.part_o_bytes + pl.part_ml_bytes);
  p.B = B;
  p.n_q = n_q;
  p.n_kv = n_kv;
  p.G = n_q / n_kv;
  p.cap = capacity;
  p.window = window;
  p.chunk = pl.chunk;
  p.max_chunks = pl.max_chunks;
  p.max_len = max_len;
  p.scale_log2e = 1.4426950408889634f / sqrtf((float)head_dim);
  hipStream_t s = (hipStream_t)stream;
  // persistent grid: one workgroup of eight waves per CU, fewer when there is less work; batches
  // beyond ATT_MAX_BATCH sequences (the kernel keeps four ints per sequence in LDS) are sliced
  GPTOSS_REQUIRE(B <= ATT_MAX_BATCH * (int)(AttnPlan::ticket_bytes / sizeof(int)), GPTOSS_ERR_DIM,
                 "attn_decode: at most %d sequences per call", ATT_MAX_BATCH * (int)(AttnPlan::ticket_bytes / sizeof(int)));
  // tickets are only used for long contexts (512-slot chunks: an item then lasts tens of
  // microseconds, against which one atomic is nothing) when a slice can have three or more rounds
  // of items; the counters start at zero (a fill kernel rather than a memset, so that the call can
  // be captured in a graph)
  bool any_tickets = false;
  for (int b0 = 0; b0 < B; b0 += ATT_MAX_BATCH) {
    const int nb = (B - b0 < ATT_MAX_BATCH) ? B - b0 : ATT_MAX_BATCH;
    const long long items = (long long)nb * n_kv * pl.max_chunks;
    long long grid = (items + ATT_WAVES - 1) / ATT_WAVES;
    if (grid > 256) grid = 256;
    if (pl.chunk >= 512 && items / (grid * ATT_WAVES) >= 3) any_tickets = true;
  }
  if (any_tickets) {
    int rc = run_fill_int(p.ticket, (int)(AttnPlan::ticket_bytes / sizeof(int)), 0, s);
    if (rc != GPTOSS_OK) return rc;
  } else {
    p.ticket = nullptr;
  }
  {
    TraceScope ts("attn_decode", s);
    for (int b0 = 0; b0 < B; b0 += ATT_MAX_BATCH) {
      AttnParams ps = p;
      if (p.ticket) ps.ticket = p.ticket + b0 / ATT_MAX_BATCH;
      ps.B = (B - b0 < ATT_MAX_BATCH) ? B - b0 : ATT_MAX_BATCH;
      ps.q = p.q + (size_t)b0 * n_q * head_dim;
      ps.kc = p.kc + (size_t)b0 * n_kv * capacity * head_dim;
      ps.vc = p.vc + (size_t)b0 * n_kv * capacity * head_dim;
      ps.lens = p.lens + b0;
      ps.out = p.out + (size_t)b0 * n_q * head_dim;
      ps.part_o = p.part_o + (size_t)b0 * pl.max_chunks * n_q * head_dim;
      ps.part_ml = p.part_ml + (size_t)b0 * pl.max_chunks * n_q * 2;
      long long items = (long long)ps.B * n_kv * pl.max_chunks;
      int grid = (int)((items + ATT_WAVES - 1) / ATT_WAVES);
      if (grid > 256) grid = 256;
      const size_t smem = sizeof(int) * (4 * (size_t)ps.B + 1);
      if (head_dim == 64) attn_decode_kernel<64><<<grid, ATT_THREADS, smem, s>>>(ps);
      else attn_decode_kernel<32><<<grid, ATT_THREADS, smem, s>>>(ps);
    }
  }
  GPTOSS_LAUNCH_CHECK("attn_decode_kernel");
  if (pl.max_chunks > 1) {
    int per_block = 256 / (head_dim / 4);
    int rgrid = (B * n_q + per_block - 1) / per_block;
    TraceScope ts("attn_reduce", s);
    if (head_dim == 64) attn_reduce_kernel<64><<<rgrid, 256, 0, s>>>(p);
    else attn_reduce_kernel<32><<<rgrid, 256, 0, s>>>(p);
    GPTOSS_LAUNCH_CHECK("attn_reduce_kernel");
  }
  return GPTOSS_OK;
}
