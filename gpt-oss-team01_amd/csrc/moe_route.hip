// MoE routing for gfx950: router GEMM (bf16 MFMA 16x16x32), top-k + softmax gating with wave
// shuffles, and a stable counting sort of the (token,slot) pairs by expert built from wave
// ballots and an LDS histogram (no global atomics), which also emits the tile list that the
// grouped GEMMs schedule from.
#include <mutex>

#include "common.hpp"
#include "gemm.hpp"

namespace gptoss {

// ------------------------------------------------------------------------------------------------
// Top-k + softmax for one token held by a group of 32 lanes: lane j holds experts j, j+32, ...
// Selection = k rounds of (local best, 5-step butterfly) ordered by (value desc, expert id asc);
// softmax over the k picked values with exp in float and the sum and division in double
// (run.cpp:319-337).  Every lane of the group must call; lane 0 of the group writes.
// ------------------------------------------------------------------------------------------------
template <int NJ>
__device__ __forceinline__ void topk_softmax_group(const float (&v)[NJ], int sub, int E, int k,
                                                   bool live, float *__restrict__ w_out,
                                                   int *__restrict__ i_out) {
  uint32_t used = 0;
  float pick_v[8];
  int pick_i[8];
  constexpr int NONE = 0x7fffffff;
#pragma unroll
  for (int s = 0; s < 8; s++) {
    pick_v[s] = -INFINITY;
    pick_i[s] = 0;
    if (s < k) {
      float bv = -INFINITY;
      int bi = NONE;
#pragma unroll
      for (int j = 0; j < NJ; j++) {
        int e = sub + 32 * j;
        bool ok = !((used >> j) & 1u) && e < E;
        if (ok && (bi == NONE || v[j] > bv || (v[j] == bv && e < bi))) {
          bv = v[j];
          bi = e;
        }
      }
#pragma unroll
      for (int m = 16; m >= 1; m >>= 1) {
        float ov = __shfl_xor(bv, m, 64);
        int oi = __shfl_xor(bi, m, 64);
        if (oi != NONE && (bi == NONE || ov > bv || (ov == bv && oi < bi))) {
          bv = ov;
          bi = oi;
        }
      }
      if (bi != NONE && (bi & 31) == sub) used |= 1u << (bi >> 5);
      pick_v[s] = bv;
      pick_i[s] = bi;
    }
  }
  if (live && sub == 0) {
    float ex[8];
    double sum = 0.0;
#pragma unroll
    for (int s = 0; s < 8; s++) {
      ex[s] = (s < k) ? expf(pick_v[s] - pick_v[0]) : 0.f;
      sum += ex[s];
    }
#pragma unroll
    for (int s = 0; s < 8; s++) {
      if (s < k) {
        w_out[s] = (float)((double)ex[s] / sum);
        i_out[s] = pick_i[s];
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Router GEMM: logits[B,E] = t[B,H] . Wr[E,H]^T + br.  One workgroup = 16 token rows x all experts;
// its 8 waves split the K loop (k-steps of 32, interleaved), request all their operands up front
// and reduce through LDS.  With topk_w != nullptr the workgroup also gates its 16 tokens (32
// lanes per token) while the logits are still in LDS.
// ------------------------------------------------------------------------------------------------
constexpr int ROUTER_WAVES = 8;
// k-steps whose operands a wave requests before its first MFMA: as many as ~150 registers hold,
// so that a hidden size of 2880 with up to 32 experts is a single round of loads
constexpr int router_steps(int nb) { return nb <= 2 ? 12 : (nb <= 4 ? 7 : (nb <= 8 ? 4 : 2)); }

// What the NORM form of the router kernel does first: x += residual, t = RMSNorm(x) * weight for the
// workgroup's own token rows.
struct RouterNorm {
  float *x;               // [B,H] residual stream, updated in place
  const float *residual;  // [B,H] or nullptr
  const float *weight;    // [H]
  bf16_t *t_out;          // [B,H]
};

// NB: number of 16-expert column blocks held per wave.  NORM: the workgroup first normalises its
// rows (the arithmetic of rmsnorm_rows_kernel: 256 threads per row, the same element-to-thread
// assignment and summation order, so t is the same to the bit), writes x and t to memory, keeps t in
// LDS and multiplies from there: one launch and one read of t less than norm kernel + router kernel.
template <int NB, bool NORM>
__global__ __launch_bounds__(ROUTER_WAVES * 64) void router_gemm_kernel(
    const bf16_t *__restrict__ t, const bf16_t *__restrict__ wr, const float *__restrict__ br,
    float *__restrict__ logits, int B, int H, int E, int k, float *__restrict__ topk_w,
    int *__restrict__ topk_i, int rows_per_wg, RouterNorm nrm) {
  __shared__ float red[ROUTER_WAVES][16][NB * 16 + 1];
  extern __shared__ __attribute__((aligned(16))) unsigned char t_rows_raw[];  // NORM: [rows_per_wg][H] bf16
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // rows_per_wg <= 16 token rows are this workgroup's; the other MFMA rows repeat the last of them
  const int r0 = blockIdx.x * rows_per_wg;
  const int arow = min(r0 + min(lane & 15, rows_per_wg - 1), B - 1);
  const int kq = (lane >> 4) * 8;
  const bf16_t *ap = t + (size_t)arow * H + kq;
  if constexpr (NORM) {
    constexpr int VPT = 4;  // rows of up to 4096 floats
    __shared__ double nred[2][4];
    bf16_t *t_rows = reinterpret_cast<bf16_t *>(t_rows_raw);
    const int grp = threadIdx.x >> 8, tg = threadIdx.x & 255;  // two groups of 256 threads, a row each
    for (int rr = 0; rr < rows_per_wg; rr += 2) {
      const int lr = rr + grp;
      const bool live = lr < rows_per_wg && r0 + lr < B;
      const size_t row = (size_t)(r0 + lr) * H;
      f32x4 v[VPT];
      double ss = 0.0;
#pragma unroll
      for (int i = 0; i < VPT; i++) {
        const int h = (tg + 256 * i) * 4;
        v[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (live && h < H) {
          v[i] = *reinterpret_cast<const f32x4 *>(nrm.x + row + h);
          if (nrm.residual) {
            const f32x4 r = *reinterpret_cast<const f32x4 *>(nrm.residual + row + h);
#pragma unroll
            for (int q = 0; q < 4; q++) v[i][q] = __fadd_rn(v[i][q], r[q]);
            *reinterpret_cast<f32x4 *>(nrm.x + row + h) = v[i];
          }
#pragma unroll
          for (int q = 0; q < 4; q++) ss += (double)__fmul_rn(v[i][q], v[i][q]);
        }
      }
      for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, 64);
      if (lane == 0) nred[grp][(threadIdx.x >> 6) & 3] = ss;
      __syncthreads();
      ss = nred[grp][0] + nred[grp][1] + nred[grp][2] + nred[grp][3];
      ss /= H;
      ss += 1e-5f;
      const double inv = (double)(1.0f / sqrtf((float)ss));
#pragma unroll
      for (int i = 0; i < VPT; i++) {
        const int h = (tg + 256 * i) * 4;
        if (live && h < H) {
          const f32x4 w = *reinterpret_cast<const f32x4 *>(nrm.weight + h);
          f32x4 o;
#pragma unroll
          for (int q = 0; q < 4; q++) o[q] = (float)((double)w[q] * (inv * (double)v[i][q]));
          const u32x2 pk = u32x2{pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
          *reinterpret_cast<u32x2 *>(nrm.t_out + row + h) = pk;
          *reinterpret_cast<u32x2 *>(t_rows + (size_t)lr * H + h) = pk;
        }
      }
      __syncthreads();   // nred is reused by the next pair of rows; after the last pair: t_rows complete
    }
    ap = t_rows + (size_t)(arow - r0) * H + kq;
  }
  f32x4 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};
  constexpr int ROUTER_MAX_STEPS = router_steps(NB);
  const int ksteps = H / 32;
  for (int ks0 = wave; ks0 < ksteps; ks0 += ROUTER_WAVES * ROUTER_MAX_STEPS) {
    u32x4 a[ROUTER_MAX_STEPS], b[ROUTER_MAX_STEPS][NB];
#pragma unroll
    for (int u = 0; u < ROUTER_MAX_STEPS; u++) {
      const int ks = min(ks0 + u * ROUTER_WAVES, ksteps - 1);
      a[u] = *reinterpret_cast<const u32x4 *>(ap + ks * 32);
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        int e = min(nb * 16 + (lane & 15), E - 1);
        b[u][nb] = *reinterpret_cast<const u32x4 *>(wr + (size_t)e * H + ks * 32 + kq);
      }
    }
#pragma unroll
    for (int u = 0; u < ROUTER_MAX_STEPS; u++) {
      if (ks0 + u * ROUTER_WAVES < ksteps) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
          acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[u]), as_bf16x8(b[u][nb]), acc[nb], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int nb = 0; nb < NB; nb++)
#pragma unroll
    for (int i = 0; i < 4; i++) red[wave][(lane >> 4) * 4 + i][nb * 16 + (lane & 15)] = acc[nb][i];
  __syncthreads();
  // 32 lanes per token row: sum the partial products, add the bias, publish, gate
  const int row = threadIdx.x >> 5, sub = threadIdx.x & 31;
  const bool live = row < rows_per_wg && r0 + row < B;
  constexpr int NJ = (NB + 1) / 2;
  float v[NJ];
#pragma unroll
  for (int j = 0; j < NJ; j++) {
    const int e = sub + 32 * j;
    float x = -INFINITY;
    if (e < E) {
      x = 0.f;
#pragma unroll
      for (int w = 0; w < ROUTER_WAVES; w++) x += red[w][row][e];
      if (br) x += br[e];
      if (live) logits[(size_t)(r0 + row) * E + e] = x;
    }
    v[j] = x;
  }
  if (topk_w != nullptr) {
    const size_t o = (size_t)(live ? r0 + row : 0) * k;
    topk_softmax_group<NJ>(v, sub, E, k, live, topk_w + o, topk_i + o);
  }
}

// ------------------------------------------------------------------------------------------------
// Stand-alone gating from logits in memory: 32 lanes per token, two tokens per wave.
// ------------------------------------------------------------------------------------------------
template <int NJ>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const float *__restrict__ logits, int B,
                                                           int E, int k, float *__restrict__ topk_w,
                                                           int *__restrict__ topk_i) {
  const int sub = threadIdx.x & 31;
  const int token = (blockIdx.x * 256 + threadIdx.x) >> 5;
  const bool live = token < B;
  const float *row = logits + (size_t)(live ? token : 0) * E;
  float v[NJ];
#pragma unroll
  for (int j = 0; j < NJ; j++) {
    int e = sub + 32 * j;
    v[j] = (live && e < E) ? row[e] : -INFINITY;
  }
  const size_t o = (size_t)(live ? token : 0) * k;
  topk_softmax_group<NJ>(v, sub, E, k, live, topk_w + o, topk_i + o);
}

// ------------------------------------------------------------------------------------------------
// Stable counting sort of P = B*k pairs by expert in ONE workgroup of 1024 threads (16 waves).
// Each wave owns a contiguous range of pairs.  Inside a 64-pair step the lanes holding the same
// expert are found with log2(E) ballots; the lowest such lane adds their count to the wave's own
// LDS histogram row, so no atomics are needed and the order is the pair order (stable).
// ------------------------------------------------------------------------------------------------
constexpr int SORT_THREADS = 1024;
constexpr int SORT_WAVES = SORT_THREADS / 64;

__device__ __forceinline__ uint64_t same_expert_mask(int e, bool valid, int nbits) {
  uint64_t mask = __ballot(valid);
  for (int b = 0; b < nbits; b++) {
    bool bit = (e >> b) & 1;
    uint64_t bal = __ballot(valid && bit);
    mask &= bit ? bal : ~bal;
  }
  return mask;
}

constexpr int SORT_CHUNK = 8;  // 64-pair steps whose expert ids a wave requests at once

// Exclusive prefix sum over up to 256 values held 4 per lane by one wave (lane l owns entries
// 4l..4l+3); returns the lane's own exclusive prefixes through ex[] and the grand total.
__device__ __forceinline__ int wave_scan4(const int (&v)[4], int (&ex)[4]) {
  const int lane = threadIdx.x & 63;
  int sum = v[0] + v[1] + v[2] + v[3];
  int inc = sum;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    int o = __shfl_up(inc, d, 64);
    if (lane >= d) inc += o;
  }
  int run = inc - sum;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    ex[i] = run;
    run += v[i];
  }
  return __shfl(inc, 63, 64);
}

// From the experts' pair counts total[E] (LDS): the experts' offsets into offs[E+1] (LDS), and, when
// `publish` is set, to memory together with the tile list, the tiles' blocks and the cut positions
// of the work list.  Called by one whole wave (wave 0 of a workgroup); cost_pre / tile_pre are E
// ints of LDS scratch each.
__device__ __forceinline__ void group_finish(const int *total, int *offs, int *cost_pre, int *tile_pre, int E,
                                             bool publish, int *__restrict__ expert_offsets,
                                             int *__restrict__ tiles, int rows_per_tile,
                                             int *__restrict__ xcd_bounds, int cost0) {
  const int lane = threadIdx.x & 63;
  int cnt[4], nt[4], off_ex[4], tile_ex[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int e = lane * 4 + i;
    cnt[i] = (e < E) ? total[e] : 0;
    nt[i] = (rows_per_tile > 0) ? (cnt[i] + rows_per_tile - 1) / rows_per_tile : 0;
  }
  const int all = wave_scan4(cnt, off_ex);
  const int n_tiles = wave_scan4(nt, tile_ex);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int e = lane * 4 + i;
    if (e < E) {
      offs[e] = off_ex[i];
      if (publish) expert_offsets[e] = off_ex[i];
      if (publish && tiles != nullptr && rows_per_tile > 0) {
        for (int t = 0; t < nt[i]; t++) {
          int *tp = tiles + 1 + 3 * (tile_ex[i] + t);
          tp[0] = e;
          tp[1] = off_ex[i] + t * rows_per_tile;
          tp[2] = min(rows_per_tile, cnt[i] - t * rows_per_tile);
          // the block of up to MOE_TILE_BLOCK tiles of this expert that the tile belongs to
          if (xcd_bounds != nullptr) {
            const int b0 = t - t % MOE_TILE_BLOCK;
            xcd_bounds[XCD_BOUNDS_INTS + tile_ex[i] + t] = ((tile_ex[i] + b0) << 8) | min(MOE_TILE_BLOCK, nt[i] - b0);
          }
        }
      }
    }
  }
  if (lane == 0) {
    offs[E] = all;
    if (publish) expert_offsets[E] = all;
    if (publish && tiles != nullptr && rows_per_tile > 0) tiles[0] = n_tiles;
  }
  // Where to cut the tile list into 8 parts (one per XCD) of equal estimated cost: a tile costs
  // cost0 + 2 per 32-row block (half units), all work items of a tile cost the same, and a cut may
  // fall inside a tile (between two of its column tiles), hence the 16-bit fraction.
  if (publish && xcd_bounds != nullptr && tiles != nullptr && rows_per_tile > 0) {
    const int cfull = cost0 + 2 * (rows_per_tile / 32);
    auto last_cost = [&](int count, int n) { return cost0 + 2 * ((count - (n - 1) * rows_per_tile + 31) / 32); };
    int cost[4], cpre[4];
#pragma unroll
    for (int i = 0; i < 4; i++) cost[i] = (nt[i] > 0) ? (nt[i] - 1) * cfull + last_cost(cnt[i], nt[i]) : 0;
    const int ctot = wave_scan4(cost, cpre);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int e = lane * 4 + i;
      if (e < E) {
        cost_pre[e] = cpre[i];
        tile_pre[e] = tile_ex[i];
      }
    }
    // lane x finds cut x: the last expert whose cost prefix is <= x/8 of the total has a tile under
    // the cut (experts without rows share their successor's prefix).  All quantities fit 32 bits:
    // ctot < 2^15 tiles * (cost0 + 16).
    if (lane < 8) {
      int bound = 0;
      if (ctot > 0) {
        const int target = (lane * ctot) >> 3;
        int lo = 0, hi = E - 1;
        while (lo < hi) {
          const int mid = (lo + hi + 1) >> 1;
          if (cost_pre[mid] <= target) lo = mid;
          else hi = mid - 1;
        }
        const int count = offs[lo + 1] - offs[lo];
        const int nte = (count + rows_per_tile - 1) / rows_per_tile;
        // float quotient (operands < 2^24) with a one-step correction instead of integer division
        const int a = target - cost_pre[lo];
        const float rcp_cfull = __builtin_amdgcn_rcpf((float)cfull);
        int t = (int)((float)a * rcp_cfull);
        t -= (t * cfull > a) ? 1 : 0;
        t += ((t + 1) * cfull <= a) ? 1 : 0;
        t = min(t, nte - 1);
        const int rest = a - t * cfull;
        const float inv = (t == nte - 1) ? __builtin_amdgcn_rcpf((float)last_cost(count, nte)) : rcp_cfull;
        bound = ((tile_pre[lo] + t) << 16) | min(65535, (int)((float)rest * 65536.0f * inv));
      }
      xcd_bounds[lane] = bound;
    }
    if (lane == 0) xcd_bounds[8] = n_tiles << 16;
  }
}

__global__ __launch_bounds__(SORT_THREADS) void group_sort_kernel(
    const int *__restrict__ topk_i, int P, int E, int nbits, int *__restrict__ expert_offsets,
    int *__restrict__ sorted_pair_ids, int *__restrict__ inv_perm, int *__restrict__ tiles,
    int rows_per_tile, int *__restrict__ xcd_bounds, int cost0) {
  extern __shared__ int smem[];
  int *hist = smem;                    // [SORT_WAVES][E] per-wave counts, then per-wave cursors
  int *total = hist + SORT_WAVES * E;  // [E]
  int *offs = total + E;               // [E+1]
  int *cost_pre = offs + E + 1;        // [E] exclusive prefix of the experts' estimated cost
  int *tile_pre = cost_pre + E;        // [E] first tile of every expert
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));

  for (int i = threadIdx.x; i < SORT_WAVES * E; i += SORT_THREADS) hist[i] = 0;
  __syncthreads();

  const int steps_total = (P + 63) / 64;
  const int steps_per_wave = (steps_total + SORT_WAVES - 1) / SORT_WAVES;
  const int p_begin = wave * steps_per_wave * 64;
  const int p_end = min(P, p_begin + steps_per_wave * 64);
  int *myhist = hist + wave * E;

  // expert ids of SORT_CHUNK steps are requested together, so their latencies overlap
  auto load_chunk = [&](int p0, int (&e)[SORT_CHUNK]) {
#pragma unroll
    for (int u = 0; u < SORT_CHUNK; u++) {
      const int p = p0 + u * 64 + lane;
      e[u] = (p < p_end) ? topk_i[p] : -1;
    }
  };

  for (int p0 = p_begin; p0 < p_end; p0 += 64 * SORT_CHUNK) {
    int e[SORT_CHUNK];
    load_chunk(p0, e);
#pragma unroll
    for (int u = 0; u < SORT_CHUNK; u++) {
      if (p0 + u * 64 < p_end) {  // wave-uniform
        const bool valid = (e[u] >= 0 && e[u] < E);
        const uint64_t mask = same_expert_mask(e[u], valid, nbits);
        if (valid && (mask & lt_mask) == 0) myhist[e[u]] += __popcll(mask);
      }
    }
  }
  __syncthreads();

  // per expert: exclusive prefix over waves (turns counts into in-expert start ranks), and totals
  for (int e = threadIdx.x; e < E; e += SORT_THREADS) {
    int run = 0;
#pragma unroll
    for (int w = 0; w < SORT_WAVES; w++) {
      int c = hist[w * E + e];
      hist[w * E + e] = run;
      run += c;
    }
    total[e] = run;
  }
  __syncthreads();

  // expert offsets, tile list and cut positions: wave 0
  if (wave == 0)
    group_finish(total, offs, cost_pre, tile_pre, E, true, expert_offsets, tiles, rows_per_tile, xcd_bounds, cost0);
  __syncthreads();

  for (int p0 = p_begin; p0 < p_end; p0 += 64 * SORT_CHUNK) {
    int e[SORT_CHUNK];
    load_chunk(p0, e);
#pragma unroll
    for (int u = 0; u < SORT_CHUNK; u++) {
      if (p0 + u * 64 < p_end) {
        const int p = p0 + u * 64 + lane;
        const bool valid = (e[u] >= 0 && e[u] < E);
        const uint64_t mask = same_expert_mask(e[u], valid, nbits);
        if (valid) {
          const int rank = myhist[e[u]] + __popcll(mask & lt_mask);
          const int dst = offs[e[u]] + rank;
          sorted_pair_ids[dst] = p;
          inv_perm[p] = dst;
        }
        // all lanes of the wave have read myhist before the leaders update it (wave-ordered LDS ops)
        if (valid && (mask & lt_mask) == 0) myhist[e[u]] += __popcll(mask);
      }
    }
  }
}


// ---- the same sort by many workgroups (prompt passes, large batches) ---------------------------
// One workgroup of 16 waves per 1024 pairs, one 64-pair step per wave.  First kernel: every pair's
// rank among the pairs of its expert inside its workgroup (to rank[], which may be inv_perm) and
// the workgroup's pair count per expert (wg_hist [G][E]).  Second kernel: every workgroup sums the
// counts of the workgroups before it, derives the experts' offsets and scatters its pairs;
// workgroup 0 also writes the offsets, the tile list and the cut positions.  The order inside an
// expert is (workgroup, wave, lane) = pair order, as in the one-workgroup kernel.
constexpr int SORT_PARALLEL_MIN_PAIRS = 8192;

__global__ __launch_bounds__(SORT_THREADS) void group_count_kernel(const int *__restrict__ topk_i, int P, int E,
                                                                   int nbits, int *__restrict__ wg_hist,
                                                                   int *__restrict__ rank) {
  extern __shared__ int smem[];  // [SORT_WAVES][E]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int i = threadIdx.x; i < SORT_WAVES * E; i += SORT_THREADS) smem[i] = 0;
  __syncthreads();
  const int p = blockIdx.x * SORT_THREADS + threadIdx.x;
  const int e = (p < P) ? topk_i[p] : -1;
  const bool valid = (e >= 0 && e < E);
  const uint64_t mask = same_expert_mask(e, valid, nbits);
  if (valid && (mask & lt_mask) == 0) smem[wave * E + e] = __popcll(mask);
  __syncthreads();
  for (int x = threadIdx.x; x < E; x += SORT_THREADS) {
    int run = 0;
#pragma unroll
    for (int w = 0; w < SORT_WAVES; w++) {
      const int c = smem[w * E + x];
      smem[w * E + x] = run;
      run += c;
    }
    wg_hist[(size_t)blockIdx.x * E + x] = run;
  }
  __syncthreads();
  if (valid) rank[p] = smem[wave * E + e] + __popcll(mask & lt_mask);
}

__global__ __launch_bounds__(SORT_THREADS) void group_scatter_kernel(
    const int *__restrict__ topk_i, int P, int E, const int *__restrict__ wg_hist, const int *rank,
    int *__restrict__ expert_offsets, int *__restrict__ sorted_pair_ids, int *inv_perm, int *__restrict__ tiles,
    int rows_per_tile, int *__restrict__ xcd_bounds, int cost0) {
  extern __shared__ int smem[];
  int *before = smem;          // [E] pairs of the expert in the workgroups before this one
  int *total = before + E;     // [E]
  int *offs = total + E;       // [E+1]
  int *cost_pre = offs + E + 1;
  int *tile_pre = cost_pre + E;
  const int wave = threadIdx.x >> 6;
  const int G = gridDim.x;
  for (int x = threadIdx.x; x < E; x += SORT_THREADS) {
    int run = 0, mine = 0;
    for (int g = 0; g < G; g++) {
      if (g == (int)blockIdx.x) mine = run;
      run += wg_hist[(size_t)g * E + x];
    }
    before[x] = mine;
    total[x] = run;
  }
  __syncthreads();
  if (wave == 0)
    group_finish(total, offs, cost_pre, tile_pre, E, blockIdx.x == 0, expert_offsets, tiles, rows_per_tile,
                 xcd_bounds, cost0);
  __syncthreads();
  const int p = blockIdx.x * SORT_THREADS + threadIdx.x;
  const int e = (p < P) ? topk_i[p] : -1;
  if (e >= 0 && e < E) {
    const int dst = offs[e] + before[e] + rank[p];   // rank may alias inv_perm: read before the write below
    sorted_pair_ids[dst] = p;
    inv_perm[p] = dst;
  }
}


// gating only: logits [B,E] -> top-k weights and ids
int run_topk_softmax(const float *logits, int B, int E, int k, float *topk_w, int *topk_i, hipStream_t s) {
  dim3 grid(cdiv(B * 32, 256)), block(256);
  int nj = cdiv(E, 32);
  TraceScope ts("topk_softmax", s);
  if (nj <= 1) topk_softmax_kernel<1><<<grid, block, 0, s>>>(logits, B, E, k, topk_w, topk_i);
  else if (nj <= 2) topk_softmax_kernel<2><<<grid, block, 0, s>>>(logits, B, E, k, topk_w, topk_i);
  else if (nj <= 4) topk_softmax_kernel<4><<<grid, block, 0, s>>>(logits, B, E, k, topk_w, topk_i);
  else topk_softmax_kernel<8><<<grid, block, 0, s>>>(logits, B, E, k, topk_w, topk_i);
  GPTOSS_LAUNCH_CHECK("topk_softmax_kernel");
  return GPTOSS_OK;
}

static int router_rows_per_wg(int B) {
  int rows_per_wg = 16;
  while (rows_per_wg > 4 && cdiv(B, rows_per_wg) < 256) rows_per_wg >>= 1;
  return rows_per_wg;
}

// logits (+ optional gating of the same tokens) in one launch
int run_router(const void *t, const void *w_router, const float *b_router, float *logits, int B,
               int H, int E, int k, float *topk_w, int *topk_i, hipStream_t s) {
  // 16 token rows per workgroup fill the MFMA, but a thousand tokens are then only 64 workgroups;
  // with fewer rows each (the rest of the MFMA rows idle) all CUs take part in what is a
  // latency-bound launch: every workgroup reads the whole router matrix from L2 either way
  // (1024 tokens over 32 experts: 19.7 us with 16 rows, 16.7 with 8, 15.6 with 4, 27 with 2)
  const int rows_per_wg = router_rows_per_wg(B);
  dim3 grid(cdiv(B, rows_per_wg)), block(ROUTER_WAVES * 64);
  const bf16_t *tp = (const bf16_t *)t, *wp = (const bf16_t *)w_router;
  int nb = cdiv(E, 16);
  const RouterNorm none{nullptr, nullptr, nullptr, nullptr};
  TraceScope ts(topk_w ? "router_gemm_topk" : "router_gemm", s);
  if (nb <= 1) router_gemm_kernel<1, false><<<grid, block, 0, s>>>(tp, wp, b_router, logits, B, H, E, k, topk_w, topk_i, rows_per_wg, none);
  else if (nb <= 2) router_gemm_kernel<2, false><<<grid, block, 0, s>>>(tp, wp, b_router, logits, B, H, E, k, topk_w, topk_i, rows_per_wg, none);
  else if (nb <= 4) router_gemm_kernel<4, false><<<grid, block, 0, s>>>(tp, wp, b_router, logits, B, H, E, k, topk_w, topk_i, rows_per_wg, none);
  else if (nb <= 8) router_gemm_kernel<8, false><<<grid, block, 0, s>>>(tp, wp, b_router, logits, B, H, E, k, topk_w, topk_i, rows_per_wg, none);
  else router_gemm_kernel<16, false><<<grid, block, 0, s>>>(tp, wp, b_router, logits, B, H, E, k, topk_w, topk_i, rows_per_wg, none);
  GPTOSS_LAUNCH_CHECK("router_gemm_kernel");
  return GPTOSS_OK;
}


template <int NB>
static int launch_norm_router(const RouterNorm &nrm, const bf16_t *wp, const float *b_router, float *logits, int B, int H,
                              int E, int k, float *topk_w, int *topk_i, int rows_per_wg, size_t dyn, hipStream_t s) {
  // the kernel's LDS (router partial sums + the rows of t) exceeds what a launch gets by default
  constexpr int MAX_DEV = 64;
  static std::mutex mu;
  static size_t raised[MAX_DEV];
  int dev = 0;
  GPTOSS_HIP(hipGetDevice(&dev));
  GPTOSS_REQUIRE(dev >= 0 && dev < MAX_DEV, GPTOSS_ERR_STATE, "router: device ordinal %d outside 0..%d", dev, MAX_DEV - 1);
  auto kern = router_gemm_kernel<NB, true>;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (raised[dev] < dyn) {
      GPTOSS_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)dyn));
      raised[dev] = dyn;
    }
  }
  TraceScope ts("norm_router_gemm_topk", s);
  hipLaunchKernelGGL(kern, dim3(cdiv(B, rows_per_wg)), dim3(ROUTER_WAVES * 64), dyn, s, nrm.t_out, wp, b_router, logits, B,
                     H, E, k, topk_w, topk_i, rows_per_wg, nrm);
  GPTOSS_LAUNCH_CHECK("router_gemm_kernel (with norm)");
  return GPTOSS_OK;
}

bool norm_router_applies(int B, int H, int E, const float *x, const float *residual, const float *weight,
                         const void *t_out) {
  const int nb = cdiv(E, 16) <= 1 ? 1 : cdiv(E, 16) <= 2 ? 2 : cdiv(E, 16) <= 4 ? 4 : cdiv(E, 16) <= 8 ? 8 : 16;
  const size_t lds = (size_t)ROUTER_WAVES * 16 * (nb * 16 + 1) * 4 + (size_t)router_rows_per_wg(B) * H * 2 + 256;
  // With more than four rows per workgroup (batches of more than ~1000 rows) the rows a workgroup
  // normalises one after the other cost more than the launch the fusion saves (8192 rows: 2.58 ms
  // per 24 layers against 2.23 ms for the two kernels; 1024 rows: 0.63 against 0.71 ms).
  return B > 0 && router_rows_per_wg(B) <= 4 && H % 32 == 0 && H <= 4096 && lds <= 160 * 1024 && aligned(x, 16) && aligned(weight, 16) &&
         aligned(t_out, 16) && (!residual || aligned(residual, 16));
}

// x += residual; t_out = RMSNorm(x) * weight; logits = t_out . Wr^T + br; gating: one launch
int run_norm_router(float *x, const float *residual, const float *weight, void *t_out, const void *w_router,
                    const float *b_router, float *logits, int B, int H, int E, int k, float *topk_w, int *topk_i,
                    hipStream_t s) {
  GPTOSS_REQUIRE(norm_router_applies(B, H, E, x, residual, weight, t_out), GPTOSS_ERR_DIM,
                 "norm + router: shape or alignment outside the fused kernel's range (H=%d E=%d)", H, E);
  const int rows_per_wg = router_rows_per_wg(B);
  const RouterNorm nrm{x, residual, weight, (bf16_t *)t_out};
  const bf16_t *wp = (const bf16_t *)w_router;
  const size_t dyn = (size_t)rows_per_wg * H * 2;
  const int nb = cdiv(E, 16);
  if (nb <= 1) return launch_norm_router<1>(nrm, wp, b_router, logits, B, H, E, k, topk_w, topk_i, rows_per_wg, dyn, s);
  if (nb <= 2) return launch_norm_router<2>(nrm, wp, b_router, logits, B, H, E, k, topk_w, topk_i, rows_per_wg, dyn, s);
  if (nb <= 4) return launch_norm_router<4>(nrm, wp, b_router, logits, B, H, E, k, topk_w, topk_i, rows_per_wg, dyn, s);
  if (nb <= 8) return launch_norm_router<8>(nrm, wp, b_router, logits, B, H, E, k, topk_w, topk_i, rows_per_wg, dyn, s);
  return launch_norm_router<16>(nrm, wp, b_router, logits, B, H, E, k, topk_w, topk_i, rows_per_wg, dyn, s);
}

}  // namespace gptoss

using namespace gptoss;

extern "C" int gptoss_router_gemm(const void *t, const void *w_router, const float *b_router,
                                  float *logits, int B, int H, int E, void *stream) {
  GPTOSS_REQUIRE(t && w_router && logits, GPTOSS_ERR_NULL, "router_gemm: null pointer");
  GPTOSS_REQUIRE(B >= 0 && H > 0 && H % 32 == 0 && E >= 1 && E <= 256, GPTOSS_ERR_DIM,
                 "router_gemm: need H %% 32 == 0 and 1 <= E <= 256 (B=%d H=%d E=%d)", B, H, E);
  GPTOSS_REQUIRE(aligned(t, 16) && aligned(w_router, 16), GPTOSS_ERR_ALIGN,
                 "router_gemm: t and w_router must be 16-byte aligned");
  if (B == 0) return GPTOSS_OK;
  return run_router(t, w_router, b_router, logits, B, H, E, 0, nullptr, nullptr, (hipStream_t)stream);
}

extern "C" int gptoss_moe_max_tiles(int B, int k, int E, int rows_per_tile) {
  if (rows_per_tile <= 0 || B < 0 || k <= 0 || E <= 0) return 0;
  long long P = (long long)B * k;
  return (int)(P / rows_per_tile) + E;
}

static int moe_route_impl(const float *logits, int B, int E, int k, float *topk_w, int *topk_i,
                          int *expert_offsets, int *sorted_pair_ids, int *inv_perm, int *tiles,
                          int rows_per_tile, int *xcd_bounds, int tile_cost0_x2, void *stream, bool gate,
                          int *sort_scratch);

// grouping only: topk_i was already written by the fused router kernel
int gptoss::run_group(int B, int E, int k, float *topk_w, int *topk_i, int *expert_offsets,
                      int *sorted_pair_ids, int *inv_perm, int *tiles, int rows_per_tile,
                      int *xcd_bounds, int tile_cost0_x2, hipStream_t s, int *sort_scratch) {
  // the cut positions hold the tile index in 15 bits
  if (gptoss_moe_max_tiles(B, k, E, rows_per_tile) >= 32768) xcd_bounds = nullptr;
  return moe_route_impl(nullptr, B, E, k, topk_w, topk_i, expert_offsets, sorted_pair_ids, inv_perm,
                        tiles, rows_per_tile, xcd_bounds, tile_cost0_x2, s, false, sort_scratch);
}

extern "C" int gptoss_moe_route(const float *logits, int B, int E, int k, float *topk_w,
                                int *topk_i, int *expert_offsets, int *sorted_pair_ids,
                                int *inv_perm, int *tiles, int rows_per_tile, void *stream) {
  return moe_route_impl(logits, B, E, k, topk_w, topk_i, expert_offsets, sorted_pair_ids, inv_perm,
                        tiles, rows_per_tile, nullptr, 0, stream, true, nullptr);
}

static int moe_route_impl(const float *logits, int B, int E, int k, float *topk_w, int *topk_i,
                          int *expert_offsets, int *sorted_pair_ids, int *inv_perm, int *tiles,
                          int rows_per_tile, int *xcd_bounds, int tile_cost0_x2, void *stream, bool gate,
                          int *sort_scratch) {
  GPTOSS_REQUIRE(expert_offsets, GPTOSS_ERR_NULL, "moe_route: null pointer");
  GPTOSS_REQUIRE(B <= 0 || ((logits || !gate) && topk_w && topk_i && sorted_pair_ids && inv_perm),
                 GPTOSS_ERR_NULL, "moe_route: null pointer");
  GPTOSS_REQUIRE(E >= 1 && E <= 256 && k >= 1 && k <= 8 && k <= E && B >= 0, GPTOSS_ERR_DIM,
                 "moe_route: need 1 <= k <= min(8,E), E <= 256 (B=%d E=%d k=%d)", B, E, k);
  GPTOSS_REQUIRE((long long)B * k < (1ll << 30), GPTOSS_ERR_DIM, "moe_route: B*k too large");
  bool tile_ok = rows_per_tile >= 0 && rows_per_tile <= 256 && rows_per_tile % 32 == 0;
  GPTOSS_REQUIRE(tile_ok, GPTOSS_ERR_DIM, "moe_route: rows_per_tile must be 0 or a multiple of 32 up to 256");
  GPTOSS_REQUIRE(rows_per_tile == 0 || tiles, GPTOSS_ERR_NULL, "moe_route: tiles is NULL");
  hipStream_t s = (hipStream_t)stream;
  if (B > 0 && gate) {
    int rc = run_topk_softmax(logits, B, E, k, topk_w, topk_i, s);
    if (rc != GPTOSS_OK) return rc;
  }
  int nbits = 0;
  while ((1 << nbits) < E) nbits++;
  size_t smem = sizeof(int) * ((size_t)SORT_WAVES * E + E + (E + 1) + 2 * (size_t)E);
  const int P = B * k;
  if (sort_scratch != nullptr && P >= SORT_PARALLEL_MIN_PAIRS) {
    const int G = cdiv(P, SORT_THREADS);
    TraceScope ts("group_sort", s);
    group_count_kernel<<<G, SORT_THREADS, sizeof(int) * SORT_WAVES * E, s>>>(topk_i, P, E, nbits, sort_scratch,
                                                                           inv_perm);
    GPTOSS_LAUNCH_CHECK("group_count_kernel");
    group_scatter_kernel<<<G, SORT_THREADS, sizeof(int) * (5 * (size_t)E + 1), s>>>(
        topk_i, P, E, sort_scratch, inv_perm, expert_offsets, sorted_pair_ids, inv_perm,
        rows_per_tile ? tiles : nullptr, rows_per_tile, xcd_bounds, tile_cost0_x2);
    GPTOSS_LAUNCH_CHECK("group_scatter_kernel");
    return GPTOSS_OK;
  }
  {
    TraceScope ts("group_sort", s);
    group_sort_kernel<<<1, SORT_THREADS, smem, s>>>(topk_i, B * k, E, nbits, expert_offsets,
                                                    sorted_pair_ids, inv_perm,
                                                    rows_per_tile ? tiles : nullptr, rows_per_tile,
                                                    xcd_bounds, tile_cost0_x2);
  }
  GPTOSS_LAUNCH_CHECK("group_sort_kernel");
  return GPTOSS_OK;
}
