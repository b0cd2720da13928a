// The grouped / dense bf16 GEMM for MANY rows (prompt passes: thousands of rows, ~1000 per expert),
// where the launch is bound by the matrix cores and not by streaming W.
//
// gemm_kernel.hpp feeds every MFMA one fresh LDS fragment (a wave owns 32 columns and all rows of
// the tile), which caps it at ~70 % of the MFMA rate before anything else is counted.  Here a
// workgroup of four waves (one per SIMD) owns a 256 x 256 tile and a wave a 128 x 128 quarter of
// it: 4 W fragments and 4 A fragments per k-step feed 16 MFMAs, half a fragment per MFMA.  Both
// operands go from global memory straight into LDS with global_load_lds_dwordx4 (no staging
// registers, no LDS store instructions), and the load pipeline runs on from one work item into
// the next.
//   W: stages of 32 k in four buffers, three in flight, in the same packed fragment order as
//      everywhere else (a fragment lands in LDS as it is read).
//   A: chunks of 64 k in three buffers, two in flight: a load instruction moves 8 rows x 128 bytes,
//      whole cache lines.  (Rows of 64 bytes, one 32-k stage at a time, fetch every line twice, once per half:
//      the loads of A then cost 2-3 times those of W, 55-65 us of a 265 us launch.)  The eight
//      16-byte pieces of a row are XOR-swizzled by (row >> 1) & 7, so fragment reads are free of
//      bank conflicts; the token gather of GEMM1 is a per-lane row offset of the load.
// The loads are inline assembly, invisible to the compiler's wait counting, and the loop has no
// other vector memory operation: every s_waitcnt vmcnt(N) is counted by hand (N = loads issued
// behind the one waited for; stores of the previous item's epilogue that are still in flight only
// make a wait stricter).
// Same operand roles (W fragment first: lane = token row, registers = channels), same k order and
// the same epilogue code as gemm_kernel.hpp, so the results are bit-identical to it.  Three forms:
// gather + SwiGLU (GEMM1 of a prompt pass), plain fp32 output (GEMM2, the projections), and the row
// arg-max of the classifier, which writes no products at all and is the fastest of the three.
#include <mutex>

#include "gemm_kernel.hpp"

namespace gptoss {

constexpr int TALL_THREADS = 256;
constexpr int TALL_BK = 32;   // k of a W stage; an A chunk is two of them

// A workgroup is WR x WC waves (four in all), a wave RB x CB blocks of 32 x 32 outputs.
template <int WR_, int WC_, int RB_, int CB_>
struct TallShape {
  static_assert(WR_ * WC_ == 4, "four waves, one per SIMD");
  static constexpr int WR = WR_, WC = WC_, RB = RB_, CB = CB_;
  static constexpr int BM = WR * RB * 32, BN = WC * CB * 32;
  static constexpr int NSTW = 4;                        // W stage buffers, NSTW - 1 in flight
  static constexpr int W_BYTES = WC * CB * 2048;        // a W stage: a column block's two k-steps are 2 KB
  static constexpr int A_BYTES = BM * 128;              // an A chunk: 128 bytes of every row
  static constexpr int A_OFF = NSTW * W_BYTES;          // three A chunk buffers behind the W stages
  static constexpr int SMEM = A_OFF + 3 * A_BYTES;      // 160 KB for the 256 x 256 tile: all of a CU's LDS
  static constexpr int LW = WC * CB * 2 / 4;            // load instructions per wave: W fragments of a stage,
  static constexpr int LA = BM / 8 / 4;                 // 8-row pieces of an A chunk
  static_assert(WC * CB * 2 % 4 == 0 && BM % 32 == 0, "the loads are shared out evenly");
  static_assert(SMEM <= 160 * 1024, "LDS of a CU");
  static constexpr int NM = RB * CB, NR = RB + CB;      // MFMAs and fragment reads of a k-step
  static_assert(LW % 2 == 0 && LA % 4 == 0, "a k-step issues half a W stage and a quarter of an A chunk");
  static_assert(NM >= NR + 2 * (LA / 4 + LW / 2), "room for a k-step's reads and loads between its MFMAs");
};

__device__ __forceinline__ void tall_dma(unsigned lds_addr, uint32_t voff, const void *sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(
                   __builtin_amdgcn_readfirstlane(lds_addr)),
               "v"(voff), "s"(sbase)
               : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
template <typename T>
__device__ __forceinline__ const T *uniform_ptr(const T *q) {
  const uint64_t v = reinterpret_cast<uint64_t>(q);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return reinterpret_cast<const T *>(((uint64_t)hi << 32) | lo);
}

// where one work item's operands come from, for this wave's share of the loads
template <class SH>
struct TallSrc {
  const unsigned char *w[SH::LW];  // stage 0 of the W fragments this wave loads
  uint32_t a[SH::LA];              // byte offsets of this lane's piece of the A rows it loads
  int mat, row0, rows, ct;
};

template <class SH, bool GATHER, int EPI>
__global__ __launch_bounds__(TALL_THREADS, 1) void tall_gemm_kernel(GemmParams p) {
  constexpr int RB = SH::RB, CB = SH::CB, LW = SH::LW, LA = SH::LA, LW1 = SH::LW / 2, LA1 = SH::LA / 4;
  constexpr int NM = SH::NM, NR = SH::NR, NSTW = SH::NSTW;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = w / SH::WC, wc = w % SH::WC;   // the wave's part of the tile
  const int K = p.K, N = p.N;
  const int S = K / TALL_BK;                    // even: K % 64 == 0
  const unsigned lds_base =
      __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)lds);
  const unsigned char *abase = reinterpret_cast<const unsigned char *>(p.A);

  // ---- work list: the order of grouped_gemm_kernel (gemm_kernel.hpp), with tiles of BM rows --------
  const const_as<int> tiles = constant_ptr(p.tiles), bounds = constant_ptr(p.xcd_bounds);
  const int n_tiles = p.tiles ? tiles[0] : (p.dense_rows + SH::BM - 1) / SH::BM;
  const int total = n_tiles * p.n_col_tiles;
  const int per_xcd = gridDim.x >> 3;
  const int xcd = blockIdx.x & 7;
  int lo, hi;
  if (p.xcd_bounds) {
    auto item = [&](int b) { return (b >> 16) * p.n_col_tiles + (((b & 0xffff) * p.n_col_tiles) >> 16); };
    lo = item(bounds[xcd]);
    hi = item(bounds[xcd + 1]);
  } else {
    const int chunk = (total + 7) >> 3;
    lo = xcd * chunk;
    hi = min(total, lo + chunk);
  }
  int j = blockIdx.x >> 3;
  auto valid = [&](int jj) { return lo + jj < hi; };
  if (!valid(j)) return;
  // which tile, which matrix, and this wave's share of the W loads
  auto decode = [&](int jj, TallSrc<SH> &t) {
    const int work = lo + jj;
    int tile;
    if (p.tiles && p.tile_block > 1 && p.xcd_bounds) {
      const int info = bounds[XCD_BOUNDS_INTS + work / p.n_col_tiles];
      const int first = info >> 8, th = info & 255;
      const int v = work - first * p.n_col_tiles;
      t.ct = v / th;
      tile = first + (v - t.ct * th);
    } else if (p.tiles) {
      tile = work / p.n_col_tiles;
      t.ct = work - tile * p.n_col_tiles;
    } else {
      t.ct = work / n_tiles;
      tile = work - t.ct * n_tiles;
    }
    if (p.tiles) {
      t.mat = tiles[1 + 3 * tile];
      t.row0 = tiles[2 + 3 * tile];
      t.rows = tiles[3 + 3 * tile];
    } else {
      t.mat = 0;
      t.row0 = tile * SH::BM;
      t.rows = min(SH::BM, p.dense_rows - t.row0);
    }
    t.ct = __builtin_amdgcn_readfirstlane(t.ct);
    t.mat = __builtin_amdgcn_readfirstlane(t.mat);
    t.row0 = __builtin_amdgcn_readfirstlane(t.row0);
    t.rows = __builtin_amdgcn_readfirstlane(t.rows);
    // W fragment f of a stage = (column block f / 2 of the tile, k-step f % 2); a block beyond N repeats the last one
    const unsigned char *wm = reinterpret_cast<const unsigned char *>(p.W) + (size_t)t.mat * N * K * 2;
#pragma unroll
    for (int q = 0; q < LW; q++) {
      const int f = w * LW + q;
      const int cb = min(t.ct * (SH::WC * CB) + (f >> 1), N / 32 - 1);
      t.w[q] = uniform_ptr(wm + ((size_t)cb * (K / 16) + (f & 1)) * 1024);
    }
  };
  // A: load instruction q of this wave moves 8 tile rows, eight lanes per row and one 16-byte piece
  // per lane: the lane at position p of row r fetches piece p ^ ((r >> 1) & 7).  Rows past the
  // tile's last one repeat it (their results are not stored).  The pair ids of a gathered tile are
  // read through the constant address space: scalar loads, which the vector-memory counter of the
  // hand-counted waits does not see.
  auto a_offsets = [&](TallSrc<SH> &t) {
    const const_as<int> ids = constant_ptr(p.row_ids);
#pragma unroll
    for (int q = 0; q < LA; q++) {
      const int r0 = (w * LA + q) * 8, r = r0 + (lane >> 3);
      int src;
      if (GATHER) {
        src = ids[t.row0 + min(r0, t.rows - 1)];
#pragma unroll
        for (int i = 1; i < 8; i++) {
          const int id = ids[t.row0 + min(r0 + i, t.rows - 1)];
          src = (lane >> 3) == i ? id : src;
        }
        src /= p.top_k;
      } else {
        src = t.row0 + min(r, t.rows - 1);
      }
      const int c = (lane & 7) ^ ((r >> 1) & 7);
      t.a[q] = ((uint32_t)src * (uint32_t)K) * 2u + (uint32_t)c * 16u;
    }
  };

  // W load instruction q of this wave for stage s of an item, into W buffer buf
  const uint32_t voff_w = lane * 16;
  auto issue_w = [&](const TallSrc<SH> &t, int s, int buf, int q) {
    tall_dma(lds_base + buf * SH::W_BYTES + (w * LW + q) * 1024, voff_w, t.w[q] + (size_t)s * 2048);
  };
  // A load instruction q of this wave for chunk c of an item, into A buffer buf
  auto issue_a = [&](const TallSrc<SH> &t, int c, int buf, int q) {
    tall_dma(lds_base + SH::A_OFF + buf * SH::A_BYTES + (w * LA + q) * 1024, t.a[q], abase + (size_t)c * 128);
  };

  f32x16 acc[CB][RB];   // [column block][row block]
  const int sw = ((lane & 31) >> 1) & 7, h = lane >> 5;
  const unsigned a_rd = SH::A_OFF + (wr * RB * 32 + (lane & 31)) * 128;
  unsigned a_k[4];      // where the lane finds its piece of k-step x of a chunk
#pragma unroll
  for (int x = 0; x < 4; x++) a_k[x] = (unsigned)(((2 * x + h) ^ sw) << 4);
  const unsigned w_rd = (wc * CB) * 2 * 1024 + lane * 16;
  bf16x8 F[2][NR];      // two fragment sets: [0, CB) W column blocks, [CB, CB + RB) A row blocks
  // fragment read number i of a k-step, in the order the MFMAs want them: W0, every A, the other W;
  // x = the k-step's number inside its A chunk
  auto rd = [&](int wbuf, int kk, int abuf, int x, int set, int i) {
    const int f = i == 0 ? 0 : (i <= RB ? CB + i - 1 : i - RB);
    if (f < CB)
      F[set][f] = as_bf16x8(*reinterpret_cast<const u32x4 *>(lds + wbuf * SH::W_BYTES + w_rd + (f * 2 + kk) * 1024));
    else
      F[set][f] = as_bf16x8(
          *reinterpret_cast<const u32x4 *>(lds + abuf * SH::A_BYTES + a_rd + (f - CB) * 32 * 128 + a_k[x]));
  };
  // one k-step: NM MFMAs out of fragment set `set`; with the first NR of them the fragment reads of
  // the next k-step (into the other set), behind those whatever loads `loads(m)` issues
  auto kstep = [&](int set, int wbuf, int kk, int abuf, int x, auto &&loads) {
#pragma unroll
    for (int m = 0; m < NM; m++) {
      acc[m / RB][m % RB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[set][m / RB], F[set][CB + m % RB],
                                                                    acc[m / RB][m % RB], 0, 0, 0);
      if (m < NR) rd(wbuf, kk, abuf, x, set ^ 1, m);
      loads(m);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  TallSrc<SH> cur, nxt;
  decode(j, cur);
  a_offsets(cur);
  // The first loads go out in the order the stage loop would have issued them, so that its waits
  // count right from the first stage on: chunk 0 and W stage 0, then a quarter of chunk 1 with
  // every half of W stages 1 and 2.
#pragma unroll
  for (int q = 0; q < LA; q++) issue_a(cur, 0, 0, q);
#pragma unroll
  for (int q = 0; q < LW; q++) issue_w(cur, 0, 0, q);
#pragma unroll
  for (int x = 0; x < 4; x++) {
#pragma unroll
    for (int q = 0; q < LA1; q++) issue_a(cur, 1, 1, x * LA1 + q);
#pragma unroll
    for (int q = 0; q < LW1; q++) issue_w(cur, 1 + (x >> 1), 1 + (x >> 1), (x & 1) * LW1 + q);
  }
  wait_vmcnt<4 * (LA1 + LW1)>();   // chunk 0 and stage 0 have landed; the loads behind them may be on their way
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < NR; i++) rd(0, 0, 0, 0, 0, i);
  __builtin_amdgcn_sched_barrier(0);
  int g = 0;   // running stage count (even at the start of every item): W buffer g & 3
  int ab = 0;  // A buffer of the current chunk: the running chunk count modulo 3
  while (true) {
    const int jn = j + per_xcd;
    const bool more = valid(jn);
    nxt = cur;  // past the last item the pipeline requests this item's first loads again, and drops them
    if (more) {
      decode(jn, nxt);
      a_offsets(nxt);
    }
#pragma unroll
    for (int i = 0; i < CB; i++)
#pragma unroll
      for (int r = 0; r < RB; r++)
#pragma unroll
        for (int x = 0; x < 16; x++) acc[i][r][x] = 0.f;
    for (int s = 0; s < S; s += 2, g += 2) {
      // ---- even stage s: the first half of A chunk s / 2 --------------------------------------
      const int ab1 = ab == 2 ? 0 : ab + 1, ab2 = ab1 == 2 ? 0 : ab1 + 1;
      const bool wrap_a = s + 4 >= S;             // the chunk requested now: two ahead, or one of the next item's first two
      const bool wrap_w0 = s + 3 >= S, wrap_w1 = s + 4 >= S;
      TallSrc<SH> sa, s0, s1;
#pragma unroll
      for (int q = 0; q < LA; q++) sa.a[q] = wrap_a ? nxt.a[q] : cur.a[q];
#pragma unroll
      for (int q = 0; q < LW; q++) {
        s0.w[q] = wrap_w0 ? nxt.w[q] : cur.w[q];
        s1.w[q] = wrap_w1 ? nxt.w[q] : cur.w[q];
      }
      const int ca = (wrap_a ? s + 4 - S : s + 4) >> 1;
      const int sw0 = wrap_w0 ? s + 3 - S : s + 3, sw1 = wrap_w1 ? s + 4 - S : s + 4;
      __builtin_amdgcn_sched_barrier(0);
      // Every k-step issues a quarter of A chunk s / 2 + 2, into the buffer that chunk s / 2 - 1 left
      // (every wave is past the barrier of the stage that read it last), and half of a W stage,
      // behind the fragment reads: loads(x, ...) places them after MFMAs NR, NR + 2, ...
      auto loads = [&](int m, int x, const TallSrc<SH> &sw_, int st, int wbuf, int half) {
#pragma unroll
        for (int q = 0; q < LA1; q++)
          if (m == NR + 2 * q) issue_a(sa, ca, ab2, x * LA1 + q);
#pragma unroll
        for (int q = 0; q < LW1; q++)
          if (m == NR + 2 * (LA1 + q)) issue_w(sw_, st, wbuf, half * LW1 + q);
      };
      kstep(0, g & 3, 1, ab, 1, [&](int m) { loads(m, 0, s0, sw0, (g + 3) & 3, 0); });
      // behind W stage s+1 were issued the loads of two k-steps of stage s-1 and of one of stage s
      wait_vmcnt<3 * (LA1 + LW1)>();
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      kstep(1, (g + 1) & 3, 0, ab, 2, [&](int m) { loads(m, 1, s0, sw0, (g + 3) & 3, 1); });
      // ---- odd stage s+1: the second half of the chunk -----------------------------------------
      kstep(0, (g + 1) & 3, 1, ab, 3, [&](int m) { loads(m, 2, s1, sw1, (g + 4) & 3, 0); });
      // W stage s+2, and with it the A chunk that the next stage starts (its last loads went out in
      // front of that stage's), must have landed
      wait_vmcnt<3 * (LA1 + LW1)>();
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      kstep(1, (g + 2) & 3, 0, ab1, 0, [&](int m) { loads(m, 3, s1, sw1, (g + 4) & 3, 1); });
      ab = ab1;
    }
    // epilogue: the wave's column blocks, each with its row blocks.  The empty asm pins a column
    // block's accumulators in their AGPRs until the block before it has been stored: left alone,
    // the compiler copies every accumulator to VGPRs where the stage loop ends, and spills.
    if constexpr (EPI == EPI_ARGMAX) {
      // Row-wise arg-max of the wave's CB x 32 columns without writing the products.  A lane holds
      // one row of each row block and 16 channels of each column block: it scans them in ascending
      // column order with a strict >, so the lowest column wins a tie; the two half-waves are merged
      // with the same rule, and the first 32 lanes write the (value, column) pair of their rows for
      // this half of the column tile.
      float bv[RB];
      int bi[RB];
#pragma unroll
      for (int r = 0; r < RB; r++) {
        bv[r] = -INFINITY;
        bi[r] = 0x7fffffff;
      }
      const const_as<float> bias = constant_ptr(p.bias);
#pragma unroll
      for (int i = 0; i < CB; i++) {
#pragma unroll
        for (int r = 0; r < RB; r++) asm volatile("" : "+a"(acc[i][r]));
        const int n0 = cur.ct * SH::BN + (wc * CB + i) * 32;
        if (n0 < N) {
#pragma unroll
          for (int gq = 0; gq < 16; gq++) {
            const int c_lo = n0 + (gq >> 2) * 8 + (gq & 3), c_hi = c_lo + 4;
            float b = 0.f;
            if (p.bias) {
              const float b_lo = bias[c_lo], b_hi = bias[c_hi];
              b = h ? b_hi : b_lo;
            }
            const int col = h ? c_hi : c_lo;
#pragma unroll
            for (int r = 0; r < RB; r++) {
              const float v = acc[i][r][gq] + b;
              if (v > bv[r]) {
                bv[r] = v;
                bi[r] = col;
              }
            }
          }
        }
      }
#pragma unroll
      for (int r = 0; r < RB; r++) {
        const float ov = __shfl_xor(bv[r], 32, 64);
        const int oi = __shfl_xor(bi[r], 32, 64);
        if (ov > bv[r] || (ov == bv[r] && oi < bi[r])) {
          bv[r] = ov;
          bi[r] = oi;
        }
        const int row = (wr * RB + r) * 32 + lane;
        if (lane < 32 && row < cur.rows) {
          const size_t o = (size_t)(cur.row0 + row) * (SH::WC * p.n_col_tiles) + cur.ct * SH::WC + wc;
          p.amax_val[o] = bv[r];
          p.amax_idx[o] = bi[r];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < CB; i++) {
#pragma unroll
        for (int r = 0; r < RB; r++) asm volatile("" : "+a"(acc[i][r]));
        const int n0 = cur.ct * SH::BN + (wc * CB + i) * 32;
        if (n0 < N)
          epilogue_store<RB, EPI, true>(p, cur.mat, cur.row0 + wr * RB * 32, cur.rows - wr * RB * 32, n0, lane,
                                        acc[i]);
      }
    }
    if (!more) break;
    j = jn;
    cur = nxt;
  }
  // loads into LDS are still in flight: the workgroup must not give its LDS back before they land
  wait_vmcnt<0>();
}

template <class SH, bool GATHER, int EPI>
static int launch_tall(const GemmParams &p, int max_tiles, hipStream_t s) {
  constexpr int MAX_DEV = 64;
  static std::mutex mu;
  static bool raised[MAX_DEV];
  int dev = 0;
  GPTOSS_HIP(hipGetDevice(&dev));
  GPTOSS_REQUIRE(dev >= 0 && dev < MAX_DEV, GPTOSS_ERR_STATE, "run_gemm: device ordinal %d outside 0..%d", dev, MAX_DEV - 1);
  auto kern = tall_gemm_kernel<SH, GATHER, EPI>;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (!raised[dev]) {
      GPTOSS_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     SH::SMEM));
      raised[dev] = true;
    }
  }
  GemmParams q = p;
  q.n_col_tiles = cdiv(p.N, SH::BN);
  const int total = max_tiles * q.n_col_tiles;
  int grid = ((total + 7) / 8) * 8;
  if (grid > 256) grid = 256;
  if (grid == 0) return GPTOSS_OK;
  {
    TraceScope ts(EPI == EPI_ARGMAX ? "gemm_argmax" : GATHER ? "gemm1_gather_swiglu" : "gemm_f32", s);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(TALL_THREADS), SH::SMEM, s, q);
  }
  GPTOSS_LAUNCH_CHECK("tall_gemm_kernel");
  return GPTOSS_OK;
}

// The shape in use.  Tiles of 128 rows for the dense GEMMs of a decode step of 1024 rows (128 x 96,
// 128, 160 and 192 columns, on an earlier form of this kernel with 32-k stages for both operands)
// came out bit-identical as well, and 3-4 us ahead of the streaming kernels' 41-43 us on the two
// projections of the 20B shape: a wave that owns 3 to 6 output blocks has 4 to 6 fragment reads per
// k-step of 100-200 cycles and nothing else to run while they are on their way, so even without any
// load or store such a launch takes 21-28 us where its MFMAs alone take 15.  128 x 128 tiles with two
// workgroups per CU (80 KB of LDS each, on this form of the kernel) did not move that either: 48 and
// 41 us against 43 and 43.  Not worth a second dispatch rule.
using Tall256 = TallShape<2, 2, 4, 4>;   // 256 x 256

bool gemm_tall_applies(const GemmParams &p, bool gather, int epi) {
  const bool kind = (gather && epi == EPI_SWIGLU) || (!gather && epi == EPI_F32) ||
                    (!gather && epi == EPI_ARGMAX && p.tiles == nullptr && p.amax_val && p.amax_idx);
  // whole A chunks of 64 k, and at least 8 stages: an item's first loads are requested during the
  // last four stages of the item before it
  static_assert(2 * TALL_BK == 64, "gemm_tall_shape_ok states the chunk size");
  return kind && !p.w_mxfp4 && gemm_tall_shape_ok(p.N, p.K, 0);
}

int run_gemm_tall(const GemmParams &p, bool gather, int epi, int max_tiles, long long max_rows, hipStream_t s) {
  GPTOSS_REQUIRE(gemm_tall_applies(p, gather, epi), GPTOSS_ERR_DIM,
                 "run_gemm: 256-row tiles need bf16 weights, K %% 64 == 0, K >= 256, N %% 32 == 0 and the "
                 "gather+SwiGLU, plain fp32 or dense arg-max form (gather=%d epi=%d N=%d K=%d)", (int)gather, epi, p.N, p.K);
  // a row of A is addressed by a 32-bit byte offset
  GPTOSS_REQUIRE(max_rows * p.K * 2 < (1ll << 32), GPTOSS_ERR_DIM,
                 "run_gemm: 256-row tiles need rows x K below 2^31 elements (rows<=%lld K=%d)", max_rows, p.K);
  static_assert(Tall256::WC == 2, "dense_gemm reports two arg-max pairs per row and column tile");
  if (epi == EPI_ARGMAX) return launch_tall<Tall256, false, EPI_ARGMAX>(p, max_tiles, s);
  if (gather) return launch_tall<Tall256, true, EPI_SWIGLU>(p, max_tiles, s);
  return launch_tall<Tall256, false, EPI_F32>(p, max_tiles, s);
}

}  // namespace gptoss
