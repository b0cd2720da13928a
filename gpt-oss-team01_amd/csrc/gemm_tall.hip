// The grouped / dense bf16 GEMM for MANY rows (prompt passes: thousands of rows, ~1000 per expert),
// where the launch is bound by the matrix cores and not by streaming W.
//
// gemm_kernel.hpp feeds every MFMA one fresh LDS fragment (a wave owns 32 columns and all rows of
// the tile), which caps it at ~70 % of the MFMA rate before anything else is counted.  Here a
// workgroup of four waves (one per SIMD) owns a 256 x 256 tile and a wave a 128 x 128 quarter of
// it: 4 W fragments and 4 A fragments per k-step feed 16 MFMAs, half a fragment per MFMA.  Both
// operands go from global memory straight into LDS with global_load_lds_dwordx4 (no staging
// registers, no LDS store instructions) through four stages of 32 k; three stages are in flight;
// the load pipeline runs on from one work item into the next.  W is read in the same packed
// fragment order as everywhere else (a fragment lands in LDS as it is read); A rows are 64 bytes
// per stage, their four 16-byte chunks XOR-swizzled by (row >> 1) & 3 so that fragment reads are
// free of bank conflicts; the token gather of GEMM1 is a per-lane row offset of the load.
// The loads are inline assembly, invisible to the compiler's wait counting, and the loop has no
// other vector memory operation: every s_waitcnt vmcnt(N) is counted by hand (N = loads issued
// behind the one waited for; stores of the previous item's epilogue that are still in flight only
// make a wait stricter).
// Same operand roles (W fragment first: lane = token row, registers = channels), same k order and
// the same epilogue code as gemm_kernel.hpp, so the results are bit-identical to it.
#include <mutex>

#include "gemm_kernel.hpp"

namespace gptoss {

constexpr int TALL_THREADS = 256;
constexpr int TALL_BM = 256, TALL_BN = 256, TALL_BK = 32;
constexpr int TALL_STAGE = 32768;   // bytes: 8 column blocks x 2 k-steps x 1 KB of W, then 256 rows x 64 B of A
constexpr int TALL_NST = 4;
constexpr int TALL_IDS = TALL_NST * TALL_STAGE;  // behind the stages: 256 pair ids of the next item
constexpr int TALL_LOADS = 8;       // load instructions per wave and stage: 2 x 2 of W, 4 of A

__device__ __forceinline__ void tall_dma(unsigned lds_addr, uint32_t voff, const void *sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(
                   __builtin_amdgcn_readfirstlane(lds_addr)),
               "v"(voff), "s"(sbase)
               : "memory");
}
// two consecutive fragments (1 KB apart in memory and in LDS) with one M0
__device__ __forceinline__ void tall_dma2(unsigned lds_addr, uint32_t voff, const void *sbase) {
  asm volatile(
      "s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\tglobal_load_lds_dwordx4 %1, %2 offset:1024" ::"s"(
          __builtin_amdgcn_readfirstlane(lds_addr)),
      "v"(voff), "s"(sbase)
      : "memory");
}

// the sorted pair ids of 64 rows of the NEXT work item, one per lane, into LDS through the same counted pipeline
__device__ __forceinline__ void tall_dma_ids(unsigned lds_addr, uint32_t voff, const void *sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(
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
struct TallSrc {
  const unsigned char *w[2];  // first fragment of column blocks 2 wave, 2 wave + 1 of the tile
  uint32_t a[4];              // byte offsets of this lane's chunk of its four A rows
  int mat, row0, rows, ct;
};

template <bool GATHER, int EPI>
__global__ __launch_bounds__(TALL_THREADS, 1) void tall_gemm_kernel(GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = w >> 1, wc = w & 1;   // the wave's 128 x 128 quarter of the tile
  const int K = p.K, N = p.N;
  const int S = K / TALL_BK;
  const unsigned lds_base =
      __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)lds);
  const unsigned char *abase = reinterpret_cast<const unsigned char *>(p.A);
  const int *ids_lds = reinterpret_cast<const int *>(lds + TALL_IDS);

  // ---- work list: the order of grouped_gemm_kernel (gemm_kernel.hpp), with 256-row tiles --------
  const const_as<int> tiles = constant_ptr(p.tiles), bounds = constant_ptr(p.xcd_bounds);
  const int n_tiles = p.tiles ? tiles[0] : (p.dense_rows + TALL_BM - 1) / TALL_BM;
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
  auto decode = [&](int jj, TallSrc &t) {
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
      t.row0 = tile * TALL_BM;
      t.rows = min(TALL_BM, p.dense_rows - t.row0);
    }
    t.ct = __builtin_amdgcn_readfirstlane(t.ct);
    t.mat = __builtin_amdgcn_readfirstlane(t.mat);
    t.row0 = __builtin_amdgcn_readfirstlane(t.row0);
    t.rows = __builtin_amdgcn_readfirstlane(t.rows);
    // this wave loads column blocks 2w and 2w+1 of the tile's eight (a block beyond N repeats the last one)
    const unsigned char *wm = reinterpret_cast<const unsigned char *>(p.W) + (size_t)t.mat * N * K * 2;
#pragma unroll
    for (int q = 0; q < 2; q++) {
      const int cb = min(t.ct * 8 + 2 * w + q, N / 32 - 1);
      t.w[q] = uniform_ptr(wm + ((size_t)cb * (K / 16)) * 1024);
    }
  };
  // A: load instruction q of this wave moves tile rows (4w + q) * 16 .. + 16, four lanes per row and
  // one 16-byte chunk per lane; rows past the tile's last one repeat it (their results are not stored)
  auto a_offsets = [&](TallSrc &t, bool from_lds) {
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int r = (w * 4 + q) * 16 + (lane >> 2);
      int src;
      if (GATHER) src = (from_lds ? ids_lds[r] : p.row_ids[t.row0 + min(r, t.rows - 1)]) / p.top_k;
      else src = t.row0 + min(r, t.rows - 1);
      const int c = (lane & 3) ^ ((r >> 1) & 3);
      t.a[q] = ((uint32_t)src * (uint32_t)K) * 2u + (uint32_t)c * 16u;
    }
  };

  // one stage = 6 issue slots: 0, 1 = the two k-steps of W column block 2w + slot, 2..5 = A pieces
  const uint32_t voff_w = lane * 16;
  auto issue = [&](const TallSrc &t, int s, int buf, int slot) {
    const unsigned sb = lds_base + buf * TALL_STAGE;
    if (slot < 2) tall_dma2(sb + (2 * w + slot) * 2048, voff_w, t.w[slot] + (size_t)s * 2048);
    else tall_dma(sb + 16384 + (w * 4 + slot - 2) * 1024, t.a[slot - 2], abase + (size_t)s * 64);
  };

  f32x16 acc[4][4];   // [column block][row block]
  const int sw = ((lane & 31) >> 1) & 3, h = lane >> 5;
  const unsigned a_rd = 16384 + (wr * 128 + (lane & 31)) * 64;
  const unsigned a_k[2] = {(unsigned)(((0 + h) ^ sw) << 4), (unsigned)(((2 + h) ^ sw) << 4)};
  const unsigned w_rd = (wc * 4) * 2 * 1024 + lane * 16;
  bf16x8 F[2][8];     // two fragment sets: [0..3] W column blocks, [4..7] A row blocks
  auto rd = [&](int buf, int kk, int set, int f) {
    const unsigned char *sb = lds + buf * TALL_STAGE;
    if (f < 4) F[set][f] = as_bf16x8(*reinterpret_cast<const u32x4 *>(sb + w_rd + (f * 2 + kk) * 1024));
    else F[set][f] = as_bf16x8(*reinterpret_cast<const u32x4 *>(sb + a_rd + (f - 4) * 32 * 64 + a_k[kk]));
  };
  constexpr int RO[8] = {0, 4, 5, 6, 7, 1, 2, 3};  // read order: what the first MFMAs need first

  TallSrc cur, nxt;
  decode(j, cur);
  a_offsets(cur, false);
#pragma unroll
  for (int q = 0; q < 3; q++)
#pragma unroll
    for (int m = 0; m < 6; m++) issue(cur, q, q, m);
  wait_vmcnt<2 * TALL_LOADS>();   // stage 0 has landed; stages 1 and 2 may be on their way
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int f = 0; f < 8; f++) rd(0, 0, 0, RO[f]);
  __builtin_amdgcn_sched_barrier(0);
  int g = 0;  // running stage count: the buffer of a stage is its count & 3
  while (true) {
    const int jn = j + per_xcd;
    const bool more = valid(jn);
    nxt = cur;  // past the last item the pipeline requests this item's first stages again, and drops them
    if (more) {
      decode(jn, nxt);
      if (GATHER) {
        // One more load in the queue, in front of the five of stage g+3: the wait of this stage is one
        // load stricter than it needs to be, and the wait of the next stage (13 younger loads) covers
        // this load, so the ids are in LDS, written and read by this wave alone, from stage 2 on.
        const int r = min(w * 64 + lane, nxt.rows - 1);
        tall_dma_ids(lds_base + TALL_IDS + w * 256, (uint32_t)r * 4u, uniform_ptr(p.row_ids + nxt.row0));
      } else {
        a_offsets(nxt, false);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int r = 0; r < 4; r++)
#pragma unroll
        for (int x = 0; x < 16; x++) acc[i][r][x] = 0.f;
    for (int s = 0; s < S; s++, g++) {
      if (GATHER && s == 2 && more) a_offsets(nxt, true);
      const int cb = g & 3, nb = (g + 1) & 3, pb = (g + 3) & 3;
      const bool wrap = s + 3 >= S;
      const int s3 = wrap ? s + 3 - S : s + 3;
      TallSrc src;
#pragma unroll
      for (int q = 0; q < 2; q++) src.w[q] = wrap ? nxt.w[q] : cur.w[q];
#pragma unroll
      for (int q = 0; q < 4; q++) src.a[q] = wrap ? nxt.a[q] : cur.a[q];
      __builtin_amdgcn_sched_barrier(0);
      // k-step 0 of the stage: its fragments are in set 0; read those of k-step 1, request half of stage g+3
#pragma unroll
      for (int m = 0; m < 16; m++) {
        acc[m >> 2][m & 3] =
            __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[0][m >> 2], F[0][4 + (m & 3)], acc[m >> 2][m & 3], 0, 0, 0);
        if (m < 8) rd(cb, 1, 1, RO[m]);
        else if (m >= 10 && (m & 1) == 0) issue(src, s3, pb, (m - 10) >> 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      // behind stage g+1 were issued stage g+2 (8 loads) and five loads of stage g+3
      wait_vmcnt<TALL_LOADS + 5>();
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      // k-step 1: read k-step 0 of the next stage, request the other half of stage g+3
#pragma unroll
      for (int m = 0; m < 16; m++) {
        acc[m >> 2][m & 3] =
            __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[1][m >> 2], F[1][4 + (m & 3)], acc[m >> 2][m & 3], 0, 0, 0);
        if (m < 8) rd(nb, 0, 0, RO[m]);
        else if (m >= 10 && (m & 1) == 0) issue(src, s3, pb, 3 + ((m - 10) >> 1));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // epilogue: the wave's four column blocks, each with its four 32-row blocks.  The empty asm pins
    // a column block's accumulators in their AGPRs until the block before it has been stored: left
    // alone, the compiler copies all 256 of them to VGPRs where the stage loop ends, and spills.
#pragma unroll
    for (int i = 0; i < 4; i++) {
      asm volatile("" : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]), "+a"(acc[i][3]));
      const int n0 = cur.ct * TALL_BN + (wc * 4 + i) * 32;
      if (n0 < N) epilogue_store<4, EPI, true>(p, cur.mat, cur.row0 + wr * 128, cur.rows - wr * 128, n0, lane, acc[i]);
    }
    if (!more) break;
    j = jn;
    cur = nxt;
  }
  // loads into LDS are still in flight: the workgroup must not give its LDS back before they land
  wait_vmcnt<0>();
}

template <bool GATHER, int EPI>
static int launch_tall(const GemmParams &p, int max_tiles, hipStream_t s) {
  constexpr int MAX_DEV = 64;
  static std::mutex mu;
  static bool raised[MAX_DEV];
  int dev = 0;
  GPTOSS_HIP(hipGetDevice(&dev));
  GPTOSS_REQUIRE(dev >= 0 && dev < MAX_DEV, GPTOSS_ERR_STATE, "run_gemm: device ordinal %d outside 0..%d", dev, MAX_DEV - 1);
  auto kern = tall_gemm_kernel<GATHER, EPI>;
  const size_t smem = (size_t)TALL_NST * TALL_STAGE + TALL_BM * 4;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (!raised[dev]) {
      GPTOSS_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)smem));
      raised[dev] = true;
    }
  }
  const int total = max_tiles * p.n_col_tiles;
  int grid = ((total + 7) / 8) * 8;
  if (grid > 256) grid = 256;
  if (grid == 0) return GPTOSS_OK;
  {
    TraceScope ts(GATHER ? "gemm1_gather_swiglu" : "gemm_f32", s);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(TALL_THREADS), smem, s, p);
  }
  GPTOSS_LAUNCH_CHECK("tall_gemm_kernel");
  return GPTOSS_OK;
}

bool gemm_tall_applies(const GemmParams &p, bool gather, int epi) {
  const bool kind = (gather && epi == EPI_SWIGLU) || (!gather && epi == EPI_F32);
  return kind && !p.w_mxfp4 && p.K % TALL_BK == 0 && p.K >= 8 * TALL_BK && p.N % 32 == 0;
}

// p.n_col_tiles must count 256-column tiles (it does: gemm_col_tiles); tiles of at most 256 rows
int run_gemm_tall(const GemmParams &p, bool gather, int epi, int max_tiles, long long max_rows, hipStream_t s) {
  GPTOSS_REQUIRE(gemm_tall_applies(p, gather, epi), GPTOSS_ERR_DIM,
                 "run_gemm: 256-row tiles need bf16 weights, K %% 32 == 0, K >= 256, N %% 32 == 0 and the gather+SwiGLU "
                 "or plain fp32 form (gather=%d epi=%d N=%d K=%d)", (int)gather, epi, p.N, p.K);
  // a row of A is addressed by a 32-bit byte offset
  GPTOSS_REQUIRE(max_rows * p.K * 2 < (1ll << 32), GPTOSS_ERR_DIM,
                 "run_gemm: 256-row tiles need rows x K below 2^31 elements (rows<=%lld K=%d)", max_rows, p.K);
  if (gather) return launch_tall<true, EPI_SWIGLU>(p, max_tiles, s);
  return launch_tall<false, EPI_F32>(p, max_tiles, s);
}

}  // namespace gptoss
