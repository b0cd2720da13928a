// Grouped (per-expert) and dense bf16 GEMMs for gfx950 built on v_mfma_f32_32x32x16_bf16.
//
//   C[rows, N] = A[rows, K] . W[N, K]^T      rows = the tokens routed to one expert (or a slice
//                                            of a dense batch), W = that expert's matrix
//
// Shape of the problem at decode time: a few hundred rows per expert against 25 M weights per
// expert, i.e. every weight is used by ~128 rows and the kernel is bound by streaming W from
// HBM.  The design follows from that:
//   * W is stored in MFMA-fragment order (gptoss_pack_weight): the 1 KB a wave needs for one
//     32-column x 16-k operand is contiguous, so each wave streams its own columns with
//     perfectly coalesced 128-bit loads straight into registers (no LDS hop, no reuse needed:
//     a workgroup covers all rows of its tile, up to 256, so W is read once);
//   * the activations (shared by the 4 waves) go through a double-buffered, padded LDS tile; the
//     token gather of the reference's pack step is folded into that load;
//   * a workgroup = 256 virtual columns x up to 256 rows; each wave owns 64 columns as two
//     B fragments and reuses every A fragment it reads from LDS for two MFMAs;
//   * work items come from the device-built tile list (expert,row0,rows), mapped so that the
//     workgroups of one XCD walk consecutive column tiles of the same expert (A stays in that
//     XCD's L2);
//   * epilogues: +bias -> fp32, or +bias -> clamped SwiGLU -> bf16 with gate and up of a pair in
//     the same lane (arranged by the packing order, so no cross-lane traffic).
#include <type_traits>

#include "common.hpp"
#include "gemm.hpp"

namespace gptoss {

constexpr int GEMM_THREADS = 256;
constexpr int BK = 64;            // k per LDS slab (4 MFMA k-steps)
constexpr int LDS_ROW = BK + 8;   // padded row length in bf16 elements (144 B)
constexpr int BN = 256;           // virtual columns per workgroup (4 waves x 64)

// One (row tile, column tile) work item with a compile-time number of 32-row blocks, so every
// loop below is fully unrolled and every global load is unconditional (the wait counters the
// compiler derives stay exact and the prefetches stay in flight across iterations).
// MXFP4 operand expansion.  One dword holds the lane's 8 e2m1 codes of a k-step (element j < 4 in
// the low nibble of byte j, element j >= 4 in the high nibble of byte j-4).  tab[] holds the eight
// positive bf16 magnitudes already multiplied by the block's power-of-two scale, as byte tables
// for v_perm_b32: tab[0]/tab[1] = low bytes of entries 0-3 / 4-7, tab[2]/tab[3] = high bytes.
struct Fp4Table {
  uint32_t lo_a, lo_b, hi_a, hi_b;
};

__device__ __forceinline__ Fp4Table fp4_table(uint32_t e8m0) {
  // bf16 bit patterns of 0, .5 | 1, 1.5 | 2, 3 | 4, 6 as pairs; the exponent field starts at bit 7
  // d * 0x00800080 adds d to both exponent fields: for negative d the borrow out of the low half
  // is undone by the carry of the low-half addition below
  const uint32_t dd = (e8m0 - 127u) * 0x00800080u;
  const uint32_t t01 = 0x3F000000u + ((e8m0 - 127u) << 23);  // entry 0 stays +0
  const uint32_t t23 = 0x3FC03F80u + dd;
  const uint32_t t45 = 0x40404000u + dd;
  const uint32_t t67 = 0x40C04080u + dd;
  Fp4Table t;
  // v_perm_b32(S0, S1, sel): selector values 0-3 pick bytes of S1, 4-7 bytes of S0
  t.lo_a = __builtin_amdgcn_perm(t23, t01, 0x06040200u);
  t.hi_a = __builtin_amdgcn_perm(t23, t01, 0x07050301u);
  t.lo_b = __builtin_amdgcn_perm(t67, t45, 0x06040200u);
  t.hi_b = __builtin_amdgcn_perm(t67, t45, 0x07050301u);
  return t;
}

__device__ __forceinline__ u32x4 fp4_expand(uint32_t w, const Fp4Table &t) {
  const uint32_t m_lo = w & 0x07070707u, m_hi = (w >> 4) & 0x07070707u;
  uint32_t l0 = __builtin_amdgcn_perm(t.lo_b, t.lo_a, m_lo);
  uint32_t h0 = __builtin_amdgcn_perm(t.hi_b, t.hi_a, m_lo) | ((w << 4) & 0x80808080u);
  uint32_t l1 = __builtin_amdgcn_perm(t.lo_b, t.lo_a, m_hi);
  uint32_t h1 = __builtin_amdgcn_perm(t.hi_b, t.hi_a, m_hi) | (w & 0x80808080u);
  // interleave low and high bytes into bf16 pairs: elements 0,1 | 2,3 | 4,5 | 6,7
  return u32x4{__builtin_amdgcn_perm(h0, l0, 0x05010400u), __builtin_amdgcn_perm(h0, l0, 0x07030602u),
               __builtin_amdgcn_perm(h1, l1, 0x05010400u), __builtin_amdgcn_perm(h1, l1, 0x07030602u)};
}

template <int MB, bool GATHER, int EPI, bool FP4>
__device__ __forceinline__ void gemm_tile(const GemmParams &p, bf16_t *lds, int lds_stage, int mat,
                                          int row0, int rows, int ct) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int K = p.K, N = p.N;
  const int n0_raw = ct * BN + wave * 64;
  const bool wave_active = n0_raw < N;
  const int n0 = wave_active ? n0_raw : N - 64;  // idle waves of the last column tile redo a valid one
  const int nslab = K / BK;
  const int ksteps = K / 16;

  // ---- A: each thread moves one 16-byte chunk per 32-row block and slab -----------------------
  const int a_row = tid >> 3, a_kc = tid & 7;
  uint32_t a_off[MB];
#pragma unroll
  for (int i = 0; i < MB; i++) {
    int r = a_row + 32 * i;
    int src = 0;
    if (r < rows) {
      if (GATHER) src = p.row_ids[row0 + r] / p.top_k;
      else src = row0 + r;
    } else if (!GATHER) {
      src = row0;
    }
    a_off[i] = (uint32_t)src * (uint32_t)K + a_kc * 8;
  }
  u32x4 areg[MB];
  auto load_a = [&](int s) {
#pragma unroll
    for (int i = 0; i < MB; i++) areg[i] = *reinterpret_cast<const u32x4 *>(p.A + a_off[i] + s * BK);
  };
  bf16_t *a_dst = lds + a_row * LDS_ROW + a_kc * 8;
  auto store_a = [&](int stage) {
#pragma unroll
    for (int i = 0; i < MB; i++)
      *reinterpret_cast<u32x4 *>(a_dst + stage * lds_stage + 32 * i * LDS_ROW) = areg[i];
  };

  // ---- B: two fragment streams per wave, three slabs in the register ring ---------------------
  // bf16: 4 x 16 bytes per fragment and slab.  MXFP4: 16 bytes of codes (the lane's 8 codes of each
  // of the 4 k-steps) + 2 scale bytes (one e8m0 per 32 k) per fragment and slab.
  constexpr int BQ = FP4 ? 1 : 4;
  const bf16_t *wbase = nullptr;
  const unsigned char *cbase = nullptr, *sbase = nullptr;
  size_t frag_stride = 0, sfrag_stride = 0;
  if (FP4) {
    const size_t mat_bytes = (size_t)N * K / 2 + (size_t)N * K / 32;
    const unsigned char *mb_ = reinterpret_cast<const unsigned char *>(p.W) + (size_t)mat * mat_bytes;
    cbase = mb_ + ((size_t)(n0 >> 5) * nslab * 64 + lane) * 16;
    sbase = mb_ + (size_t)N * K / 2 + ((size_t)(n0 >> 5) * nslab * 32 + (lane & 31)) * 2;
    frag_stride = (size_t)nslab * 1024;
    sfrag_stride = (size_t)nslab * 64;
  } else {
    wbase = p.W + (size_t)mat * N * K + ((size_t)(n0 >> 5) * ksteps * 64 + lane) * 8;
    frag_stride = (size_t)ksteps * 512;  // elements between adjacent 32-column blocks
  }
  u32x4 breg[3][2][BQ];
  uint32_t sreg[3][2];
  auto load_b = [&](int s, auto ring) {
    constexpr int R = decltype(ring)::value;
#pragma unroll
    for (int f = 0; f < 2; f++) {
      if (FP4) {
        breg[R][f][0] = *reinterpret_cast<const u32x4 *>(cbase + f * frag_stride + (size_t)s * 1024);
        sreg[R][f] = *reinterpret_cast<const unsigned short *>(sbase + f * sfrag_stride + (size_t)s * 64);
      } else {
#pragma unroll
        for (int kk = 0; kk < 4; kk++)
          breg[R][f][kk % BQ] = *reinterpret_cast<const u32x4 *>(wbase + f * frag_stride +
                                                                 (size_t)(s * 4 + kk) * 512);
      }
    }
  };

  f32x16 acc[MB][2];
#pragma unroll
  for (int i = 0; i < MB; i++)
#pragma unroll
    for (int f = 0; f < 2; f++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][f][r] = 0.f;

  const bf16_t *a_src = lds + (lane & 31) * LDS_ROW + (lane >> 5) * 8;
  auto compute = [&](int stage, auto ring) {
    constexpr int R = decltype(ring)::value;
    const bf16_t *base = a_src + stage * lds_stage;
    Fp4Table tab[2][2];
    if (FP4) {
#pragma unroll
      for (int f = 0; f < 2; f++) {
        tab[f][0] = fp4_table(sreg[R][f] & 0xffu);
        tab[f][1] = fp4_table((sreg[R][f] >> 8) & 0xffu);
      }
    }
#pragma unroll
    for (int kk = 0; kk < 4; kk++) {
      bf16x8 b0, b1;
      if (FP4) {
        b0 = as_bf16x8(fp4_expand(breg[R][0][0][kk], tab[0][kk >> 1]));
        b1 = as_bf16x8(fp4_expand(breg[R][1][0][kk], tab[1][kk >> 1]));
      } else {
        b0 = as_bf16x8(breg[R][0][kk % BQ]);
        b1 = as_bf16x8(breg[R][1][kk % BQ]);
      }
#pragma unroll
      for (int i = 0; i < MB; i++) {
        bf16x8 a = as_bf16x8(*reinterpret_cast<const u32x4 *>(base + i * 32 * LDS_ROW + kk * 16));
        acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b0, acc[i][0], 0, 0, 0);
        acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b1, acc[i][1], 0, 0, 0);
      }
    }
  };

  using R0 = std::integral_constant<int, 0>;
  using R1 = std::integral_constant<int, 1>;
  using R2 = std::integral_constant<int, 2>;
  const int last = nslab - 1;

  load_b(0, R0{});
  load_b(min(1, last), R1{});
  load_a(0);
  store_a(0);
  load_a(min(1, last));
  __syncthreads();

  // slab s: prefetch B and A of slab s+2 (clamped at the end: a harmless re-read), multiply slab
  // s, publish A of slab s+1 to the other LDS stage.
  auto body = [&](int s, auto ring, auto ring_next2) {
    load_b(min(s + 2, last), ring_next2);
    compute(s & 1, ring);
    store_a((s + 1) & 1);
    load_a(min(s + 2, last));
    __syncthreads();
  };
  int s = 0;
  for (; s + 3 <= nslab; s += 3) {
    body(s, R0{}, R2{});
    body(s + 1, R1{}, R0{});
    body(s + 2, R2{}, R1{});
  }
  if (s < nslab) {
    body(s, R0{}, R2{});
    if (s + 1 < nslab) body(s + 1, R1{}, R0{});
  }

  if (!wave_active) return;

  // ---- epilogue ------------------------------------------------------------------------------
  const int c = lane & 31, rsub = (lane >> 5) * 4;
  if (EPI == EPI_SWIGLU) {
    const int half_n = N >> 1;
    const int j = (n0 >> 1) + c;  // pair index: gate = row 2j, up = row 2j+1 of the .bin matrix
    float bg = 0.f, bu = 0.f;
    if (p.bias) {
      bg = p.bias[(size_t)mat * N + 2 * j];
      bu = p.bias[(size_t)mat * N + 2 * j + 1];
    }
    bf16_t *o = reinterpret_cast<bf16_t *>(p.out);
    const float L = p.limit;
#pragma unroll
    for (int i = 0; i < MB; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int row = i * 32 + (r >> 2) * 8 + rsub + (r & 3);
        if (row < rows) {
          float g = acc[i][0][r] + bg, u = acc[i][1][r] + bu;
          g = fminf(g, L);
          u = fminf(fmaxf(u, -L), L);
          float v = g * (1.0f / (1.0f + expf(-1.702f * g)));
          v *= (u + 1.0f);
          o[(size_t)(row0 + row) * half_n + j] = f32_to_bf16(v);
        }
      }
    }
  } else {
#pragma unroll
    for (int f = 0; f < 2; f++) {
      const int col = n0 + f * 32 + c;
      float bv = p.bias ? p.bias[(size_t)mat * N + col] : 0.f;
#pragma unroll
      for (int i = 0; i < MB; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          int row = i * 32 + (r >> 2) * 8 + rsub + (r & 3);
          if (row < rows) {
            float v = acc[i][f][r] + bv;
            if (EPI == EPI_F32)
              reinterpret_cast<float *>(p.out)[(size_t)(row0 + row) * N + col] = v;
            else
              reinterpret_cast<bf16_t *>(p.out)[(size_t)(row0 + row) * N + col] = f32_to_bf16(v);
          }
        }
      }
    }
  }
}

template <int MBMAX, bool GATHER, int EPI, bool FP4>
__global__ __launch_bounds__(GEMM_THREADS) void grouped_gemm_kernel(GemmParams p) {
  constexpr int BM = MBMAX * 32;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);  // [2][BM][LDS_ROW]
  constexpr int STAGE = BM * LDS_ROW;

  // ---- which (row tile, column tile) is this workgroup's: workgroups are dealt round-robin to
  // the 8 XCDs, so XCD x takes the x-th contiguous eighth of the work list -----------------------
  const int n_tiles = p.tiles ? p.tiles[0] : (p.dense_rows + BM - 1) / BM;
  const int total = n_tiles * p.n_col_tiles;
  const int chunk = (total + 7) >> 3;
  const int slot = blockIdx.x >> 3;
  if (slot >= chunk) return;
  const int work = (blockIdx.x & 7) * chunk + slot;
  if (work >= total) return;
  const int tile = work / p.n_col_tiles, ct = work - tile * p.n_col_tiles;
  int mat, row0, rows;
  if (p.tiles) {
    mat = p.tiles[1 + 3 * tile];
    row0 = p.tiles[2 + 3 * tile];
    rows = p.tiles[3 + 3 * tile];
  } else {
    mat = 0;
    row0 = tile * BM;
    rows = min(BM, p.dense_rows - row0);
  }
  const int mb = (rows + 31) >> 5;
  if (MBMAX >= 8 && mb > 6) {
    if (mb == 8) gemm_tile<(MBMAX >= 8 ? 8 : MBMAX), GATHER, EPI, FP4>(p, lds, STAGE, mat, row0, rows, ct);
    else gemm_tile<(MBMAX >= 8 ? 7 : MBMAX), GATHER, EPI, FP4>(p, lds, STAGE, mat, row0, rows, ct);
  } else if (MBMAX >= 8 && mb > 4) {
    if (mb == 6) gemm_tile<(MBMAX >= 8 ? 6 : MBMAX), GATHER, EPI, FP4>(p, lds, STAGE, mat, row0, rows, ct);
    else gemm_tile<(MBMAX >= 8 ? 5 : MBMAX), GATHER, EPI, FP4>(p, lds, STAGE, mat, row0, rows, ct);
  } else if (MBMAX >= 4 && mb > 2) {
    if (mb == 4) gemm_tile<(MBMAX >= 4 ? 4 : MBMAX), GATHER, EPI, FP4>(p, lds, STAGE, mat, row0, rows, ct);
    else gemm_tile<(MBMAX >= 4 ? 3 : MBMAX), GATHER, EPI, FP4>(p, lds, STAGE, mat, row0, rows, ct);
  } else if (MBMAX >= 2 && mb == 2) {
    gemm_tile<(MBMAX >= 2 ? 2 : MBMAX), GATHER, EPI, FP4>(p, lds, STAGE, mat, row0, rows, ct);
  } else {
    gemm_tile<1, GATHER, EPI, FP4>(p, lds, STAGE, mat, row0, rows, ct);
  }
}

// Weighted combine: out[b,:] (+)= sum over the token's k experts, in ascending expert order (the
// order of the reference CPU loop, run.cpp:642-704), of w * y2[row of that pair].  Products and
// sums are rounded separately, as that loop rounds them.
__global__ __launch_bounds__(256) void combine_kernel(const float *__restrict__ y2,
                                                      const float *__restrict__ topk_w,
                                                      const int *__restrict__ inv_perm,
                                                      float *__restrict__ out, int H, int k,
                                                      int accumulate) {
  const int b = blockIdx.x;
  int rows[8];
  float w[8];
#pragma unroll
  for (int s = 0; s < 8; s++) {
    rows[s] = (s < k) ? inv_perm[(size_t)b * k + s] : 0x7fffffff;
    w[s] = (s < k) ? topk_w[(size_t)b * k + s] : 0.f;
  }
  // sorted position grows with expert id, so ordering by row orders by expert
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j + 1 < 8 - i; j++)
      if (rows[j] > rows[j + 1]) {
        int tr = rows[j]; rows[j] = rows[j + 1]; rows[j + 1] = tr;
        float tw = w[j]; w[j] = w[j + 1]; w[j + 1] = tw;
      }
  for (int h = threadIdx.x * 4; h < H; h += 256 * 4) {
    f32x4 agg = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 8; s++) {
      if (s < k) {
        f32x4 v = *reinterpret_cast<const f32x4 *>(y2 + (size_t)rows[s] * H + h);
#pragma unroll
        for (int q = 0; q < 4; q++) agg[q] = __fadd_rn(agg[q], __fmul_rn(v[q], w[s]));
      }
    }
    f32x4 *op = reinterpret_cast<f32x4 *>(out + (size_t)b * H + h);
    if (accumulate) {
      f32x4 prev = *op;
#pragma unroll
      for (int q = 0; q < 4; q++) agg[q] = __fadd_rn(prev[q], agg[q]);
    }
    *op = agg;
  }
}

// Repack row-major [n_out, n_in] matrices into fragment order:
//   dst[((nb*KS + ks)*64 + lane)*8 + j] = W[row(nb*32 + lane%32)][ks*16 + (lane/32)*8 + j]
// With GLU pairing, virtual row v of a 64-row wave tile maps to pair (v/64)*32 + v%32, gate for
// the first 32 virtual rows and up for the second 32.
template <typename SRC>
__global__ __launch_bounds__(256) void pack_weight_kernel(const SRC *__restrict__ src,
                                                          bf16_t *__restrict__ dst, int n_out,
                                                          int n_in, int glu) {
  const int ksteps = n_in / 16;
  const size_t frags_per_mat = (size_t)(n_out / 32) * ksteps;
  const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;  // one (fragment, lane) per thread
  const size_t frag = gid >> 6;
  const int lane = (int)(gid & 63);
  const int mat = blockIdx.y;
  if (frag >= frags_per_mat) return;
  const int nb = (int)(frag / ksteps), ks = (int)(frag - (size_t)nb * ksteps);
  int v = nb * 32 + (lane & 31);
  int row = v;
  if (glu) row = 2 * ((v >> 6) * 32 + (v & 31)) + ((v >> 5) & 1);
  const SRC *sp = src + ((size_t)mat * n_out + row) * n_in + ks * 16 + (lane >> 5) * 8;
  uint32_t o[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    if constexpr (sizeof(SRC) == 4) {
      o[j] = pack_bf16x2((float)sp[2 * j], (float)sp[2 * j + 1]);
    } else {
      o[j] = (uint32_t)sp[2 * j] | ((uint32_t)sp[2 * j + 1] << 16);
    }
  }
  u32x4 *dp = reinterpret_cast<u32x4 *>(dst + ((size_t)mat * frags_per_mat + frag) * 512 + lane * 8);
  *dp = u32x4{o[0], o[1], o[2], o[3]};
}

// MXFP4 repack: blocks [n_out, n_in/2] (low nibble = even element) and e8m0 scales [n_out, n_in/32]
// -> per (32-column block, 64-k slab): 64 lanes x 16 bytes of codes, then 32 x 2 scale bytes.
__global__ __launch_bounds__(256) void pack_mxfp4_kernel(const unsigned char *__restrict__ blocks,
                                                         const unsigned char *__restrict__ scales,
                                                         unsigned char *__restrict__ dst, int n_out,
                                                         int n_in, int glu) {
  const int nslab = n_in / 64;
  const size_t items = (size_t)(n_out / 32) * nslab;          // (column block, slab)
  const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;  // one (item, lane) per thread
  const size_t item = gid >> 6;
  const int lane = (int)(gid & 63);
  const int mat = blockIdx.y;
  if (item >= items) return;
  const int nb = (int)(item / nslab), slab = (int)(item - (size_t)nb * nslab);
  int v = nb * 32 + (lane & 31);
  int row = v;
  if (glu) row = 2 * ((v >> 6) * 32 + (v & 31)) + ((v >> 5) & 1);
  const size_t mat_bytes = (size_t)n_out * n_in / 2 + (size_t)n_out * n_in / 32;
  const unsigned char *brow = blocks + ((size_t)mat * n_out + row) * (n_in / 2);
  const unsigned char *srow = scales + ((size_t)mat * n_out + row) * (n_in / 32);
  unsigned char *md = dst + (size_t)mat * mat_bytes;
  uint32_t w[4];
#pragma unroll
  for (int kk = 0; kk < 4; kk++) {
    const int k0 = (slab * 4 + kk) * 16 + (lane >> 5) * 8;  // the lane's 8 consecutive k
    uint32_t src = *reinterpret_cast<const uint32_t *>(brow + k0 / 2);  // nibble j = element k0+j
    uint32_t o = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      uint32_t code = (src >> (4 * j)) & 0xfu;
      o |= code << ((j < 4) ? (8 * j) : (8 * (j - 4) + 4));
    }
    w[kk] = o;
  }
  *reinterpret_cast<u32x4 *>(md + (item * 64 + lane) * 16) = u32x4{w[0], w[1], w[2], w[3]};
  if (lane < 32) {
    unsigned char *sd = md + (size_t)n_out * n_in / 2 + (item * 32 + lane) * 2;
    sd[0] = srow[slab * 2];
    sd[1] = srow[slab * 2 + 1];
  }
}

template <int MB, bool GATHER, int EPI, bool FP4 = false>
static int launch_gemm(const GemmParams &p, int max_tiles, hipStream_t s) {
  static bool attr_done = false;
  size_t smem = (size_t)2 * MB * 32 * LDS_ROW * sizeof(bf16_t);
  auto kern = grouped_gemm_kernel<MB, GATHER, EPI, FP4>;
  if (!attr_done) {
    GPTOSS_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    attr_done = true;
  }
  int total = max_tiles * p.n_col_tiles;
  int grid = ((total + 7) / 8) * 8;
  if (grid == 0) return GPTOSS_OK;
  {
    TraceScope ts(FP4 ? (GATHER ? "gemm1_gather_swiglu_mxfp4" : "gemm_f32_mxfp4") : GATHER ? "gemm1_gather_swiglu" : (EPI == EPI_F32 ? "gemm_f32" : (EPI == EPI_BF16 ? "gemm_bf16" : "gemm_swiglu")), s);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(GEMM_THREADS), smem, s, p);
  }
  GPTOSS_LAUNCH_CHECK("grouped_gemm_kernel");
  return GPTOSS_OK;
}

// Host-side dispatcher used by the MoE layer and the engine.  rows_per_tile selects MB.
int run_gemm(const GemmParams &p, bool gather, int epi, int rows_per_tile, int max_tiles,
             hipStream_t s) {
#define GPTOSS_GEMM_CASE(MBV)                                                                  \
  if (rows_per_tile == MBV * 32 && p.w_mxfp4) {                                                \
    if (gather && epi == EPI_SWIGLU) return launch_gemm<MBV, true, EPI_SWIGLU, true>(p, max_tiles, s); \
    if (!gather && epi == EPI_F32) return launch_gemm<MBV, false, EPI_F32, true>(p, max_tiles, s); \
  } else if (rows_per_tile == MBV * 32) {                                                      \
    if (gather && epi == EPI_SWIGLU) return launch_gemm<MBV, true, EPI_SWIGLU>(p, max_tiles, s); \
    if (!gather && epi == EPI_F32) return launch_gemm<MBV, false, EPI_F32>(p, max_tiles, s);    \
    if (!gather && epi == EPI_BF16) return launch_gemm<MBV, false, EPI_BF16>(p, max_tiles, s);  \
    if (!gather && epi == EPI_SWIGLU) return launch_gemm<MBV, false, EPI_SWIGLU>(p, max_tiles, s); \
  }
  GPTOSS_GEMM_CASE(1)
  GPTOSS_GEMM_CASE(2)
  GPTOSS_GEMM_CASE(4)
  GPTOSS_GEMM_CASE(8)
#undef GPTOSS_GEMM_CASE
  return fail(GPTOSS_ERR_DIM, "run_gemm: unsupported combination (rows_per_tile=%d gather=%d epi=%d)",
              rows_per_tile, (int)gather, epi);
}

int run_combine(const float *y2, const float *topk_w, const int *inv_perm, float *out, int B, int H,
                int k, int accumulate, hipStream_t s) {
  if (B == 0) return GPTOSS_OK;
  {
    TraceScope ts("combine", s);
    combine_kernel<<<B, 256, 0, s>>>(y2, topk_w, inv_perm, out, H, k, accumulate);
  }
  GPTOSS_LAUNCH_CHECK("combine_kernel");
  return GPTOSS_OK;
}

}  // namespace gptoss

using namespace gptoss;

extern "C" size_t gptoss_packed_weight_bytes(int n_mat, int n_out, int n_in) {
  if (n_mat <= 0 || n_out <= 0 || n_in <= 0) return 0;
  return (size_t)n_mat * n_out * n_in * sizeof(bf16_t);
}

extern "C" int gptoss_pack_weight(const void *src, void *dst, int n_mat, int n_out, int n_in,
                                  int flags, void *stream) {
  GPTOSS_REQUIRE(src && dst, GPTOSS_ERR_NULL, "pack_weight: null pointer");
  const int glu = (flags & GPTOSS_PACK_GLU) ? 1 : 0;
  GPTOSS_REQUIRE(n_mat >= 1 && n_out > 0 && n_in > 0 && n_out % (glu ? 64 : 32) == 0 && n_in % 64 == 0,
                 GPTOSS_ERR_DIM, "pack_weight: need n_out %% %d == 0 and n_in %% 64 == 0 (n_out=%d n_in=%d)",
                 glu ? 64 : 32, n_out, n_in);
  GPTOSS_REQUIRE(aligned(src, 16) && aligned(dst, 16), GPTOSS_ERR_ALIGN,
                 "pack_weight: pointers must be 16-byte aligned");
  size_t threads = (size_t)(n_out / 32) * (n_in / 16) * 64;
  dim3 grid((unsigned)((threads + 255) / 256), n_mat);
  hipStream_t s = (hipStream_t)stream;
  if (flags & GPTOSS_PACK_SRC_FP32)
    pack_weight_kernel<float><<<grid, 256, 0, s>>>((const float *)src, (bf16_t *)dst, n_out, n_in, glu);
  else
    pack_weight_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t *)src, (bf16_t *)dst, n_out, n_in, glu);
  GPTOSS_LAUNCH_CHECK("pack_weight_kernel");
  return GPTOSS_OK;
}

extern "C" size_t gptoss_packed_mxfp4_bytes(int n_mat, int n_out, int n_in) {
  if (n_mat <= 0 || n_out <= 0 || n_in <= 0) return 0;
  return (size_t)n_mat * ((size_t)n_out * n_in / 2 + (size_t)n_out * n_in / 32);
}

extern "C" int gptoss_pack_mxfp4(const void *blocks, const void *scales, void *dst, int n_mat,
                                 int n_out, int n_in, int flags, void *stream) {
  GPTOSS_REQUIRE(blocks && scales && dst, GPTOSS_ERR_NULL, "pack_mxfp4: null pointer");
  const int glu = (flags & GPTOSS_PACK_GLU) ? 1 : 0;
  GPTOSS_REQUIRE(n_mat >= 1 && n_out > 0 && n_in > 0 && n_out % (glu ? 64 : 32) == 0 && n_in % 64 == 0,
                 GPTOSS_ERR_DIM, "pack_mxfp4: need n_out %% %d == 0 and n_in %% 64 == 0 (n_out=%d n_in=%d)",
                 glu ? 64 : 32, n_out, n_in);
  GPTOSS_REQUIRE(aligned(blocks, 4) && aligned(dst, 16), GPTOSS_ERR_ALIGN,
                 "pack_mxfp4: blocks must be 4-byte and dst 16-byte aligned");
  size_t threads = (size_t)(n_out / 32) * (n_in / 64) * 64;
  dim3 grid((unsigned)((threads + 255) / 256), n_mat);
  pack_mxfp4_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const unsigned char *)blocks,
                                                          (const unsigned char *)scales,
                                                          (unsigned char *)dst, n_out, n_in, glu);
  GPTOSS_LAUNCH_CHECK("pack_mxfp4_kernel");
  return GPTOSS_OK;
}
