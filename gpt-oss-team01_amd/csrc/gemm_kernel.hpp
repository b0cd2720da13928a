// Grouped (per-expert) and dense bf16 GEMMs for gfx950 built on v_mfma_f32_32x32x16_bf16.
//
//   C[rows, N] = A[rows, K] . W[N, K]^T      rows = the tokens routed to one expert (or a slice
//                                            of a dense batch), W = that expert's matrix
//
// Shape of the problem at decode time: a few hundred rows per expert against 25 M weights per
// expert, i.e. every weight is used by ~128 rows and the kernel is bound by streaming W from
// HBM.  The design follows from that:
//   * W is stored in MFMA-fragment order (gptoss_pack_weight): the 1 KB a wave needs for one
//     32-column x 16-k operand is contiguous, so each wave streams its own 32 columns with
//     perfectly coalesced 128-bit loads straight into registers (no LDS hop, no reuse needed:
//     a workgroup covers all rows of its tile, up to 160, so W is read from HBM once);
//   * the activations (shared by the 8 waves) go through a three-stage, padded LDS tile; the
//     token gather of the reference's pack step is folded into that load;
//   * a workgroup = 8 waves = 256 columns x up to 160 rows, each wave keeping at most 80
//     accumulator registers, so two waves share a SIMD: one wave's MFMAs, epilogue or prologue
//     overlap the other's waits on memory;
//   * the kernel is persistent (one workgroup per CU, two for the small-tile MXFP4 kernels); its
//     work items come from the device-built tile list (expert,row0,rows), mapped so that the workgroups of one XCD walk consecutive
//     column tiles of the same expert (A stays in that XCD's L2), and the register ring of W keeps
//     streaming across work items;
//   * the MFMAs compute the transposed tile (W fragment first), so a lane ends up with one token
//     row and 16 channels: stores are 8/16 bytes wide, and since the packing order puts the gates
//     of 16 (gate,up) pairs in channels 0-15 of a wave's block and their ups in channels 16-31,
//     each pair sits in two registers of the same lane;
//   * epilogues: +bias -> fp32, or +bias -> clamped SwiGLU -> bf16.
#pragma once

#include <type_traits>

#include "common.hpp"
#include "gemm.hpp"

namespace gptoss {

constexpr int GEMM_WAVES = 8;
constexpr int GEMM_THREADS = GEMM_WAVES * 64;
constexpr int BK = 64;            // k per LDS slab (4 MFMA k-steps)
constexpr int LDS_ROW = BK + 8;   // padded row length in bf16 elements (144 B)
constexpr int BN = GEMM_WAVES * 32;  // columns per workgroup
constexpr int HOLD_ROW = BN / 2 + 8;  // row of a SwiGLU output tile that waits in LDS: 128 outputs + padding (272 B)

// MXFP4 operand expansion.  One dword holds the lane's 8 e2m1 codes of a k-step in checkpoint
// order (byte j = elements 2j in the low and 2j+1 in the high nibble), which is what the hardware
// conversion takes: v_cvt_scalef32_pk_bf16_fp4 turns one byte into the bf16 pair (value * scale),
// exact for a power-of-two scale inside the bf16 normal range.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float fp4_scale(uint32_t e8m0) {
  return __builtin_bit_cast(float, e8m0 << 23);  // 2^(e8m0 - 127)
}

__device__ __forceinline__ u32x4 fp4_expand(uint32_t w, float scale) {
  return u32x4{__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 0)),
               __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 1)),
               __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 2)),
               __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 3))};
}

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// Where one wave's W fragment stream of a work item starts (wave-uniform; each lane adds its own
// 16 bytes, or 2 scale bytes, when loading).
struct WStream {
  const bf16_t *w;           // bf16: first fragment of the wave's 32-column block
  const unsigned char *c;    // MXFP4: codes
  const unsigned char *sc;   // MXFP4: scales
};

template <bool FP4>
__device__ __forceinline__ WStream w_stream(const GemmParams &p, int mat, int ct, int wave) {
  const int K = p.K, N = p.N;
  int n0 = ct * BN + wave * 32;
  if (n0 >= N) n0 = N - 32;  // idle waves of the last column tile stream a valid block again
  WStream st{nullptr, nullptr, nullptr};
  if (FP4) {
    const int nslab = K / BK;
    const size_t mat_bytes = (size_t)N * K / 2 + (size_t)N * K / 32;
    const unsigned char *mb_ = reinterpret_cast<const unsigned char *>(p.W) + (size_t)mat * mat_bytes;
    st.c = mb_ + (size_t)(n0 >> 5) * nslab * 1024;
    st.sc = mb_ + (size_t)N * K / 2 + (size_t)(n0 >> 5) * nslab * 64;
  } else {
    st.w = p.W + (size_t)mat * N * K + (size_t)(n0 >> 5) * (K / 16) * 512;
  }
  return st;
}

// Register ring holding NRING slabs of the wave's W operand (bf16: 4 x 16 bytes per lane and
// slab; MXFP4: 16 bytes of codes + 2 scale bytes).
template <int NRING, bool FP4>
struct WRing {
  static constexpr int BQ = FP4 ? 1 : 4;
  u32x4 b[NRING][BQ];
  uint32_t s[NRING];
};

// A 16-byte load of W.  ONCE: the bytes are used by this workgroup alone (an expert with a single row
// tile, a dense GEMM of one row tile), so they are requested with the non-temporal hint and leave the
// caches to what is read again, the activation rows and the outputs that the next kernel reads (GEMM1
// of the 1024-token layer 222 -> 213 us, the combine behind GEMM2 14.5 -> 12.9 us).  Where row tiles
// share W through L2 the hint costs 5-8 %, so it is decided per work item.
template <bool ONCE>
__device__ __forceinline__ u32x4 w_fetch(const void *q) {
  if (ONCE) return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(q));
  return *reinterpret_cast<const u32x4 *>(q);
}

template <int NRING, bool FP4, bool ONCE, int R>
__device__ __forceinline__ void w_load(WRing<NRING, FP4> &ring, const WStream &st, int slab, int lane,
                                       std::integral_constant<int, R>) {
  if (FP4) {
    ring.b[R][0] = w_fetch<ONCE>(st.c + (size_t)slab * 1024 + lane * 16);
    ring.s[R] = *reinterpret_cast<const unsigned short *>(st.sc + (size_t)slab * 64 + (lane & 31) * 2);
  } else {
#pragma unroll
    for (int kk = 0; kk < 4; kk++)
      ring.b[R][kk % WRing<NRING, FP4>::BQ] = w_fetch<ONCE>(st.w + (size_t)(slab * 4 + kk) * 512 + lane * 8);
  }
}

// Epilogue of one wave's 32-column block at column n0: MB accumulator blocks of 32 rows starting
// at row0, of which `rows` are real (rows <= 0: nothing is stored).
// The MFMAs take the W fragment as their first operand, i.e. they compute the transposed tile:
// a lane holds one token row (lane%32 of each 32-row block) and 16 of the wave's 32 output
// channels, channel g*8 + h*4 + q in result register g*4 + q (h = lane/32).  Four consecutive
// channels of a row are therefore four consecutive registers of one lane, which makes every
// store 8 or 16 bytes wide and keeps each (gate, up) pair inside a lane.
// Biases are wave-uniform per register and half-wave: they come in through scalar loads, which
// do not queue behind the vector loads already in flight for the next item.
// CONST_BIAS: read the biases through the constant address space, for a kernel whose asm statements
// would otherwise turn these loads into vector loads.
// hold != nullptr (SwiGLU form only): the tile goes to LDS instead of memory, row r of the tile at
// hold + r * HOLD_ROW, this wave's 16 outputs from column hold_col on.
template <int MB, int EPI, bool CONST_BIAS = false>
__device__ __forceinline__ void epilogue_store(const GemmParams &p, int mat, int row0, int rows, int n0,
                                               int lane, const f32x16 (&acc)[MB], bf16_t *hold = nullptr,
                                               int hold_col = 0) {
  const int N = p.N;
  const int tok = lane & 31;
  const bool hi = lane >= 32;
  const int h4 = hi ? 4 : 0;
  using BiasPtr = std::conditional_t<CONST_BIAS, const_as<float>, const float *>;
  const BiasPtr bp = (BiasPtr)(p.bias ? p.bias + (size_t)mat * N + n0 : nullptr);
  if (EPI == EPI_SWIGLU) {
    // channels 0-15 of the wave are the gates of pairs j0..j0+15, channels 16-31 their ups; in the
    // unpacked matrix pair j is rows 2j (gate) and 2j+1 (up), so its biases are bp[2jj], bp[2jj+1]
    const int half_n = N >> 1;
    float bg[8], bu[8];
#pragma unroll
    for (int g = 0; g < 2; g++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int jlo = g * 8 + q, jhi = jlo + 4;
        const float g_lo = bp ? bp[2 * jlo] : 0.f, g_hi = bp ? bp[2 * jhi] : 0.f;
        const float u_lo = bp ? bp[2 * jlo + 1] : 0.f, u_hi = bp ? bp[2 * jhi + 1] : 0.f;
        bg[g * 4 + q] = hi ? g_hi : g_lo;
        bu[g * 4 + q] = hi ? u_hi : u_lo;
      }
    // address = wave-uniform base (scalar registers) + a 32-bit per-lane element offset
    bf16_t *o = reinterpret_cast<bf16_t *>(p.out) + (size_t)row0 * half_n + (n0 >> 1);
    const uint32_t lane_off = (uint32_t)tok * (uint32_t)half_n + (uint32_t)h4;
    const float L = p.limit;
    const int row_lim = rows - tok;  // block i of this lane is a real row iff i*32 < row_lim
#pragma unroll
    for (int i = 0; i < MB; i++) {
      if (i * 32 < row_lim) {
        bf16_t *orow = o + (size_t)((uint32_t)(i * 32) * (uint32_t)half_n);
#pragma unroll
        for (int g = 0; g < 2; g++) {
          float v[4];
#pragma unroll
          for (int q = 0; q < 4; q++) {
            float gate = acc[i][g * 4 + q] + bg[g * 4 + q];
            float up = acc[i][(g + 2) * 4 + q] + bu[g * 4 + q];
            gate = fminf(gate, L);
            up = fminf(fmaxf(up, -L), L);
            // gate * sigmoid(1.702 gate) * (up + 1); exp2 and the hardware reciprocal are accurate
            // to a few ulp of fp32, far inside the bf16 rounding of the result
            const float e = __builtin_amdgcn_exp2f(-1.702f * 1.4426950408889634f * gate);
            v[q] = gate * __builtin_amdgcn_rcpf(1.0f + e) * (up + 1.0f);
          }
          const u32x2 pk = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
          if (hold) *reinterpret_cast<u32x2 *>(hold + (i * 32 + tok) * HOLD_ROW + hold_col + h4 + g * 8) = pk;
          else *reinterpret_cast<u32x2 *>(orow + lane_off + g * 8) = pk;
        }
      }
    }
  } else {
    float bv[16];
#pragma unroll
    for (int g = 0; g < 4; g++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const float lo = bp ? bp[g * 8 + q] : 0.f, hi_v = bp ? bp[g * 8 + 4 + q] : 0.f;
        bv[g * 4 + q] = hi ? hi_v : lo;
      }
    const uint32_t lane_off = (uint32_t)tok * (uint32_t)N + (uint32_t)h4;
    const int row_lim = rows - tok;
#pragma unroll
    for (int i = 0; i < MB; i++) {
      if (i * 32 < row_lim) {
        const size_t row_off = (size_t)((uint32_t)(row0 + i * 32) * (uint32_t)N) + n0;
#pragma unroll
        for (int g = 0; g < 4; g++) {
          float v[4];
#pragma unroll
          for (int q = 0; q < 4; q++) v[q] = acc[i][g * 4 + q] + bv[g * 4 + q];
          if (EPI == EPI_F32)
            *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(p.out) + row_off + lane_off + g * 8) =
                f32x4{v[0], v[1], v[2], v[3]};
          else
            *reinterpret_cast<u32x2 *>(reinterpret_cast<bf16_t *>(p.out) + row_off + lane_off + g * 8) =
                u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        }
      }
    }
  }
}

// One (row tile, column tile) work item with a compile-time number of 32-row blocks, so every
// loop below is fully unrolled and every global load of W is unconditional.  On entry the ring
// holds slabs 0..NRING-2 of this item's W stream; while the last slabs are multiplied the ring is
// refilled from `next` (the stream of the workgroup's next work item), so the HBM stream of W
// never drains between work items.  On exit the ring holds slabs 0..NRING-2 of `next`.
template <int MB, int MBMAX, int NRING, bool GATHER, int EPI, bool FP4, bool ONCE>
__device__ __forceinline__ void gemm_tile(const GemmParams &p, bf16_t *lds, int mat, int row0, int rows,
                                          int ct, WRing<NRING, FP4> &ring, const WStream &cur,
                                          const WStream &next, bf16_t *hold = nullptr) {
  constexpr int LDS_STAGE = MBMAX * 32 * LDS_ROW;  // elements per A stage
  constexpr int D = NRING - 1;                     // slabs of W in flight
  constexpr int BQ = WRing<NRING, FP4>::BQ;
  constexpr int APASS = GEMM_THREADS / 8;          // rows moved per pass of the workgroup
  constexpr int AC = (MB * 32 + APASS - 1) / APASS;  // 16-byte A chunks per thread and slab
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = p.K, N = p.N;
  const int n0 = ct * BN + wave * 32;
  const bool wave_active = n0 < N;
  const int nslab = K / BK;

  // ---- A: the workgroup moves APASS rows x 8 chunks of 16 bytes per pass ----------------------
  const int a_row = tid >> 3, a_kc = tid & 7;
  uint32_t a_off[AC];
  bool a_live[AC];
#pragma unroll
  for (int i = 0; i < AC; i++) {
    const int r = a_row + APASS * i;
    a_live[i] = r < MB * 32;
    int src = GATHER ? 0 : row0;
    if (r < rows) {
      if (GATHER) src = p.row_ids[row0 + r] / p.top_k;
      else src = row0 + r;
    }
    a_off[i] = (uint32_t)src * (uint32_t)K + a_kc * 8;
  }
  // Register sets for A in flight.  With bf16 weights a slab's rows are requested one iteration
  // before they are stored to LDS; with MXFP4 weights the iterations are short (a quarter of the
  // W bytes), so two sets alternate and every request has two iterations to complete.
  constexpr int APF = FP4 ? 2 : 1;
  u32x4 areg[APF][AC];
  auto load_a = [&](int s, auto psel) {
    constexpr int P = decltype(psel)::value % APF;
#pragma unroll
    for (int i = 0; i < AC; i++)
      if (a_live[i]) areg[P][i] = *reinterpret_cast<const u32x4 *>(p.A + a_off[i] + s * BK);
  };
  bf16_t *a_dst = lds + a_row * LDS_ROW + a_kc * 8;
  auto store_a = [&](int stage, bool zero, auto psel) {
    constexpr int P = decltype(psel)::value % APF;
#pragma unroll
    for (int i = 0; i < AC; i++)
      if (a_live[i])
        *reinterpret_cast<u32x4 *>(a_dst + stage * LDS_STAGE + APASS * i * LDS_ROW) =
            zero ? u32x4{0u, 0u, 0u, 0u} : areg[P][i];
  };

  f32x16 acc[MB];
#pragma unroll
  for (int i = 0; i < MB; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[i][r] = 0.f;

  const bf16_t *a_src = lds + (lane & 31) * LDS_ROW + (lane >> 5) * 8;
  bf16x8 af[2][MB];
  auto compute = [&](int stage, int next_stage, auto rsel, auto &&after_kstep) {
    constexpr int R = decltype(rsel)::value;
    const bf16_t *base = a_src + stage * LDS_STAGE;
    const bf16_t *nbase = a_src + next_stage * LDS_STAGE;
    float scale[2] = {0.f, 0.f};  // of k 0-31 and k 32-63 of the slab
    if (FP4) {
      scale[0] = fp4_scale(ring.s[R] & 0xffu);
      scale[1] = fp4_scale((ring.s[R] >> 8) & 0xffu);
    }
    // af[0] already holds the fragments of k-step 0 (requested before the previous barrier).  The
    // fragments of k-step kk+1 are requested before the MFMAs of k-step kk are issued (bf16: before
    // those of the last k-step, the first fragments of the next slab, whose stage is complete since
    // the previous barrier), and the scheduling fences keep the compiler from sinking those reads
    // next to their uses (bf16; with MXFP4 weights the compiler is left free to weave the operand
    // expansion between the MFMAs, measured 2 % faster).  after_kstep(kk) is what else the iteration
    // has to issue, placed behind the MFMAs of a k-step so that it costs no time of its own.
#pragma unroll
    for (int kk = 0; kk < 4; kk++) {
      if (kk + 1 < 4) {
#pragma unroll
        for (int i = 0; i < MB; i++)
          af[(kk + 1) & 1][i] =
              as_bf16x8(*reinterpret_cast<const u32x4 *>(base + i * 32 * LDS_ROW + (kk + 1) * 16));
      } else if (!FP4) {
#pragma unroll
        for (int i = 0; i < MB; i++)
          af[0][i] = as_bf16x8(*reinterpret_cast<const u32x4 *>(nbase + i * 32 * LDS_ROW));
      }
      bf16x8 b;
      if (FP4) b = as_bf16x8(fp4_expand(ring.b[R][0][kk], scale[kk >> 1]));
      else b = as_bf16x8(ring.b[R][kk % BQ]);
      if (!FP4) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < MB; i++)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, af[kk & 1][i], acc[i], 0, 0, 0);
      after_kstep(kk);
      if (!FP4) __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto read_first_frags = [&](int stage) {
    const bf16_t *base = a_src + stage * LDS_STAGE;
#pragma unroll
    for (int i = 0; i < MB; i++)
      af[0][i] = as_bf16x8(*reinterpret_cast<const u32x4 *>(base + i * 32 * LDS_ROW));
  };

  // Three LDS stages for A: slab s is multiplied from stage s%3 while slab s+2 is being written
  // to stage (s+2)%3, so the first fragments of slab s+1 (complete since the previous barrier) can
  // be requested before this iteration's barrier and their latency is hidden behind it.
  // The slab loop runs a multiple of NRING iterations so the ring is back at index 0 for the next
  // item; the (at most NRING-1) padding iterations multiply zero A rows.
  const int last = nslab - 1;
  const int padded = (nslab + NRING - 1) / NRING * NRING;
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  if constexpr (APF == 2) {
    load_a(0, P0{});
    load_a(min(1, last), P1{});
    store_a(0, false, P0{});
    store_a(1, nslab <= 1, P1{});
    load_a(min(2, last), P0{});
    load_a(min(3, last), P1{});
  } else {
    // slabs 0 and 1 are requested together (the second into registers that are only live here), so
    // the prologue waits for one round trip to memory instead of two
    u32x4 first[AC];
    load_a(0, P0{});
#pragma unroll
    for (int i = 0; i < AC; i++)
      if (a_live[i]) first[i] = *reinterpret_cast<const u32x4 *>(p.A + a_off[i] + min(1, last) * BK);
    store_a(0, false, P0{});
#pragma unroll
    for (int i = 0; i < AC; i++)
      if (a_live[i])
        *reinterpret_cast<u32x4 *>(a_dst + LDS_STAGE + APASS * i * LDS_ROW) =
            (nslab <= 1) ? u32x4{0u, 0u, 0u, 0u} : first[i];
    load_a(min(2, last), P0{});
  }
  __syncthreads();
  read_first_frags(0);

  int st = 0;  // s % 3
  auto body = [&](int s, auto rsel, auto psel) {
    constexpr int R = decltype(rsel)::value;
    using Refill = std::integral_constant<int, (R + D) % NRING>;
    // ring slot consumed at iteration s+D: slab s+D of this item, nothing useful while padding,
    // then the first slabs of the next item
    const int t = s + D;
    const bool wrap = t >= padded;
    const WStream &wsrc = wrap ? next : cur;
    const int wslab = min(wrap ? t - padded : t, last);
    const int st1 = (st == 2) ? 0 : st + 1, st2 = (st1 == 2) ? 0 : st1 + 1;
    // bf16: everything the iteration issues besides MFMAs and fragment reads sits behind the MFMAs
    // of a k-step.  Without the token gather (dense GEMMs, GEMM2) each of the refill slab's four
    // 1 KB fragments is requested after one k-step (classifier -6 %, projections of a prompt pass
    // -5 %); GEMM1 keeps all four requests at the top of the iteration, where its HBM-bound stream
    // measured 2 % faster.  The rows of slab s+2 go to LDS after k-step 1 and the next rows are
    // requested after k-step 2 (GEMM1 of a prompt pass -5 %; after k-steps 0 and 1: no gain).
    constexpr bool W_PER_KSTEP = !FP4 && !GATHER;
    if constexpr (!W_PER_KSTEP) w_load<NRING, FP4, ONCE>(ring, wsrc, wslab, lane, Refill{});
    compute(st, st1, rsel, [&](int kk) {
      if constexpr (W_PER_KSTEP)
        ring.b[Refill::value][kk % BQ] = w_fetch<ONCE>(wsrc.w + (size_t)(wslab * 4 + kk) * 512 + lane * 8);
      if constexpr (!FP4) {
        if (kk == 1) store_a(st2, s + 2 >= nslab, psel);  // rows of slab s+2 (zeros while padding)
        if (kk == 2) load_a(min(s + 2 + APF, last), psel);
      }
    });
    if constexpr (FP4) {
      store_a(st2, s + 2 >= nslab, psel);
      load_a(min(s + 2 + APF, last), psel);
      read_first_frags(st1);
    }
    st = st1;
    __syncthreads();
  };
  if constexpr (APF == 2) {
    // the register set alternates with the parity of s: pairs of NRING-iteration groups, then one
    // more group when their number is odd
    int s = 0;
    for (; s + 2 * NRING <= padded; s += 2 * NRING)
      static_for<0, 2 * NRING>([&](auto r) {
        constexpr int Q = decltype(r)::value;
        body(s + Q, std::integral_constant<int, Q % NRING>{}, std::integral_constant<int, Q & 1>{});
      });
    if (s < padded)
      static_for<0, NRING>([&](auto r) {
        constexpr int Q = decltype(r)::value;
        body(s + Q, std::integral_constant<int, Q>{}, std::integral_constant<int, Q & 1>{});
      });
  } else {
    for (int s = 0; s < padded; s += NRING)
      static_for<0, NRING>([&](auto r) { body(s + (int)decltype(r)::value, r, P0{}); });
  }

  if (EPI == EPI_ARGMAX) {
    // Row-wise arg-max of this workgroup's 256 columns without writing the products: every lane
    // reduces its 16 channels (ascending, strict >, so the lowest column wins a tie), the two
    // half-waves are merged, the 8 waves meet in LDS (free since the last barrier) and one thread
    // per row writes the tile's (value, column) pair.
    float *rv = reinterpret_cast<float *>(lds);
    int *ri = reinterpret_cast<int *>(lds) + GEMM_WAVES * MBMAX * 32;
    const int tok = lane & 31, h4 = (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < MB; i++) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      if (wave_active) {
#pragma unroll
        for (int g = 0; g < 4; g++)
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const int col = n0 + g * 8 + h4 + q;
            const float v = acc[i][g * 4 + q] + (p.bias ? p.bias[(size_t)mat * N + col] : 0.f);
            if (v > bv) {
              bv = v;
              bi = col;
            }
          }
      }
      const float ov = __shfl_xor(bv, 32, 64);
      const int oi = __shfl_xor(bi, 32, 64);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
      if (lane < 32) {
        rv[wave * (MBMAX * 32) + i * 32 + tok] = bv;
        ri[wave * (MBMAX * 32) + i * 32 + tok] = bi;
      }
    }
    __syncthreads();
    if (tid < MB * 32 && tid < rows) {
      float bv = rv[tid];
      int bi = ri[tid];
#pragma unroll
      for (int w = 1; w < GEMM_WAVES; w++) {
        const float v = rv[w * (MBMAX * 32) + tid];
        if (v > bv) {  // later waves hold higher columns: ties keep the earlier one
          bv = v;
          bi = ri[w * (MBMAX * 32) + tid];
        }
      }
      p.amax_val[(size_t)(row0 + tid) * p.n_col_tiles + ct] = bv;
      p.amax_idx[(size_t)(row0 + tid) * p.n_col_tiles + ct] = bi;
    }
    return;
  }
  if (!wave_active) return;

  epilogue_store<MB, EPI>(p, mat, row0, rows, n0, lane, acc, hold, wave * 16);
}

// Kernels that keep two finished SwiGLU tiles in LDS until the workgroup's last item is done (see
// grouped_gemm_kernel): GEMM1 with bf16 weights, whose bf16 tile of up to 160 x 128 outputs fits twice
// behind the A stages of one workgroup per CU (156 KB at 160 rows).
constexpr bool gemm_holds_output(bool gather, int epi, bool fp4) { return gather && epi == EPI_SWIGLU && !fp4; }

// NRING: slabs of W held in registers per wave, NRING-1 of them in flight.  Three everywhere
// except the 64-row MXFP4 kernels, where a slab costs 5 registers and two more ring slots fit under
// the 128 registers of two workgroups per CU: four slabs in flight measured 4-10 % faster there
// (1024 tokens on 32 experts: 192 + 110 -> 178 + 104 us), nothing or worse for the other tile sizes.
constexpr int GEMM_NRING = 3;
constexpr int gemm_nring(int mbmax, bool fp4) { return (fp4 && mbmax == 2) ? 5 : GEMM_NRING; }

// MXFP4 kernels for tiles of up to 96 rows are compiled for 128 registers, so that two workgroups
// (four waves per SIMD) share a CU: with a quarter of the weight bytes per MFMA the kernel is no
// longer bound by the W stream but by everything around the MFMAs (load latency, LDS round trips,
// prologues and epilogues), and a second workgroup fills those gaps better than larger tiles do
// (64-row tiles on 16 waves: -6 % on a 4096-token layer of 128 experts, -9 % / -14 % on GEMM1 /
// GEMM2 of a 1024-token layer of 32 experts against 160-row tiles on 8 waves).  With bf16 weights
// the same change measured nothing: those kernels follow the W stream.
constexpr bool gemm_two_per_cu(int mbmax, bool fp4) { return fp4 && mbmax <= 3; }

// Persistent kernel: the grid is one workgroup of 8 waves per CU; workgroups are dealt round-robin
// to the 8 XCDs, XCD x owns the x-th contiguous part of the work list (consecutive column tiles
// of the same expert, so that expert's rows stay in that XCD's L2) and its workgroups walk that
// part with a stride of the number of workgroups per XCD.  The parts hold equal numbers of items,
// or, when the grouping kernel supplied cut positions, equal estimated cost (experts with many
// rows next to experts with few would otherwise leave some XCDs idle early).
template <int MBMAX, bool GATHER, int EPI, bool FP4>
__global__ __launch_bounds__(GEMM_THREADS, (gemm_two_per_cu(MBMAX, FP4) ? 4 : 2)) void grouped_gemm_kernel(GemmParams p) {
  constexpr int BM = MBMAX * 32;
  constexpr int NRING = gemm_nring(MBMAX, FP4);
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);  // [3][BM][LDS_ROW], then [2][BM][HOLD_ROW] where outputs are held
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  const int n_tiles = p.tiles ? p.tiles[0] : (p.dense_rows + BM - 1) / BM;
  const int total = n_tiles * p.n_col_tiles;
  const int per_xcd = gridDim.x >> 3;
  const int xcd = blockIdx.x & 7;
  int lo, hi;  // this XCD's part of the work list
  if (p.xcd_bounds) {
    auto item = [&](int b) { return (b >> 16) * p.n_col_tiles + (((b & 0xffff) * p.n_col_tiles) >> 16); };
    lo = item(p.xcd_bounds[xcd]);
    hi = item(p.xcd_bounds[xcd + 1]);
  } else {
    const int chunk = (total + 7) >> 3;
    lo = xcd * chunk;
    hi = min(total, lo + chunk);
  }
  int j = blockIdx.x >> 3;
  auto valid = [&](int jj) { return lo + jj < hi; };
  if (!valid(j)) return;

  struct Item {
    int mat, row0, rows, ct;
    int once;  // no other row tile multiplies this item's W (an int: the struct has no padding to copy)
  };
  auto decode = [&](int jj) {
    const int work = lo + jj;
    Item it;
    int tile;
    if (p.tiles && p.tile_block > 1 && p.xcd_bounds) {
      // grouped, experts with several row tiles: the row tiles of one expert form blocks of up to
      // MOE_TILE_BLOCK tiles (table behind the cut positions) that are walked column tile by
      // column tile, so that the workgroups of an XCD share each column tile of the expert's
      // weights among the block's row tiles as well as each row tile among a few column tiles.
      // A block covers the work indices [first * n_col_tiles, (first + count) * n_col_tiles).
      const int info = p.xcd_bounds[XCD_BOUNDS_INTS + work / p.n_col_tiles];
      const int first = info >> 8, th = info & 255;
      const int v = work - first * p.n_col_tiles;
      it.ct = v / th;
      tile = first + (v - it.ct * th);
      // a block of one tile is an expert's only block unless the expert has 8 k + 1 tiles
      it.once = th == 1 && (tile == 0 || p.tiles[1 + 3 * (tile - 1)] != p.tiles[1 + 3 * tile]);
    } else if (p.tiles) {
      // grouped: column tiles of one row tile are neighbours (the tile's gathered rows stay in L2)
      tile = work / p.n_col_tiles;
      it.ct = work - tile * p.n_col_tiles;
      it.once = false;
    } else {
      // dense: row tiles of one column tile are neighbours, so an XCD reads its share of W from
      // memory once and serves the other row tiles from its L2 (W is the larger operand)
      it.ct = work / n_tiles;
      tile = work - it.ct * n_tiles;
      it.once = n_tiles == 1;
    }
    if (p.tiles) {
      it.mat = p.tiles[1 + 3 * tile];
      it.row0 = p.tiles[2 + 3 * tile];
      it.rows = p.tiles[3 + 3 * tile];
    } else {
      it.mat = 0;
      it.row0 = tile * BM;
      it.rows = min(BM, p.dense_rows - it.row0);
    }
    return it;
  };

  // bf16 GEMM1: the outputs of the two work items before a workgroup's last one wait in LDS (behind
  // the A stages) and are written after the last item's.  Output lines that turn dirty in L2 while
  // the other workgroups still stream W are written back in the middle of that stream, and the
  // write-backs slow the reads far beyond their share of the bytes: with three items per workgroup
  // (the 1024-token layer) the slab loops of the second and third item take 60-65 us where the first
  // item's takes 52, and 47-50 us without the stores.  Held back, the 23 MB leave the chip when the
  // reads are over: GEMM1 213 -> 203 us, the layer 0.386 -> 0.375 ms on the same box.
  constexpr bool HOLD = gemm_holds_output(GATHER, EPI, FP4);
  bf16_t *hold_base = lds + 3 * BM * LDS_ROW;
  const int n_mine = (hi - lo - j + per_xcd - 1) / per_xcd;
  int it = 0;
  int held_row0_a = 0, held_rows_a = 0, held_ct_a = 0, held_row0_b = 0, held_rows_b = 0, held_ct_b = 0;
  Item cur = decode(j);
  WStream cur_w = w_stream<FP4>(p, cur.mat, cur.ct, wave);
  WRing<NRING, FP4> ring;
  static_for<0, NRING - 1>([&](auto r) {
    w_load<NRING, FP4, false>(ring, cur_w, min((int)decltype(r)::value, p.K / BK - 1), lane, r);
  });
  while (true) {
    const int jn = j + per_xcd;
    const bool more = valid(jn);
    const Item nxt = more ? decode(jn) : cur;
    // without a next item the refill re-reads this item's first slabs: harmless and unconditional
    const WStream nxt_w = more ? w_stream<FP4>(p, nxt.mat, nxt.ct, wave) : cur_w;
    // one fully unrolled code path per number of 32-row blocks actually present in the tile
    const int mb = (cur.rows + 31) >> 5;
    bf16_t *hold_ptr = nullptr;
    if (HOLD && it >= n_mine - 3 && it < n_mine - 1) {
      const int slot = it & 1;
      hold_ptr = hold_base + slot * (BM * HOLD_ROW);
      if (slot == 0) {
        held_row0_a = cur.row0;
        held_rows_a = cur.rows;
        held_ct_a = cur.ct;
      } else {
        held_row0_b = cur.row0;
        held_rows_b = cur.rows;
        held_ct_b = cur.ct;
      }
    }
    bool done = false;
    static_for<1, MBMAX + 1>([&](auto m) {
      constexpr int M = decltype(m)::value;
      if (!done && (mb == M || M == MBMAX)) {
        // the refill of the ring from the next item follows this item's choice
        if (!FP4 && cur.once)   // MXFP4 weights: a quarter of the bytes, not bound by their stream; one path keeps the 128-register kernels free of spills
          gemm_tile<M, MBMAX, NRING, GATHER, EPI, FP4, true>(p, lds, cur.mat, cur.row0, cur.rows, cur.ct, ring,
                                                             cur_w, nxt_w, hold_ptr);
        else
          gemm_tile<M, MBMAX, NRING, GATHER, EPI, FP4, false>(p, lds, cur.mat, cur.row0, cur.rows, cur.ct, ring,
                                                              cur_w, nxt_w, hold_ptr);
        done = true;
      }
    });
    if (!more) break;
    // every wave must be done reading this item's last A slab before the next prologue overwrites it
    __syncthreads();
    it++;
    j = jn;
    cur = nxt;
    cur_w = nxt_w;
  }
  if (HOLD) {
    __syncthreads();
    const int half_n = p.N >> 1;
    auto flush = [&](int slot, int row0, int rows, int ct) {
      const bf16_t *src = hold_base + slot * (BM * HOLD_ROW);
      bf16_t *dst = reinterpret_cast<bf16_t *>(p.out) + (size_t)row0 * half_n + ct * (BN / 2);
      for (int idx = threadIdx.x; idx < rows * 16; idx += GEMM_THREADS) {
        const int row = idx >> 4, ch = (idx & 15) * 8;
        if (ct * (BN / 2) + ch < half_n)
          *reinterpret_cast<u32x4 *>(dst + (size_t)row * half_n + ch) =
              *reinterpret_cast<const u32x4 *>(src + row * HOLD_ROW + ch);
      }
    };
    flush(0, held_row0_a, held_rows_a, held_ct_a);
    flush(1, held_row0_b, held_rows_b, held_ct_b);
  }
}

template <int MBMAX, bool HOLD = false>
constexpr size_t gemm_smem_bytes() {
  return (size_t)3 * MBMAX * 32 * LDS_ROW * sizeof(bf16_t) + (HOLD ? (size_t)2 * MBMAX * 32 * HOLD_ROW * sizeof(bf16_t) : 0);
}

// The kernels use more dynamic LDS than a launch gets by default; the limit is raised for every
// instantiation of a translation unit in one go (gemm_prepare_device in moe_gemm.hip, once per
// device), not at an instantiation's first launch, so a first call may sit inside a graph capture
// and concurrent first calls from several host threads do not race.
template <int MBMAX, bool GATHER, int EPI, bool FP4>
hipError_t gemm_set_attr() {
  return hipFuncSetAttribute(reinterpret_cast<const void *>(grouped_gemm_kernel<MBMAX, GATHER, EPI, FP4>),
                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_smem_bytes<MBMAX, gemm_holds_output(GATHER, EPI, FP4)>());
}

template <int MBMAX, bool GATHER, int EPI, bool FP4>
int launch_gemm(const GemmParams &p, int max_tiles, hipStream_t s) {
  const size_t smem = gemm_smem_bytes<MBMAX, gemm_holds_output(GATHER, EPI, FP4)>();
  auto kern = grouped_gemm_kernel<MBMAX, GATHER, EPI, FP4>;
  int total = max_tiles * p.n_col_tiles;
  int grid = ((total + 7) / 8) * 8;
  // resident workgroups: one of 8 waves (2 per SIMD) per CU, or two where the registers allow
  const int resident = gemm_two_per_cu(MBMAX, FP4) ? 512 : 256;
  if (grid > resident) grid = resident;
  if (grid == 0) return GPTOSS_OK;
  {
    TraceScope ts(EPI == EPI_ARGMAX ? "gemm_argmax"
                  : FP4 ? (GATHER ? "gemm1_gather_swiglu_mxfp4" : "gemm_f32_mxfp4")
                        : (GATHER ? "gemm1_gather_swiglu" : "gemm_f32"), s);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(GEMM_THREADS), smem, s, p);
  }
  GPTOSS_LAUNCH_CHECK("grouped_gemm_kernel");
  return GPTOSS_OK;
}

// the two operand/epilogue combinations in use, for every row-tile size
#define GPTOSS_GEMM_INSTANTIATE(FP4V)                                                          \
  template int launch_gemm<1, true, EPI_SWIGLU, FP4V>(const GemmParams &, int, hipStream_t);   \
  template int launch_gemm<2, true, EPI_SWIGLU, FP4V>(const GemmParams &, int, hipStream_t);   \
  template int launch_gemm<3, true, EPI_SWIGLU, FP4V>(const GemmParams &, int, hipStream_t);   \
  template int launch_gemm<4, true, EPI_SWIGLU, FP4V>(const GemmParams &, int, hipStream_t);   \
  template int launch_gemm<5, true, EPI_SWIGLU, FP4V>(const GemmParams &, int, hipStream_t);   \
  template int launch_gemm<1, false, EPI_F32, FP4V>(const GemmParams &, int, hipStream_t);     \
  template int launch_gemm<2, false, EPI_F32, FP4V>(const GemmParams &, int, hipStream_t);     \
  template int launch_gemm<3, false, EPI_F32, FP4V>(const GemmParams &, int, hipStream_t);     \
  template int launch_gemm<4, false, EPI_F32, FP4V>(const GemmParams &, int, hipStream_t);     \
  template int launch_gemm<5, false, EPI_F32, FP4V>(const GemmParams &, int, hipStream_t);     \
  template int launch_gemm<1, false, EPI_ARGMAX, FP4V>(const GemmParams &, int, hipStream_t);  \
  template int launch_gemm<2, false, EPI_ARGMAX, FP4V>(const GemmParams &, int, hipStream_t);  \
  template int launch_gemm<3, false, EPI_ARGMAX, FP4V>(const GemmParams &, int, hipStream_t);  \
  template int launch_gemm<4, false, EPI_ARGMAX, FP4V>(const GemmParams &, int, hipStream_t);  \
  template int launch_gemm<5, false, EPI_ARGMAX, FP4V>(const GemmParams &, int, hipStream_t);

#define GPTOSS_GEMM_ATTR_ROW(M, FP4V)                                            \
  if (err == hipSuccess) err = gemm_set_attr<M, true, EPI_SWIGLU, FP4V>();       \
  if (err == hipSuccess) err = gemm_set_attr<M, false, EPI_F32, FP4V>();         \
  if (err == hipSuccess) err = gemm_set_attr<M, false, EPI_ARGMAX, FP4V>();

#define GPTOSS_GEMM_SET_ATTRS(NAME, FP4V) \
  hipError_t NAME() {                     \
    hipError_t err = hipSuccess;          \
    GPTOSS_GEMM_ATTR_ROW(1, FP4V)         \
    GPTOSS_GEMM_ATTR_ROW(2, FP4V)         \
    GPTOSS_GEMM_ATTR_ROW(3, FP4V)         \
    GPTOSS_GEMM_ATTR_ROW(4, FP4V)         \
    GPTOSS_GEMM_ATTR_ROW(5, FP4V)         \
    return err;                           \
  }

}  // namespace gptoss
