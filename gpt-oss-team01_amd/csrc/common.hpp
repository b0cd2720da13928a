// Shared device/host helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/gptoss_mi355.h"

namespace gptoss {

// ---- error plumbing (host) -------------------------------------------------------------------
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);

#define GPTOSS_REQUIRE(cond, code, ...)                 \
  do {                                                  \
    if (!(cond)) return ::gptoss::fail(code, __VA_ARGS__); \
  } while (0)

#define GPTOSS_HIP(call)                                                                       \
  do {                                                                                         \
    hipError_t err__ = (call);                                                                 \
    if (err__ != hipSuccess)                                                                   \
      return ::gptoss::fail(GPTOSS_ERR_HIP, "%s: %s (%s:%d)", #call, hipGetErrorString(err__), \
                            __FILE__, __LINE__);                                               \
  } while (0)

#define GPTOSS_LAUNCH_CHECK(name)                                                           \
  do {                                                                                      \
    hipError_t err__ = hipGetLastError();                                                   \
    if (err__ != hipSuccess)                                                                \
      return ::gptoss::fail(GPTOSS_ERR_HIP, "launch %s: %s", name, hipGetErrorString(err__)); \
  } while (0)

// ---- kernel timing hook (host) ----------------------------------------------------------------
// When the calling thread has armed a trace (gptoss_trace_set), every kernel launch made by an
// entry point is bracketed by a start/stop event pair on the launch stream.
struct TraceScope {
  TraceScope(const char *name, hipStream_t stream);
  ~TraceScope();
  int slot;
  hipStream_t stream;
};

static inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
static inline int cdiv(int a, int b) { return (a + b - 1) / b; }

// ---- device types ----------------------------------------------------------------------------
typedef uint16_t bf16_t;  // raw bf16 bits
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int WAVE = 64;

__device__ __forceinline__ float bf16_to_f32(bf16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// round-to-nearest-even, NaN stays NaN: gfx950 converts in hardware (v_cvt_pk_bf16_f32)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(bf16_t, static_cast<__bf16>(f));
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}

// A pointer to data that nothing writes while the kernel runs, in the constant address space: a load
// through it with a wave-uniform address is a scalar load whatever the kernel stores or clobbers
// elsewhere (a generic pointer falls back to vector loads once the compiler sees a possible writer,
// an asm statement with a memory clobber included).
template <typename T>
using const_as = const __attribute__((address_space(4))) T *;
template <typename T>
__device__ __forceinline__ const_as<T> constant_ptr(const T *q) {
  return (const_as<T>)(q);
}

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) {
  union {
    u32x4 u;
    bf16x8 b;
  } c;
  c.u = v;
  return c.b;
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & (WAVE - 1); }

// ---- KV cache layout ---------------------------------------------------------------------------
// One array per layer: for every (sequence, kv head) capacity/64 blocks of 64 slots; a block holds
// the K rows of its slots, [64][D] bf16, followed by their V in the operand order of the second
// attention MFMA, [2 groups of 32 slots][D/16][64 lanes][8].  A wave that walks a sequence reads
// one contiguous 256*D-byte unit per 64 slots; position p lives in slot p % capacity.
constexpr int KV_BLOCK = 64;
__host__ __device__ __forceinline__ size_t kv_plane_elems(int cap, int D) { return (size_t)cap * D * 2; }
// first element of the block that holds `slot` of (seq, g)
__device__ __forceinline__ size_t kv_block_off(int seq, int g, int n_kv, int cap, int D, int slot) {
  return ((size_t)(seq * n_kv + g) * (cap >> 6) + (slot >> 6)) * (size_t)(2 * KV_BLOCK * D);
}
// element offsets inside a block
__device__ __forceinline__ int kv_k_elem(int slot, int d, int D) { return (slot & 63) * D + d; }
__device__ __forceinline__ int kv_v_elem(int slot, int d, int D) {
  const int tt = slot & 31, within = tt & 15;
  const int lane = (within >> 2) * 16 + (d & 15);
  const int j = (tt >> 4) * 4 + (within & 3);
  return KV_BLOCK * D + (((slot & 63) >> 5) * (D >> 4) + (d >> 4)) * 512 + lane * 8 + j;
}

}  // namespace gptoss
