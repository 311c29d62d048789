// Shared helpers for the gfx950 DiT-MoE kernels: error reporting for the
// C ABI, element types, and 64-lane wavefront primitives.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/dice_moe.h"

namespace dice {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
// LDS staging is written as packed bf16 and read back as raw 16-byte chunks;
// these views may alias anything.
typedef u32x4_t __attribute__((may_alias)) u32x4_any_t;
typedef u32x2_t __attribute__((may_alias)) u32x2_any_t;

constexpr int kWave = 64;

// Orders LDS traffic between the lanes of one wavefront: LDS writes issued
// before are complete and visible to every lane after.  (Lanes exchange data
// through LDS in the GEMM epilogues; without a barrier here the compiler may
// run one side of a divergent branch's reads ahead of the other side's
// writes.)  Deliberately not a fence: a fence would also wait for every
// outstanding global load and store.
__device__ __forceinline__ void wave_lds_sync() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_wave_barrier();
}

// Workgroup barrier for data exchanged through LDS: waits for this wave's LDS
// traffic only, not for its outstanding global loads and stores (which
// __syncthreads() would drain first).
__device__ __forceinline__ void block_lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
}

// Records a printf-style message for dice_last_error() and returns `code`.
int fail(int code, const char *fmt, ...);

#define DICE_REQUIRE(cond, code, ...)          \
  do {                                         \
    if (!(cond)) return ::dice::fail((code), __VA_ARGS__); \
  } while (0)

// Returns DICE_ERR_LAUNCH with the runtime's message when a HIP call fails.
#define DICE_HIP(call)                                                              \
  do {                                                                              \
    hipError_t e_ = (call);                                                         \
    if (e_ != hipSuccess) return ::dice::fail(DICE_ERR_LAUNCH, "%s: %s", #call, hipGetErrorString(e_)); \
  } while (0)

// Checks the launch that was just enqueued.
inline int launch_status(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(DICE_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return DICE_OK;
}

inline size_t dtype_size(int dt) {
  switch (dt) {
    case DICE_F32: return 4;
    case DICE_BF16: return 2;
    case DICE_F16: return 2;
    case DICE_FP8_E4M3: return 1;
    default: return 0;
  }
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }
__device__ __forceinline__ float to_f32(f16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float v) { return (f16_t)v; }

// Sum / max over the 64 lanes of a wavefront; every lane gets the result and
// the combination order is fixed (xor butterfly), so results are reproducible.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ int wave_sum_i32(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

}  // namespace dice
