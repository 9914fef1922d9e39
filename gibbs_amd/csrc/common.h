// Shared declarations of the gfx950 kernels: element types, the error channel that the
// Python side reads, and small wave/block reductions (64-wide wavefronts).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

typedef __bf16 bf16;

// Element type tags passed across the C interface.
enum { GIBBS_F32 = 0, GIBBS_BF16 = 1 };

#define GIBBS_EXPORT extern "C" __attribute__((visibility("default")))

// Records a message for gibbs_last_error() and returns a non-zero status.
int gibbs_fail(const char* fmt, ...);

#define GIBBS_REQUIRE(cond, ...)                 \
  do {                                           \
    if (!(cond)) return gibbs_fail(__VA_ARGS__); \
  } while (0)

// Status of the launch that was just queued.
#define GIBBS_LAUNCH_STATUS(what)                                                      \
  do {                                                                                 \
    hipError_t e_ = hipGetLastError();                                                 \
    if (e_ != hipSuccess) return gibbs_fail("%s: %s", what, hipGetErrorString(e_));    \
    return 0;                                                                          \
  } while (0)

static inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16 v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_float<bf16>(float v) { return (bf16)v; }

constexpr int WAVE = 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `scratch` holds
// one float per wave.  The order of additions is fixed by the thread layout alone.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int n_waves = (blockDim.x + WAVE - 1) / WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < n_waves; ++i) total += scratch[i];
  return total;
}

// Every file of the library sees the entry points' prototypes, so that a definition whose signature has
// drifted from what the native step (step_plan.hip) calls does not compile.
#include "kernels.h"
