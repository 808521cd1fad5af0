// Shared helpers of the HIP kernels: element types, wave reductions, error reporting.
// Everything here is written for gfx950 (CDNA4): 64-lane waves, 160 KB LDS per CU.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;

#define MI_WAVE 64

// Every entry point returns 0 on success.  On refusal it returns a negative code
// and leaves a message that mi_last_error() returns.
#define MI_OK 0
#define MI_ERR_SHAPE (-1)
#define MI_ERR_LAUNCH (-2)
#define MI_ERR_LIMIT (-3)

void mi_set_error(const char* fmt, ...);

#define MI_REQUIRE(cond, ...)        \
  do {                               \
    if (!(cond)) {                   \
      mi_set_error(__VA_ARGS__);     \
      return MI_ERR_SHAPE;           \
    }                                \
  } while (0)

#define MI_CHECK_LAUNCH(name)                                               \
  do {                                                                      \
    hipError_t mi_err_ = hipGetLastError();                                 \
    if (mi_err_ != hipSuccess) {                                            \
      mi_set_error("%s: launch failed: %s", name, hipGetErrorString(mi_err_)); \
      return MI_ERR_LAUNCH;                                                 \
    }                                                                       \
  } while (0)

// dtype codes shared with the Python side
#define MI_F32 0
#define MI_BF16 1

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

// A load of data that a kernel reads once and nobody reads again soon (the weights of a
// product with few rows, the keys and values of a decode step): marked non-temporal, so that
// it does not push what is reused out of the caches.  Measured on MI355X, long reads run at
// 7.0-7.1 TB/s with this mark against 6.1-6.3 TB/s without it.
template <typename T>
__device__ __forceinline__ T load_streamed(const T* p) {
  return __builtin_nontemporal_load(p);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, MI_WAVE));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, MI_WAVE);
  return v;
}

// Sum over a whole block in a fixed order: lanes by butterfly, waves one after another.
// `scratch` holds at least blockDim.x / 64 floats.  All threads get the result.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / MI_WAVE;
  const int lane = threadIdx.x % MI_WAVE;
  const int n_waves = (blockDim.x + MI_WAVE - 1) / MI_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < n_waves; ++w) total += scratch[w];
  return total;
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }
