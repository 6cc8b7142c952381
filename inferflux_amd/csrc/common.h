// Shared helpers of the HIP kernels (gfx950, wave64).
//
// Element types are passed as integer codes (DT_F32, DT_BF16) and turned into template
// arguments at the extern "C" boundary.  All arithmetic is done in float; bf16 is a
// storage type only.  Every entry point returns 0 on success or a hipError_t / negative
// code; ifx_last_error() of the same library returns the text for a negative code.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#define DT_F32 0
#define DT_BF16 1

typedef __bf16 bf16_t;

#define WAVE 64

static thread_local char g_ifx_error[512];

#define IFX_FAIL(...)                                         \
  do {                                                        \
    snprintf(g_ifx_error, sizeof(g_ifx_error), __VA_ARGS__);  \
    return -1;                                                \
  } while (0)

#define IFX_REQUIRE(cond, ...) \
  do {                         \
    if (!(cond)) IFX_FAIL(__VA_ARGS__); \
  } while (0)

#define IFX_LAUNCH_CHECK()                      \
  do {                                          \
    hipError_t e__ = hipGetLastError();         \
    if (e__ != hipSuccess) {                    \
      snprintf(g_ifx_error, sizeof(g_ifx_error), "launch failed: %s", hipGetErrorString(e__)); \
      return (int)e__;                          \
    }                                           \
    return 0;                                   \
  } while (0)

#define IFX_DEFINE_LAST_ERROR() \
  extern "C" const char* ifx_last_error() { return g_ifx_error; }

__device__ __forceinline__ float to_f(float v) { return v; }
__device__ __forceinline__ float to_f(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f(float v);
template <> __device__ __forceinline__ float from_f<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f<bf16_t>(float v) { return (bf16_t)v; }

// Load element i of an array whose element type is only known at run time.
__device__ __forceinline__ float load_dyn(const void* p, int dtype, size_t i) {
  return dtype == DT_F32 ? ((const float*)p)[i] : (float)((const bf16_t*)p)[i];
}

// Butterfly reductions over the 64 lanes of a wave.  The order of the additions is fixed by
// the lane numbers, so a result never depends on what else runs on the chip.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `red` holds 16 floats.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int nw = (blockDim.x + WAVE - 1) / WAVE;
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int nw = (blockDim.x + WAVE - 1) / WAVE;
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  float t = red[0];
  for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
  return t;
}
