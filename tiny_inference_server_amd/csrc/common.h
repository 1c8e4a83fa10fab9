// Shared helpers for the gfx950 kernels: storage types, wave64 and block reductions, error reporting.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

typedef __bf16 bf16;

#define TIS_WAVE 64

// dtype codes shared with the Python binding
#define TIS_F32 0
#define TIS_BF16 1

template <typename T> __device__ __forceinline__ float to_f(T v);
template <> __device__ __forceinline__ float to_f<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f<bf16>(bf16 v) { return static_cast<float>(v); }

template <typename T> __device__ __forceinline__ T from_f(float v);
template <> __device__ __forceinline__ float from_f<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f<bf16>(float v) { return static_cast<bf16>(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = TIS_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, TIS_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = TIS_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, TIS_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads. `scratch` holds 16 floats of LDS. Every thread gets the result.
// The order of additions depends only on the block size, never on the data or the grid.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / TIS_WAVE, lane = threadIdx.x % TIS_WAVE;
  const int nw = (blockDim.x + TIS_WAVE - 1) / TIS_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float r = 0.f;
  for (int i = 0; i < nw; ++i) r += scratch[i];
  return r;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int wave = threadIdx.x / TIS_WAVE, lane = threadIdx.x % TIS_WAVE;
  const int nw = (blockDim.x + TIS_WAVE - 1) / TIS_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float r = scratch[0];
  for (int i = 1; i < nw; ++i) r = fmaxf(r, scratch[i]);
  return r;
}

// ---- error reporting: every entry point returns 0 or a negative code and leaves a message here ----
static thread_local char tis_error_text[512];

static inline int tis_fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
#include <stdarg.h>
static inline int tis_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(tis_error_text, sizeof(tis_error_text), fmt, ap);
  va_end(ap);
  return -1;
}
static inline int tis_launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return tis_fail("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}
#define TIS_EXPORT extern "C" __attribute__((visibility("default")))
#define TIS_DEFINE_LAST_ERROR(prefix) \
  TIS_EXPORT const char* prefix##_last_error() { return tis_error_text; }
