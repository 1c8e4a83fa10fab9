// Row-wise kernels: token embedding, the reference's RMSNorm, embedding fused with that norm,
// row gather from activations or per-request state, row copies into state, SwiGLU gating.
// One workgroup per row; every reduction runs in 32-bit in an order fixed by the block size.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_rowwise)

static constexpr int ROW_THREADS = 256;

// y = x * sqrt(D) / (||x||_2 + eps) * gain    (reference main_models_new.py:38-42: eps is added to the norm)
template <typename T>
__device__ __forceinline__ void rmsnorm_row(const T* __restrict__ x, const float* __restrict__ gain,
                                            T* __restrict__ y, int D, float eps, float* scratch) {
  float ss = 0.f;
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    float v = to_f(x[i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float mul = sqrtf((float)D) / (sqrtf(ss) + eps);
  for (int i = threadIdx.x; i < D; i += blockDim.x) y[i] = from_f<T>(to_f(x[i]) * mul * gain[i]);
}

template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void rmsnorm_kernel(const T* x, long x_ld, const float* gain, T* y,
                                                              long y_ld, int D, float eps) {
  __shared__ float scratch[16];
  const long r = blockIdx.x;
  rmsnorm_row<T>(x + r * x_ld, gain, y + r * y_ld, D, eps, scratch);
}

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

// The same norm for bfloat16 rows whose width is a multiple of 8 and whose rows start on 16 bytes: every thread
// moves 16 bytes at a time and keeps its values in registers between the two passes.
template <int PER_THREAD>
__global__ __launch_bounds__(ROW_THREADS) void rmsnorm_bf16_vec_kernel(const bf16* __restrict__ x, long x_ld,
                                                                       const float* __restrict__ gain,
                                                                       bf16* __restrict__ y, long y_ld, int D,
                                                                       float eps) {
  __shared__ float scratch[16];
  const long r = blockIdx.x;
  const bf16* xr = x + r * x_ld;
  bf16* yr = y + r * y_ld;
  bf16x8 v[PER_THREAD];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < PER_THREAD; ++i) {
    const int c = (i * ROW_THREADS + threadIdx.x) * 8;
    if (c < D) {
      v[i] = *reinterpret_cast<const bf16x8*>(xr + c);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = static_cast<float>(v[i][e]);
        ss += f * f;
      }
    }
  }
  ss = block_sum(ss, scratch);
  const float mul = sqrtf((float)D) / (sqrtf(ss) + eps);
#pragma unroll
  for (int i = 0; i < PER_THREAD; ++i) {
    const int c = (i * ROW_THREADS + threadIdx.x) * 8;
    if (c < D) {
      const float4 g0 = *reinterpret_cast<const float4*>(gain + c), g1 = *reinterpret_cast<const float4*>(gain + c + 4);
      const float g[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
      bf16x8 w;
#pragma unroll
      for (int e = 0; e < 8; ++e) w[e] = static_cast<__bf16>(static_cast<float>(v[i][e]) * mul * g[e]);
      *reinterpret_cast<bf16x8*>(yr + c) = w;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void embedding_kernel(const T* table, const int* tokens, T* out,
                                                                long out_ld, int D) {
  const long r = blockIdx.x;
  const T* src = table + (long)tokens[r] * D;
  for (int i = threadIdx.x; i < D; i += blockDim.x) out[r * out_ld + i] = src[i];
}

template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void embedding_rmsnorm_kernel(const T* table, const int* tokens,
                                                                        const float* gain, T* out, long out_ld,
                                                                        int D, float eps) {
  __shared__ float scratch[16];
  const long r = blockIdx.x;
  rmsnorm_row<T>(table + (long)tokens[r] * D, gain, out + r * out_ld, D, eps, scratch);
}

// out[r] = index[r] >= 0 ? src[index[r]] : state[-index[r]-1]
template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void gather_rows_kernel(const T* src, long src_ld, const T* state,
                                                                  long state_ld, const int* index, T* out,
                                                                  long out_ld, int D) {
  const long r = blockIdx.x;
  const int ix = index[r];
  const T* from = ix >= 0 ? src + (long)ix * src_ld : state + (long)(-ix - 1) * state_ld;
  for (int i = threadIdx.x; i < D; i += blockDim.x) out[r * out_ld + i] = from[i];
}

// dst[dst_index[i]] = src[src_index[i]]
template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void copy_rows_kernel(const T* src, long src_ld, const int* src_index,
                                                                T* dst, long dst_ld, const int* dst_index, int D) {
  const long i = blockIdx.x;
  const T* from = src + (long)src_index[i] * src_ld;
  T* to = dst + (long)dst_index[i] * dst_ld;
  for (int c = threadIdx.x; c < D; c += blockDim.x) to[c] = from[c];
}

// The gate for bfloat16 rows of a width that is a multiple of 8, 16-byte aligned: eight outputs per thread.
__global__ __launch_bounds__(ROW_THREADS) void swiglu_bf16_vec_kernel(const bf16* __restrict__ gu, long gu_ld,
                                                                      bf16* __restrict__ out, long out_ld, int F) {
  const long r = blockIdx.x;
  const int f = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (f >= F) return;
  const bf16x8 a = *reinterpret_cast<const bf16x8*>(gu + r * gu_ld + 2 * f);
  const bf16x8 b = *reinterpret_cast<const bf16x8*>(gu + r * gu_ld + 2 * f + 8);
  bf16x8 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float g0 = static_cast<float>(a[2 * e]), u0 = static_cast<float>(a[2 * e + 1]);
    const float g1 = static_cast<float>(b[2 * e]), u1 = static_cast<float>(b[2 * e + 1]);
    o[e] = static_cast<__bf16>(g0 / (1.f + expf(-g0)) * u0);
    o[4 + e] = static_cast<__bf16>(g1 / (1.f + expf(-g1)) * u1);
  }
  *reinterpret_cast<bf16x8*>(out + r * out_ld + f) = o;
}

// out[r, f] = silu(gu[r, 2f]) * gu[r, 2f + 1]: gate and up columns come interleaved  (reference main_models_new.py:51)
template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void swiglu_kernel(const T* gu, long gu_ld, T* out, long out_ld, int F) {
  const long r = blockIdx.x;
  const int f = blockIdx.y * blockDim.x + threadIdx.x;
  if (f >= F) return;
  const float g = to_f(gu[r * gu_ld + 2 * f]);
  const float u = to_f(gu[r * gu_ld + 2 * f + 1]);
  out[r * out_ld + f] = from_f<T>(g / (1.f + expf(-g)) * u);
}

#define DISPATCH(dtype, CALL)                                         \
  if ((dtype) == TIS_F32) { typedef float T; CALL; }                  \
  else if ((dtype) == TIS_BF16) { typedef bf16 T; CALL; }             \
  else return tis_fail("unknown dtype code %d", (int)(dtype));

TIS_EXPORT int tis_rmsnorm(int dtype, const void* x, long x_ld, const float* gain, void* y, long y_ld, int rows,
                           int D, float eps, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1) return tis_fail("rmsnorm: bad size rows=%d D=%d", rows, D);
  if (dtype == TIS_BF16 && D % 8 == 0 && D <= 8 * 8 * ROW_THREADS && x_ld % 8 == 0 && y_ld % 8 == 0 &&
      (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0 && (uintptr_t)gain % 16 == 0) {
    const int per_thread = (D / 8 + ROW_THREADS - 1) / ROW_THREADS;
#define VEC(P) rmsnorm_bf16_vec_kernel<P><<<rows, ROW_THREADS, 0, stream>>>((const bf16*)x, x_ld, gain, (bf16*)y, y_ld, D, eps)
    if (per_thread <= 1) VEC(1);
    else if (per_thread <= 2) VEC(2);
    else if (per_thread <= 4) VEC(4);
    else VEC(8);
#undef VEC
    return tis_launch_status("rmsnorm");
  }
  DISPATCH(dtype, (rmsnorm_kernel<T><<<rows, ROW_THREADS, 0, stream>>>((const T*)x, x_ld, gain, (T*)y, y_ld, D, eps)))
  return tis_launch_status("rmsnorm");
}

TIS_EXPORT int tis_embedding(int dtype, const void* table, const int* tokens, void* out, long out_ld, int rows,
                             int D, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1) return tis_fail("embedding: bad size rows=%d D=%d", rows, D);
  DISPATCH(dtype, (embedding_kernel<T><<<rows, ROW_THREADS, 0, stream>>>((const T*)table, tokens, (T*)out, out_ld, D)))
  return tis_launch_status("embedding");
}

TIS_EXPORT int tis_embedding_rmsnorm(int dtype, const void* table, const int* tokens, const float* gain, void* out,
                                     long out_ld, int rows, int D, float eps, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1) return tis_fail("embedding_rmsnorm: bad size rows=%d D=%d", rows, D);
  DISPATCH(dtype, (embedding_rmsnorm_kernel<T><<<rows, ROW_THREADS, 0, stream>>>((const T*)table, tokens, gain,
                                                                                 (T*)out, out_ld, D, eps)))
  return tis_launch_status("embedding_rmsnorm");
}

TIS_EXPORT int tis_gather_rows(int dtype, const void* src, long src_ld, const void* state, long state_ld,
                               const int* index, void* out, long out_ld, int rows, int D, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1) return tis_fail("gather_rows: bad size rows=%d D=%d", rows, D);
  DISPATCH(dtype, (gather_rows_kernel<T><<<rows, ROW_THREADS, 0, stream>>>((const T*)src, src_ld, (const T*)state,
                                                                           state_ld, index, (T*)out, out_ld, D)))
  return tis_launch_status("gather_rows");
}

TIS_EXPORT int tis_copy_rows(int dtype, const void* src, long src_ld, const int* src_index, void* dst, long dst_ld,
                             const int* dst_index, int count, int D, hipStream_t stream) {
  if (count == 0) return 0;
  if (count < 0 || D < 1) return tis_fail("copy_rows: bad size count=%d D=%d", count, D);
  DISPATCH(dtype, (copy_rows_kernel<T><<<count, ROW_THREADS, 0, stream>>>((const T*)src, src_ld, src_index, (T*)dst,
                                                                          dst_ld, dst_index, D)))
  return tis_launch_status("copy_rows");
}

TIS_EXPORT int tis_swiglu(int dtype, const void* gu, long gu_ld, void* out, long out_ld, int rows, int F,
                          hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || F < 1) return tis_fail("swiglu: bad size rows=%d F=%d", rows, F);
  if ((F + ROW_THREADS - 1) / ROW_THREADS > 65535) return tis_fail("swiglu: width %d exceeds the grid", F);
  if (dtype == TIS_BF16 && F % 8 == 0 && gu_ld % 8 == 0 && out_ld % 8 == 0 && (uintptr_t)gu % 16 == 0 &&
      (uintptr_t)out % 16 == 0) {
    dim3 vgrid(rows, (F / 8 + ROW_THREADS - 1) / ROW_THREADS);
    swiglu_bf16_vec_kernel<<<vgrid, ROW_THREADS, 0, stream>>>((const bf16*)gu, gu_ld, (bf16*)out, out_ld, F);
    return tis_launch_status("swiglu");
  }
  dim3 grid(rows, (F + ROW_THREADS - 1) / ROW_THREADS);
  DISPATCH(dtype, (swiglu_kernel<T><<<grid, ROW_THREADS, 0, stream>>>((const T*)gu, gu_ld, (T*)out, out_ld, F)))
  return tis_launch_status("swiglu");
}
