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
  dim3 grid(rows, (F + ROW_THREADS - 1) / ROW_THREADS);
  DISPATCH(dtype, (swiglu_kernel<T><<<grid, ROW_THREADS, 0, stream>>>((const T*)gu, gu_ld, (T*)out, out_ld, F)))
  return tis_launch_status("swiglu");
}
