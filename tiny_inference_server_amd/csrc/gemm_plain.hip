// C[M,N] = A[M,K] . W[N,K]^T (+ R[M,N]) with plain 32-bit multiply-adds: the matrix product of the true
// 32-bit path, and of any shape the faster kernels refuse. No matrix-core instruction and no reduced
// precision mode is used here; inputs may be stored as float or bfloat16 and are widened exactly.
// Each output element sums its K products in the same order whatever M is, so a row's result does not
// depend on the other rows of the batch.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_gemm_plain)

static constexpr int GP_BM = 64, GP_BN = 64, GP_BK = 16, GP_THREADS = 256;

template <typename TI, typename TO>
__global__ __launch_bounds__(GP_THREADS) void gemm_plain_kernel(const TI* __restrict__ A, long lda,
                                                                const TI* __restrict__ W, long ldw,
                                                                const TO* __restrict__ R, long ldr, TO* __restrict__ C,
                                                                long ldc, int M, int N, int K) {
  __shared__ float As[GP_BK][GP_BM + 4];
  __shared__ float Ws[GP_BK][GP_BN + 4];
  const int t = threadIdx.x;
  const int tx = t % 16, ty = t / 16;
  const long m0 = (long)blockIdx.y * GP_BM, n0 = (long)blockIdx.x * GP_BN;
  const int lrow = t / 4, lk = (t % 4) * 4;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GP_BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      const long am = m0 + lrow, wn = n0 + lrow;
      As[lk + e][lrow] = (am < M && k < K) ? to_f(A[am * lda + k]) : 0.f;
      Ws[lk + e][lrow] = (wn < N && k < K) ? to_f(W[wn * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GP_BK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const long m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (R) v += to_f(R[m * ldr + n]);
      C[m * ldc + n] = from_f<TO>(v);
    }
  }
}

// in_dtype / out_dtype: 0 float, 1 bfloat16. Supported: (0,0), (1,1), (1,0).
TIS_EXPORT int tis_gemm_plain(int in_dtype, int out_dtype, const void* A, long lda, const void* W, long ldw,
                              const void* R, long ldr, void* C, long ldc, int M, int N, int K, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (M < 0 || N < 0 || K < 1) return tis_fail("gemm: bad size M=%d N=%d K=%d", M, N, K);
  dim3 grid((N + GP_BN - 1) / GP_BN, (M + GP_BM - 1) / GP_BM);
  if (grid.y > 65535) return tis_fail("gemm: %d rows exceed the grid", M);
  if (in_dtype == TIS_F32 && out_dtype == TIS_F32)
    gemm_plain_kernel<float, float><<<grid, GP_THREADS, 0, stream>>>((const float*)A, lda, (const float*)W, ldw,
                                                                     (const float*)R, ldr, (float*)C, ldc, M, N, K);
  else if (in_dtype == TIS_BF16 && out_dtype == TIS_BF16)
    gemm_plain_kernel<bf16, bf16><<<grid, GP_THREADS, 0, stream>>>((const bf16*)A, lda, (const bf16*)W, ldw,
                                                                   (const bf16*)R, ldr, (bf16*)C, ldc, M, N, K);
  else if (in_dtype == TIS_BF16 && out_dtype == TIS_F32)
    gemm_plain_kernel<bf16, float><<<grid, GP_THREADS, 0, stream>>>((const bf16*)A, lda, (const bf16*)W, ldw,
                                                                    (const float*)R, ldr, (float*)C, ldc, M, N, K);
  else
    return tis_fail("gemm: unsupported dtype pair in=%d out=%d", in_dtype, out_dtype);
  return tis_launch_status("gemm_plain");
}
