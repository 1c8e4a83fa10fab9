// Attention of query rows over paged keys and values: the kernel for every head size and for 32-bit.
//
// One workgroup per (row, query head). The row at position p of a request sees the keys at positions
// [max(0, p - window + 1), p] of that request (window 0: all of them), found through the request's block
// table. Query head h reads key/value head h / group_size (reference paged_attention_kernels.py:49).
// Scores, maximum, sum and the output accumulate in 32-bit (reference paged_attention_kernels.py:86-108);
// masked keys are never read, so what a reused page still holds cannot reach the result.
// A page holds a head's keys as [slot][head_dim] and its values as [head_dim][slot].
// A position encoding that works on the scores brings one slope per query head: the score of key j for the row at
// position p gets slope[h] * (j - p) added (a bias linear in the distance; null: none).
// Keys are walked in chunks of a fixed size with a running maximum, so the order of every sum depends on
// the row's own length only, not on what else is in the batch.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_attention_generic)

static constexpr int AG_THREADS = 256;
static constexpr int AG_CHUNK = 1024;
static constexpr int AG_MAX_HD = 256;

template <typename T>
__global__ __launch_bounds__(AG_THREADS) void attention_generic_kernel(
    const T* __restrict__ q, long q_ld, const T* __restrict__ plane, const int* __restrict__ block_tables, int bt_ld,
    const int* __restrict__ row_seq, const int* __restrict__ positions, T* __restrict__ out, long out_ld,
    int group_size, int n_kv_heads, int HD, int page_size, int window, float scale, const float* __restrict__ slopes) {
  __shared__ float qs[AG_MAX_HD];
  __shared__ float sc[AG_CHUNK];
  __shared__ float red[16];
  __shared__ float accm[AG_THREADS];

  const long r = blockIdx.x;
  const int h = blockIdx.y;
  const int kvh = h / group_size;
  const int t = threadIdx.x;
  const int pos = positions[r];
  const int* bt = block_tables + (long)row_seq[r] * bt_ld;
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int kv_end = pos + 1;
  const float slope = slopes ? slopes[h] : 0.f;

  for (int d = t; d < HD; d += AG_THREADS) qs[d] = to_f(q[r * q_ld + (long)h * HD + d]) * scale;
  __syncthreads();

  const long page_stride = 2L * n_kv_heads * page_size * HD;
  const long k_off = (long)kvh * page_size * HD;
  const long v_off = ((long)n_kv_heads + kvh) * page_size * HD;

  const int groups = AG_THREADS / HD;  // HD <= 256 so at least 1
  const int g = t / HD, d = t % HD;
  const bool pv_thread = g < groups;

  float m = -INFINITY, l = 0.f, acc = 0.f;
  for (int c0 = first; c0 < kv_end; c0 += AG_CHUNK) {
    const int n = min(AG_CHUNK, kv_end - c0);
    float cmax = -INFINITY;
    for (int i = t; i < n; i += AG_THREADS) {
      const int j = c0 + i;
      const T* kp = plane + (long)bt[j / page_size] * page_stride + k_off + (long)(j % page_size) * HD;
      float s = 0.f;
      for (int e = 0; e < HD; ++e) s += qs[e] * to_f(kp[e]);
      if (slopes) s += slope * (float)(j - pos);
      sc[i] = s;
      cmax = fmaxf(cmax, s);
    }
    cmax = block_max(cmax, red);
    const float m_new = fmaxf(m, cmax);
    float csum = 0.f;
    for (int i = t; i < n; i += AG_THREADS) {
      const float p = expf(sc[i] - m_new);
      sc[i] = p;
      csum += p;
    }
    csum = block_sum(csum, red);  // its barriers also publish sc[]
    const float rescale = expf(m - m_new);  // 0 on the first chunk (m = -inf)
    l = l * rescale + csum;
    acc *= rescale;
    m = m_new;
    if (pv_thread) {
      for (int i = g; i < n; i += groups) {
        const int j = c0 + i;
        const T* vp = plane + (long)bt[j / page_size] * page_stride + v_off + (j % page_size);
        acc += sc[i] * to_f(vp[(long)d * page_size]);  // values lie transposed: [head_dim][slot]
      }
    }
    __syncthreads();  // sc[] is rewritten by the next chunk
  }
  accm[t] = pv_thread ? acc : 0.f;
  __syncthreads();
  if (t < HD) {
    float o = 0.f;
    for (int gg = 0; gg < groups; ++gg) o += accm[gg * HD + t];
    out[r * out_ld + (long)h * HD + t] = from_f<T>(o / l);
  }
}

TIS_EXPORT int tis_attention_generic(int dtype, const void* q, long q_ld, const void* plane, const int* block_tables,
                                     int bt_ld, const int* row_seq, const int* positions, void* out, long out_ld,
                                     int rows, int n_heads, int n_kv_heads, int head_dim, int page_size, int window,
                                     float scale, const float* slopes, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || n_heads < 1 || n_kv_heads < 1 || n_heads % n_kv_heads || page_size < 1 || window < 0)
    return tis_fail("attention: bad size rows=%d heads=%d kv_heads=%d page=%d window=%d", rows, n_heads, n_kv_heads,
                    page_size, window);
  if (head_dim < 1 || head_dim > AG_MAX_HD)
    return tis_fail("attention: head size %d is outside this kernel's range 1..%d", head_dim, AG_MAX_HD);
  if (n_heads > 65535) return tis_fail("attention: %d heads exceed the grid", n_heads);
  dim3 grid(rows, n_heads);
  const int group = n_heads / n_kv_heads;
  if (dtype == TIS_F32)
    attention_generic_kernel<float><<<grid, AG_THREADS, 0, stream>>>(
        (const float*)q, q_ld, (const float*)plane, block_tables, bt_ld, row_seq, positions, (float*)out, out_ld, group,
        n_kv_heads, head_dim, page_size, window, scale, slopes);
  else if (dtype == TIS_BF16)
    attention_generic_kernel<bf16><<<grid, AG_THREADS, 0, stream>>>(
        (const bf16*)q, q_ld, (const bf16*)plane, block_tables, bt_ld, row_seq, positions, (bf16*)out, out_ld, group,
        n_kv_heads, head_dim, page_size, window, scale, slopes);
  else
    return tis_fail("unknown dtype code %d", dtype);
  return tis_launch_status("attention_generic");
}
