// Rotary position encoding of queries and keys, fused with the write of keys and values into cache pages.
//
// Input rows hold [q heads | k heads | v heads] as one projection wrote them. Queries are rotated in place,
// keys are rotated on their way into the page, values are copied. The rotation runs in 32-bit on a table of
// (cos, sin) per position and pair. Pairs are (j, j + head_dim/2) in the "half" pairing (reference
// main_models_new.py:71-80) or (2j, 2j+1) in the "interleaved" pairing; a null table means no rotation.
//
// With `paired` the q and k heads of the input come with the two members of every rotary pair side by side
// (pair j at columns 2j and 2j+1 of the head: the order in which the fused projection's weight rows are kept);
// the rotated queries then go, in their natural order, to a separate output.
//
// One cache plane is laid out [page][key or value][kv head][...]: a head's keys of a page as [slot][head_dim],
// its values transposed as [head_dim][slot], which is how the matrix-core attention kernel wants to load them.
#include <algorithm>

#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_rope_cache)

static constexpr int RC_THREADS = 256;

// A row's heads (q, then k, then v) are spread over gridDim.y workgroups of four waves; a wave takes its
// workgroup's heads in turn. Few heads a wave keep the chain of dependent loads short.
template <typename T>
__global__ __launch_bounds__(RC_THREADS) void rope_write_kv_kernel(T* __restrict__ qkv, long ld,
                                                                   const int* __restrict__ positions,
                                                                   const int* __restrict__ write_slots,
                                                                   const float2* __restrict__ table,
                                                                   T* __restrict__ plane, int n_heads, int n_kv_heads,
                                                                   int head_dim, int page_size, int interleaved,
                                                                   int write_cache, int paired, T* __restrict__ q_out,
                                                                   long q_out_ld) {
  const long r = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int half = head_dim / 2;
  const int total = n_heads + 2 * n_kv_heads;
  const int slot = write_cache ? write_slots[r] : 0;
  const int page = slot / page_size, off = slot % page_size;
  const float2* cs = table ? table + (long)positions[r] * half : nullptr;

  for (int hh = blockIdx.y * (RC_THREADS / 64) + (threadIdx.x >> 6); hh < total;
       hh += gridDim.y * (RC_THREADS / 64)) {   // [0, n_heads): q, then k heads, then v heads
    T* row = qkv + r * ld + (long)hh * head_dim;
    const bool is_q = hh < n_heads;
    const bool is_v = hh >= n_heads + n_kv_heads;
    T* dst = row;  // queries are rewritten where they are, unless a separate output is given
    if (is_q && q_out) dst = q_out + r * q_out_ld + (long)hh * head_dim;
    if (!is_q) {
      if (!write_cache) continue;  // keys and values that are not kept have no reader
      const int kvh = is_v ? hh - n_heads - n_kv_heads : hh - n_heads;
      T* head = plane + (((long)page * 2 + (is_v ? 1 : 0)) * n_kv_heads + kvh) * page_size * head_dim;
      if (is_v) {  // values: [head_dim][slot]
        for (int i = lane; i < head_dim; i += 64) head[(long)i * page_size + off] = row[i];
        continue;
      }
      dst = head + (long)off * head_dim;
    }
    if (cs == nullptr) {
      if (paired) {
        for (int j = lane; j < half; j += 64) {
          dst[interleaved ? 2 * j : j] = row[2 * j];
          dst[interleaved ? 2 * j + 1 : j + half] = row[2 * j + 1];
        }
      } else if (dst != row) {
        for (int i = lane; i < head_dim; i += 64) dst[i] = row[i];
      }
      continue;
    }
    for (int j = lane; j < half; j += 64) {
      const int a = interleaved ? 2 * j : j;
      const int b = interleaved ? 2 * j + 1 : j + half;
      const float x1 = to_f(row[paired ? 2 * j : a]), x2 = to_f(row[paired ? 2 * j + 1 : b]);
      const float c = cs[j].x, s = cs[j].y;
      // q*cos + rotate_half(q)*sin with rotate_half = [-x2, x1]
      const float y1 = x1 * c - x2 * s;
      const float y2 = x2 * c + x1 * s;
      dst[a] = from_f<T>(y1);
      dst[b] = from_f<T>(y2);
    }
  }
}

TIS_EXPORT int tis_rope_write_kv(int dtype, void* qkv, long ld, const int* positions, const int* write_slots,
                                 const float* table, void* plane, int rows, int n_heads, int n_kv_heads, int head_dim,
                                 int page_size, int interleaved, int write_cache, int paired, void* q_out,
                                 long q_out_ld, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || n_heads < 1 || n_kv_heads < 1 || head_dim < 2 || (head_dim & 1) || page_size < 1)
    return tis_fail("rope_write_kv: bad size rows=%d heads=%d kv_heads=%d head_dim=%d page=%d", rows, n_heads,
                    n_kv_heads, head_dim, page_size);
  if (paired && !q_out) return tis_fail("rope_write_kv: paired input needs a separate output for the queries");
  const int total_heads = n_heads + 2 * n_kv_heads;
  // measured on MI355X with 18 heads of 128: few rows like their heads spread wide (64 rows: 3.5 us over five
  // workgroups a row against 4.5 over one), thousands of rows like two workgroups a row (10.3 against 11.1 us)
  const int wide = (total_heads + RC_THREADS / 64 - 1) / (RC_THREADS / 64);
  dim3 grid(rows, std::max(1, std::min(rows < 256 ? 5 : 2, wide)));
  if (dtype == TIS_F32)
    rope_write_kv_kernel<float><<<grid, RC_THREADS, 0, stream>>>((float*)qkv, ld, positions, write_slots, (const float2*)table,
                                                         (float*)plane, n_heads, n_kv_heads, head_dim, page_size,
                                                         interleaved, write_cache, paired, (float*)q_out, q_out_ld);
  else if (dtype == TIS_BF16)
    rope_write_kv_kernel<bf16><<<grid, RC_THREADS, 0, stream>>>((bf16*)qkv, ld, positions, write_slots, (const float2*)table,
                                                        (bf16*)plane, n_heads, n_kv_heads, head_dim, page_size,
                                                        interleaved, write_cache, paired, (bf16*)q_out, q_out_ld);
  else
    return tis_fail("unknown dtype code %d", dtype);
  return tis_launch_status("rope_write_kv");
}
