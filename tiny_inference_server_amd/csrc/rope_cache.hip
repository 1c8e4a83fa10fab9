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

// The same for many rows of a pair-ordered bfloat16 projection (a prompt portion), sixteen rows a workgroup.
// Queries and keys: a lane takes four pairs (16 bytes in, two 8-byte runs out), so a wave does four (row, head)
// items an instruction instead of one. Values: the sixteen rows of a head pass through LDS and leave transposed,
// lanes side by side along the rows: rows of a portion have consecutive slots, so a wave's 2-byte stores fall
// into runs of up to 32 bytes ([head_dim][slot] keeps a page's slots of one element together) instead of
// sixty-four separate places.
static constexpr int RB = 16;            // rows of a workgroup
typedef __attribute__((ext_vector_type(8))) __bf16 rc_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 rc_bf16x4;

__global__ __launch_bounds__(RC_THREADS) void rope_write_kv_rows_kernel(
    const bf16* __restrict__ qkv, long ld, const int* __restrict__ positions, const int* __restrict__ write_slots,
    const float2* __restrict__ table, bf16* __restrict__ plane, int rows, int n_heads, int n_kv_heads, int head_dim,
    int page_size, int write_cache, bf16* __restrict__ q_out, long q_out_ld) {
  __shared__ bf16 tile[RB][256 + 8];      // one head of sixteen rows; head sizes up to 256
  const long r0 = (long)blockIdx.x * RB;
  const int n_rows = (int)min((long)RB, rows - r0);
  const int half = head_dim / 2, pieces = head_dim / 8;     // a piece: four pairs, 16 bytes
  const int rotated = n_heads + (write_cache ? n_kv_heads : 0);
  // queries and keys of this workgroup's share of the heads: piece after piece over (head, row, piece)
  for (int hh = blockIdx.y; hh < rotated; hh += gridDim.y) {
    for (int i = threadIdx.x; i < n_rows * pieces; i += RC_THREADS) {
      const int row = i / pieces, piece = i % pieces;
      const long r = r0 + row;
      const rc_bf16x8 x = *reinterpret_cast<const rc_bf16x8*>(qkv + r * ld + (long)hh * head_dim + piece * 8);
      const float4* cs = reinterpret_cast<const float4*>(table + (long)positions[r] * half + piece * 4);
      const float4 cs01 = cs[0], cs23 = cs[1];
      const float c[4] = {cs01.x, cs01.z, cs23.x, cs23.z}, sn[4] = {cs01.y, cs01.w, cs23.y, cs23.w};
      rc_bf16x4 y1, y2;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x1 = static_cast<float>(x[2 * e]), x2 = static_cast<float>(x[2 * e + 1]);
        y1[e] = static_cast<__bf16>(x1 * c[e] - x2 * sn[e]);
        y2[e] = static_cast<__bf16>(x2 * c[e] + x1 * sn[e]);
      }
      bf16* dst;
      if (hh < n_heads) {
        dst = q_out + r * q_out_ld + (long)hh * head_dim;
      } else {
        const int slot = write_slots[r];
        dst = plane + (((long)(slot / page_size) * 2) * n_kv_heads + (hh - n_heads)) * page_size * head_dim +
              (long)(slot % page_size) * head_dim;
      }
      *reinterpret_cast<rc_bf16x4*>(dst + piece * 4) = y1;
      *reinterpret_cast<rc_bf16x4*>(dst + half + piece * 4) = y2;
    }
  }
  if (!write_cache) return;
  // values
  const int row_t = threadIdx.x % RB, d_t = threadIdx.x / RB;          // on the way out: rows side by side
  long v_dst = 0;
  if (row_t < n_rows) {
    const int slot = write_slots[r0 + row_t];
    v_dst = ((long)(slot / page_size) * 2 + 1) * n_kv_heads * page_size * head_dim + slot % page_size;
  }
  for (int kvh = blockIdx.y; kvh < n_kv_heads; kvh += gridDim.y) {
    __syncthreads();                                                     // the tile's last readers are done
    for (int i = threadIdx.x; i < n_rows * pieces; i += RC_THREADS) {
      const int row = i / pieces, piece = i % pieces;
      *reinterpret_cast<rc_bf16x8*>(&tile[row][piece * 8]) = *reinterpret_cast<const rc_bf16x8*>(
          qkv + (r0 + row) * ld + (long)(n_heads + n_kv_heads + kvh) * head_dim + piece * 8);
    }
    __syncthreads();
    if (row_t < n_rows)
      for (int d = d_t; d < head_dim; d += RC_THREADS / RB)
        plane[v_dst + ((long)kvh * head_dim + d) * page_size] = tile[row_t][d];
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
  if (dtype == TIS_BF16 && paired && !interleaved && table && rows >= 4 * RB && head_dim % 8 == 0 && head_dim <= 256 &&
      ld % 8 == 0 && q_out_ld % 4 == 0 && ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)q_out % 8) == 0 &&
      (!write_cache || (uintptr_t)plane % 8 == 0)) {
    dim3 grid((rows + RB - 1) / RB, std::min(total_heads, 4));
    rope_write_kv_rows_kernel<<<grid, RC_THREADS, 0, stream>>>((const bf16*)qkv, ld, positions, write_slots,
                                                              (const float2*)table, (bf16*)plane, rows, n_heads,
                                                              n_kv_heads, head_dim, page_size, write_cache,
                                                              (bf16*)q_out, q_out_ld);
    return tis_launch_status("rope_write_kv_rows");
  }
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
