// Attention over paged keys and values on the matrix cores (bfloat16, gfx950), for decode rows and for
// portions of prompts alike. Compiled for one head size: -DTIS_HD=<multiple of 16, at most 256>.
// Two kernels and a merge: the wave kernel described next, and further down the tile kernel that takes long
// portions (a workgroup of four waves sharing keys and values through LDS).
//
// Wave kernel. One wavefront owns an *item*: up to 16*NB query columns that share a request and a key/value head, a
// column being (row, query head): n_rows consecutive positions of the request times the group's query heads.
// A decode row is an item of one row; all query heads of its group share one pass over the keys, so keys
// and values are read once per group, not once per query head. A long key range is cut into splits that
// different wavefronts take; a second kernel merges their partial results.
//
// Per step of 32 keys (two tiles of 16, each inside one page; page sizes are multiples of 16):
//   S^T[key, col] = K[key, :] . Q[col, :]      v_mfma_f32_16x16x32_bf16, A = keys straight from the page
//                                              ([slot][head_dim]: 16 bytes per lane), B = queries in registers
//   mask by select (key <= the column's position, key inside its window), running maximum and sum per column
//   in 32-bit, base-2 exponentials with log2(e)/sqrt(head_dim) folded into the scale
//   O^T[d, col] += V^T[d, key] . P^T[key, col] A = values straight from the page, which holds them transposed
//                                              ([head_dim][slot]: 8 bytes per lane and tile), B = P rounded to
//                                              bfloat16 (as the reference does before P.V:
//                                              paged_attention_kernels.py:108), exactly as S^T left it in registers
// Both products put the column on the lane, so the softmax statistics never cross lanes except for the
// reduction over the four key groups, and this kernel uses no LDS. Masked keys are read (their page is mapped), but their
// scores are replaced by -inf and their values by zero before either is used in arithmetic, so what an earlier
// owner left in a page never reaches a result.
#include <algorithm>
#include <mutex>
#include <type_traits>

#include "common.h"
#include "attention_mfma.h"

#ifndef TIS_HD
#error "compile with -DTIS_HD=<head size>"
#endif
static_assert(TIS_HD % 16 == 0 && TIS_HD >= 16 && TIS_HD <= 256, "head size must be a multiple of 16, at most 256");

TIS_DEFINE_LAST_ERROR(tis_attention_mfma)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

static constexpr int HD = TIS_HD;
static constexpr int DC = (HD + 31) / 32;   // 32-wide chunks of the head for Q.K
static constexpr int DB = HD / 16;          // 16-wide blocks of the head for P.V

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x4 load4(const bf16* p) { return *reinterpret_cast<const bf16x4*>(p); }

// the largest / the sum of a value over the four lanes that hold one column (they differ in lane bits 4 and 5),
// by the row and half swaps of gfx950: no trip through LDS
__device__ __forceinline__ float column_max(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
// the largest of three numbers that are not NaN payloads to be quieted: one instruction (fmaxf would first copy each
// operand through a maximum with itself)
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float column_sum(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// PS16: pages of exactly 16 tokens. A 16-key tile is then a whole page, page indices are shifts, and a lane's
// offsets inside a page never change: the loads of a step need no address arithmetic beyond the page's base.
template <int NB, bool PS16>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(NB <= 2 ? 2 : 1))) void attention_mfma_kernel(
    const bf16* __restrict__ q, long q_ld, const bf16* __restrict__ plane, const int* __restrict__ block_tables,
    int bt_ld, const int* __restrict__ row_seq, const int* __restrict__ positions, const int2* __restrict__ items,
    bf16* __restrict__ out, long out_ld, float* __restrict__ part_o, float2* __restrict__ part_ml, int group_size,
    int n_kv_heads, int n_heads, int page_size_arg, int window, float scale_log2, int n_splits, int min_steps,
    int split_stride, int* __restrict__ row_splits) {
  const int page_size = PS16 ? 16 : page_size_arg;
  const int item = blockIdx.x, kvh = blockIdx.y;
  int split = blockIdx.z;
  const int lane = threadIdx.x, c16 = lane & 15, g = lane >> 4;
  // Three ways to an item. No item list: every item is the single row of its own index (a step of decoded tokens),
  // which saves the wave one of the dependent loads it starts with. A list of (first row, rows). Or, for decoded
  // tokens of requests whose lengths differ widely (min_steps < 0), a list planned on the host with one entry per
  // wave: (row, split + 65536 * the row's splits, position, line of the block table); it brings what the wave would
  // otherwise load next, so it costs no further trip to memory, and a row < 0 pads the list to its fixed length.
  int row0, n_rows, p_first, seq, planned_splits = 0;
  if (min_steps < 0) {
    const int4 e = reinterpret_cast<const int4*>(items)[item];
    if (e.x < 0) return;
    row0 = e.x;
    n_rows = 1;
    split = e.y & 0xffff;
    planned_splits = e.y >> 16;
    p_first = e.z;
    seq = e.w;
  } else {
    row0 = items ? items[item].x : item;
    n_rows = items ? items[item].y : 1;
    seq = row_seq[row0];
    p_first = positions[row0];
  }
  const int* bt = block_tables + (long)seq * bt_ld;
  const int p_last = p_first + n_rows - 1;

  // the lane's column in each block
  int col_row[NB], col_head[NB], col_pos[NB], col_lo[NB];
  bool col_ok[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int c = nb * 16 + c16;
    const int ro = c / group_size;
    col_ok[nb] = ro < n_rows;
    col_row[nb] = row0 + (col_ok[nb] ? ro : 0);
    col_head[nb] = kvh * group_size + c % group_size;
    col_pos[nb] = col_ok[nb] ? p_first + ro : -1;
    col_lo[nb] = (window > 0 && col_pos[nb] - window + 1 > 0) ? col_pos[nb] - window + 1 : 0;
  }

  // queries: the B operand of S^T, kept in registers for the whole key range
  bf16x8 qb[NB][DC];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) {
      const int d = dc * 32 + g * 8;
      bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (col_ok[nb] && d < HD) v = load8(q + (long)col_row[nb] * q_ld + (long)col_head[nb] * HD + d);
      qb[nb][dc] = v;
    }

  // this wave's share of the item's keys, in steps of 32 from a multiple of 32
  int k_lo = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
  k_lo &= ~31;
  const int k_hi = p_last + 1;
  const int lo_last = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;   // the largest window start
  const int n_steps = (k_hi - k_lo + 31) / 32;
  // The grid offers every item n_splits waves a kv head. With min_steps an item takes only as many of them as
  // leaves each at least that many steps, so that short items are not cut into crumbs while long ones (the last
  // rows of a prompt, whose chain of steps would otherwise set the kernel's time) are; the rest return at once.
  // row_splits tells the merge how many partial results each row has (one: the output is already final).
  int item_splits = n_splits;
  if (min_steps > 0) item_splits = max(1, min(n_splits, n_steps / min_steps));
  if (min_steps < 0) item_splits = max(1, min(n_splits, planned_splits));
  if (split >= item_splits) return;
  if (row_splits && kvh == 0 && split == 0 && lane < n_rows) row_splits[row0 + lane] = item_splits;
  const int per_split = (n_steps + item_splits - 1) / item_splits;
  const int s_begin = split * per_split;
  const int s_end = min(n_steps, s_begin + per_split);

  const long page_stride = 2L * n_kv_heads * page_size * HD;
  const long k_head = (long)kvh * page_size * HD;
  const long v_head = ((long)n_kv_heads + kvh) * page_size * HD;

  f32x4 o[NB][DB];
  float m[NB], l[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    m[nb] = -INFINITY;
    l[nb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db) o[nb][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  // One step's keys and values in registers. A step's loads are all issued together, one step ahead of the
  // products that use them, and the page ids two steps ahead, so that a wave always has a step's worth of
  // requests in flight instead of waiting out a chain of dependent loads per step.
  struct Tiles {
    bf16x8 k[2][DC];
    bf16x8 v[DB];
    bool ok[2];
  };
  // Every load below is unconditional: a tile that lies past the item's keys, or a step past the wave's share,
  // reads page 0 instead (always mapped, and finite) and is masked afterwards. Without branches around the loads
  // the compiler can wait for exactly the loads a product needs while the next step's are still in flight.
  auto page_ids = [&](int s, int (&pg)[2]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key0 = k_lo + s * 32 + t * 16;
      const bool ok = s < s_end && key0 < k_hi;
      const int got = bt[ok ? (PS16 ? key0 >> 4 : key0 / page_size) : 0];
      pg[t] = ok ? got : -1;
    }
  };
  auto load_tiles = [&](int s, const int (&pg)[2], Tiles& T) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key0 = k_lo + s * 32 + t * 16;
      const int slot0 = PS16 ? 0 : key0 % page_size;
      T.ok[t] = pg[t] >= 0;
      const bf16* base = plane + (long)(T.ok[t] ? pg[t] : 0) * page_stride;
      const bf16* kp = base + k_head + (long)(slot0 + c16) * HD;
      const bf16* vp = base + v_head + (long)c16 * page_size + slot0 + g * 4;
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) {
        const int d = dc * 32 + g * 8;
        const bool d_ok = (HD % 32 == 0) || d < HD;
        const bf16x8 ka = load8(kp + (d_ok ? d : 0));
        T.k[t][dc] = d_ok ? ka : (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
      }
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const bf16x4 h = load4(vp + (long)db * 16 * page_size);
#pragma unroll
        for (int e = 0; e < 4; ++e) T.v[db][t * 4 + e] = h[e];
      }
    }
  };
  auto consume = [&](int s, Tiles& T) {
    const int kb = k_lo + s * 32;
    // S^T = K . Q^T
    f32x4 st[2][NB];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) st[t][nb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dc = 0; dc < DC; ++dc)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          st[t][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(T.k[t][dc], qb[nb][dc], st[t][nb], 0, 0, 0);
    }
    // mask, running maximum and sum per column, P in bfloat16 as the B operand of the second product.
    // A step whose 32 keys lie inside every column's range needs no mask at all (most steps of a long row).
    const bool full = T.ok[0] && T.ok[1] && kb + 31 <= p_first && kb >= lo_last;
    if (!full) {
      // Values of keys that no column of the item may see (slots past its last position, keys before its window,
      // tiles past its range) are set to zero and not merely weighted by zero: what lies there is whatever an
      // earlier owner of the page left, possibly not even finite.
      const int lo_first = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int key = kb + t * 16 + g * 4 + e;
          if (!(T.ok[t] && key <= p_last && key >= lo_first)) {
#pragma unroll
            for (int db = 0; db < DB; ++db) T.v[db][t * 4 + e] = static_cast<__bf16>(0.f);
          }
        }
      // one branch a step around all the masking, not one around each score
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = kb + t * 16 + g * 4 + i;
            const bool ok = T.ok[t] && key <= col_pos[nb] && key >= col_lo[nb];
            st[t][nb][i] = ok ? st[t][nb][i] : -INFINITY;
          }
    }
    bf16x8 pb[NB];
    float alpha[NB];
    bool grew = false;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float sv[8];
      float tmax = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float v = st[t][nb][i];   // unscaled: the scale (positive) goes into the exponent's multiply-add
          sv[t * 4 + i] = v;
          tmax = fmaxf(tmax, v);
        }
      tmax = column_max(tmax) * scale_log2;
      // m is the exponent that P, the sum and the output are taken relative to. It follows the running maximum
      // only when that has grown by more than 2^8 beyond it, so it settles after a row's first keys and the
      // rescaling below becomes rare; until then P stays below 256, well inside bfloat16, and sum and output
      // share the factor, which cancels in their ratio.
      const bool move = tmax > m[nb] + 8.f || m[nb] == -INFINITY;
      const float m_new = move ? fmaxf(m[nb], tmax) : m[nb];
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;   // a column with no key yet: everything stays 0
      grew = grew || (move && m_new > m[nb]);
      alpha[nb] = __builtin_amdgcn_exp2f(m[nb] - m_use);
      float psum = 0.f;
      bf16x8 pv;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = __builtin_amdgcn_exp2f(fmaf(sv[e], scale_log2, -m_use));   // arguments are <= 8
        psum += p;
        pv[e] = static_cast<__bf16>(p);
      }
      pb[nb] = pv;
      l[nb] = l[nb] * alpha[nb] + psum;      // the lane's share; the four key groups are added at the end
      m[nb] = m_new;
    }
    // O^T = O^T * alpha + V^T . P^T. The running maximum settles after the first keys of a row; while no
    // column of the wave has a new maximum every alpha is exactly 1 and the accumulators are left alone.
    if (__builtin_amdgcn_ballot_w64(grew) != 0) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[nb][db][i] *= alpha[nb];
    }
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        o[nb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(T.v[db], pb[nb], o[nb][db], 0, 0, 0);
  };

  if (NB >= 2) {
    // Wide items (rows of prompt portions) are bound by instruction issue, not by memory: they keep one step's
    // tiles only, which leaves registers for a second wave per SIMD to fill the gaps, and prefetch just the page
    // ids. (A second set of tiles to load ahead into would live in accumulator registers and cost some 180 copy
    // instructions a step: measured slower even where a wave has its SIMD to itself.)
    if (s_begin < s_end) {
      Tiles ta;
      int pa[2], pn[2];
      page_ids(s_begin, pa);
      for (int s = s_begin; s < s_end; ++s) {
        load_tiles(s, pa, ta);
        page_ids(s + 1, pn);
        consume(s, ta);
        pa[0] = pn[0];
        pa[1] = pn[1];
      }
    }
  } else if (s_begin < s_end) {
    Tiles ta, tb;
    int pa[2], pn[2], pq[2];
    page_ids(s_begin, pa);
    page_ids(s_begin + 1, pn);
    load_tiles(s_begin, pa, ta);
    for (int s = s_begin; s < s_end; s += 2) {
      // pn holds the page ids of step s+1; loads past the end are harmless and never consumed
      page_ids(s + 2, pq);
      load_tiles(s + 1, pn, tb);
      consume(s, ta);
      page_ids(s + 3, pn);
      load_tiles(s + 2, pq, ta);
      if (s + 1 < s_end) consume(s + 1, tb);
    }
  }

  // the lane holds, for its column, the outputs d = db*16 + g*4 + {0..3}
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const float lt = column_sum(l[nb]);
    if (!col_ok[nb]) continue;
    if (item_splits == 1) {
      const float inv = 1.f / lt;
      bf16* dst = out + (long)col_row[nb] * out_ld + (long)col_head[nb] * HD + g * 4;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        bf16x4 w;
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = static_cast<__bf16>(o[nb][db][i] * inv);
        *reinterpret_cast<bf16x4*>(dst + db * 16) = w;
      }
    } else {
      const long slot = ((long)col_row[nb] * n_heads + col_head[nb]) * split_stride + split;
      float* dst = part_o + slot * HD + g * 4;
#pragma unroll
      for (int db = 0; db < DB; ++db) *reinterpret_cast<f32x4*>(dst + db * 16) = o[nb][db];
      if (g == 0) part_ml[slot] = make_float2(m[nb], lt);
    }
  }
}

// ---- Long portions of prompts: a workgroup of four waves shares every step's keys and values through LDS ----
//
// A wave of the kernel above fetches its keys and values itself, so the rows of a prompt read each key once per
// 16*NB columns, and a wave waits out the fetch of every step. Here a *tile* is up to TW * (32 / group size)
// consecutive rows of one request; its four waves own 32 columns each, one a lane pair, and walk the tile's keys
// together. Each step's 32 keys and values are copied once from the pages into LDS, two steps ahead of the products
// that read them, by loads that write LDS directly (global_load_lds: no registers, no store instructions), and every
// wave takes its operands from there. LDS holds them in the order the products read them: 16-byte pieces, 16 pieces
// that a quarter of a wave reads together side by side, so that reads meet no bank conflict and need no padding; a
// copying lane picks the piece of the page that belongs in its slot.
//
// Both products are v_mfma_f32_32x32x16_bf16, with the column on the lane as in the wave kernel:
//   S^T[32 keys, 32 columns] = K . Q^T over the head in steps of 16; lane (c, h) of the result holds column c and the
//       score rows 8b + 4h + k (b, k < 4) in accumulator 4b + k
//   O^T[32 of the head, 32 columns] += V^T . P^T over the keys in two halves of 16; as the second operand lane (c, h)
//       must hold P of the keys 8h .. 8h+7 of a half
// So that P can stay in the registers S^T left it in, score row 8b + 4h + k is made to be key 16 (b >> 1) + 8h +
// 4 (b & 1) + k: inside each 16-key tile the rows' bits 2 and 3 change places, which costs nothing, since the copying
// lane picks its key anyway. Accumulators 0..7 of a lane are then the keys 8h.. of the first half and 8..15 those of
// the second, in order.
static constexpr int TW = 4;               // waves of a tile
static constexpr int TCOLS = 32;           // columns of a wave
static constexpr int TBUF = 3;             // LDS buffers: step s+1's keys, step s's values, and step s+2 being written
static constexpr int NCH = HD / 8;         // 16-byte pieces of one key
static constexpr int TCH = 4 * HD;         // pieces of a step's keys, and of its values: HD / 16 fetches of 64
static constexpr int TPT = (TCH + TW * 64 - 1) / (TW * 64);   // fetches a wave issues, of each
static constexpr int KC = HD / 16;         // 16-wide steps of the head for K.Q
static constexpr int DT = (HD + 31) / 32;  // 32-high blocks of the head for V.P
// keys:   piece (t, dch, r) = key t*16 + (r with bits 2 and 3 exchanged), elements dch*8.. at piece index
//         (t*NCH + dch)*16 + r
// values: piece (t, db, gh, c16) = element db*16 + c16 of the head, keys t*16 + gh*8.. at ((t*DB + db)*2 + gh)*16 + c16
typedef __attribute__((ext_vector_type(16))) float f32x16;

#pragma clang diagnostic ignored "-Winline-asm"   // M0 in a clobber list: meant
// One 16-byte piece per lane from global memory straight into LDS: lane i's piece lands at lds_base + 16 * i
// (global_load_lds_dwordx4; the LDS base travels in M0). Written in assembly because the compiler orders every later
// LDS read behind such a load, whichever buffer it reads, which would undo the prefetch; so the compiler does not
// count these loads either, and whoever reads the pieces waits for them (vmcnt) and for the other waves (barrier).
__device__ __forceinline__ void copy_to_lds(const bf16* src, const bf16* lds_base) {
  const unsigned base = (unsigned)(uintptr_t)(const __attribute__((address_space(3))) bf16*)lds_base;
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(base) : "memory", "m0");
}
// the same with the source as a scalar address (the same on all lanes) plus each lane's offset in bytes
__device__ __forceinline__ void copy_to_lds(const bf16* src, unsigned lane_bytes, const bf16* lds_base) {
  const unsigned base = (unsigned)(uintptr_t)(const __attribute__((address_space(3))) bf16*)lds_base;
  const uint64_t a = (uint64_t)src;       // into scalar registers, whatever the compiler made of the address so far
  const uint64_t scalar = ((uint64_t)(unsigned)__builtin_amdgcn_readfirstlane((int)(a >> 32)) << 32) |
                          (unsigned)__builtin_amdgcn_readfirstlane((int)a);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_bytes), "s"(scalar), "s"(base) : "memory", "m0");
}
// the larger / the sum of a value on the two lanes that hold one column of a tile (they differ in lane bit 5)
__device__ __forceinline__ float pair_max(float v) {
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float pair_sum(float v) {
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// (heads wider than 128 need more than 256 registers a lane: one wave a SIMD)
template <bool PS16>
__global__ __launch_bounds__(TW * 64) __attribute__((amdgpu_waves_per_eu(HD <= 128 ? 2 : 1))) void attention_tile_kernel(
    const bf16* __restrict__ q, long q_ld, const bf16* __restrict__ plane, const int* __restrict__ block_tables,
    int bt_ld, const int* __restrict__ row_seq, const int* __restrict__ positions, const int2* __restrict__ tiles,
    bf16* __restrict__ out, long out_ld, float* __restrict__ part_o, float2* __restrict__ part_ml, int group_size,
    int n_kv_heads, int n_heads, int page_size_arg, int window, float scale_log2, int n_splits, int max_steps,
    int split_stride, int* __restrict__ row_splits) {
  __shared__ __attribute__((aligned(16))) bf16 k_lds[TBUF][TCH * 8];
  __shared__ __attribute__((aligned(16))) bf16 v_lds[TBUF][TCH * 8];
  const int page_size = PS16 ? 16 : page_size_arg;
  const int tile = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
  // the wave's number is the same on all its lanes: said so, what follows from it is scalar arithmetic and branches
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, c32 = lane & 31, h = lane >> 5;
  const int t_row0 = tiles[tile].x, t_rows = tiles[tile].y;
  const int* bt = block_tables + (long)row_seq[t_row0] * bt_ld;
  const int tp_first = positions[t_row0], tp_last = tp_first + t_rows - 1;

  // the wave's rows of the tile; a wave past the tile's last row only helps with the copies
  const int rows_per_wave = TCOLS / group_size;
  const int n_rows = max(0, min(rows_per_wave, t_rows - wave * rows_per_wave));
  const bool active = n_rows > 0;
  const int row0 = t_row0 + (active ? wave * rows_per_wave : 0);
  const int p_first = tp_first + (active ? wave * rows_per_wave : 0);
  const int p_last = p_first + n_rows - 1;

  // the lane's column: a row of the wave and a query head of the group
  const int ro = c32 / group_size;
  const bool col_ok = ro < n_rows;
  const int col_row = row0 + (col_ok ? ro : 0);
  const int col_head = kvh * group_size + c32 % group_size;
  const int col_pos = col_ok ? p_first + ro : -1;
  const int col_lo = (window > 0 && col_pos - window + 1 > 0) ? col_pos - window + 1 : 0;
  bf16x8 qb[KC];
#pragma unroll
  for (int kc = 0; kc < KC; ++kc) {
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (col_ok) v = load8(q + (long)col_row * q_ld + (long)col_head * HD + kc * 16 + h * 8);
    qb[kc] = v;
  }

  // the tile's keys and this workgroup's share of them, as in the wave kernel
  const int t_lo = (window > 0 && tp_first - window + 1 > 0) ? tp_first - window + 1 : 0;   // first key any row sees
  const int k_lo = t_lo & ~31;
  const int k_hi = tp_last + 1;
  const int n_steps = (k_hi - k_lo + 31) / 32;
  // as many splits as keep each no longer than max_steps (the host's bound on the chain of steps one workgroup walks)
  const int item_splits = max(1, min(n_splits, (n_steps + max_steps - 1) / max_steps));
  if (split >= item_splits) return;                   // the whole workgroup, before any barrier
  if (row_splits && kvh == 0 && split == 0 && tid < t_rows) row_splits[t_row0 + tid] = item_splits;
  const int per_split = (n_steps + item_splits - 1) / item_splits;
  const int s_begin = split * per_split;
  const int s_end = min(n_steps, s_begin + per_split);
  const int w_lo = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;    // first key the wave sees
  const int lo_last = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;

  const long page_stride = 2L * n_kv_heads * page_size * HD;
  const long k_head = (long)kvh * page_size * HD;
  const long v_head = ((long)n_kv_heads + kvh) * page_size * HD;

  // No running maximum yet: a finite number far below any score, so that differences with it stay numbers (a
  // column none of whose keys has counted so far keeps it, with a sum of zero; the merge gives such a part no weight).
  // `over`: the raw score from which on the maximum has to move.
  constexpr float NO_MAX = -1e30f;
  const float per_scale = 1.f / scale_log2;
  f32x16 o[DT];
  float m = NO_MAX, l = 0.f, over = (NO_MAX + 8.f) * per_scale;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;

  // What the loop below spends per step is instructions, of any kind: a wave issues one every four cycles at best,
  // and the matrix instructions of the other wave on its SIMD do not hide the rest. So whatever a step can know in
  // advance is worked out here, once, as ranges of steps:
  //   mine:   steps with a key that some row of this wave sees (others are skipped: past its last row, before its
  //           first window)
  //   free:   steps all of whose keys every row of the wave sees (no masking)
  //   inside: steps all of whose keys some row of the tile sees (their values need no guarding, see below)
  const int mine_lo = max(s_begin, (w_lo - k_lo) >> 5), mine_hi = active ? min(s_end, ((p_last - k_lo) >> 5) + 1) : 0;
  const int free_lo = (lo_last - k_lo + 31) >> 5, free_hi = (p_first + 1 - k_lo) >> 5;
  const int in_lo = (t_lo - k_lo + 31) >> 5, in_hi = (tp_last + 1 - k_lo) >> 5;

  // Where a step's keys and values lie: every wave keeps, in a line of LDS of its own, the addresses of a run of 64
  // 16-key tiles (32 steps), worked out by one lane each from one vector load a run; a step reads its two from there.
  // (Fetched step by step the page ids would be scalar loads, and the waits for LDS data wait for outstanding scalar
  // loads as well: a round trip to memory every step.) A tile past the request's keys, or on a page that a window
  // has passed and given back (-1 in the table), reads page 0, which is always mapped; its scores are masked below,
  // and so are its values.
  struct TileAddress { const bf16* keys; const bf16* values; };      // of slot 0 of kv head 0, element 0
  __shared__ __attribute__((aligned(16))) TileAddress run_tiles[TW][64];
  int run_first = s_begin;
  auto load_run = [&](int s0) {
    const int key0 = k_lo + (2 * s0 + lane) * 16;
    const int pg = bt[key0 < k_hi ? (PS16 ? key0 >> 4 : key0 / page_size) : 0];
    const bf16* page = plane + (long)(key0 < k_hi && pg >= 0 ? pg : 0) * page_stride;
    const int slot0 = PS16 ? 0 : key0 % page_size;
    run_tiles[wave][lane] = TileAddress{page + (long)slot0 * HD, page + slot0};
    run_first = s0;
  };

  // A lane's pieces of a step as offsets from those addresses: they never change. With a head size in steps of 32
  // all pieces of a fetch lie in the same 16-key tile, and the address is scalar.
  constexpr bool T_UNIFORM = HD % 32 == 0;
  constexpr bool T_IS_J = 2 * HD == TW * 64;     // fetch j holds the pieces of tile j
  unsigned k_off[TPT], v_off[TPT];       // in elements; less than a page
  int piece_t[TPT];
#pragma unroll
  for (int j = 0; j < TPT; ++j) {
    const int c = tid + j * (TW * 64);                      // the piece's index in LDS
    const int t = c / (2 * HD);                             // keys and values alike
    piece_t[j] = T_IS_J ? j : T_UNIFORM ? __builtin_amdgcn_readfirstlane(t) : t;
    const int key_in_tile = (c & 3) | ((c & 4) << 1) | ((c & 8) >> 1);
    k_off[j] = (unsigned)k_head + key_in_tile * HD + ((c >> 4) % NCH) * 8;
    v_off[j] = (unsigned)v_head + (((c >> 5) % DB) * 16 + (c & 15)) * page_size + ((c >> 4) & 1) * 8;
  }

  // A step on its way from the pages to LDS buffer `buf`.
  auto stage = [&](int s, int buf) {
    if (s - run_first >= 32) load_run(s);
    const TileAddress* at = &run_tiles[wave][2 * (s - run_first)];
    const bf16 *kbase[2], *vbase[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (T_UNIFORM) {
        const uint64_t ka = (uint64_t)at[t].keys, va = (uint64_t)at[t].values;
        kbase[t] = (const bf16*)(((uint64_t)(unsigned)__builtin_amdgcn_readfirstlane((int)(ka >> 32)) << 32) |
                                 (unsigned)__builtin_amdgcn_readfirstlane((int)ka));
        vbase[t] = (const bf16*)(((uint64_t)(unsigned)__builtin_amdgcn_readfirstlane((int)(va >> 32)) << 32) |
                                 (unsigned)__builtin_amdgcn_readfirstlane((int)va));
      } else {
        kbase[t] = at[t].keys;
        vbase[t] = at[t].values;
      }
    }
#pragma unroll
    for (int j = 0; j < TPT; ++j) {
      if (TCH % (TW * 64) != 0 && wave * 64 + j * (TW * 64) >= TCH) break;
      if (T_UNIFORM) copy_to_lds(kbase[piece_t[j]], k_off[j] * 2, &k_lds[buf][(wave + j * TW) * 512]);
      else copy_to_lds(kbase[piece_t[j]] + k_off[j], &k_lds[buf][(wave + j * TW) * 512]);
    }
#pragma unroll
    for (int j = 0; j < TPT; ++j) {
      if (TCH % (TW * 64) != 0 && wave * 64 + j * (TW * 64) >= TCH) break;
      if (T_UNIFORM) copy_to_lds(vbase[piece_t[j]], v_off[j] * 2, &v_lds[buf][(wave + j * TW) * 512]);
      else copy_to_lds(vbase[piece_t[j]] + v_off[j], &v_lds[buf][(wave + j * TW) * 512]);
    }
  };
  // the copies this wave has issued are in LDS
  auto staged = [&]() { asm volatile("s_waitcnt vmcnt(0)" : : : "memory"); };

  // S^T of one step. Lane (c, h) supplies score row c (tile c >> 4, row c & 15 of it), elements kc*16 + h*8.. of the head.
  auto scores = [&](int buf, f32x16& st) {
    const bf16* kp = &k_lds[buf][(((c32 >> 4) * NCH + h) * 16 + (c32 & 15)) * 8];
#pragma unroll
    for (int i = 0; i < 16; ++i) st[i] = 0.f;
#pragma unroll
    for (int kc = 0; kc < KC; ++kc)
      st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(load8(kp + kc * 256), qb[kc], st, 0, 0, 0);
  };
  // a step's scores without the keys that the column may not see (steps outside `free` only); accumulator i of
  // lane (c, h) is key 16 (i >> 3) + 8h + (i & 7) of the step
  auto mask = [&](int s, f32x16& st) {
    asm volatile("; a step with masked keys");   // (keeps the compiler from doing this on every step, by selects)
    const int kb = k_lo + s * 32 + h * 8;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = kb + (i >> 3) * 16 + (i & 7);
      st[i] = (key <= col_pos && key >= col_lo) ? st[i] : -INFINITY;
    }
  };
  // The running maximum of a column follows its scores in jumps: it moves only when a score exceeds it by more than
  // 2^8, so that weights stay below 2^8 and, on most steps, nothing moves. Whether anything does is asked of every
  // lane's own scores first; only then are the maxima of a column's two lanes brought together, the sum and the
  // output so far scaled down (alpha is exactly 1 for a column that stays).
  auto follow_maximum = [&](const f32x16& st) {
    const float tmax = max3(max3(max3(st[0], st[1], st[2]), max3(st[3], st[4], st[5]), max3(st[6], st[7], st[8])),
                            max3(st[9], st[10], st[11]), max3(max3(st[12], st[13], st[14]), st[15], st[15]));
    if (__builtin_amdgcn_ballot_w64(tmax > over) == 0) return;
    const float top = pair_max(tmax) * scale_log2;
    const float m_new = top > m + 8.f ? top : m;
    const float alpha = __builtin_amdgcn_exp2f(m - m_new);
    m = m_new;
    over = (m_new + 8.f) * per_scale;
    l *= alpha;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
  };
  // the weights of a step's keys: P in bfloat16 as the second operand of V.P, one for each half of the keys, and their
  // sum in 32-bit
  auto weights = [&](const f32x16& st, bf16x8 (&pb)[2]) {
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float p = __builtin_amdgcn_exp2f(fmaf(st[i], scale_log2, -m));
      psum += p;
      pb[i >> 3][i & 7] = static_cast<__bf16>(p);
    }
    l += psum;
  };
  // O^T += V^T . P^T. Lane (c, h) supplies element dt*32 + c of the head, keys 8h.. of each half.
  auto values = [&](int buf, const bf16x8 (&pb)[2]) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const int db = 2 * dt + (c32 >> 4);
      const bool d_ok = (HD % 32 == 0) || db < DB;
      const bf16* vp = &v_lds[buf][(((d_ok ? db : 0) * 2 + h) * 16 + (c32 & 15)) * 8];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        bf16x8 va = load8(vp + half * DB * 256);
        if (!d_ok) va = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb[half], o[dt], 0, 0, 0);
      }
    }
  };
  // A step outside `inside` holds keys that no row of the tile may see (past its last position, before its first
  // window, past its last page). Their weights are zero, but their values are whatever an earlier owner of the page
  // left, possibly not even finite, and zero times that is no number. Such a step's values are therefore set to zero
  // in LDS, a turn before any wave multiplies by them: wave w takes the 8 keys w*8.. of the step, a lane a piece
  // (8 keys of one element of the head) at a time. The barrier that ends the turn publishes it.
  auto zero_unseen_values = [&](int s, int buf) {
    const int key0 = k_lo + s * 32 + wave * 8;
    if (key0 >= t_lo && key0 + 7 <= tp_last) return;
    for (int piece = lane; piece < 16 * DB; piece += 64) {
      bf16* vp = &v_lds[buf][((((wave >> 1) * DB + (piece >> 4)) * 2 + (wave & 1)) * 16 + (piece & 15)) * 8];
      bf16x8 v = load8(vp);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (key0 + e < t_lo || key0 + e > tp_last) v[e] = static_cast<__bf16>(0.f);
      *reinterpret_cast<bf16x8*>(vp) = v;
    }
  };
  auto mine = [&](int s) { return s >= mine_lo && s < mine_hi; };

  if (s_begin < s_end) {
    // Steps s_begin and s_begin + 1 go to LDS before the loop; turn s copies step s + 2, multiplies out the scores of
    // step s + 1 (into `ahead`) and finishes step s (from `now`). Buffer of step s: (s - s_begin) % TBUF.
    load_run(s_begin);
    stage(s_begin, 0);
    if (s_begin + 1 < s_end) stage(s_begin + 1, 1);
    staged();
    __syncthreads();
    if (s_begin < in_lo || s_begin >= in_hi) {     // the same for all waves
      zero_unseen_values(s_begin, 0);
      __syncthreads();
    }
    f32x16 st_even, st_odd;
    scores(0, st_even);
    if (s_begin < free_lo || s_begin >= free_hi) mask(s_begin, st_even);
    // The scores of the step ahead are multiplied out whether or not this wave will use them (a wave skips few
    // steps, and after the split's last step they are thrown away): so they are defined on every path, and the
    // compiler keeps them where they are instead of copying them about.
    auto turn = [&](int s, int buf, f32x16& now, f32x16& ahead) {
      const int buf1 = buf + 1 == TBUF ? 0 : buf + 1, buf2 = buf1 + 1 == TBUF ? 0 : buf1 + 1;
      if (s + 2 < s_end) stage(s + 2, buf2);
      bf16x8 pb[2];
      scores(buf1, ahead);
      follow_maximum(now);
      weights(now, pb);
      values(buf, pb);
      if (s + 1 < free_lo || s + 1 >= free_hi) mask(s + 1, ahead);
      if ((s + 1 < in_lo || s + 1 >= in_hi) && s + 1 < s_end) zero_unseen_values(s + 1, buf1);
      // everyone has read step s's buffer (the copy of step s + 3 overwrites it) and step s + 2 has arrived
      staged();
      __syncthreads();
      return buf1;
    };
    int buf = 0;                                   // of step s
    for (int s = s_begin; s < s_end; s += 2) {     // two turns a round: the scores change places without being moved
      buf = turn(s, buf, st_even, st_odd);
      if (s + 1 >= s_end) break;
      buf = turn(s + 1, buf, st_odd, st_even);
    }
  }

  // accumulator 4b + k of lane (c, h) and block dt is element dt*32 + 8b + 4h + k of the head
  const float lt = pair_sum(l);
  if (!col_ok) return;
  if (item_splits == 1) {
    const float inv = 1.f / lt;
    bf16* dst = out + (long)col_row * out_ld + (long)col_head * HD + h * 4;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        if (HD % 32 != 0 && dt * 32 + b * 8 >= HD) continue;
        bf16x4 w;
#pragma unroll
        for (int k = 0; k < 4; ++k) w[k] = static_cast<__bf16>(o[dt][b * 4 + k] * inv);
        *reinterpret_cast<bf16x4*>(dst + dt * 32 + b * 8) = w;
      }
  } else {
    const long slot = ((long)col_row * n_heads + col_head) * split_stride + split;
    float* dst = part_o + slot * HD + h * 4;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        if (HD % 32 != 0 && dt * 32 + b * 8 >= HD) continue;
        *reinterpret_cast<f32x4*>(dst + dt * 32 + b * 8) = (f32x4){o[dt][b * 4], o[dt][b * 4 + 1], o[dt][b * 4 + 2], o[dt][b * 4 + 3]};
      }
    if (h == 0) part_ml[slot] = make_float2(m == NO_MAX ? -INFINITY : m, lt);
  }
}

// out[row, head, :] = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s      (reference paged_attention_kernels.py:121-204)
// Four groups of 64 lanes take the splits in turn, a lane holding up to four outputs; the groups' sums meet in
// LDS and are added in a fixed order. All loads of a lane are independent, so they overlap.
static constexpr int MG = 4;             // split groups per workgroup
static constexpr int MD = (HD + 63) / 64;  // outputs per lane

__global__ __launch_bounds__(MG * 64) void attention_merge_kernel(const float* __restrict__ part_o,
                                                                  const float2* __restrict__ part_ml,
                                                                  bf16* __restrict__ out, long out_ld, int n_heads,
                                                                  int max_splits, const int* __restrict__ row_splits) {
  __shared__ float so[MG][MD][64];
  const long row = blockIdx.x;
  const int head = blockIdx.y;
  const int grp = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n_splits = row_splits ? row_splits[row] : max_splits;   // partial results of this row
  if (n_splits <= 1) return;                                        // its output is final already
  const long base = (row * n_heads + head) * max_splits;
  // every wave reads the splits' (maximum, sum) pairs with one split per lane, so that the reads go out together
  // and not one after the other; the weights stay on the lanes and are handed round by index
  float M = -INFINITY;
  for (int s0 = 0; s0 < n_splits; s0 += 64)
    if (s0 + lane < n_splits) M = fmaxf(M, part_ml[base + s0 + lane].x);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off, 64));
  float acc[MD];
#pragma unroll
  for (int j = 0; j < MD; ++j) acc[j] = 0.f;
  float L = 0.f;
  for (int s0 = 0; s0 < n_splits; s0 += 64) {
    const int cnt = min(64, n_splits - s0);
    // the group's partial outputs of this chunk are asked for before the weights are known: one round trip, not two
    float v[64 / MG][MD];
#pragma unroll
    for (int q = 0; q < 64 / MG; ++q) {
      const int i = grp + q * MG;
#pragma unroll
      for (int j = 0; j < MD; ++j) {
        const int d = j * 64 + lane;
        v[q][j] = (i < cnt && d < HD) ? part_o[(base + s0 + i) * HD + d] : 0.f;
      }
    }
    float w = 0.f;
    if (lane < cnt) {
      const float2 ml = part_ml[base + s0 + lane];
      if (ml.x != -INFINITY) {   // else: a split that held no key of this row; its partial output means nothing
        w = exp2f(ml.x - M);
        L += w * ml.y;
      }
    }
#pragma unroll
    for (int q = 0; q < 64 / MG; ++q) {
      const float wi = __shfl(w, min(grp + q * MG, 63), 64);
#pragma unroll
      for (int j = 0; j < MD; ++j)
        if (wi != 0.f) acc[j] += wi * v[q][j];
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) L += __shfl_xor(L, off, 64);
#pragma unroll
  for (int j = 0; j < MD; ++j) so[grp][j][lane] = acc[j];
  __syncthreads();
  if (grp != 0) return;
#pragma unroll
  for (int j = 0; j < MD; ++j) {
    const int d = j * 64 + lane;
    if (d >= HD) continue;
    float t = so[0][j][lane];
#pragma unroll
    for (int gq = 1; gq < MG; ++gq) t += so[gq][j][lane];
    out[row * out_ld + (long)head * HD + d] = static_cast<__bf16>(t / L);
  }
}

// The same merge for many rows (prompt portions): a workgroup takes four heads of a row, one a wave, and a row that
// was not split costs one load. With a workgroup per (row, head) the thousands of rows of a prompt would mean tens of
// thousands of workgroups; with a wave taking several heads in turn, each head's two round trips to memory follow
// the previous head's.
__global__ __launch_bounds__(MG * 64) void attention_merge_rows_kernel(const float* __restrict__ part_o,
                                                                       const float2* __restrict__ part_ml,
                                                                       bf16* __restrict__ out, long out_ld,
                                                                       int n_heads, int max_splits,
                                                                       const int* __restrict__ row_splits) {
  const long row = blockIdx.x;
  const int n_splits = row_splits ? row_splits[row] : max_splits;
  if (n_splits <= 1) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int head = blockIdx.y * MG + wave;
  if (head >= n_heads) return;
  const long base = (row * n_heads + head) * max_splits;
  float acc[MD];
#pragma unroll
  for (int j = 0; j < MD; ++j) acc[j] = 0.f;
  float M = -INFINITY, L = 0.f;
  for (int s0 = 0; s0 < n_splits; s0 += 64)
    if (s0 + lane < n_splits) M = fmaxf(M, part_ml[base + s0 + lane].x);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off, 64));
  for (int s0 = 0; s0 < n_splits; s0 += 64) {
    float w = 0.f;
    if (s0 + lane < n_splits) {
      const float2 ml = part_ml[base + s0 + lane];
      if (ml.x != -INFINITY) {
        w = exp2f(ml.x - M);
        L += w * ml.y;
      }
    }
    const int cnt = min(64, n_splits - s0);
    for (int i = 0; i < cnt; ++i) {
      const float wi = __shfl(w, i, 64);
#pragma unroll
      for (int j = 0; j < MD; ++j) {
        const int d = j * 64 + lane;
        if (d < HD && wi != 0.f) acc[j] += wi * part_o[(base + s0 + i) * HD + d];
      }
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) L += __shfl_xor(L, off, 64);
#pragma unroll
  for (int j = 0; j < MD; ++j) {
    const int d = j * 64 + lane;
    if (d < HD) out[row * out_ld + (long)head * HD + d] = static_cast<__bf16>(acc[j] / L);
  }
}

TIS_EXPORT int tis_attention_mfma_head_dim() { return HD; }
// columns (row, query head of a group) that one wave of a tile holds; a tile has four waves
TIS_EXPORT int tis_attention_mfma_tile_columns() { return TCOLS; }

// items: (first row, rows) pairs; the rows of an item are consecutive positions of one request and
// rows * group_size <= 16 * nb. Null: n_items single rows, item i being row i. tiles: (first row, rows) pairs for the
// workgroup kernel, rows <= 4 * (tis_attention_mfma_tile_columns() / group_size); items and tiles together hold every row once.
// n_splits / tile_splits: what the grid offers an item / a tile. part_o / part_ml: workspace where either exceeds
// one, [rows][heads][S][HD] floats and [rows][heads][S] float pairs, S the larger of the two. min_steps > 0: an item
// uses min(n_splits, its steps of 32 keys / min_steps) splits; a tile uses as many as keep each at most
// tile_max_steps long; row_splits [rows] receives each row's count.
// min_steps == -1: `items` holds n_items entries of four integers, one per wave and key/value head, planned on the
// host for single rows: (row, split + 65536 * splits of the row, position, block-table line), row < 0 for padding;
// n_splits is then the most splits any row may have (the partial results' stride).
// A second stream for the tile kernel where a step has tiles and items: the two kernels share no rows, one is bound
// by the matrix cores and LDS, the other by memory, and side by side they take less than one after the other. Set
// once per device by the owner of the streams (null: everything on the caller's stream). Both streams must have
// the default priority.
struct SideStream {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
};
static SideStream g_side[64];
static std::mutex g_side_mutex;      // set-up and launches may come from different threads

// The second stream of the current device, as it was last set (a copy: the caller does not hold the lock).
static SideStream side_of_current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return SideStream();
  std::lock_guard<std::mutex> lock(g_side_mutex);
  return g_side[dev];
}

// How many partial results a row and head may have: what both entry points size and lay out the workspace by.
static int split_stride(int n_items, int n_tiles, int n_splits, int tile_splits) {
  return std::max(n_items > 0 ? n_splits : 1, n_tiles > 0 ? tile_splits : 1);
}

TIS_EXPORT int tis_attention_mfma_side_stream(hipStream_t side) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return tis_fail("attention_mfma: no current device");
  std::lock_guard<std::mutex> lock(g_side_mutex);
  SideStream& st = g_side[dev];
  if (side && !st.fork) {
    if (hipEventCreateWithFlags(&st.fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&st.join, hipEventDisableTiming) != hipSuccess)
      return tis_fail("attention_mfma: no events for the second stream");
  }
  st.stream = side;
  return 0;
}

static int attention_launch(const void* q, long q_ld, const void* plane, const int* block_tables, int bt_ld,
                            const int* row_seq, const int* positions, const int* items, int n_items, int nb,
                            const int* tiles, int n_tiles, void* out, long out_ld, float* part_o,
                            float* part_ml, int rows, int n_heads, int n_kv_heads, int head_dim, int page_size,
                            int window, float scale, int n_splits, int min_steps, int tile_splits,
                            int tile_max_steps, int* row_splits, hipStream_t stream) {
  if ((n_items == 0 && n_tiles == 0) || rows == 0) return 0;
  if (n_items < 0 || n_tiles < 0 || (n_tiles > 0 && !tiles)) return tis_fail("attention_mfma: bad item counts %d, %d", n_items, n_tiles);
  if (head_dim != HD) return tis_fail("attention_mfma: built for head size %d, called with %d", HD, head_dim);
  if (n_heads < 1 || n_kv_heads < 1 || n_heads % n_kv_heads)
    return tis_fail("attention_mfma: %d query heads over %d key/value heads", n_heads, n_kv_heads);
  const int group = n_heads / n_kv_heads;
  if (n_items > 0) {
    if (nb != 1 && nb != 2 && nb != 4) return tis_fail("attention_mfma: %d column blocks; 1, 2 or 4 are built", nb);
    if (group > 16 * nb) return tis_fail("attention_mfma: a group of %d query heads does not fit %d columns", group, 16 * nb);
  } else {
    n_splits = 1;
  }
  if (n_tiles > 0 && group > TCOLS) return tis_fail("attention_mfma: a group of %d query heads does not fit a tile's wave", group);
  if (n_tiles > 0 && 4L * n_kv_heads * page_size * HD >= (1L << 31))
    return tis_fail("attention_mfma: a page of %d key/value heads x %d slots is too large for the tile kernel's 32-bit offsets", n_kv_heads, page_size);
  if (n_tiles == 0) tile_splits = 1;
  if (page_size < 16 || page_size % 16) return tis_fail("attention_mfma: page size %d is no multiple of 16", page_size);
  if (n_splits < 1 || n_splits > 65535 || tile_splits < 1 || tile_splits > 65535 || n_kv_heads > 65535)
    return tis_fail("attention_mfma: bad grid %d x %d (tiles: %d)", n_kv_heads, n_splits, tile_splits);
  const int stride = split_stride(n_items, n_tiles, n_splits, tile_splits);
  if (stride > 1 && (!part_o || !part_ml)) return tis_fail("attention_mfma: %d splits need a workspace", stride);
  if (min_steps < -1 || (min_steps == -1 && (!items || n_items < 1)))
    return tis_fail("attention_mfma: min_steps=%d; -1 goes with a planned list of single rows", min_steps);
  if (min_steps == -1 && ((uintptr_t)items % 16))
    return tis_fail("attention_mfma: a planned list's entries of four integers must be 16-byte aligned");
  if (min_steps != 0 && n_splits > 1 && !row_splits)
    return tis_fail("attention_mfma: splits chosen item by item (min_steps=%d) need the per-row count array", min_steps);
  if (n_tiles > 0 && tile_max_steps < 1) return tis_fail("attention_mfma: a tile's splits need a longest chain of at least one step");
  if (n_tiles > 0 && stride > 1 && (!row_splits || (n_items > 0 && min_steps == 0)))
    return tis_fail("attention_mfma: tiles beside split key ranges need the per-row count array, and items that take their splits by their own length");
  if (stride == 1 || (n_tiles == 0 && min_steps == 0)) row_splits = nullptr;
  if ((q_ld % 8) || (out_ld % 4) || ((uintptr_t)q % 16) || ((uintptr_t)out % 8) || ((uintptr_t)plane % 16))
    return tis_fail("attention_mfma: q, out and the cache plane must be 16-byte aligned with row strides in steps of 8");
  const float scale_log2 = scale * 1.4426950408889634f;
  int rc = 0;
  hipStream_t tile_stream = stream;
  SideStream side;
  bool forked = false;
  if (n_items > 0 && n_tiles > 0) {
    side = side_of_current_device();
    if (side.stream && side.stream != stream) {
      // the tiles wait for what came before this call, not for the items
      if (hipEventRecord(side.fork, stream) != hipSuccess) return tis_fail("attention_mfma: the second stream could not be joined to the first");
      if (hipStreamWaitEvent(side.stream, side.fork, 0) != hipSuccess) return tis_fail("attention_mfma: the second stream could not be joined to the first");
      forked = true;
      tile_stream = side.stream;
    }
  }
  // From here on the second stream hangs off the first: whatever happens, it is joined again before this function
  // returns, so that a stream capture never ends with a branch left open.
  // (the items first: their single waves spread over the chip and leave every compute unit room for a tile's
  // workgroup; tiles launched first fill the units' LDS and registers and the items wait for them to finish: 64 decoded
  // tokens beside a 2,048-token prompt 180 instead of 122 us)
  if (n_items > 0) {
    dim3 grid(n_items, n_kv_heads, min_steps < 0 ? 1 : n_splits);
#define LAUNCH(NBV, PSV)                                                                                              \
  attention_mfma_kernel<NBV, PSV><<<grid, 64, 0, stream>>>(                                                      \
      (const bf16*)q, q_ld, (const bf16*)plane, block_tables, bt_ld, row_seq, positions, (const int2*)items,     \
      (bf16*)out, out_ld, part_o, (float2*)part_ml, group, n_kv_heads, n_heads, page_size, window, scale_log2,   \
      n_splits, min_steps, stride, row_splits)
    if (page_size == 16) {
      if (nb == 1) LAUNCH(1, true);
      else if (nb == 2) LAUNCH(2, true);
      else LAUNCH(4, true);
    } else {
      if (nb == 1) LAUNCH(1, false);
      else if (nb == 2) LAUNCH(2, false);
      else LAUNCH(4, false);
    }
#undef LAUNCH
    rc = tis_launch_status("attention_mfma");
  }
  if (n_tiles > 0 && rc == 0) {
    dim3 grid(n_tiles, n_kv_heads, tile_splits);
#define LAUNCH(PSV)                                                                                                   \
  attention_tile_kernel<PSV><<<grid, TW * 64, 0, tile_stream>>>(                                                      \
      (const bf16*)q, q_ld, (const bf16*)plane, block_tables, bt_ld, row_seq, positions, (const int2*)tiles,     \
      (bf16*)out, out_ld, part_o, (float2*)part_ml, group, n_kv_heads, n_heads, page_size, window, scale_log2,   \
      tile_splits, tile_max_steps, stride, row_splits)
    if (page_size == 16) LAUNCH(true);
    else LAUNCH(false);
#undef LAUNCH
    rc = tis_launch_status("attention_tile");
  }
  if (forked && (hipEventRecord(side.join, side.stream) != hipSuccess ||
                 hipStreamWaitEvent(stream, side.join, 0) != hipSuccess))
    return tis_fail("attention_mfma: the first stream could not wait for the second");
  if (rc) return rc;
  if (stride > 1) {
    if ((long)rows * n_heads > 8192) {
      dim3 mgrid(rows, (n_heads + MG - 1) / MG);
      attention_merge_rows_kernel<<<mgrid, MG * 64, 0, stream>>>(part_o, (const float2*)part_ml, (bf16*)out, out_ld,
                                                                 n_heads, stride, row_splits);
    } else {
      dim3 mgrid(rows, n_heads);
      attention_merge_kernel<<<mgrid, MG * 64, 0, stream>>>(part_o, (const float2*)part_ml, (bf16*)out, out_ld,
                                                            n_heads, stride, row_splits);
    }
    rc = tis_launch_status("attention_merge");
  }
  return rc;
}

TIS_EXPORT int tis_attention_mfma(const void* q, long q_ld, const void* plane, const int* block_tables, int bt_ld,
                                  const int* row_seq, const int* positions, const int* items, int n_items, int nb,
                                  const int* tiles, int n_tiles, void* out, long out_ld, float* part_o,
                                  float* part_ml, int rows, int n_heads, int n_kv_heads, int head_dim, int page_size,
                                  int window, float scale, int n_splits, int min_steps, int tile_splits,
                                  int tile_max_steps, int* row_splits, hipStream_t stream) {
  return attention_launch(q, q_ld, plane, block_tables, bt_ld, row_seq, positions, items, n_items, nb, tiles, n_tiles,
                          out, out_ld, part_o, part_ml, rows, n_heads, n_kv_heads, head_dim, page_size, window, scale,
                          n_splits, min_steps, tile_splits, tile_max_steps, row_splits, stream);
}

// ---- the same without a workspace argument: partial results in memory that this library owns for good ----
//
// The array below is the workspace of tis_attention_mfma_static. Every GPU on which this library's code is loaded holds
// a copy of it, at an address of its own, until the process ends. In host code the array's name is only a handle for
// hipGetSymbolAddress: the device address is asked for once per device, with that device current, and kept; kernels,
// like those of tis_attention_mfma, get the address as an argument.
static __device__ __align__(256) float scratch[TIS_ATTENTION_STATIC_FLOATS];

static constexpr int kMaxDevices = 64;
static float* g_scratch_ptr[kMaxDevices];     // null until the device's first call
static std::mutex g_scratch_mutex;

static int scratch_of_current_device(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return tis_fail("attention_mfma_static: no current device: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return tis_fail("attention_mfma_static: device %d is beyond the %d this library keeps track of", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    float* ptr = nullptr;
    e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return tis_fail("attention_mfma_static: the workspace's address on device %d is not to be had: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

TIS_EXPORT long tis_attention_mfma_static_floats() { return TIS_ATTENTION_STATIC_FLOATS; }

TIS_EXPORT int tis_attention_mfma_static(const void* q, long q_ld, const void* plane, const int* block_tables, int bt_ld,
                                         const int* row_seq, const int* positions, const int* items, int n_items,
                                         int nb, const int* tiles, int n_tiles, void* out, long out_ld, int rows,
                                         int n_heads, int n_kv_heads, int head_dim, int page_size, int window,
                                         float scale, int n_splits, int min_steps, int tile_splits, int tile_max_steps,
                                         hipStream_t stream) {
  if ((n_items == 0 && n_tiles == 0) || rows == 0) return 0;
  if (rows < 0 || n_heads < 1 || n_splits < 1 || tile_splits < 1)
    return tis_fail("attention_mfma_static: bad sizes rows=%d heads=%d splits=%d, %d", rows, n_heads, n_splits, tile_splits);
  const int stride = split_stride(n_items, n_tiles, n_splits, tile_splits);
  float *part_o = nullptr, *part_ml = nullptr;
  int* row_splits = nullptr;
  if (stride > 1) {
    // [rows][heads][stride][HD] partial outputs, [rows][heads][stride] (maximum, sum) pairs, [rows] split counts.
    // Nothing of it has to start at zero: every slot that the merge reads has been written by this call before.
    const long o_floats = (long)rows * n_heads * stride * HD, ml_floats = (long)rows * n_heads * stride * 2;
    const long need = o_floats + ml_floats + rows;
    if (need > (long)TIS_ATTENTION_STATIC_FLOATS)
      return tis_fail("attention_mfma_static: %d rows x %d heads x %d splits need %ld floats of partial results; the "
                      "built-in workspace holds %ld (fewer splits or rows, or tis_attention_mfma with a workspace of "
                      "the caller's)", rows, n_heads, stride, need, (long)TIS_ATTENTION_STATIC_FLOATS);
    float* base = nullptr;
    if (scratch_of_current_device(&base)) return -1;
    part_o = base;
    part_ml = base + o_floats;
    row_splits = reinterpret_cast<int*>(base + o_floats + ml_floats);
  }
  return attention_launch(q, q_ld, plane, block_tables, bt_ld, row_seq, positions, items, n_items, nb, tiles, n_tiles,
                          out, out_ld, part_o, part_ml, rows, n_heads, n_kv_heads, head_dim, page_size, window, scale,
                          n_splits, min_steps, tile_splits, tile_max_steps, row_splits, stream);
}
