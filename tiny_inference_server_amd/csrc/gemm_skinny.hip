// C[M,N] = f(A[M,K]) . W[N,K]^T for few rows: the matrix product of decode steps, where the job is to stream W from
// HBM once, on v_mfma_f32_16x16x32_bf16 (gfx950). Two kernels. The first (below) takes up to 8 rows against a
// matrix of up to 2,048 rows: operands go straight from memory into registers and a workgroup owns only 8 output
// columns, so that a narrow matrix still gives a workgroup to every compute unit. The staged kernel (further down)
// takes everything else: operands pass through LDS by direct loads, in panels of 16 or 32 rows of X, one per
// blockIdx.y, each an independent product over the same weights (the panels of a column tile run side by side, so
// the weights come from HBM once and from the caches after that). That is right for a few panels; for many, every
// panel streams all of W again, which only a product tiled in both directions avoids: it still gives the right
// result, slowly. Measured on MI355X (microseconds, first kernel / staged): at 8 rows the 1536x1536 product 4.8 / 5.0
// and the 1536x4096 one 7.3 / 8.2, but 2304x1536 6.3 / 5.5, 8192x1536 8.2 / 7.2, the 147 MB output table 35.5 / 30.4;
// at 16 rows the staged kernel wins everywhere (8192x1536: 8.7 / 7.3, 1536x4096: 10.5 / 8.4).
//
// The first kernel:
// One workgroup owns 16 rows of W (16 output columns; 8 in the variant that is built, see R below) over the whole of
// K; its waves take the 32-wide steps of K in turn, so together they read each weight row in contiguous runs. W rows
// are the A operand straight from global memory (16 bytes per lane), the activations are the B operand straight
// from L2 (they are a few KB and every workgroup reads the same ones), so no LDS is used for operands. Partial sums
// of the waves are added through LDS in a fixed order: a row's result does not depend on M or on the other rows.
//
// Fused around the product, so that a layer needs fewer launches and no round trips for small tensors:
//   NORM      the reference's RMSNorm of the input rows (main_models_new.py:38-42): the activations are multiplied
//             by the gain on the way in, their squares are summed as they pass, and the row factor
//             sqrt(K) / (||x|| + eps) is applied to the 32-bit sums at the end (the factor is per row, so it
//             commutes with the product)
//   RESIDUAL  C += R
//   SWIGLU    W holds gate and up rows interleaved (gate_0, up_0, gate_1, ...): out[:, f] = silu(c[2f]) * c[2f+1]
//             (main_models_new.py:51), written [M, N/2]
//   ROPE      the q/k/v projection: rotary encoding of q and k by the row's position, q written out, k and v
//             written into the row's cache slot (main_models_new.py:75-80, block_table.py:6-28); see RopeArgs
// Output bfloat16 or float (the output table writes 32-bit logits).
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_gemm_skinny)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;


enum { EPI_NONE = 0, EPI_RESIDUAL = 1, EPI_SWIGLU = 2, EPI_ROPE = 3 };

// What the rotary epilogue needs beyond the product: the rows of W are [q heads | k heads | v heads], and inside
// every q and k head the rows are ordered so that the two members of a rotary pair are neighbours
// (pair j at rows 2j and 2j+1). The epilogue rotates each pair by the row's position, puts queries back in
// their natural order into `C` ([M, n_heads*head_dim]) and writes keys and values into the cache page of the
// row's slot: keys as [slot][head_dim], values transposed as [head_dim][slot].
struct RopeArgs {
  const int* positions;
  const int* write_slots;
  const float2* table;     // [position][pair] (cos, sin); null: no rotation
  bf16* plane;
  int n_heads, n_kv_heads, head_dim, page_size, interleaved, write_cache;
};

// GS_WAVES: waves per workgroup; U: steps of K whose loads a wave issues together before the first product.
// Eight waves of three or four steps measured best on MI355X for K of 1536 to 4096 (5.6 us for a 25 MB matrix,
// 23 us for the 147 MB output table: 80 % of the HBM peak); four waves where K is too short to feed eight. Batches
// of eight steps, or sixteen waves, so that all of a wave's loads are in flight at once, measured the same within
// noise (the gated product at 64 rows slower: fewer workgroups fit a compute unit).
//
// MB: blocks of 16 rows of X that share every weight tile a wave loads, and CT: column tiles of 16 a workgroup
// owns. One of each is built. With two row blocks a wave fetches its own pieces of twice the activations, 16 bytes a
// lane from 16 different rows, and that is what its time went to (down product, 12.6 MB: 7.3 us at 8 rows, 10.4 at
// 16, 14.7 at 32); with two column tiles the staged kernel is faster for the same shapes.
//
// R: with 16 output columns per workgroup a matrix of 1536 rows gives 96 workgroups, and a compute unit draws
// only about 24 GB/s, so the 160 idle units cost more than the product. For M <= 16/R rows a workgroup
// therefore owns only 16/R columns and fills the 16 rows of the matrix operand with R different 32-wide chunks of
// K for those columns; the activation operand holds the same R chunks side by side. Of the 16x16 result only
// the R diagonal blocks (chunk r of the weights against chunk r of the activations) mean anything; they are
// added up with the waves' partial sums. R times as many workgroups, each step covers 32 R of K.
template <int MB, bool NORM, int EPI, typename TO, int GS_WAVES, int U, int R, int CT>
__global__ __launch_bounds__(GS_WAVES * 64) void gemm_skinny_kernel(
    const bf16* __restrict__ X, long x_ld, const bf16* __restrict__ W, const float* __restrict__ gain, float eps,
    const bf16* __restrict__ R_in, long r_ld, TO* __restrict__ C, long c_ld, int M, int N, int K, RopeArgs rope) {
  static_assert(MB == 1 || R == 1, "several row blocks go with full column tiles only");
  static_assert(CT == 1 || (R == 1 && (EPI == EPI_NONE || EPI == EPI_SWIGLU)), "two column tiles: plain and gated products");
  constexpr int COLS = 16 / R;   // output columns of a workgroup, and the most rows of X a block takes
  constexpr int GH = 4 / R;      // lane groups of four result rows per chunk
  __shared__ float red[GS_WAVES][MB][CT][64][4];
  __shared__ float red_ss[GS_WAVES][MB][16];

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, c16 = lane & 15, g = lane >> 4;
  const int chunk = c16 / COLS, sub = c16 % COLS;   // the lane's chunk of a step; its weight row and its activation row
  const int n0 = blockIdx.x * COLS * CT;
  // the workgroup's panel of rows: everything below sees only these
  {
    const long m0 = (long)blockIdx.y * (MB * 16);
    X += m0 * x_ld;
    C += m0 * c_ld;
    if (EPI == EPI_RESIDUAL) R_in += m0 * r_ld;
    if (EPI == EPI_ROPE) {
      rope.positions += m0;
      if (rope.write_slots) rope.write_slots += m0;
    }
    M = min(M - (int)m0, MB * 16);
  }
  const int steps = (K + 32 * R - 1) / (32 * R);
  bool w_ok[CT];
  const bf16* wrow[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    w_ok[ct] = n0 + ct * 16 + sub < N;
    wrow[ct] = W + (long)(w_ok[ct] ? n0 + ct * 16 + sub : 0) * K + chunk * 32 + g * 8;
  }
  bool x_ok[MB];
  const bf16* xrow[MB];
  f32x4 acc[MB][CT];
  float ss[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    x_ok[mb] = mb * 16 + sub < M;
    xrow[mb] = X + (long)(x_ok[mb] ? mb * 16 + sub : 0) * x_ld + chunk * 32 + g * 8;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc[mb][ct] = (f32x4){0.f, 0.f, 0.f, 0.f};
    ss[mb] = 0.f;
  }

  // What the epilogue wants from memory (the residual; the row's position, rotary factors and cache slot) is asked
  // for here, by the lanes that will use it, so that its round trips run beside the weights' and not after them.
  // Result lane (g, c16) of wave 0: columns n_out .. n_out + 3 of the rows mb * 16 + c16.
  const bool out_lane = wave == 0 && g < GH && c16 < COLS;
  const int n_out = n0 + g * 4;
  float res[MB][4];
  float2 cs[MB][2];
  int slot[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = mb * 16 + c16;
#pragma unroll
    for (int i = 0; i < 4; ++i) res[mb][i] = 0.f;
    cs[mb][0] = cs[mb][1] = make_float2(1.f, 0.f);
    slot[mb] = 0;
    if (!out_lane || m >= M) continue;
    if (EPI == EPI_RESIDUAL) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n_out + i < N) res[mb][i] = static_cast<float>(R_in[(long)m * r_ld + n_out + i]);
    }
    if (EPI == EPI_ROPE && n_out < N) {
      const int hd = rope.head_dim;
      const int head = n_out / hd, e0 = n_out % hd;
      if (head < rope.n_heads + rope.n_kv_heads && rope.table) {
        const long at = (long)rope.positions[m] * (hd / 2) + e0 / 2;
        cs[mb][0] = rope.table[at];
        cs[mb][1] = rope.table[at + 1];
      }
      if (head >= rope.n_heads && rope.write_cache) slot[mb] = rope.write_slots[m];
    }
  }

  // U steps at a time: all their loads are issued before the first product, so that a wave keeps several
  // rows' worth of HBM requests in flight
  for (int s0 = wave; s0 < steps; s0 += U * GS_WAVES) {
    bf16x8 a[U][CT];
    bf16x8 b[U][MB];
    float gv[U][8];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * GS_WAVES;
      const int k = s * (32 * R) + chunk * 32 + g * 8;
      const bool k_ok = s < steps && k < K;   // K is a multiple of 8, so a lane's 8 values are all inside or all outside
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        a[u][ct] = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
        if (w_ok[ct] && k_ok) a[u][ct] = *reinterpret_cast<const bf16x8*>(wrow[ct] + (long)s * (32 * R));
      }
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        b[u][mb] = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
        if (x_ok[mb] && k_ok) b[u][mb] = *reinterpret_cast<const bf16x8*>(xrow[mb] + (long)s * (32 * R));
      }
      if (NORM) {
        const float4 g0 = k_ok ? *reinterpret_cast<const float4*>(gain + k) : make_float4(0.f, 0.f, 0.f, 0.f);
        const float4 g1 = k_ok ? *reinterpret_cast<const float4*>(gain + k + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        gv[u][0] = g0.x; gv[u][1] = g0.y; gv[u][2] = g0.z; gv[u][3] = g0.w;
        gv[u][4] = g1.x; gv[u][5] = g1.y; gv[u][6] = g1.z; gv[u][7] = g1.w;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        bf16x8 bv = b[u][mb];
        if (NORM) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float xf = static_cast<float>(bv[e]);
            ss[mb] += xf * xf;
            bv[e] = static_cast<__bf16>(xf * gv[u][e]);
          }
        }
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
          acc[mb][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][ct], bv, acc[mb][ct], 0, 0, 0);
      }
    }
  }

  // add the partial sums of the waves and of the chunks in a fixed order
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][mb][ct][lane][i] = acc[mb][ct][i];
    if (NORM) {
      float t = ss[mb];
      t += __shfl_xor(t, 16, 64);
      t += __shfl_xor(t, 32, 64);
      if (g == 0) red_ss[wave][mb][c16] = t;
    }
  }
  __syncthreads();
  if (wave != 0) return;
  // result lane (gh, c): columns n0 + 4 gh + i of the rows mb * 16 + c; chunk r's share sits with lane (r GH + gh, r COLS + c)
  const int gh = lane >> 4, c = lane & 15;
  if (gh >= GH || c >= COLS) return;
#pragma unroll
  for (int mbct = 0; mbct < MB * CT; ++mbct) {
    const int mb = mbct / CT, ct = mbct % CT;
    const int n = n0 + ct * 16 + gh * 4;   // the lane's four consecutive output columns
    const int m = mb * 16 + c;
    if (m >= M) continue;
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float t = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int src = (r * GH + gh) * 16 + r * COLS + c;
#pragma unroll
        for (int w = 0; w < GS_WAVES; ++w) t += red[w][mb][ct][src][i];
      }
      v[i] = t;
    }
    if (NORM) {
      float t = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int w = 0; w < GS_WAVES; ++w) t += red_ss[w][mb][r * COLS + c];
      }
      const float mul = sqrtf((float)K) / (sqrtf(t) + eps);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] *= mul;
    }
    if (EPI == EPI_ROPE) {
      if (n >= N) continue;          // N is a multiple of head_dim, head_dim of 4: the lane's columns are all in or out
      const int hd = rope.head_dim, half = hd / 2;
      const int head = n / hd, e0 = n % hd;      // e0 is a multiple of 4: two whole pairs
      const bool is_q = head < rope.n_heads, is_v = head >= rope.n_heads + rope.n_kv_heads;
      float y[4] = {v[0], v[1], v[2], v[3]};
      int d[4];                                   // where the lane's four values belong inside the head
      if (is_v) {
#pragma unroll
        for (int i = 0; i < 4; ++i) d[i] = e0 + i;
      } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int pair = e0 / 2 + j;
          d[2 * j] = rope.interleaved ? 2 * pair : pair;
          d[2 * j + 1] = rope.interleaved ? 2 * pair + 1 : pair + half;
          if (rope.table) {
            const float x1 = v[2 * j], x2 = v[2 * j + 1];
            y[2 * j] = x1 * cs[mb][j].x - x2 * cs[mb][j].y;
            y[2 * j + 1] = x2 * cs[mb][j].x + x1 * cs[mb][j].y;
          }
        }
      }
      if (is_q) {
#pragma unroll
        for (int i = 0; i < 4; ++i) C[(long)m * c_ld + (long)head * hd + d[i]] = from_f<TO>(y[i]);
      } else if (rope.write_cache) {
        const int page = slot[mb] / rope.page_size, off = slot[mb] % rope.page_size;
        const int kvh = is_v ? head - rope.n_heads - rope.n_kv_heads : head - rope.n_heads;
        bf16* hp = rope.plane + (((long)page * 2 + (is_v ? 1 : 0)) * rope.n_kv_heads + kvh) * rope.page_size * hd;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (is_v) hp[(long)d[i] * rope.page_size + off] = static_cast<__bf16>(y[i]);
          else hp[(long)off * hd + d[i]] = static_cast<__bf16>(y[i]);
        }
      }
    } else if (EPI == EPI_SWIGLU) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (n + 2 * j + 1 < N) {
          const float gt = v[2 * j], up = v[2 * j + 1];
          C[(long)m * c_ld + n / 2 + j] = from_f<TO>(gt / (1.f + __expf(-gt)) * up);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (n + i < N) {
          float t = v[i];
          if (EPI == EPI_RESIDUAL) t += res[mb][i];
          C[(long)m * c_ld + n + i] = from_f<TO>(t);
        }
      }
    }
  }
}

// ---- the staged kernel: operands through LDS ----
//
// What a workgroup of the kernel above spends its time on, as soon as it has more than a few rows or columns, is
// the waiting for its own loads: every wave fetches its pieces of X, 16 bytes a lane from 16 different rows, and of
// W likewise, into registers it must hold until the products. Here a workgroup of eight waves
// owns CT * 16 columns and a panel of MB * 16 rows over the whole of K and walks K in chunks of 256: a chunk's
// weight rows and activation rows (512 bytes each) are copied into LDS by loads that write LDS directly
// (global_load_lds_dwordx4: no registers; a wave's load is two whole 512-byte runs), NSTAGE - 1 chunks ahead of the
// products, and wave w takes the w-th 32-wide step of the chunk for all CT * MB tiles, so the waves' partial sums are
// added at the end as above, in a fixed order. A row's 32 pieces of 16 bytes lie in LDS with their index XORed by
// the row's number in its tile, so that the 16 rows an operand fetch reads for one piece index fall into 16
// different bank groups; the copying lane picks the piece that belongs in its slot. With NORM the gains of a chunk
// are staged the same way (1 KB, by wave 0).
#pragma clang diagnostic ignored "-Winline-asm"   // M0 in a clobber list: meant
// One 16-byte piece per lane from global memory straight into LDS: lane i's piece lands at lds_base + 16 * i. In
// assembly, because the compiler would order every later LDS read behind such a load, whichever buffer it reads; so
// the compiler does not count these loads either, and whoever reads the pieces waits for them (vmcnt) and for the
// other waves (barrier).
__device__ __forceinline__ void copy16_to_lds(const void* src, const void* lds_base) {
  // (the base is the same on every lane: into a scalar register, whatever the compiler made of it so far)
  const unsigned base = (unsigned)__builtin_amdgcn_readfirstlane(
      (int)(unsigned)(uintptr_t)(const __attribute__((address_space(3))) unsigned char*)lds_base);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(base) : "memory", "m0");
}
template <int N_LATER>
__device__ __forceinline__ void wait_all_but() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N_LATER) : "memory");
}

template <int MB, int CT, bool NORM, int EPI, typename TO, int NSTAGE>
__global__ __launch_bounds__(512) void gemm_staged_kernel(
    const bf16* __restrict__ X, long x_ld, const bf16* __restrict__ W, const float* __restrict__ gain, float eps,
    const bf16* __restrict__ R_in, long r_ld, TO* __restrict__ C, long c_ld, int M, int N, int K, RopeArgs rope) {
  constexpr int WAVES = 8, KC = 256;
  constexpr int ROWS = 16 * (CT + MB);            // rows of a stage: the weight tiles' first, then the activations'
  constexpr int STAGE = ROWS * 512 + (NORM ? 1024 : 0);
  constexpr int L = CT + MB;                      // loads of a stage that every wave issues (wave 0: one more for the gains)
  constexpr int RED = WAVES * MB * CT * 1024 + WAVES * MB * 16 * 4;     // the waves' partial sums at the end
  constexpr int LDS_BYTES = NSTAGE * STAGE > RED ? NSTAGE * STAGE : RED;
  static_assert(LDS_BYTES <= 160 * 1024, "stages exceed the LDS of a compute unit");
  static_assert(L * (NSTAGE - 1) + NSTAGE <= 63, "more loads in flight than the counter counts");
  __shared__ __attribute__((aligned(1024))) unsigned char lds[LDS_BYTES];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, c16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (16 * CT);
  {
    const long m0 = (long)blockIdx.y * (MB * 16);
    X += m0 * x_ld;
    C += m0 * c_ld;
    if (EPI == EPI_RESIDUAL) R_in += m0 * r_ld;
    if (EPI == EPI_ROPE) {
      rope.positions += m0;
      if (rope.write_slots) rope.write_slots += m0;
    }
    M = min(M - (int)m0, MB * 16);
  }

  // What this wave copies of every chunk: L pairs of rows; lane l takes slot l & 31 of row 2 * pair + (l >> 5), which
  // holds the piece (slot ^ row's number in its tile) of the row's 512 bytes. Rows past the matrix read a row inside.
  const bf16* row_ptr[L];
  int piece_k[L];
#pragma unroll
  for (int i = 0; i < L; ++i) {
    const int row = 2 * (i * WAVES + wave) + (lane >> 5);
    piece_k[i] = ((lane & 31) ^ (row & 15)) * 8;
    if (row < 16 * CT) {
      const int n = n0 + row;
      row_ptr[i] = W + (long)(n < N ? n : N - 1) * K;
    } else {
      const int m = row - 16 * CT;
      row_ptr[i] = X + (long)(m < M ? m : 0) * x_ld;
    }
  }
  const int n_chunks = (K + KC - 1) / KC;
  auto issue = [&](int c) {
    unsigned char* st = lds + (c % NSTAGE) * STAGE;
    const int k0 = c * KC;
#pragma unroll
    for (int i = 0; i < L; ++i) {
      const int k = k0 + piece_k[i];
      copy16_to_lds(row_ptr[i] + (k < K ? k : 0), st + (i * WAVES + wave) * 1024);
    }
    if (NORM && wave == 0) {
      const int k = k0 + lane * 4;
      copy16_to_lds(gain + (k < K ? k : 0), st + ROWS * 512);
    }
  };

  // What the epilogue wants from memory, asked for before the main loop by the lanes that will use it. Tile t of the
  // MB x CT tiles is finished by wave t % 8; a result lane (g, c16) holds columns n_out .. n_out + 3 of row m_out.
  constexpr int TILES = MB * CT, TPW = (TILES + WAVES - 1) / WAVES;
  float res[TPW][4];
  float2 cs[TPW][2];
  int slot[TPW];
#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    const int t = j * WAVES + wave, mb = t / CT, ct = t % CT;
    const int m = mb * 16 + c16, n_out = n0 + ct * 16 + g * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) res[j][i] = 0.f;
    cs[j][0] = cs[j][1] = make_float2(1.f, 0.f);
    slot[j] = 0;
    if (t >= TILES || m >= M) continue;
    if (EPI == EPI_RESIDUAL) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n_out + i < N) res[j][i] = static_cast<float>(R_in[(long)m * r_ld + n_out + i]);
    }
    if (EPI == EPI_ROPE && n_out < N) {
      const int hd = rope.head_dim;
      const int head = n_out / hd, e0 = n_out % hd;
      if (head < rope.n_heads + rope.n_kv_heads && rope.table) {
        const long at = (long)rope.positions[m] * (hd / 2) + e0 / 2;
        cs[j][0] = rope.table[at];
        cs[j][1] = rope.table[at + 1];
      }
      if (head >= rope.n_heads && rope.write_cache) slot[j] = rope.write_slots[m];
    }
  }

  f32x4 acc[MB][CT];
  float ss[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    ss[mb] = 0.f;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc[mb][ct] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

#pragma unroll
  for (int c = 0; c < NSTAGE - 1; ++c)
    if (c < n_chunks) issue(c);
  const int piece = ((wave * 4 + g) ^ c16) * 16;      // where this lane's 16 bytes of a row lie in a stage
  for (int c = 0; c < n_chunks; ++c) {
    // this wave's copies of chunk c have landed: all but those of the chunks issued after it may be outstanding
    // (wave 0 has issued one more per chunk, so it waits a little longer than it must)
    const int later = min(n_chunks - 1 - c, NSTAGE - 2);
    if (later <= 0) wait_all_but<0>();
    else if (later == 1) wait_all_but<L>();
    else if (later == 2) wait_all_but<2 * L>();
    else wait_all_but<(NSTAGE - 2) * L>();
    // ... and everybody's: and every wave is done with chunk c - 1, whose stage the next copies overwrite
    __builtin_amdgcn_s_barrier();
    if (c + NSTAGE - 1 < n_chunks) issue(c + NSTAGE - 1);
    const unsigned char* st = lds + (c % NSTAGE) * STAGE;
    const bool k_ok = c * KC + wave * 32 + g * 8 < K;     // K is a multiple of 8: a lane's 8 values are all in or all out
    bf16x8 a[CT], b[MB];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) a[ct] = *reinterpret_cast<const bf16x8*>(st + (ct * 16 + c16) * 512 + piece);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) b[mb] = *reinterpret_cast<const bf16x8*>(st + ((CT + mb) * 16 + c16) * 512 + piece);
    float gv[8];
    if (NORM) {
      const float4 g0 = *reinterpret_cast<const float4*>(st + ROWS * 512 + wave * 128 + g * 32);
      const float4 g1 = *reinterpret_cast<const float4*>(st + ROWS * 512 + wave * 128 + g * 32 + 16);
      gv[0] = g0.x; gv[1] = g0.y; gv[2] = g0.z; gv[3] = g0.w;
      gv[4] = g1.x; gv[5] = g1.y; gv[6] = g1.z; gv[7] = g1.w;
    }
    if (!k_ok) {       // past the end of K (the last chunk): whatever was copied there counts as zero
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) a[ct] = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) b[mb] = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int e = 0; e < 8; ++e) gv[e] = 0.f;
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      bf16x8 bv = b[mb];
      if (NORM) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float xf = static_cast<float>(bv[e]);
          ss[mb] += xf * xf;
          bv[e] = static_cast<__bf16>(xf * gv[e]);
        }
      }
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
        acc[mb][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ct], bv, acc[mb][ct], 0, 0, 0);
    }
  }

  // the waves' partial sums, over the stages (every wave is done reading them)
  __builtin_amdgcn_s_barrier();
  float(*red)[MB][CT][64][4] = reinterpret_cast<float(*)[MB][CT][64][4]>(lds);
  float(*red_ss)[MB][16] = reinterpret_cast<float(*)[MB][16]>(lds + WAVES * MB * CT * 1024);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][mb][ct][lane][i] = acc[mb][ct][i];
    if (NORM) {
      float t = ss[mb];
      t += __shfl_xor(t, 16, 64);
      t += __shfl_xor(t, 32, 64);
      if (g == 0) red_ss[wave][mb][c16] = t;
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    const int t = j * WAVES + wave, mb = t / CT, ct = t % CT;
    if (t >= TILES) continue;
    const int n = n0 + ct * 16 + g * 4;      // the lane's four consecutive output columns
    const int m = mb * 16 + c16;
    if (m >= M) continue;
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) s += red[w][mb][ct][lane][i];
      v[i] = s;
    }
    if (NORM) {
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) s += red_ss[w][mb][c16];
      const float mul = sqrtf((float)K) / (sqrtf(s) + eps);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] *= mul;
    }
    if (EPI == EPI_ROPE) {
      if (n >= N) continue;
      const int hd = rope.head_dim, half = hd / 2;
      const int head = n / hd, e0 = n % hd;
      const bool is_q = head < rope.n_heads, is_v = head >= rope.n_heads + rope.n_kv_heads;
      float y[4] = {v[0], v[1], v[2], v[3]};
      int d[4];
      if (is_v) {
#pragma unroll
        for (int i = 0; i < 4; ++i) d[i] = e0 + i;
      } else {
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const int pair = e0 / 2 + jj;
          d[2 * jj] = rope.interleaved ? 2 * pair : pair;
          d[2 * jj + 1] = rope.interleaved ? 2 * pair + 1 : pair + half;
          if (rope.table) {
            const float x1 = v[2 * jj], x2 = v[2 * jj + 1];
            y[2 * jj] = x1 * cs[j][jj].x - x2 * cs[j][jj].y;
            y[2 * jj + 1] = x2 * cs[j][jj].x + x1 * cs[j][jj].y;
          }
        }
      }
      if (is_q) {
#pragma unroll
        for (int i = 0; i < 4; ++i) C[(long)m * c_ld + (long)head * hd + d[i]] = from_f<TO>(y[i]);
      } else if (rope.write_cache) {
        const int page = slot[j] / rope.page_size, off = slot[j] % rope.page_size;
        const int kvh = is_v ? head - rope.n_heads - rope.n_kv_heads : head - rope.n_heads;
        bf16* hp = rope.plane + (((long)page * 2 + (is_v ? 1 : 0)) * rope.n_kv_heads + kvh) * rope.page_size * hd;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (is_v) hp[(long)d[i] * rope.page_size + off] = static_cast<__bf16>(y[i]);
          else hp[(long)off * hd + d[i]] = static_cast<__bf16>(y[i]);
        }
      }
    } else if (EPI == EPI_SWIGLU) {
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        if (n + 2 * jj + 1 < N) {
          const float gt = v[2 * jj], up = v[2 * jj + 1];
          C[(long)m * c_ld + n / 2 + jj] = from_f<TO>(gt / (1.f + __expf(-gt)) * up);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (n + i < N) {
          float s = v[i];
          if (EPI == EPI_RESIDUAL) s += res[j][i];
          C[(long)m * c_ld + n + i] = from_f<TO>(s);
        }
      }
    }
  }
}

// (these can be set from outside: the kernel tests make small matrices take the wide path, and measurements compare
// panel heights)
static int g_wide_tiles = 256;   // from this many 32-column workgroups on (one a compute unit), a workgroup takes two column tiles
TIS_EXPORT void tis_gemm_skinny_wide_tiles(int n_workgroups) { g_wide_tiles = n_workgroups; }
static int g_staged_stages = 0;    // measurements: stages of LDS of the staged kernel, 2 or 4 (0: as chosen below)
static int g_staged_always = 0;    // measurements and tests: the staged kernel also where the first one would be chosen
TIS_EXPORT void tis_gemm_skinny_staged_always(int on) { g_staged_always = on; }
static int g_units = 256;          // compute units of the device: set by whoever knows (the default is an MI355X)
TIS_EXPORT void tis_gemm_skinny_staged_stages(int stages) { g_staged_stages = stages; }
TIS_EXPORT void tis_gemm_skinny_units(int n) { if (n > 0) g_units = n; }

template <bool NORM, int EPI, typename TO>
static int launch_staged(const void* X, long x_ld, const void* W, const float* gain, float eps, const void* R, long r_ld,
                         void* C, long c_ld, int M, int N, int K, hipStream_t stream, RopeArgs rope) {
  // Up to 16 rows one block of rows; beyond, panels of 32 rows: what a workgroup draws from L2 and HBM is what bounds it (about 50 GB/s), so small panels on
  // many workgroups beat panels of 64 rows wherever they were measured (64 rows, 0.9B widths, us, panels of 32 / of
  // 64: down 10.7 / 14.9, attention output 6.3 / 8.2, q/k/v 8.6 / 10.0, gate-up 11.2 / 11.7).
  const int mb = M <= 16 ? 1 : 2;
  const int panels = (M + mb * 16 - 1) / (mb * 16);
  if (panels > 65535) return tis_fail("gemm_skinny: %d rows are more panels than a grid holds", M);
  if (NORM && ((uintptr_t)gain % 16)) return tis_fail("gemm_skinny: the norm's gains must be 16-byte aligned");
  // two column tiles a workgroup where that still leaves a workgroup for every compute unit: the panel's activations,
  // which a workgroup copies in full, then serve twice as many weights
  int ct = 1;
  if constexpr (EPI == EPI_NONE || EPI == EPI_SWIGLU) {
    if ((long)((N + 31) / 32) * panels >= g_wide_tiles) ct = 2;
  }
  const dim3 grid((N + 16 * ct - 1) / (16 * ct), panels);
  // Stages of LDS: four (three chunks in flight) while every workgroup has a compute unit to itself; two, so that two
  // or three workgroups share a unit, once there are more workgroups than units (gate-up at 64 rows: 11.2 us with
  // two stages, 14.0 with four; down at 64 rows, 192 workgroups: 10.7 with four, 13.5 with two).
  int ns = (long)grid.x * grid.y > g_units ? 2 : 4;
  if (g_staged_stages) ns = g_staged_stages;
#define STAGED(MBV, CTV, NS)                                                                                      \
  if (mb == MBV && ct == CTV && ns == NS) {                                                                       \
    gemm_staged_kernel<MBV, CTV, NORM, EPI, TO, NS><<<grid, 512, 0, stream>>>(                                    \
        (const bf16*)X, x_ld, (const bf16*)W, gain, eps, (const bf16*)R, r_ld, (TO*)C, c_ld, M, N, K, rope);      \
    return 0;                                                                                                     \
  }
  STAGED(2, 1, 4) STAGED(2, 1, 2) STAGED(1, 1, 4) STAGED(1, 1, 2)
  if constexpr (EPI == EPI_NONE || EPI == EPI_SWIGLU) { STAGED(2, 2, 4) STAGED(2, 2, 2) STAGED(1, 2, 4) STAGED(1, 2, 2) }
#undef STAGED
  return tis_fail("gemm_skinny: no staged kernel for %d column tiles and %d stages", ct, ns);
}

template <bool NORM, int EPI, typename TO>
static int launch(const void* X, long x_ld, const void* W, const float* gain, float eps, const void* R, long r_ld,
                  void* C, long c_ld, int M, int N, int K, hipStream_t stream, RopeArgs rope = RopeArgs()) {
  // Which kernel. Up to 8 rows of a matrix of at most 2,048 rows (the attention output and down products) the first
  // kernel, with 8 columns a workgroup: twice the workgroups of 16-column tiles, where those would leave more than
  // half of the 256 compute units idle (N = 1536: 6.2 instead of 8.2 us for K = 4096, 4.1 instead of 4.8 for K = 1536;
  // the staged kernel there: 8.2 and 5.0). Everything else the staged kernel, which from 9 rows on, and for wider
  // matrices at any row count, is the faster one (0.9B widths, 8 rows, us, first / staged: gate-up 8.2 / 7.2, q/k/v
  // 6.3 / 5.5, output table 35.5 / 30.4; 16 rows: gate-up 8.7 / 7.3, down 10.5 / 8.4, q/k/v 6.7 / 5.5).
  const bool narrow = M <= 8 && (N + 15) / 16 <= 128 && !g_staged_always;
  if (!narrow) return launch_staged<NORM, EPI, TO>(X, x_ld, W, gain, eps, R, r_ld, C, c_ld, M, N, K, stream, rope);
  constexpr int r = 2;
  const int steps = (K + 32 * r - 1) / (32 * r);
  int waves, u;
  if (steps >= 24) {
    waves = 8;
    const int per_wave = (steps + 7) / 8;
    u = (per_wave % 3 == 0 && per_wave % 4 != 0) ? 3 : 4;
  } else {
    waves = 4;
    u = (steps % 3 == 0 && steps % 4 != 0) || steps == 12 ? 3 : 4;
  }
  const dim3 grid((N + 16 / r - 1) / (16 / r), 1);
#define CFG(WV, UV)                                                                                              \
  if (waves == WV && u == UV) {                                                                                  \
    gemm_skinny_kernel<1, NORM, EPI, TO, WV, UV, r, 1><<<grid, WV * 64, 0, stream>>>(                            \
        (const bf16*)X, x_ld, (const bf16*)W, gain, eps, (const bf16*)R, r_ld, (TO*)C, c_ld, M, N, K, rope);     \
    return 0;                                                                                                    \
  }
  CFG(4, 3) CFG(4, 4) CFG(8, 3) CFG(8, 4)
#undef CFG
  return tis_fail("gemm_skinny: no kernel for %d waves of %d steps", waves, u);
}

template <bool NORM, int EPI, typename TO>
static int launch_mb(const void* X, long x_ld, const void* W, const float* gain, float eps, const void* R, long r_ld,
                     void* C, long c_ld, int M, int N, int K, hipStream_t stream, RopeArgs rope = RopeArgs()) {
  if (launch<NORM, EPI, TO>(X, x_ld, W, gain, eps, R, r_ld, C, c_ld, M, N, K, stream, rope)) return -1;
  return tis_launch_status("gemm_skinny");
}

// epilogue: 0 none, 1 residual, 2 swiglu. out_dtype: 0 float, 1 bfloat16. gain == null: no norm.
TIS_EXPORT int tis_gemm_skinny(const void* X, long x_ld, const void* W, const float* gain, float eps, const void* R,
                               long r_ld, void* C, long c_ld, int M, int N, int K, int epilogue, int out_dtype,
                               hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (M < 0) return tis_fail("gemm_skinny: %d rows", M);
  if (N < 1 || K < 8 || K % 8) return tis_fail("gemm_skinny: N=%d K=%d; K must be a multiple of 8", N, K);
  if (x_ld % 8 || ((uintptr_t)X % 16) || ((uintptr_t)W % 16))
    return tis_fail("gemm_skinny: activations and weights must be 16-byte aligned with row strides in steps of 8");
  if (epilogue == EPI_RESIDUAL && !R) return tis_fail("gemm_skinny: residual epilogue without a residual");
  if (epilogue == EPI_SWIGLU && (N % 2)) return tis_fail("gemm_skinny: gate/up rows come in pairs, N=%d is odd", N);
  const bool norm = gain != nullptr;
#define GO(NORMV, EPIV, TOV) return launch_mb<NORMV, EPIV, TOV>(X, x_ld, W, gain, eps, R, r_ld, C, c_ld, M, N, K, stream)
  if (out_dtype == TIS_BF16) {
    if (epilogue == EPI_NONE) { if (norm) GO(true, EPI_NONE, bf16); else GO(false, EPI_NONE, bf16); }
    if (epilogue == EPI_RESIDUAL) { if (norm) GO(true, EPI_RESIDUAL, bf16); else GO(false, EPI_RESIDUAL, bf16); }
    if (epilogue == EPI_SWIGLU) { if (norm) GO(true, EPI_SWIGLU, bf16); else GO(false, EPI_SWIGLU, bf16); }
  } else if (out_dtype == TIS_F32) {
    if (epilogue == EPI_NONE) { if (norm) GO(true, EPI_NONE, float); else GO(false, EPI_NONE, float); }
  }
#undef GO
  return tis_fail("gemm_skinny: unsupported epilogue %d with output dtype %d", epilogue, out_dtype);
}

// The q/k/v projection of an attention layer with the rotary encoding and the cache write in its epilogue.
// W: [(n_heads + 2 n_kv_heads) * head_dim, K] with rotary pairs on neighbouring rows (see RopeArgs). Q out: [M, n_heads*head_dim].
TIS_EXPORT int tis_gemm_skinny_qkv_rope(const void* X, long x_ld, const void* W, const float* gain, float eps, void* Q,
                                        long q_ld, int M, int K, const int* positions, const int* write_slots,
                                        const float* table, void* plane, int n_heads, int n_kv_heads, int head_dim,
                                        int page_size, int interleaved, int write_cache, hipStream_t stream) {
  if (M == 0) return 0;
  if (M < 0) return tis_fail("gemm_skinny: %d rows", M);
  if (K < 8 || K % 8) return tis_fail("gemm_skinny: K=%d must be a multiple of 8", K);
  if (n_heads < 1 || n_kv_heads < 1 || head_dim < 4 || head_dim % 4 || page_size < 1)
    return tis_fail("gemm_skinny: heads=%d kv_heads=%d head_dim=%d (a multiple of 4) page=%d", n_heads, n_kv_heads,
                    head_dim, page_size);
  if (x_ld % 8 || ((uintptr_t)X % 16) || ((uintptr_t)W % 16))
    return tis_fail("gemm_skinny: activations and weights must be 16-byte aligned with row strides in steps of 8");
  RopeArgs rope;
  rope.positions = positions;
  rope.write_slots = write_slots;
  rope.table = (const float2*)table;
  rope.plane = (bf16*)plane;
  rope.n_heads = n_heads;
  rope.n_kv_heads = n_kv_heads;
  rope.head_dim = head_dim;
  rope.page_size = page_size;
  rope.interleaved = interleaved;
  rope.write_cache = write_cache;
  const int N = (n_heads + 2 * n_kv_heads) * head_dim;
  if (gain) return launch_mb<true, EPI_ROPE, bf16>(X, x_ld, W, gain, eps, nullptr, 0, Q, q_ld, M, N, K, stream, rope);
  return launch_mb<false, EPI_ROPE, bf16>(X, x_ld, W, gain, eps, nullptr, 0, Q, q_ld, M, N, K, stream, rope);
}
