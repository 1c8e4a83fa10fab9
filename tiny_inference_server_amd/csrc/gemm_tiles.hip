// C[M,N] = X[M,K] . W[N,K]^T (+ R[M,N]) in bfloat16 for many rows at widths where the library's product is not used:
// a product tiled in both directions on v_mfma_f32_32x32x16_bf16 (gfx950), operands through LDS by direct loads.
// (The few-row kernel takes such a product in panels of 32 rows, each of which streams all of W again: 0.25 to 0.3
// PFLOP/s at 2,048 rows. This kernel reaches 0.45 to 0.95 on the same shapes; the library's kernels, where they may be
// used, 0.5 to 1.3.) The reference's engine uses a library product here (x @ W, main_models_new.py:19-20).
//
// A workgroup of four waves (2 x 2) owns a tile of 128 rows x 128 or 64 columns, or one of eight waves (2 x 4) a tile
// of 256 x 256 where that still gives every compute unit a workgroup, and walks K in steps of 64. A step's
// operand rows, 128 bytes each, are copied into LDS by global_load_lds_dwordx4 (no registers; eight lanes read one
// row's 128 bytes), one step ahead of the products, into one of two buffers; two workgroups share a compute unit and
// fill each other's waits. A row's eight 16-byte pieces lie in LDS with their index XORed by half the row's number:
// an operand fetch reads one piece index of 32 rows, LDS serves sixteen lanes at a time, and sixteen rows of 128
// bytes are eight such indices at each of two offsets in the 256 bytes that the banks span, so no two of them meet
// (XORed by the row's number itself, rows r and r + 8 did: half of the LDS's busy cycles were bank conflicts). The
// copying lane picks the piece that belongs in its slot. The result tile is computed transposed (W's rows are the first operand), so that a
// lane ends up with four consecutive columns of one row: 8-byte stores, and the residual read the same way.
// A row's sums run over K in the same order whatever M is: its result does not depend on the other rows.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_gemm_tiles)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

static constexpr int GT_BK = 64, GT_PIECES = GT_BK / 8;

// what lanes past the end of K read in the last step: zeros
static __device__ __attribute__((aligned(16))) unsigned char gt_zeros[16];

#pragma clang diagnostic ignored "-Winline-asm"   // M0 in a clobber list: meant
// One 16-byte piece per lane from global memory straight into LDS: lane i's piece lands at lds_addr + 16 * i. In
// assembly, because the compiler would order every later LDS read behind such a load, whichever buffer it reads; so
// the compiler does not count these loads either, and whoever reads the pieces waits for them (vmcnt) and for the
// other waves (barrier).
__device__ __forceinline__ void gt_copy16(const void* scalar_src, unsigned lane_bytes, unsigned lds_addr) {
  const uint64_t a = (uint64_t)scalar_src;
  const uint64_t sc = ((uint64_t)(unsigned)__builtin_amdgcn_readfirstlane((int)(a >> 32)) << 32) |
                      (unsigned)__builtin_amdgcn_readfirstlane((int)a);
  const unsigned base = (unsigned)__builtin_amdgcn_readfirstlane((int)lds_addr);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_bytes), "s"(sc), "s"(base) : "memory", "m0");
}
// the same with every lane's own address
__device__ __forceinline__ void gt_copy16(const void* lane_src, unsigned lds_addr) {
  const unsigned base = (unsigned)__builtin_amdgcn_readfirstlane((int)lds_addr);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(lane_src), "s"(base) : "memory", "m0");
}

// BM x BN: the workgroup's tile; WM x WN: its waves, each with (BM / WM) x (BN / WN) of it
template <int BM, int BN, int WM, int WN, bool RESIDUAL, typename TO>
__global__ __launch_bounds__(WM * WN * 64) void gemm_tiles_kernel(
    const bf16* __restrict__ X, long x_ld, const bf16* __restrict__ W, const bf16* R, long r_ld, TO* C, long c_ld,
    int M, int N, int K) {
  constexpr int BK = GT_BK, PCS = GT_PIECES, ROWS = BM + BN, GT_WAVES = WM * WN;
  constexpr int STAGE = ROWS * BK * 2;                  // bytes of a buffer: X's rows, then W's
  constexpr int LPW = ROWS * PCS / 64 / GT_WAVES;       // loads of a step that each wave issues, 8 rows each
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;   // 32 x 32 result tiles of a wave
  static_assert(ROWS * PCS % (64 * GT_WAVES) == 0 && TM >= 1 && TN >= 1 && 2 * STAGE <= 160 * 1024, "tile sizes");
  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * STAGE];
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, r32 = lane & 31, h = lane >> 5;
  const int wm = wave / WN, wn = wave % WN;
  const int tiles_m = (M + BM - 1) / BM;
  const long m0 = (long)(blockIdx.x % tiles_m) * BM, n0 = (long)(blockIdx.x / tiles_m) * BN;
  const unsigned lds0 = (unsigned)(uintptr_t)(const __attribute__((address_space(3))) unsigned char*)lds;

  // The wave's loads of a step: load j brings rows 8 (wave * LPW + j) .. +7 of the buffer, lane (row, slot) the piece
  // slot ^ ((row >> 1) & 7) of its row. Rows past the matrix's last are the last row again (their results are not
  // stored).
  const unsigned char* first_row[LPW];       // of the load's first row, at K offset 0 (the same on all lanes)
  unsigned lane_off[LPW];                    // the lane's piece from there, in bytes
  int lane_piece[LPW];                       // which 8 elements of a step's 64 the lane brings
#pragma unroll
  for (int j = 0; j < LPW; ++j) {
    const int row0 = (wave * LPW + j) * 8, row = row0 + (lane >> 3);
    lane_piece[j] = (lane & 7) ^ ((row >> 1) & 7);
    const bool of_x = row0 < BM;
    const long ld = of_x ? x_ld : (long)K;
    const long last = of_x ? (long)M - 1 : (long)N - 1;
    const long g_first = min(last, of_x ? m0 + row0 : n0 + (row0 - BM));
    const long g_row = min(last, of_x ? m0 + row : n0 + (row - BM));
    first_row[j] = (const unsigned char*)(of_x ? X : W) + g_first * ld * 2;
    lane_off[j] = (unsigned)((g_row - g_first) * ld * 2 + lane_piece[j] * 16);
  }
  auto stage = [&](int k0, int buf) {
#pragma unroll
    for (int j = 0; j < LPW; ++j)
      gt_copy16(first_row[j] + (long)k0 * 2, lane_off[j], lds0 + buf * STAGE + (wave * LPW + j) * 1024);
  };
  // the last step of a K that is no multiple of 64: pieces past the end come from a block of zeros
  auto stage_tail = [&](int k0, int buf) {
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
      const bool inside = k0 + lane_piece[j] * 8 < K;
      const unsigned char* src = inside ? first_row[j] + (long)k0 * 2 + lane_off[j] : gt_zeros;
      gt_copy16(src, lds0 + buf * STAGE + (wave * LPW + j) * 1024);
    }
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // operand pieces: row r of the buffer, elements 16 ks + 8 h .. of the step, at piece r * 8 + ((2 ks + h) ^ ((r >> 1) & 7))
  unsigned a_row[TM], b_row[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) a_row[i] = wm * (BM / WM) + i * 32 + r32;
#pragma unroll
  for (int j = 0; j < TN; ++j) b_row[j] = BM + wn * (BN / WN) + j * 32 + r32;

  const int nk = (K + BK - 1) / BK;
  const bool tail = K % BK != 0;
  if (tail && nk == 1) stage_tail(0, 0); else stage(0, 0);
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");      // this wave's pieces of step kt are in LDS
    __builtin_amdgcn_s_barrier();                             // ... and everyone's; everyone has read step kt - 1
    if (kt + 1 < nk) {
      if (tail && kt + 2 == nk) stage_tail((kt + 1) * BK, buf ^ 1);
      else stage((kt + 1) * BK, buf ^ 1);
    }
    const unsigned char* st = lds + buf * STAGE;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        a[i] = *(const bf16x8*)(st + (a_row[i] * PCS + ((2 * ks + h) ^ ((a_row[i] >> 1) & 7))) * 16);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        b[j] = *(const bf16x8*)(st + (b_row[j] * PCS + ((2 * ks + h) ^ ((b_row[j] >> 1) & 7))) * 16);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[j], a[i], acc[i][j], 0, 0, 0);
    }
  }

  // accumulator 4 q + e of block (i, j): row m0 + wm * (BM / WM) + i * 32 + r32, column n0 + wn * (BN / WN) + j * 32 + 8 q + 4 h + e
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const long m = m0 + wm * (BM / WM) + i * 32 + r32;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const long n = n0 + wn * (BN / WN) + j * 32 + q * 8 + h * 4;
        if (n >= N) continue;                 // (N is a multiple of 4: the four columns are inside or outside together)
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][q * 4 + e];
        if (RESIDUAL) {
          const bf16x4 r = *(const bf16x4*)(R + m * r_ld + n);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += (float)r[e];
        }
        if constexpr (sizeof(TO) == 4) {
          *(f32x4*)(C + m * c_ld + n) = (f32x4){v[0], v[1], v[2], v[3]};       // the 32-bit sums as they are
        } else {
          bf16x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = static_cast<__bf16>(v[e]);
          *(bf16x4*)(C + m * c_ld + n) = o;
        }
      }
  }
}

static int g_units = 256;      // compute units of the device: set by whoever knows (the default is an MI355X)
TIS_EXPORT void tis_gemm_tiles_units(int n) { if (n > 0) g_units = n; }

// W: [N, K] contiguous. R: null, or the residual (bfloat16) added to the product; it may be C itself (every element is
// read and then written by the same lane). out_f32: C holds 32-bit floats, the sums as they are (the output table's
// logits), and takes no residual. Sizes: K and x_ld multiples of 8, N, c_ld and r_ld multiples of 4; X and W 16-byte
// aligned, C and R 8-byte aligned (a 32-bit C 16-byte). Launches only: safe under stream capture.
TIS_EXPORT int tis_gemm_tiles(const void* X, long x_ld, const void* W, const void* R, long r_ld, void* C, long c_ld,
                              int M, int N, int K, int out_f32, hipStream_t stream) {
  if (M < 0 || N < 0 || K < 1) return tis_fail("gemm_tiles: bad size M=%d N=%d K=%d", M, N, K);
  if (M == 0 || N == 0) return 0;
  if (K % 8 || x_ld % 8 || x_ld < K) return tis_fail("gemm_tiles: K=%d and the input's row stride %ld must be multiples of 8", K, x_ld);
  if (N % 4 || c_ld % 4 || c_ld < N || (R && (r_ld % 4 || r_ld < N)))
    return tis_fail("gemm_tiles: N=%d and the row strides of the output (%ld) and residual (%ld) must be multiples of 4", N, c_ld, r_ld);
  if (((uintptr_t)X | (uintptr_t)W) % 16 || ((uintptr_t)C | (uintptr_t)R) % 8 || (out_f32 && (uintptr_t)C % 16))
    return tis_fail("gemm_tiles: inputs must be 16-byte aligned, output and residual 8-byte aligned (a 32-bit output 16-byte)");
  if (out_f32 && R) return tis_fail("gemm_tiles: a 32-bit result takes no residual");
  if ((long)x_ld * 16 >= (1L << 31) || (long)K * 16 >= (1L << 31)) return tis_fail("gemm_tiles: rows of %ld elements are too long for 32-bit offsets", x_ld);
  // The tile: 256 x 256 on eight waves where that gives every compute unit a workgroup (it moves half the bytes into
  // LDS per product that 128 x 128 does: 2,048 x 8,192 x 1,536 at 0.92 instead of 0.84 PFLOP/s); else 128 x 128 on
  // four; 128 x 64 where 128 x 128 would leave compute units without a workgroup.
  const long big = (long)((M + 255) / 256) * ((N + 255) / 256), mid = (long)((M + 127) / 128) * ((N + 127) / 128);
  const int bm = big >= g_units ? 256 : 128, bn = big >= g_units ? 256 : mid >= g_units ? 128 : 64;
  const long tiles = (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
  if (tiles >= (1L << 31)) return tis_fail("gemm_tiles: %ld tiles are more than a grid holds", tiles);
#define LAUNCH(BMV, BNV, WMV, WNV, RV, TOV)                                                                \
  gemm_tiles_kernel<BMV, BNV, WMV, WNV, RV, TOV><<<dim3((unsigned)tiles), WMV * WNV * 64, 0, stream>>>(    \
      (const bf16*)X, x_ld, (const bf16*)W, (const bf16*)R, r_ld, (TOV*)C, c_ld, M, N, K)
#define PICK(BMV, BNV, WMV, WNV)                                \
  {                                                             \
    if (out_f32) LAUNCH(BMV, BNV, WMV, WNV, false, float);      \
    else if (R) LAUNCH(BMV, BNV, WMV, WNV, true, bf16);         \
    else LAUNCH(BMV, BNV, WMV, WNV, false, bf16);               \
  }
  if (bm == 256) PICK(256, 256, 2, 4)
  else if (bn == 128) PICK(128, 128, 2, 2)
  else PICK(128, 64, 2, 2)
#undef PICK
#undef LAUNCH
  return tis_launch_status("gemm_tiles");
}
