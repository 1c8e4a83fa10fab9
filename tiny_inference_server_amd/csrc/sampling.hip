// Token sampling, one workgroup per row of logits, all in 32-bit.
//
// Order of operations as in the reference's batch_probs (server.py:22-50): repetition penalty on the
// tokens of the request's context (l > 0 ? l / pen : l * pen, each token once) -> divide by the
// temperature -> top-k -> top-p (keep a token while the probability mass of the strictly larger ones is
// <= top_p, so the token that crosses top_p stays) -> softmax over what is left -> draw.
// The reference sorts; here both cuts are thresholds over the bit pattern of the values (a radix select for
// top-k, then the few survivors are handled in LDS; a bisection for top-p without top-k), which keeps the
// same set whenever the values at the cut are distinct (ties at the top-k cut are all kept). The draw takes a uniform number per row from the caller (a stream per request, so a
// request's tokens do not depend on what else is in the batch) and inverts the cumulative distribution
// in token order. temperature == 0 or top_k == 1 is greedy: the arg-max, lowest index on ties.
//
// Two kernels with the same results. sample_regs_kernel keeps a row's values in registers (vocabularies up to
// 48 x 1024: more would spill registers) and finds the top-k cut by bisection over the key's bits with ballot counts: one pass over the logits
// and no atomics on a histogram whose few busy bins serialise the lanes (48,000 logits, k = 50: 0.02 instead of
// 0.17 ms a step). Rows it cannot finish that way (no top-k, or more than 1024 values at the cut) go on, in the same
// launch, through the general path that sample_kernel runs for every row: values in a work buffer in global memory.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_sampling)

static constexpr int SM_THREADS = 1024;

__device__ __forceinline__ unsigned order_key(float v) {
  unsigned u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// (value, index) arg-max over the block; lowest index wins ties. Result valid in every thread.
__device__ __forceinline__ void block_argmax(float& v, int& ix, float* sv, int* si) {
#pragma unroll
  for (int o = TIS_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, TIS_WAVE);
    const int oi = __shfl_xor(ix, o, TIS_WAVE);
    if (ov > v || (ov == v && oi < ix)) { v = ov; ix = oi; }
  }
  const int wave = threadIdx.x / TIS_WAVE, lane = threadIdx.x % TIS_WAVE;
  __syncthreads();
  if (lane == 0) { sv[wave] = v; si[wave] = ix; }
  __syncthreads();
  v = sv[0]; ix = si[0];
  for (int i = 1; i < SM_THREADS / TIS_WAVE; ++i)
    if (sv[i] > v || (sv[i] == v && si[i] < ix)) { v = sv[i]; ix = si[i]; }
}

struct SampleShared {
  float red[16];
  float sv[16];
  int si[16];
  float part[SM_THREADS];
  int found;
  int first_owner;
  unsigned hist[256];
  int sel_bin, sel_rem, n_cand;
  int icount[SM_THREADS];
  float cand_e[SM_THREADS];
  float cand_v[SM_THREADS];
  int cand_i[SM_THREADS];
  int counts[2][16];
};

// The n <= 1024 survivors of a top-k cut lie in sh.cand_{e,v,i}[0..n) in token order (e = exp(v - max)): top-p,
// then the draw. Every thread of the block calls it.
__device__ __forceinline__ void finish_survivors(SampleShared& sh, int n, float p_req, float u, int mi,
                                                 int* __restrict__ out_token, unsigned char* mark) {
  const int t = threadIdx.x;
  // top-p on the survivors: keep one while the mass of the strictly larger ones is <= top_p of the whole
  float zk = 0.f;
  for (int j = 0; j < n; ++j) zk += sh.cand_e[j];
  bool keep = t < n;
  if (keep && p_req > 0.f && p_req < 1.f) {
    float above = 0.f;
    for (int j = 0; j < n; ++j) above += sh.cand_v[j] > sh.cand_v[t] ? sh.cand_e[j] : 0.f;
    keep = above <= p_req * zk;
  }
  __syncthreads();
  if (t < n && !keep) sh.cand_e[t] = 0.f;
  __syncthreads();
  // inverse CDF in token order; every thread adds the same numbers in the same order, so the intervals
  // [before, before + e) of neighbours meet exactly
  float zz = 0.f, before = 0.f;
  for (int j = 0; j < n; ++j) {
    if (j == t) before = zz;
    zz += sh.cand_e[j];
  }
  const float target = u * zz;
  if (t == 0) sh.found = -1;
  __syncthreads();
  if (t < n && sh.cand_e[t] > 0.f && before <= target && target < before + sh.cand_e[t]) sh.found = sh.cand_i[t];
  __syncthreads();
  if (t == 0) {
    int pick = sh.found;
    if (pick < 0) {          // rounding left the target at the very end: the last survivor
      for (int j = n - 1; j >= 0 && pick < 0; --j)
        if (sh.cand_e[j] > 0.f) pick = sh.cand_i[j];
    }
    pick = pick >= 0 ? pick : mi;
    *out_token = pick;
    if (mark) mark[pick] = 1;
  }
}

// The general path: the row's values x[0..V) in global memory, everything with a key below `cut` already out.
// top-p by bisection, then the draw. Every thread of the block calls it.
__device__ __forceinline__ void finish_general(SampleShared& sh, const float* __restrict__ x, int V, unsigned cut,
                                               float mv, int mi, float p_req, float u, int* __restrict__ out_token,
                                               unsigned char* mark) {
  const int t = threadIdx.x;
  const int chunk = (V + SM_THREADS - 1) / SM_THREADS;
  const int lo = min(V, t * chunk), hi = min(V, lo + chunk);
  float z = 0.f;
  for (int i = t; i < V; i += SM_THREADS) {
    const float v = x[i];
    if (order_key(v) >= cut) z += expf(v - mv);
  }
  z = block_sum(z, sh.red);

  // top-p: the largest key whose mass at or above it exceeds top_p
  if (p_req > 0.f && p_req < 1.f) {
    unsigned pc = 0u;
    const float limit = p_req * z;
    for (int bit = 31; bit >= 0; --bit) {
      const unsigned cand = pc | (1u << bit);
      float mass = 0.f;
      for (int i = t; i < V; i += SM_THREADS) {
        const float v = x[i];
        const unsigned key = order_key(v);
        if (key >= cand && key >= cut) mass += expf(v - mv);
      }
      mass = block_sum(mass, sh.red);
      if (mass > limit) pc = cand;
    }
    if (pc > cut) {
      cut = pc;
      z = 0.f;
      for (int i = t; i < V; i += SM_THREADS) {
        const float v = x[i];
        if (order_key(v) >= cut) z += expf(v - mv);
      }
      z = block_sum(z, sh.red);
    }
  }

  // inverse CDF in token order: thread t owns the tokens [t*chunk, (t+1)*chunk)
  float mine = 0.f;
  for (int i = lo; i < hi; ++i) {
    const float v = x[i];
    if (order_key(v) >= cut) mine += expf(v - mv);
  }
  sh.part[t] = mine;
  if (t == 0) { sh.found = -1; sh.first_owner = SM_THREADS; }
  __syncthreads();
  if (t < TIS_WAVE) {
    // one wave scans the 1024 partial sums in order: 16 per lane, then across lanes
    float s = 0.f;
    for (int i = 0; i < SM_THREADS / TIS_WAVE; ++i) s += sh.part[t * (SM_THREADS / TIS_WAVE) + i];
    float incl = s;
#pragma unroll
    for (int o = 1; o < TIS_WAVE; o <<= 1) {
      const float up = __shfl_up(incl, o, TIS_WAVE);
      if (t >= o) incl += up;
    }
    float run = incl - s;
    for (int i = 0; i < SM_THREADS / TIS_WAVE; ++i) {
      const int ix = t * (SM_THREADS / TIS_WAVE) + i;
      const float v = sh.part[ix];
      sh.part[ix] = run;  // exclusive prefix
      run += v;
    }
  }
  __syncthreads();
  // the owner of the draw is the first thread whose running total passes the target; taking the minimum
  // over candidates keeps the choice well defined where rounding makes neighbouring intervals overlap
  const float target = u * z;
  const float before = sh.part[t];
  if (mine > 0.f && before + mine > target) atomicMin(&sh.first_owner, t);
  __syncthreads();
  if (t == sh.first_owner) {
    float run = before;
    int pick = -1;
    for (int i = lo; i < hi; ++i) {
      const float v = x[i];
      if (order_key(v) >= cut) {
        run += expf(v - mv);
        pick = i;
        if (run > target) break;
      }
    }
    sh.found = pick;
  }
  __syncthreads();
  if (t == 0) {
    const int pick = sh.found >= 0 ? sh.found : mi;  // rounding left the target past the last token: take the mode
    *out_token = pick;
    if (mark) mark[pick] = 1;
  }
}

__global__ __launch_bounds__(SM_THREADS) void sample_kernel(
    const float* __restrict__ logits, long ld, float* __restrict__ work, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ rep_penalty,
    const int* __restrict__ ctx_tokens, const int* __restrict__ ctx_offsets, const float* __restrict__ uniform,
    int* __restrict__ out_tokens, unsigned char* __restrict__ seen, long seen_ld, const int* __restrict__ seen_row) {
  __shared__ SampleShared sh;

  const long r = blockIdx.x;
  const int t = threadIdx.x;
  const float* lg = logits + r * ld;
  float* x = work + r * (long)V;
  const float temp = temperature[r];
  const int k_req = top_k[r];
  const float p_req = top_p[r];
  const float pen = rep_penalty ? rep_penalty[r] : 1.f;
  const bool greedy = (temp == 0.f) || (k_req == 1);
  const float inv_t = greedy ? 1.f : 1.f / temp;

  for (int i = t; i < V; i += SM_THREADS) x[i] = lg[i] * inv_t;
  __syncthreads();
  // The request's context comes either as a list of tokens or as a row of a table with one byte per token of
  // the vocabulary (nonzero: the token has occurred); the table's row also gets the token drawn here, so that a
  // server only ever uploads a request's context once.
  unsigned char* mark = (seen && seen_row && seen_row[r] >= 0) ? seen + (long)seen_row[r] * seen_ld : nullptr;
  if (pen != 1.f && mark) {
    for (int i = t; i < V; i += SM_THREADS) {
      if (mark[i]) {
        const float l = lg[i];
        x[i] = (l > 0.f ? l / pen : l * pen) * inv_t;
      }
    }
    __syncthreads();
  } else if (pen != 1.f && ctx_tokens) {
    // computed from the untouched logits, so a token that occurs twice is still penalised once
    for (int c = ctx_offsets[r] + t; c < ctx_offsets[r + 1]; c += SM_THREADS) {
      const int tok = ctx_tokens[c];
      if (tok >= 0 && tok < V) {
        const float l = lg[tok];
        x[tok] = (l > 0.f ? l / pen : l * pen) * inv_t;
      }
    }
    __syncthreads();
  }

  // maximum and its index
  float mv = -INFINITY;
  int mi = 0x7fffffff;
  for (int i = t; i < V; i += SM_THREADS) {
    const float v = x[i];
    if (v > mv) { mv = v; mi = i; }
  }
  block_argmax(mv, mi, sh.sv, sh.si);
  if (mi < 0 || mi >= V) mi = 0;  // only when every value is NaN
  if (greedy) {
    if (t == 0) {
      out_tokens[r] = mi;
      if (mark) mark[mi] = 1;
    }
    return;
  }

  // top-k: the k-th largest key by a radix select, eight bits a pass over a histogram of counts in LDS
  // (integer counts, so the result does not depend on the order in which threads arrive)
  unsigned cut = 0u;
  const bool has_k = k_req > 0 && k_req < V;
  if (has_k) {
    unsigned prefix = 0u;
    int remaining = k_req;
    for (int pass = 0; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      if (t < 256) sh.hist[t] = 0u;
      __syncthreads();
      for (int i = t; i < V; i += SM_THREADS) {
        const unsigned key = order_key(x[i]);
        if (pass == 0 || (key >> (shift + 8)) == (prefix >> (shift + 8))) atomicAdd(&sh.hist[(key >> shift) & 255u], 1u);
      }
      __syncthreads();
      if (t == 0) {
        int seen_n = 0, b = 255;
        for (; b > 0; --b) {
          if (seen_n + (int)sh.hist[b] >= remaining) break;
          seen_n += (int)sh.hist[b];
        }
        sh.sel_bin = b;
        sh.sel_rem = remaining - seen_n;
      }
      __syncthreads();
      prefix |= (unsigned)sh.sel_bin << shift;
      remaining = sh.sel_rem;
      __syncthreads();
    }
    cut = prefix;
  }

  // With a top-k cut the survivors are few: gather them, in token order, into LDS and finish there.
  const int chunk = (V + SM_THREADS - 1) / SM_THREADS;
  const int lo = min(V, t * chunk), hi = min(V, lo + chunk);
  if (has_k) {
    int mine_n = 0;
    for (int i = lo; i < hi; ++i) mine_n += order_key(x[i]) >= cut ? 1 : 0;
    // exclusive scan of the 1024 counts, in thread order: sixteen per lane of the first wave, then across its lanes
    sh.icount[t] = mine_n;
    __syncthreads();
    if (t < TIS_WAVE) {
      int s = 0;
      for (int i = 0; i < SM_THREADS / TIS_WAVE; ++i) s += sh.icount[t * (SM_THREADS / TIS_WAVE) + i];
      int incl = s;
#pragma unroll
      for (int o = 1; o < TIS_WAVE; o <<= 1) {
        const int up = __shfl_up(incl, o, TIS_WAVE);
        if (t >= o) incl += up;
      }
      int run = incl - s;
      for (int i = 0; i < SM_THREADS / TIS_WAVE; ++i) {
        const int ix = t * (SM_THREADS / TIS_WAVE) + i;
        const int v = sh.icount[ix];
        sh.icount[ix] = run;
        run += v;
      }
      if (t == TIS_WAVE - 1) sh.n_cand = run;
    }
    __syncthreads();
    const int n = sh.n_cand;
    if (n <= SM_THREADS) {     // more only when many values tie at the cut: then the general path below takes over
      int at = sh.icount[t];
      for (int i = lo; i < hi; ++i) {
        const float v = x[i];
        if (order_key(v) >= cut) {
          sh.cand_e[at] = expf(v - mv);
          sh.cand_v[at] = v;
          sh.cand_i[at] = i;
          ++at;
        }
      }
      __syncthreads();
      finish_survivors(sh, n, p_req, uniform[r], mi, out_tokens + r, mark);
      return;
    }
  }
  finish_general(sh, x, V, cut, mv, mi, p_req, uniform[r], out_tokens + r, mark);
}

__device__ __forceinline__ float key_value(unsigned key) {
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

// The same with the row in registers: thread t holds the keys of the tokens t, t + 1024, ... (REG of them).
template <int REG>
__global__ __launch_bounds__(SM_THREADS) void sample_regs_kernel(
    const float* __restrict__ logits, long ld, float* __restrict__ work, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ rep_penalty,
    const int* __restrict__ ctx_tokens, const int* __restrict__ ctx_offsets, const float* __restrict__ uniform,
    int* __restrict__ out_tokens, unsigned char* __restrict__ seen, long seen_ld, const int* __restrict__ seen_row) {
  __shared__ SampleShared sh;

  const long r = blockIdx.x;
  const int t = threadIdx.x;
  const float* lg = logits + r * ld;
  float* x = work + r * (long)V;
  const float temp = temperature[r];
  const int k_req = top_k[r];
  const float p_req = top_p[r];
  const float pen = rep_penalty ? rep_penalty[r] : 1.f;
  const bool greedy = (temp == 0.f) || (k_req == 1);
  const float inv_t = greedy ? 1.f : 1.f / temp;
  unsigned char* mark = (seen && seen_row && seen_row[r] >= 0) ? seen + (long)seen_row[r] * seen_ld : nullptr;

  // a penalty that comes as a token list is applied in the work buffer, as in the general kernel, and read back
  const bool by_list = pen != 1.f && !mark && ctx_tokens;
  bool in_work = false;
  if (by_list) {
    for (int i = t; i < V; i += SM_THREADS) x[i] = lg[i] * inv_t;
    __syncthreads();
    for (int c = ctx_offsets[r] + t; c < ctx_offsets[r + 1]; c += SM_THREADS) {
      const int tok = ctx_tokens[c];
      if (tok >= 0 && tok < V) {
        const float l = lg[tok];
        x[tok] = (l > 0.f ? l / pen : l * pen) * inv_t;
      }
    }
    __syncthreads();
    in_work = true;
  }

  // keys of the row's values (0 past the end of the row: below every cut that is ever tried), maximum and its index.
  // The values come in batches of CH: all of a batch's loads (logits, and the context's marks where a penalty is
  // on) are issued before any is used, so a batch costs one trip to memory and not one per value.
  constexpr int CH = REG % 16 == 0 ? 16 : 8;
  static_assert(REG % CH == 0, "values per thread come in whole batches");
  const bool by_mark = pen != 1.f && mark != nullptr;
  const float* src = by_list ? x : lg;
  unsigned key[REG];
  float mv = -INFINITY;
  int mi = 0x7fffffff;
#pragma unroll
  for (int c = 0; c < REG; c += CH) {
    float lv[CH];
    unsigned char mk[CH];
#pragma unroll
    for (int jj = 0; jj < CH; ++jj) {
      const int i = t + (c + jj) * SM_THREADS;
      lv[jj] = i < V ? src[i] : 0.f;
    }
#pragma unroll
    for (int jj = 0; jj < CH; ++jj) {
      const int i = t + (c + jj) * SM_THREADS;
      mk[jj] = (by_mark && i < V) ? mark[i] : (unsigned char)0;
    }
#pragma unroll
    for (int jj = 0; jj < CH; ++jj) {
      const int i = t + (c + jj) * SM_THREADS;
      const float l = lv[jj];
      float v = by_list ? l : l * inv_t;
      if (mk[jj]) v = (l > 0.f ? l / pen : l * pen) * inv_t;
      key[c + jj] = i < V ? order_key(v) : 0u;
      if (i < V && v > mv) { mv = v; mi = i; }
    }
  }
  block_argmax(mv, mi, sh.sv, sh.si);
  if (mi < 0 || mi >= V) mi = 0;  // only when every value is NaN
  if (greedy) {
    if (t == 0) {
      out_tokens[r] = mi;
      if (mark) mark[mi] = 1;
    }
    return;
  }

  unsigned cut = 0u;
  const bool has_k = k_req > 0 && k_req < V;
  if (has_k) {
    // The k-th largest key, bit by bit from the top: a bit stays set if at least k keys reach the candidate. Counts
    // are ballots added per wave, then over the sixteen waves through LDS (two buffers in turn: one barrier a bit).
    unsigned pc = 0u;
    int n_cut = V;
    const int wave = t / TIS_WAVE, lane = t % TIS_WAVE;
    const unsigned kmax = order_key(mv);      // no key of a number lies above it: such candidates need no count
    int turn = 0;                             // which of the two count buffers the next counted candidate uses
    for (int bit = 31; bit >= 0; --bit) {
      const unsigned cand = pc | (1u << bit);
      if (cand > kmax) continue;
      turn ^= 1;
      int c = 0;
#pragma unroll
      for (int j = 0; j < REG; ++j) {
        c += __popcll(__ballot(key[j] >= cand));
        if (j % 8 == 7) __builtin_amdgcn_sched_barrier(0);      // eight ballots in scalar registers at a time
      }
      if (lane == 0) sh.counts[turn][wave] = c;
      __syncthreads();
      int total = 0;
#pragma unroll
      for (int w = 0; w < SM_THREADS / TIS_WAVE; ++w) total += sh.counts[turn][w];
      if (total >= k_req) { pc = cand; n_cut = total; }
      if (total == k_req) break;        // exactly k keys reach the candidate: the same set as at the k-th key itself
    }
    cut = pc;
    __syncthreads();
    if (n_cut <= SM_THREADS) {
      // the survivors, in whatever order they arrive, then each to the place its token's rank gives it
      if (t == 0) sh.n_cand = 0;
      __syncthreads();
#pragma unroll
      for (int j = 0; j < REG; ++j) {
        const int i = t + j * SM_THREADS;
        if (i < V && key[j] >= cut) {
          const int at = atomicAdd(&sh.n_cand, 1);
          if (at < SM_THREADS) { sh.icount[at] = i; sh.part[at] = key_value(key[j]); }
        }
      }
      __syncthreads();
      const int n = min(sh.n_cand, SM_THREADS);
      int my_i = 0, rank = 0;
      float my_v = 0.f;
      if (t < n) {
        my_i = sh.icount[t];
        my_v = sh.part[t];
        for (int j = 0; j < n; ++j) rank += sh.icount[j] < my_i ? 1 : 0;
      }
      if (t < n) {
        sh.cand_e[rank] = expf(my_v - mv);
        sh.cand_v[rank] = my_v;
        sh.cand_i[rank] = my_i;
      }
      __syncthreads();
      finish_survivors(sh, n, p_req, uniform[r], mi, out_tokens + r, mark);
      return;
    }
  }
  if (!in_work) {
#pragma unroll
    for (int j = 0; j < REG; ++j) {
      const int i = t + j * SM_THREADS;
      if (i < V) x[i] = key_value(key[j]);
    }
    __syncthreads();
  }
  finish_general(sh, x, V, cut, mv, mi, p_req, uniform[r], out_tokens + r, mark);
}

// (tests switch the register kernel off to run the general one at every size)
static int g_sample_registers = 1;
TIS_EXPORT void tis_sample_use_registers(int on) { g_sample_registers = on; }

TIS_EXPORT int tis_sample(const float* logits, long ld, float* work, int rows, int V, const float* temperature,
                          const int* top_k, const float* top_p, const float* rep_penalty, const int* ctx_tokens,
                          const int* ctx_offsets, const float* uniform, int* out_tokens, unsigned char* seen,
                          long seen_ld, const int* seen_row, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || V < 1) return tis_fail("sample: bad size rows=%d vocab=%d", rows, V);
#define GO(KERNEL)                                                                                                \
  KERNEL<<<rows, SM_THREADS, 0, stream>>>(logits, ld, work, V, temperature, top_k, top_p, rep_penalty, ctx_tokens, \
                                          ctx_offsets, uniform, out_tokens, seen, seen_ld, seen_row)
  const int per_thread = (V + SM_THREADS - 1) / SM_THREADS;
  if (g_sample_registers && per_thread <= 8) GO(sample_regs_kernel<8>);
  else if (g_sample_registers && per_thread <= 24) GO(sample_regs_kernel<24>);
  else if (g_sample_registers && per_thread <= 48) GO(sample_regs_kernel<48>);
  else GO(sample_kernel);
#undef GO
  return tis_launch_status("sample");
}

__global__ __launch_bounds__(SM_THREADS) void argmax_kernel(const float* __restrict__ logits, long ld, int V,
                                                            int* __restrict__ out_tokens) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const long r = blockIdx.x;
  float mv = -INFINITY;
  int mi = 0x7fffffff;
  const float* row = logits + r * ld;
  if ((((uintptr_t)row) & 15) == 0) {
    // four values a load, two loads in flight; a thread meets its indices in rising order, so ">" keeps the lowest
    const int V4 = V & ~3;
    for (int i = threadIdx.x * 4; i < V4; i += 2 * SM_THREADS * 4) {
      const int j = i + SM_THREADS * 4;
      const float4 a = *reinterpret_cast<const float4*>(row + i);
      const float4 b = j < V4 ? *reinterpret_cast<const float4*>(row + j) : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
      const float va[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int at = (e < 4 ? i : j - 4) + e;
        if (va[e] > mv) { mv = va[e]; mi = at; }
      }
    }
    for (int i = V4 + threadIdx.x; i < V; i += SM_THREADS) {
      const float v = row[i];
      if (v > mv || (v == mv && i < mi)) { mv = v; mi = i; }
    }
  } else {
    for (int i = threadIdx.x; i < V; i += SM_THREADS) {
      const float v = row[i];
      if (v > mv) { mv = v; mi = i; }
    }
  }
  block_argmax(mv, mi, sv, si);
  if (threadIdx.x == 0) out_tokens[r] = (mi < 0 || mi >= V) ? 0 : mi;
}

TIS_EXPORT int tis_argmax(const float* logits, long ld, int rows, int V, int* out_tokens, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || V < 1) return tis_fail("argmax: bad size rows=%d vocab=%d", rows, V);
  argmax_kernel<<<rows, SM_THREADS, 0, stream>>>(logits, ld, V, out_tokens);
  return tis_launch_status("argmax");
}
