// Choice of the next token from rows of logits: greedy, temperature with top-p, repetition penalty.
// Nothing is sorted.
#include "common.h"
#include "no_alloc.h"
#include <mutex>

#define ST 1024   // threads per row

// ---------------------------------------------------------------- greedy
// First maximum wins (/root/reference/src/engine/tq_generate.c:30-40).
__global__ __launch_bounds__(ST) void argmax_kernel(const float* __restrict__ logits, int V, int* __restrict__ out) {
  __shared__ float bv[ST];
  __shared__ int bi[ST];
  const float* row = logits + (size_t)blockIdx.x * V;
  float best = -INFINITY;
  int idx = 0x7fffffff;
  // indices ascend within a thread, so '>' keeps the thread's first maximum
  if (V % 4 == 0 && ((size_t)row & 15) == 0) {      // 16 bytes at a time, several loads on their way at once
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const f32x4* row4 = reinterpret_cast<const f32x4*>(row);
#pragma unroll 4
    for (int c = threadIdx.x; c < V / 4; c += ST) {
      const f32x4 v = row4[c];
      const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (idx == 0x7fffffff || e[j] > best) {
          best = e[j];
          idx = 4 * c + j;
        }
    }
  } else {
    for (int i = threadIdx.x; i < V; i += ST) {
      const float v = row[i];
      if (idx == 0x7fffffff || v > best) {
        best = v;
        idx = i;
      }
    }
  }
  bv[threadIdx.x] = best;
  bi[threadIdx.x] = idx;
  __syncthreads();
  for (int s = ST / 2; s > 0; s >>= 1) {
    if (threadIdx.x < s) {
      const float ov = bv[threadIdx.x + s];
      const int oi = bi[threadIdx.x + s];
      if (oi != 0x7fffffff && (bi[threadIdx.x] == 0x7fffffff || ov > bv[threadIdx.x] ||
                               (ov == bv[threadIdx.x] && oi < bi[threadIdx.x]))) {
        bv[threadIdx.x] = ov;
        bi[threadIdx.x] = oi;
      }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) out[blockIdx.x] = bi[0] == 0x7fffffff ? 0 : bi[0];
}

TQ_API int tq_argmax(const float* logits, int R, int V, int* out, hipStream_t st) {
  if (R <= 0) return 0;
  hipLaunchKernelGGL(argmax_kernel, dim3(R), dim3(ST), 0, st, logits, V, out);
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- negative log-likelihood of a given next token
// out[r] = -(logits[r][target[r]] - max_j logits[r][j] - log sum_j exp(logits[r][j] - max)), the sum in double as
// /root/reference/tools/quant.c:577-592 takes it (a target outside the vocabulary gives NaN: the caller leaves it out, :575).
// One workgroup per row; threads and then waves are added up in a fixed order.
__global__ __launch_bounds__(ST) void nll_kernel(const float* __restrict__ logits, int V, const int* __restrict__ target,
                                                 float* __restrict__ out) {
  __shared__ float red[ST / TQ_WAVE];
  __shared__ double dred[ST / TQ_WAVE];
  const float* row = logits + (size_t)blockIdx.x * V;
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < V; i += ST) mx = fmaxf(mx, row[i]);
  mx = block_max(mx, red);
  double sum = 0.0;
  for (int i = threadIdx.x; i < V; i += ST) sum += exp((double)(row[i] - mx));
#pragma unroll
  for (int o = TQ_WAVE / 2; o > 0; o >>= 1) sum += __shfl_xor(sum, o, TQ_WAVE);
  if (threadIdx.x % TQ_WAVE == 0) dred[threadIdx.x / TQ_WAVE] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    double total = 0.0;
    for (int w = 0; w < ST / TQ_WAVE; ++w) total += dred[w];
    const int t = target[blockIdx.x];
    out[blockIdx.x] = t < 0 || t >= V ? NAN : (float)(log(total) - (double)(row[t] - mx));
  }
}

TQ_API int tq_nll(const float* logits, int R, int V, const int* target, float* out, hipStream_t st) {
  if (R <= 0) return 0;
  hipLaunchKernelGGL(nll_kernel, dim3(R), dim3(ST), 0, st, logits, V, target, out);
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- a row's probabilities as 16-bit floats, and KL against such rows
// What the reference writes per scored position with --save-logits and compares with --kl-baseline
// (/root/reference/tools/quant.c:594-636): p[j] = exp((l[j] - max) - log sum exp(l - max)) in double, made a float and
// then a 16-bit float by its own conversion (:166-174: the mantissa cut, not rounded; below 2^-14 zero; no NaN).
// KL(baseline || current) = sum over j with pb > 1e-12 of pb (log pb - log max(pc, 1e-20)) in double, pb and pc being
// the 16-bit values widened again (:175-185).  One workgroup per row, sums over threads and waves in a fixed order.
__device__ __forceinline__ unsigned short half_cut(float v) {
  const uint32_t u = __float_as_uint(v);
  const uint32_t sign = (u >> 16) & 0x8000u;
  const int e = (int)((u >> 23) & 0xffu) - 127 + 15;
  if (e <= 0) return (unsigned short)sign;
  if (e >= 31) return (unsigned short)(sign | 0x7c00u);
  return (unsigned short)(sign | ((uint32_t)e << 10) | ((u >> 13) & 0x3ffu));
}
__device__ __forceinline__ float half_widen(unsigned short h) {
  const uint32_t sign = ((uint32_t)h & 0x8000u) << 16, e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
  if (e == 0) return __uint_as_float(sign);
  if (e == 31) return __uint_as_float(sign | 0x7f800000u | (m << 13));
  return __uint_as_float(sign | ((e - 15 + 127) << 23) | (m << 13));
}
__device__ __forceinline__ double block_sum_double(double v, double* dred) {
#pragma unroll
  for (int o = TQ_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, TQ_WAVE);
  __syncthreads();
  if (threadIdx.x % TQ_WAVE == 0) dred[threadIdx.x / TQ_WAVE] = v;
  __syncthreads();
  double total = 0.0;
  for (int w = 0; w < ST / TQ_WAVE; ++w) total += dred[w];
  return total;
}

// probs (null, or [R][V]): the row's probabilities; base (null, or [R][V]) with kl [R]: KL of base against them.
__global__ __launch_bounds__(ST) void probs_half_kernel(const float* __restrict__ logits, int V,
                                                        unsigned short* __restrict__ probs,
                                                        const unsigned short* __restrict__ base, double* __restrict__ kl) {
  __shared__ float red[ST / TQ_WAVE];
  __shared__ double dred[ST / TQ_WAVE];
  const float* row = logits + (size_t)blockIdx.x * V;
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < V; i += ST) mx = fmaxf(mx, row[i]);
  mx = block_max(mx, red);
  double sum = 0.0;
  for (int i = threadIdx.x; i < V; i += ST) sum += exp((double)(row[i] - mx));
  const double log_sum = log(block_sum_double(sum, dred));
  double part = 0.0;
  for (int i = threadIdx.x; i < V; i += ST) {
    const unsigned short h = half_cut((float)exp((double)(row[i] - mx) - log_sum));
    if (probs) probs[(size_t)blockIdx.x * V + i] = h;
    if (base) {
      const float pb = half_widen(base[(size_t)blockIdx.x * V + i]);
      float pc = half_widen(h);
      if (pb > 1e-12f) {
        if (pc < 1e-20f) pc = 1e-20f;
        part += (double)pb * (log((double)pb) - log((double)pc));
      }
    }
  }
  if (base) {
    const double total = block_sum_double(part, dred);
    if (threadIdx.x == 0) kl[blockIdx.x] = total;
  }
}

TQ_API int tq_probs_half(const float* logits, int R, int V, void* probs, const void* base, double* kl, hipStream_t st) {
  if (R <= 0) return 0;
  if ((!probs && !base) || (base && !kl)) return TQ_ERR_BAD_ARG;
  hipLaunchKernelGGL(probs_half_kernel, dim3(R), dim3(ST), 0, st, logits, V, (unsigned short*)probs,
                     (const unsigned short*)base, kl);
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- repetition penalty
// For each of the last `count` tokens of a row's history, once per occurrence: a positive logit is
// divided by the penalty, any other multiplied (/root/reference/src/engine/tq_generate.c:387-400).
// One workgroup per row, a thread per entry of the history: the thread that holds a token's first entry counts the
// token's entries and applies the penalty that many times, one after the other as the walk over the history would
// (the sign of a logit does not change on the way, so the order of the entries does not matter).
#define RP_MAX 128      // entries of history per row that the parallel kernel takes
__global__ __launch_bounds__(RP_MAX) void rep_penalty_kernel(float* __restrict__ logits, int V,
                                                             const int* __restrict__ recent, int window,
                                                             const int* __restrict__ counts, float penalty) {
  __shared__ int toks[RP_MAX];
  float* row = logits + (size_t)blockIdx.x * V;
  const int n = min(counts[blockIdx.x], window), r = threadIdx.x;
  const int tok = r < n ? recent[blockIdx.x * window + r] : -1;
  toks[r] = tok;
  __syncthreads();
  if (tok < 0 || tok >= V) return;
  int times = 0;
  for (int j = 0; j < n; ++j) {
    if (toks[j] == tok) {
      if (j < r) return;      // an earlier entry holds the token and does the work
      ++times;
    }
  }
  float v = row[tok];
  for (int t = 0; t < times; ++t) v = v > 0.f ? v / penalty : v * penalty;
  row[tok] = v;
}

// The same for longer histories: one thread walks the row's history.
__global__ void rep_penalty_walk_kernel(float* __restrict__ logits, int V, const int* __restrict__ recent, int window,
                                        const int* __restrict__ counts, float penalty) {
  if (threadIdx.x != 0) return;
  float* row = logits + (size_t)blockIdx.x * V;
  const int n = min(counts[blockIdx.x], window);
  for (int r = 0; r < n; ++r) {
    const int tok = recent[blockIdx.x * window + r];
    if (tok >= 0 && tok < V) row[tok] = row[tok] > 0.f ? row[tok] / penalty : row[tok] * penalty;
  }
}

TQ_API int tq_rep_penalty(float* logits, int R, int V, const int* recent, int window, const int* counts,
                          float penalty, hipStream_t st) {
  if (R <= 0) return 0;
  if (window <= RP_MAX)
    hipLaunchKernelGGL(rep_penalty_kernel, dim3(R), dim3(RP_MAX), 0, st, logits, V, recent, window, counts, penalty);
  else
    hipLaunchKernelGGL(rep_penalty_walk_kernel, dim3(R), dim3(64), 0, st, logits, V, recent, window, counts, penalty);
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- temperature + top-p
// The reference (/root/reference/src/engine/tq_generate.c:81-156) keeps the logits within 16*T of the
// maximum, turns them into probabilities p = exp((l - max) / T) / sum, sorts them in descending order,
// cuts the list where the running sum reaches top_p, draws r = u * (that sum) and walks the list until
// the running sum reaches r.  The same choice is made here without a sort: "the running sum reaches s
// at an element of probability tau" means  S(> tau) < s <= S(>= tau), where S(>= tau) is the sum of all
// probabilities >= tau; the largest tau with S(>= tau) >= s is found by a search over the bit patterns
// of positive floats, which are ordered like the floats.  Equal probabilities are taken in order of
// index.  Sums are taken in a fixed order, but not the order of a sorted walk, so a draw that lands
// within rounding of a boundary between two tokens may fall on either.
//
// One workgroup would have to go through a row of 150,000 probabilities some twenty times (about 40 us a time:
// one compute unit alone draws little from memory).  So a row is cut into SC contiguous chunks, one workgroup each,
// and every pass over the rows is a launch: a workgroup first adds up what the chunks of its row left in the pass
// before (in chunk order, every workgroup of the row the same arithmetic) and so knows where the search stands,
// then goes through its own chunk and leaves its partial results for the next pass.  Nothing is sorted and no sum
// depends on timing.
#define SC 32            // chunks per row
#define SB 256           // threads per chunk
#define NB 8             // loads that a thread has on their way at once
#define KW 16            // candidate thresholds per pass of a search
// A pass with KW candidates leaves at most span / (KW + 1) + 1 of a span of bit patterns, and a span of KW or less
// is settled by one pass.  The probabilities that are not 0 lie within 2^-24 of the largest (exp(-16) > 2^-24), which
// is fewer than 2^28 patterns: 2^28 -> 1.6e7 -> 9.3e5 -> 5.5e4 -> 3.2e3 -> 190 -> 13 -> settled.  Only the first
// two or three passes compare every value with every candidate: later the bounds are so close that few values
// lie between them.
#define SEARCH_PASSES 7
#define PW (KW + 2)      // floats a chunk leaves per pass

// stages, in launch order
enum { ST_MAX = 0, ST_EXP, ST_NORM, ST_SEARCH_P, ST_SUMS_P = ST_SEARCH_P + SEARCH_PASSES, ST_SEARCH_R,
       ST_SUMS_R = ST_SEARCH_R + SEARCH_PASSES, ST_PICK, ST_COUNT };

struct RowState {        // what earlier passes have settled for a row; a pass reads the one that the pass before
                         // wrote and writes its own (the row's chunk 0 does), so no chunk sees it half-way
  float mx, inv_s, pmax, all;
  uint32_t lo_b, hi_b;   // bounds of the running search, as bit patterns of positive floats
  float target;          // what S(>= tau) has to reach in the running search; <= 0: no search
  float tau_p, cumulative, tau_r;
  int nth;
};

// Sum over the workgroup in a fixed order (butterfly in the wave, waves in order); every thread gets it.
__device__ __forceinline__ float chunk_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if (threadIdx.x % TQ_WAVE == 0) red[threadIdx.x / TQ_WAVE] = v;
  __syncthreads();
  float t = 0.f;
  for (int w = 0; w < SB / TQ_WAVE; ++w) t += red[w];
  return t;
}

__device__ __forceinline__ float chunk_max(float v, float* red) {
  v = wave_max(v);
  __syncthreads();
  if (threadIdx.x % TQ_WAVE == 0) red[threadIdx.x / TQ_WAVE] = v;
  __syncthreads();
  float t = red[0];
  for (int w = 1; w < SB / TQ_WAVE; ++w) t = fmaxf(t, red[w]);
  return t;
}

// The candidates of a search pass: ascending in (lo, hi]; with KW patterns or fewer left every one of them, the
// last repeated.
__device__ __forceinline__ float candidate(uint32_t lo_b, uint32_t hi_b, int j) {
  const uint32_t span = hi_b - lo_b;
  const uint32_t step = span <= KW ? (uint32_t)min(j + 1, (int)span) : (uint32_t)(((uint64_t)span * (j + 1)) / (KW + 1));
  return __uint_as_float(lo_b + step);
}

typedef float f32x4 __attribute__((ext_vector_type(4)));

// A thread fetches NB units of VEC floats at a time, all asked for before any is used.  Where unit u starts,
// counted from `first`: with OWN_RUN a thread's units follow one another, else the threads' units interleave (a
// wave's loads take whole lines).
template <int VEC, bool OWN_RUN>
__device__ __forceinline__ int unit_start(int first, int u) {
  return first + (OWN_RUN ? (int)threadIdx.x * NB + u : u * SB + (int)threadIdx.x) * VEC;
}
// What lies at or beyond `end` reads as `pad`.  (With VEC 4, first and end are multiples of 4 and the row is aligned
// to 16 bytes.)
template <int VEC, bool OWN_RUN>
__device__ __forceinline__ void load_units(const float* __restrict__ base, int first, int end, float pad,
                                           float (&v)[NB][VEC]) {
#pragma unroll
  for (int u = 0; u < NB; ++u) {
    const int i = unit_start<VEC, OWN_RUN>(first, u);
    if (VEC == 4) {
      f32x4 x = {pad, pad, pad, pad};
      if (i < end) x = *reinterpret_cast<const f32x4*>(base + i);
      v[u][0] = x.x;
      v[u][1 % VEC] = x.y;
      v[u][2 % VEC] = x.z;
      v[u][3 % VEC] = x.w;
    } else {
      v[u][0] = i < end ? base[i] : pad;
    }
  }
}

// prev, next: partial results [row][chunk][PW] of the pass before and of this one.
template <int VEC>
__global__ __launch_bounds__(SB) void sample_topp_stage_kernel(int stage, const float* __restrict__ logits, int V,
                                                               float temperature, float top_p,
                                                               const float* __restrict__ uniforms,
                                                               float* __restrict__ probs,
                                                               const RowState* __restrict__ state_prev,
                                                               RowState* __restrict__ state_next,
                                                               const float* __restrict__ prev, float* __restrict__ next,
                                                               int* __restrict__ out) {
  __shared__ float red[SB / TQ_WAVE];
  __shared__ float red_k[SB / TQ_WAVE][KW];
  __shared__ float tot_k[KW];
  constexpr int BATCH = NB * SB * VEC;
  const int row_i = blockIdx.y, chunk = blockIdx.x;
  const float* row = logits + (size_t)row_i * V;
  float* p = probs + (size_t)row_i * V;
  const int share = ((V + SC - 1) / SC + 3) / 4 * 4;
  const int b = min(V, chunk * share), e = min(V, b + share);
  const float* mine_prev = prev + (size_t)row_i * SC * PW;
  float* mine_next = next + ((size_t)row_i * SC + chunk) * PW;
  const bool writer = chunk == 0 && threadIdx.x == 0;
  const bool searching = (stage >= ST_SEARCH_P && stage < ST_SUMS_P) || (stage >= ST_SEARCH_R && stage < ST_SUMS_R);
  const bool after_search = (stage > ST_SEARCH_P && stage <= ST_SUMS_P) || (stage > ST_SEARCH_R && stage <= ST_SUMS_R);

  // the chunk's first values are asked for before anything else: what follows waits for the pass before anyway
  const float* src = stage <= ST_EXP ? row : p;
  const float pad = stage == ST_MAX ? -INFINITY : 0.f;
  float v[NB][VEC];
  if (stage != ST_PICK) load_units<VEC, false>(src, b, e, pad, v);
  RowState st = state_prev[row_i];

  // ---- where the row stands: from the chunks' results of the pass before (every workgroup of the row the same
  // arithmetic)
  if (stage == ST_EXP) {
    float mx = -INFINITY;
    for (int c = 0; c < SC; ++c) mx = fmaxf(mx, mine_prev[c * PW]);
    st.mx = mx;
  } else if (stage == ST_NORM) {
    float sum = 0.f;
    for (int c = 0; c < SC; ++c) sum += mine_prev[c * PW];
    st.inv_s = 1.0f / sum;
  } else if (stage == ST_SEARCH_P) {
    float all = 0.f, pmax = 0.f;
    for (int c = 0; c < SC; ++c) {
      all += mine_prev[c * PW];
      pmax = fmaxf(pmax, mine_prev[c * PW + 1]);
    }
    st.all = all;
    st.pmax = pmax;
    st.lo_b = max(1u, __float_as_uint(pmax * 0x1p-24f));    // no probability other than 0 lies below
    st.hi_b = __float_as_uint(pmax);
    st.target = all >= top_p ? top_p : 0.f;      // else the whole list is kept
  } else if (after_search) {
    // the search pass before: the candidates ascend and S does not grow with tau, so those that reach the target
    // come first; the first that fails is strictly larger than the last that reaches it
    if (st.target > 0.f && st.lo_b < st.hi_b) {
      if (threadIdx.x < KW) {
        float t = 0.f;
#pragma unroll
        for (int c = 0; c < SC; ++c) t += mine_prev[c * PW + threadIdx.x];
        tot_k[threadIdx.x] = t;
      }
      __syncthreads();
      int best = -1;
      for (int j = 0; j < KW; ++j)
        if (tot_k[j] >= st.target) best = j;
      const uint32_t lo_b = st.lo_b, hi_b = st.hi_b;
      if (best + 1 < KW) st.hi_b = __float_as_uint(candidate(lo_b, hi_b, best + 1)) - 1u;
      if (best >= 0) st.lo_b = __float_as_uint(candidate(lo_b, hi_b, best));
    }
    if (stage == ST_SUMS_P) st.tau_p = st.target > 0.f ? __uint_as_float(st.lo_b) : 0.f;
    if (stage == ST_SUMS_R) st.tau_r = st.target > 0.f ? __uint_as_float(st.lo_b) : st.pmax;
  } else if (stage == ST_SEARCH_R) {
    // where the sorted list is cut: the running sum first reaches top_p inside the ties of tau_p
    if (st.target > 0.f) {
      float above = 0.f;
      int ties = 0;
      for (int c = 0; c < SC; ++c) {
        above += mine_prev[c * PW];
        ties += __float_as_int(mine_prev[c * PW + 1]);
      }
      int need = (int)ceilf((top_p - above) / st.tau_p);
      need = max(1, min(need, ties));
      st.cumulative = above + (float)need * st.tau_p;
    } else {
      st.cumulative = st.all;
    }
    const float r = uniforms[row_i] * st.cumulative;
    st.lo_b = max(1u, __float_as_uint(st.pmax * 0x1p-24f));
    st.hi_b = __float_as_uint(st.pmax);
    st.target = r > 0.f ? r : 0.f;
  } else if (stage == ST_PICK) {
    st.nth = 1;
    if (st.target > 0.f) {
      float above = 0.f;
      int ties = 0;
      for (int c = 0; c < SC; ++c) {
        above += mine_prev[c * PW];
        ties += __float_as_int(mine_prev[c * PW + 1]);
      }
      const int nth = (int)ceilf((st.target - above) / st.tau_r);
      st.nth = max(1, min(nth, ties));
    }
  }
  if (writer) {
    state_next[row_i] = st;
    if (stage == ST_MAX) out[row_i] = 0;      // stays if no probability is picked (a NaN among the logits)
  }

  if (stage == ST_PICK) {
    // the nth lowest index whose probability equals tau_r: chunks are contiguous, so the ties before this chunk
    // are those that the chunks before it counted in the pass before; inside the chunk a thread counts a run of
    // its own
    __shared__ int wave_cnt[SB / TQ_WAVE];
    const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
    int k = 0;
    for (int c = 0; c < chunk; ++c) k += __float_as_int(mine_prev[c * PW + 1]);
    const int here = __float_as_int(mine_prev[chunk * PW + 1]);
    if (!(k < st.nth && st.nth <= k + here)) return;
    for (int first = b; first < e; first += BATCH) {
      load_units<VEC, true>(p, first, e, 0.f, v);
      int cnt = 0;
#pragma unroll
      for (int u = 0; u < NB; ++u)
#pragma unroll
        for (int x = 0; x < VEC; ++x) cnt += v[u][x] == st.tau_r ? 1 : 0;
      int upto = cnt;          // ties in this wave's runs up to and with this thread's
      for (int o = 1; o < TQ_WAVE; o <<= 1) {
        const int other = __shfl_up(upto, o, TQ_WAVE);
        if (lane >= o) upto += other;
      }
      __syncthreads();
      if (lane == TQ_WAVE - 1) wave_cnt[wave] = upto;
      __syncthreads();
      int before = k;
      for (int w = 0; w < wave; ++w) before += wave_cnt[w];
      before += upto - cnt;
      if (before < st.nth && st.nth <= before + cnt) {
        int seen = before;
#pragma unroll
        for (int u = 0; u < NB; ++u)
#pragma unroll
          for (int x = 0; x < VEC; ++x)
            if (v[u][x] == st.tau_r && ++seen == st.nth) out[row_i] = unit_start<VEC, true>(first, u) + x;
        // (what lies beyond the chunk's end was read as 0, and tau_r is not 0)
      }
      for (int w = 0; w < SB / TQ_WAVE; ++w) k += wave_cnt[w];
      if (k >= st.nth) return;
    }
    return;
  }

  // ---- this pass over the chunk
  const float cut = st.mx - 16.0f * temperature, inv_t = 1.0f / temperature;
  const float tau_s = stage == ST_SUMS_P ? st.tau_p : st.tau_r;
  if (searching && (!(st.target > 0.f) || st.lo_b >= st.hi_b)) return;       // nothing to search, or found already
  if (stage == ST_SUMS_P && !(st.target > 0.f)) return;
  // (without a second search, the draw being 0, tau_r is the largest probability and ST_SUMS_R counts its ties)
  float tau[KW], a[KW];
  const float lo_f = __uint_as_float(st.lo_b), hi_f = __uint_as_float(st.hi_b);
  if (searching) {
#pragma unroll
    for (int j = 0; j < KW; ++j) {
      tau[j] = candidate(st.lo_b, st.hi_b, j);
      a[j] = 0.f;
    }
  }
  float acc = 0.f, top = stage == ST_MAX ? -INFINITY : 0.f;
  int cnt = 0;
  for (int first = b; first < e; first += BATCH) {
    if (first != b) load_units<VEC, false>(src, first, e, pad, v);
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int i = unit_start<VEC, false>(first, u);
      if (stage == ST_MAX) {
#pragma unroll
        for (int x = 0; x < VEC; ++x) top = fmaxf(top, v[u][x]);
      } else if (stage == ST_EXP) {
        if (i < e) {
          float ex[VEC];
#pragma unroll
          for (int x = 0; x < VEC; ++x) {
            ex[x] = v[u][x] >= cut ? expf((v[u][x] - st.mx) * inv_t) : 0.f;
            acc += ex[x];
          }
          if (VEC == 4)
            *reinterpret_cast<f32x4*>(p + i) = f32x4{ex[0], ex[1 % VEC], ex[2 % VEC], ex[3 % VEC]};
          else
            p[i] = ex[0];
        }
      } else if (stage == ST_NORM) {
        if (i < e) {
          float n[VEC];
#pragma unroll
          for (int x = 0; x < VEC; ++x) {
            n[x] = v[u][x] * st.inv_s;
            acc += n[x];
            top = fmaxf(top, n[x]);
          }
          if (VEC == 4)
            *reinterpret_cast<f32x4*>(p + i) = f32x4{n[0], n[1 % VEC], n[2 % VEC], n[3 % VEC]};
          else
            p[i] = n[0];
        }
      } else if (searching) {
        // the candidates lie in (lo, hi]: what is above hi counts for each of them, what is not above lo for none
#pragma unroll
        for (int x = 0; x < VEC; ++x) {
          const float val = v[u][x];
          if (val > hi_f) {
            acc += val;
          } else if (val > lo_f) {
#pragma unroll
            for (int j = 0; j < KW; ++j) a[j] += val >= tau[j] ? val : 0.f;
          }
        }
      } else {      // ST_SUMS_P, ST_SUMS_R: S(> tau) and the number of ties at tau, tau being what the search found
#pragma unroll
        for (int x = 0; x < VEC; ++x) {
          if (v[u][x] > tau_s) acc += v[u][x];
          cnt += v[u][x] == tau_s ? 1 : 0;
        }
      }
    }
  }
  if (stage == ST_MAX) {
    top = chunk_max(top, red);
    if (threadIdx.x == 0) mine_next[0] = top;
  } else if (stage == ST_EXP) {
    acc = chunk_sum(acc, red);
    if (threadIdx.x == 0) mine_next[0] = acc;
  } else if (stage == ST_NORM) {
    acc = chunk_sum(acc, red);
    top = chunk_max(top, red);
    if (threadIdx.x == 0) {
      mine_next[0] = acc;
      mine_next[1] = top;
    }
  } else if (searching) {
#pragma unroll
    for (int j = 0; j < KW; ++j) a[j] = wave_sum(acc + a[j]);
    __syncthreads();
    if (threadIdx.x % TQ_WAVE == 0) {
#pragma unroll
      for (int j = 0; j < KW; ++j) red_k[threadIdx.x / TQ_WAVE][j] = a[j];
    }
    __syncthreads();
    if (threadIdx.x < KW) {
      float t = 0.f;
      for (int w = 0; w < SB / TQ_WAVE; ++w) t += red_k[w][threadIdx.x];
      mine_next[threadIdx.x] = t;
    }
  } else {
    acc = chunk_sum(acc, red);
    const float cf = chunk_sum((float)cnt, red);     // a chunk holds far fewer than 2^24 elements: exact
    if (threadIdx.x == 0) {
      mine_next[0] = acc;
      mine_next[1] = __int_as_float((int)cf);
    }
  }
}

#define STATE_FLOATS ((sizeof(RowState) + 3) / 4)

// Floats of scratch that tq_sample_topp needs for R rows (two sets each of row states and partial results).
TQ_API int64_t tq_sample_topp_scratch(int R) {
  return (int64_t)R * 2 * (STATE_FLOATS + SC * PW);
}

static int launch_sample_topp(const float* logits, int R, int V, float temperature, float top_p, const float* uniforms,
                              float* probs, float* scratch, int* out, hipStream_t st) {
  RowState* state[2] = {(RowState*)scratch, (RowState*)(scratch + (size_t)R * STATE_FLOATS)};
  float* part[2] = {scratch + (size_t)R * 2 * STATE_FLOATS, nullptr};
  part[1] = part[0] + (size_t)R * SC * PW;
  // 16 bytes at a time where every chunk of every row starts at a multiple of 16 bytes
  const bool by4 = V % 4 == 0 && ((size_t)logits & 15) == 0 && ((size_t)probs & 15) == 0;
  auto kernel = by4 ? sample_topp_stage_kernel<4> : sample_topp_stage_kernel<1>;
  for (int stage = 0; stage < ST_COUNT; ++stage)
    hipLaunchKernelGGL(kernel, dim3(SC, R), dim3(SB), 0, st, stage, logits, V, temperature, top_p, uniforms, probs,
                       state[(stage + 1) % 2], state[stage % 2], part[(stage + 1) % 2], part[stage % 2], out);
  TQ_LAUNCH_CHECK();
  return 0;
}

// probs: scratch of R * V floats; scratch: tq_sample_topp_scratch(R) floats.  temperature > 0 and top_p > 0 (the
// caller takes the greedy path otherwise).  out[r] is written for every row unless a probability is NaN; it is
// set to 0 first.
TQ_API int tq_sample_topp(const float* logits, int R, int V, float temperature, float top_p, const float* uniforms,
                          float* probs, float* scratch, int* out, hipStream_t st) {
  if (R <= 0) return 0;
  if (!(temperature > 0.f) || !(top_p > 0.f) || !scratch) return TQ_ERR_BAD_ARG;
  if (R > 65535) return TQ_ERR_UNSUPPORTED;
  return launch_sample_topp(logits, R, V, temperature, top_p, uniforms, probs, scratch, out, st);
}

// ---------------------------------------------------------------- the same choice without any allocation
// The probabilities and the passes' partial results live in an array that is part of the library's image on every
// GPU, TQ_STATIC_SAMPLE_BYTES of it (see no_alloc.h).  The array's name is only the host's handle for it: the
// address that kernels can use is looked up once per device and kept.  Nothing in the array has to start at zero:
// the first pass writes every field that a later pass reads.
#define STATIC_SCRATCH_FLOATS (TQ_STATIC_SAMPLE_MAX_ROWS * 2 * (STATE_FLOATS + SC * PW))
static __device__ __align__(256) float scratch[TQ_STATIC_SAMPLE_MAX_PROBS + STATIC_SCRATCH_FLOATS];
static_assert(sizeof(scratch) <= TQ_STATIC_SAMPLE_BYTES, "the array has outgrown the size that no_alloc.h states");

#define STATIC_MAX_DEVICES 64
static std::mutex static_lock;
static float* static_ptr[STATIC_MAX_DEVICES];      // device address of `scratch` on each GPU, once looked up

TQ_API int tq_sample_topp_static_init(void) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= STATIC_MAX_DEVICES) return TQ_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> hold(static_lock);
  if (static_ptr[dev]) return 0;
  float* ptr = nullptr;
  e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess) return (int)e;
  if (!ptr) return TQ_ERR_BAD_ARG;
  static_ptr[dev] = ptr;
  return 0;
}

TQ_API int tq_sample_topp_static(const float* logits, int R, int V, float temperature, float top_p,
                                 const float* uniforms, int* out, hipStream_t st) {
  if (R <= 0) return 0;
  if (!(temperature > 0.f) || !(top_p > 0.f) || V <= 0) return TQ_ERR_BAD_ARG;
  if (R > TQ_STATIC_SAMPLE_MAX_ROWS || (int64_t)R * V > TQ_STATIC_SAMPLE_MAX_PROBS) return TQ_ERR_UNSUPPORTED;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= STATIC_MAX_DEVICES) return TQ_ERR_UNSUPPORTED;
  float* base;
  {
    std::lock_guard<std::mutex> hold(static_lock);
    base = static_ptr[dev];
  }
  if (!base) {
    const int rc = tq_sample_topp_static_init();
    if (rc != 0) return rc;
    std::lock_guard<std::mutex> hold(static_lock);
    base = static_ptr[dev];
  }
  return launch_sample_topp(logits, R, V, temperature, top_p, uniforms, base, base + TQ_STATIC_SAMPLE_MAX_PROBS, out, st);
}
