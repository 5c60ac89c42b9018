// Choice of the next token from rows of logits: greedy, temperature with top-p, repetition penalty.
// One workgroup per row; nothing is sorted.
#include "common.h"

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

// ---------------------------------------------------------------- repetition penalty
// For each of the last `count` tokens of a row's history, once per occurrence: a positive logit is
// divided by the penalty, any other multiplied (/root/reference/src/engine/tq_generate.c:387-400).
__global__ void rep_penalty_kernel(float* __restrict__ logits, int V, const int* __restrict__ recent, int window,
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
  hipLaunchKernelGGL(rep_penalty_kernel, dim3(R), dim3(64), 0, st, logits, V, recent, window, counts, penalty);
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- temperature + top-p
// The reference (/root/reference/src/engine/tq_generate.c:81-156) keeps the logits within 16*T of the
// maximum, turns them into probabilities p = exp((l - max) / T) / sum, sorts them in descending order,
// cuts the list where the running sum reaches top_p, draws r = u * (that sum) and walks the list until
// the running sum reaches r.  The same choice is made here without a sort: "the running sum reaches s
// at an element of probability tau" means  S(> tau) < s <= S(>= tau), where S(>= tau) is the sum of all
// probabilities >= tau; the largest tau with S(>= tau) >= s is found by bisection over the bit patterns
// of positive floats, which are ordered like the floats.  Equal probabilities are taken in order of
// index.  Sums are taken in a fixed order, but not the order of a sorted walk, so a draw that lands
// within rounding of a boundary between two tokens may fall on either.
struct Sums {
  float above;   // sum of probabilities > tau
  int ties;      // number of probabilities == tau
};

__device__ Sums sums_at(const float* __restrict__ p, int V, float tau, float* red, int* redi) {
  float a = 0.f;
  int c = 0;
  for (int i = threadIdx.x; i < V; i += ST) {
    const float v = p[i];
    if (v > tau) a += v;
    c += v == tau ? 1 : 0;
  }
  Sums s;
  s.above = block_sum(a, red);
  // integer sum through the same scratch
  __syncthreads();
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  for (int o = TQ_WAVE / 2; o > 0; o >>= 1) c += __shfl_xor(c, o, TQ_WAVE);
  if (lane == 0) redi[wave] = c;
  __syncthreads();
  int tot = 0;
  for (int i = 0; i < ST / TQ_WAVE; ++i) tot += redi[i];
  s.ties = tot;
  return s;
}

// largest tau in (0, hi] such that S(>= tau) >= target; hi is the largest probability
__device__ float threshold_for(const float* __restrict__ p, int V, float target, float hi, float* red, int* redi) {
  uint32_t lo_b = 1u, hi_b = __float_as_uint(hi);   // invariant: S(>= lo) >= target (all mass), answer in [lo, hi]
  while (lo_b < hi_b) {
    const uint32_t mid = lo_b + (hi_b - lo_b + 1u) / 2u;
    const float tau = __uint_as_float(mid);
    float a = 0.f;
    for (int i = threadIdx.x; i < V; i += ST) {
      const float v = p[i];
      if (v >= tau) a += v;
    }
    a = block_sum(a, red);
    if (a >= target)
      lo_b = mid;
    else
      hi_b = mid - 1u;
  }
  return __uint_as_float(lo_b);
}

__global__ __launch_bounds__(ST) void sample_topp_kernel(const float* __restrict__ logits, int V, float temperature,
                                                         float top_p, const float* __restrict__ uniforms,
                                                         float* __restrict__ probs, int* __restrict__ out) {
  __shared__ float red[ST / TQ_WAVE];
  __shared__ int redi[ST / TQ_WAVE];
  __shared__ int chosen;
  const float* row = logits + (size_t)blockIdx.x * V;
  float* p = probs + (size_t)blockIdx.x * V;
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < V; i += ST) mx = fmaxf(mx, row[i]);
  mx = block_max(mx, red);
  const float cut = mx - 16.0f * temperature;
  const float inv_t = 1.0f / temperature;
  float s = 0.f;
  for (int i = threadIdx.x; i < V; i += ST) {
    const float l = row[i];
    const float e = l >= cut ? expf((l - mx) * inv_t) : 0.f;
    p[i] = e;
    s += e;
  }
  s = block_sum(s, red);
  const float inv_s = 1.0f / s;
  float pmax = 0.f;
  for (int i = threadIdx.x; i < V; i += ST) {
    const float v = p[i] * inv_s;
    p[i] = v;
    pmax = fmaxf(pmax, v);
  }
  pmax = block_max(pmax, red);
  __syncthreads();

  // where the sorted list is cut: the running sum first reaches top_p inside the ties of tau_p
  float cumulative;
  float tau_p = 0.f;
  {
    float all = 0.f;
    for (int i = threadIdx.x; i < V; i += ST) all += p[i];
    all = block_sum(all, red);
    if (all >= top_p) {
      tau_p = threshold_for(p, V, top_p, pmax, red, redi);
      const Sums sp = sums_at(p, V, tau_p, red, redi);
      int need = (int)ceilf((top_p - sp.above) / tau_p);
      need = max(1, min(need, sp.ties));
      cumulative = sp.above + (float)need * tau_p;
    } else {
      cumulative = all;   // the whole list is kept
    }
  }
  const float r = uniforms[blockIdx.x] * cumulative;
  float tau_r = pmax;
  int nth = 1;
  if (r > 0.f) {
    tau_r = threshold_for(p, V, r, pmax, red, redi);
    const Sums sr = sums_at(p, V, tau_r, red, redi);
    nth = (int)ceilf((r - sr.above) / tau_r);
    nth = max(1, min(nth, sr.ties));
  }
  // the nth lowest index whose probability equals tau_r
  if (threadIdx.x == 0) chosen = -1;
  __syncthreads();
  {
    const int per = (V + ST - 1) / ST;
    const int b = threadIdx.x * per, e = min(V, b + per);
    int c = 0;
    for (int i = b; i < e; ++i) c += p[i] == tau_r ? 1 : 0;
    __shared__ int cnt[ST];
    cnt[threadIdx.x] = c;
    __syncthreads();
    int before = 0;
    for (int i = 0; i < threadIdx.x; ++i) before += cnt[i];
    if (before < nth && nth <= before + c) {
      int k = before;
      for (int i = b; i < e; ++i)
        if (p[i] == tau_r && ++k == nth) chosen = i;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    if (chosen < 0) {   // not reachable unless a probability is NaN: fall back to the largest
      chosen = 0;
      for (int i = 1; i < V; ++i)
        if (row[i] > row[chosen]) chosen = i;
    }
    out[blockIdx.x] = chosen;
  }
}

// probs: scratch of R * V floats.  temperature > 0 and top_p > 0 (the caller takes the greedy path otherwise).
TQ_API int tq_sample_topp(const float* logits, int R, int V, float temperature, float top_p, const float* uniforms,
                          float* probs, int* out, hipStream_t st) {
  if (R <= 0) return 0;
  if (!(temperature > 0.f) || !(top_p > 0.f)) return TQ_ERR_BAD_ARG;
  hipLaunchKernelGGL(sample_topp_kernel, dim3(R), dim3(ST), 0, st, logits, V, temperature, top_p, uniforms, probs,
                     out);
  TQ_LAUNCH_CHECK();
  return 0;
}
