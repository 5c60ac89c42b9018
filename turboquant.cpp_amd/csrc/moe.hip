// Routing of tokens to experts: router logits, softmax, top-k, and the order of (token, expert)
// pairs by expert that the expert products work through.
#include "common.h"

// ---------------------------------------------------------------- router
// One workgroup per token.  logit[e] = sum_j x[j] * wr[e][j] in float
// (/root/reference/src/engine/tq_moe.c:611-618).  Top-k by logit with k passes of a linear scan
// that uses >=, so among equal logits the highest index wins and ids come out by descending logit
// (tq_moe.c:626-645).  Weights:
//   renorm != 0: softmax over the selected logits (tq_moe.c:648-678);
//   renorm == 0: softmax over all experts, the selected probabilities kept as they are.
// If shared_w is given, shared_gate[t] = 1 / (1 + exp(-(x . shared_w)))  (tq_moe.c:1012-1018, with an
// exact exponential).
template <class W>
__global__ __launch_bounds__(256) void router_topk_kernel(const float* __restrict__ x, const W* __restrict__ wr,
                                                          const W* __restrict__ shared_w, int E, int topk,
                                                          int renorm, int* __restrict__ ids,
                                                          float* __restrict__ weights,
                                                          float* __restrict__ shared_gate, int H) {
  extern __shared__ float logits[];   // E
  const int t = blockIdx.x;
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE, nw = blockDim.x / TQ_WAVE;
  const float* xr = x + (size_t)t * H;
  for (int e = wave; e < E + (shared_w ? 1 : 0); e += nw) {
    const W* row = e < E ? wr + (size_t)e * H : shared_w;
    float s = 0.f;
    for (int j = lane; j < H; j += TQ_WAVE) s = fmaf(xr[j], to_f32(row[j]), s);
    s = wave_sum(s);
    if (lane == 0) {
      if (e < E)
        logits[e] = s;
      else
        shared_gate[t] = 1.0f / (1.0f + expf(-s));
    }
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  float denom = 1.f, mx = 0.f;
  if (!renorm) {
    mx = logits[0];
    for (int e = 1; e < E; ++e) mx = fmaxf(mx, logits[e]);
    denom = 0.f;
    for (int e = 0; e < E; ++e) denom += expf(logits[e] - mx);
  }
  // selection; a chosen logit is marked by NaN-free sentinel: its index is kept in ids and skipped
  float sel[64];
  for (int k = 0; k < topk; ++k) {
    int best = -1;
    float bv = -INFINITY;
    for (int e = 0; e < E; ++e) {
      bool used = false;
      for (int u = 0; u < k; ++u) used |= ids[t * topk + u] == e;
      if (!used && logits[e] >= bv) {
        bv = logits[e];
        best = e;
      }
    }
    ids[t * topk + k] = best < 0 ? 0 : best;
    sel[k] = best < 0 ? -INFINITY : bv;
  }
  if (renorm) {
    float m = sel[0];
    for (int k = 1; k < topk; ++k) m = fmaxf(m, sel[k]);
    float s = 0.f;
    for (int k = 0; k < topk; ++k) {
      sel[k] = expf(sel[k] - m);
      s += sel[k];
    }
    const float inv = s > 0.f ? 1.0f / s : 0.f;
    for (int k = 0; k < topk; ++k) weights[t * topk + k] = sel[k] * inv;
  } else {
    const float inv = 1.0f / denom;
    for (int k = 0; k < topk; ++k) weights[t * topk + k] = expf(sel[k] - mx) * inv;
  }
}

TQ_API int tq_router_topk(const float* x, const void* wr, const void* shared_w, int wtype, int E, int topk,
                          int renorm, int* ids, float* weights, float* shared_gate, int T, int H,
                          hipStream_t st) {
  if (T <= 0) return 0;
  if (topk < 1 || topk > 64 || topk > E || E > 16384) return TQ_ERR_UNSUPPORTED;
  TQ_DISPATCH_W(wtype, {
    hipLaunchKernelGGL(router_topk_kernel<W>, dim3(T), dim3(256), (size_t)E * sizeof(float), st, x, (const W*)wr,
                       (const W*)shared_w, E, topk, renorm, ids, weights, shared_gate, H);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- order of pairs by expert
// Pair i = (token i / topk, its (i % topk)-th expert ids[i]).  Pairs are put in order of expert and,
// within an expert, of i (a stable counting sort, so the order never depends on timing).  Each
// expert's run of rows starts at a multiple of `unit` rows so that a row tile of the expert
// products belongs to one expert; the rows between are marked -1.
//   sorted_token[r]  token whose activations feed row r, or -1
//   pair_slot[i]     row of pair i
//   tile_expert[j]   expert of row tile j (tiles of `unit` rows), n_tiles[0] tiles in all
// One workgroup does all of it: waves take experts in turn and find their pairs by ballot.
__global__ __launch_bounds__(1024) void moe_align_kernel(const int* __restrict__ ids, int n_pairs, int E, int topk,
                                                         int unit, int cap, int* __restrict__ sorted_token,
                                                         int* __restrict__ pair_slot, int* __restrict__ tile_expert,
                                                         int* __restrict__ n_tiles) {
  extern __shared__ int counts[];     // E counts, then E starts
  int* starts = counts + E;
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE, nw = blockDim.x / TQ_WAVE;
  for (int i = threadIdx.x; i < cap; i += blockDim.x) sorted_token[i] = -1;
  for (int e = wave; e < E; e += nw) {
    int c = 0;
    for (int b = 0; b < n_pairs; b += TQ_WAVE) {
      const int i = b + lane;
      const bool hit = i < n_pairs && ids[i] == e;
      c += __popcll(__ballot(hit));
    }
    if (lane == 0) counts[e] = c;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int row = 0, tile = 0;
    for (int e = 0; e < E; ++e) {
      starts[e] = row;
      const int nt = (counts[e] + unit - 1) / unit;
      for (int j = 0; j < nt; ++j) tile_expert[tile++] = e;
      row += nt * unit;
    }
    n_tiles[0] = tile;
  }
  __syncthreads();
  for (int e = wave; e < E; e += nw) {
    int row = starts[e];
    for (int b = 0; b < n_pairs; b += TQ_WAVE) {
      const int i = b + lane;
      const bool hit = i < n_pairs && ids[i] == e;
      const unsigned long long mask = __ballot(hit);
      if (hit) {
        const int r = row + __popcll(mask & ((1ull << lane) - 1ull));
        sorted_token[r] = i / topk;
        pair_slot[i] = r;
      }
      row += __popcll(mask);
    }
  }
}

// cap: rows that sorted_token holds, a multiple of unit and at least n_pairs + min(E, n_pairs) * (unit - 1);
// tile_expert holds cap / unit entries.
TQ_API int tq_moe_align(const int* ids, int n_pairs, int E, int topk, int unit, int cap, int* sorted_token,
                        int* pair_slot, int* tile_expert, int* n_tiles, hipStream_t st) {
  if (n_pairs <= 0) return 0;
  if (unit < 1 || cap % unit != 0 || cap < n_pairs + (E < n_pairs ? E : n_pairs) * (unit - 1) || E > 8192)
    return TQ_ERR_BAD_ARG;
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), (size_t)2 * E * sizeof(int), st, ids, n_pairs, E, topk,
                     unit, cap, sorted_token, pair_slot, tile_expert, n_tiles);
  TQ_LAUNCH_CHECK();
  return 0;
}
