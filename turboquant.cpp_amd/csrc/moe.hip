// Routing of tokens to experts: router logits, softmax, top-k, and the order of (token, expert)
// pairs by expert that the expert products work through.
#include "common.h"

// ---------------------------------------------------------------- router
// Two kernels.  router_logits: logit[t][e] = sum_j x[t][j] * wr[e][j] in float
// (/root/reference/src/engine/tq_moe.c:611-618), with the shared expert's gate vector as one more row.  A
// wave takes one row of wr at a time for a group of up to 8 tokens whose activations wait in LDS; lane l sums
// the elements j = 8 * (64 i + l) .. + 7 for i = 0, 1, ... and the lanes' sums are added by a butterfly: one
// order for every token, whatever else is in the batch.  Rows are dealt over a second grid dimension when
// there are few tokens, so that decoding does not leave the chip to eight waves.
// router_select, one wave per token: top-k by logit, k rounds of a search in which >= lets the highest index
// win among equal logits, so ids come out by descending logit (tq_moe.c:626-645).  Weights:
//   renorm != 0: softmax over the selected logits (tq_moe.c:648-678);
//   renorm == 0: softmax over all experts, the selected probabilities kept as they are.
// shared_gate[t] = 1 / (1 + exp(-(x . shared_w)))  (tq_moe.c:1012-1018, with an exact exponential).
#define RT 8   // most tokens per workgroup of router_logits

__device__ __forceinline__ void load8(const float* p, float (&w)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w; w[4] = b.x; w[5] = b.y; w[6] = b.z; w[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float (&w)[8]) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    w[2 * i] = __uint_as_float(u[i] << 16);
    w[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
  }
}

template <int TG>
__device__ __forceinline__ void router_chunk(const float* xs, int H, int j, const float (&w)[8], float (&s)[TG]) {
#pragma unroll
  for (int r = 0; r < TG; ++r) {
    const float4 a = *reinterpret_cast<const float4*>(xs + r * H + j);
    const float4 b = *reinterpret_cast<const float4*>(xs + r * H + j + 4);
    s[r] = fmaf(a.x, w[0], s[r]);
    s[r] = fmaf(a.y, w[1], s[r]);
    s[r] = fmaf(a.z, w[2], s[r]);
    s[r] = fmaf(a.w, w[3], s[r]);
    s[r] = fmaf(b.x, w[4], s[r]);
    s[r] = fmaf(b.y, w[5], s[r]);
    s[r] = fmaf(b.z, w[6], s[r]);
    s[r] = fmaf(b.w, w[7], s[r]);
  }
}

// TG: tokens per workgroup (tokens beyond T are zeros in LDS and are not stored).
template <class W, int TG>
__global__ __launch_bounds__(256) void router_logits_kernel(const float* __restrict__ x, const W* __restrict__ wr,
                                                            const W* __restrict__ shared_w, int rows, int E,
                                                            float* __restrict__ logits, int T, int H) {
  extern __shared__ float xs[];      // [TG][H]
  const int t0 = blockIdx.x * TG;
  const int nt = min(TG, T - t0);
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const bool vec = H % 8 == 0;
  if (vec) {
    const float4* src = reinterpret_cast<const float4*>(x + (size_t)t0 * H);
    float4* dst = reinterpret_cast<float4*>(xs);
    for (int i = threadIdx.x; i < TG * H / 4; i += blockDim.x) dst[i] = i < nt * H / 4 ? src[i] : make_float4(0.f, 0.f, 0.f, 0.f);
  } else {
    for (int i = threadIdx.x; i < TG * H; i += blockDim.x) xs[i] = i < nt * H ? x[(size_t)t0 * H + i] : 0.f;
  }
  __syncthreads();
  // workgroups start at different rows, so that they do not all ask for the same row at once
  const int rot = (blockIdx.x * 5) % rows;
  const int h_quad = H / (TQ_WAVE * 8 * 4) * (TQ_WAVE * 8 * 4);     // the part of a row that goes four chunks at a time
  for (int idx = blockIdx.y * 4 + wave; idx < rows; idx += gridDim.y * 4) {
    const int e = idx + rot < rows ? idx + rot : idx + rot - rows;
    const W* row = e < E ? wr + (size_t)e * H : shared_w;
    float s[TG];
#pragma unroll
    for (int r = 0; r < TG; ++r) s[r] = 0.f;
    if (vec) {
      for (int j0 = lane * 8; j0 < h_quad; j0 += TQ_WAVE * 8 * 4) {   // four chunks asked for before the first is used
        float w[4][8];
#pragma unroll
        for (int c = 0; c < 4; ++c) load8(row + j0 + c * TQ_WAVE * 8, w[c]);
#pragma unroll
        for (int c = 0; c < 4; ++c) router_chunk<TG>(xs, H, j0 + c * TQ_WAVE * 8, w[c], s);
      }
      for (int j = h_quad + lane * 8; j < H; j += TQ_WAVE * 8) {
        float w[8];
        load8(row + j, w);
        router_chunk<TG>(xs, H, j, w, s);
      }
    } else {
      for (int j = lane; j < H; j += TQ_WAVE) {
        const float w = to_f32(row[j]);
#pragma unroll
        for (int r = 0; r < TG; ++r) s[r] = fmaf(xs[r * H + j], w, s[r]);
      }
    }
#pragma unroll
    for (int r = 0; r < TG; ++r) {
      const float v = wave_sum(s[r]);
      if (lane == 0 && r < nt) logits[(size_t)(t0 + r) * rows + e] = v;
    }
  }
}

__global__ __launch_bounds__(256) void router_select_kernel(const float* __restrict__ logits, int rows, int E,
                                                            int topk, int renorm, int* __restrict__ ids,
                                                            float* __restrict__ weights,
                                                            float* __restrict__ shared_gate, int T) {
  extern __shared__ float sm[];      // [4][E]
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  float* lg = sm + wave * E;
  const float* src = logits + (size_t)t * rows;
  for (int e = lane; e < E; e += TQ_WAVE) lg[e] = src[e];
  if (rows > E && lane == 0) shared_gate[t] = 1.0f / (1.0f + expf(-src[E]));
  __builtin_amdgcn_wave_barrier();
  float mx = 0.f, denom = 1.f;
  if (!renorm) {      // softmax over all experts, before any logit is taken out
    mx = -INFINITY;
    for (int e = lane; e < E; e += TQ_WAVE) mx = fmaxf(mx, lg[e]);
    mx = wave_max(mx);
    float d = 0.f;
    for (int e = lane; e < E; e += TQ_WAVE) d += expf(lg[e] - mx);
    denom = wave_sum(d);
  }
  float sel = 0.f;    // lane k keeps the k-th selected logit
  for (int k = 0; k < topk; ++k) {
    float bv = -INFINITY;
    int bi = -1;
    for (int e = lane; e < E; e += TQ_WAVE) {
      const float v = lg[e];
      if (v >= bv) {     // e ascends: the highest index among equals
        bv = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = TQ_WAVE / 2; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, TQ_WAVE);
      const int oi = __shfl_xor(bi, o, TQ_WAVE);
      if (oi >= 0 && (bi < 0 || ov > bv || (ov == bv && oi > bi))) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi < 0) bi = 0;   // only if every logit is NaN
    if (lane == k) sel = bv;
    if (lane == 0) {
      ids[t * topk + k] = bi;
      lg[bi] = -INFINITY;   // taken out of the later rounds
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (renorm) {
    const float m = wave_max(lane < topk ? sel : -INFINITY);
    const float p = lane < topk ? expf(sel - m) : 0.f;
    const float s = wave_sum(p);
    if (lane < topk) weights[t * topk + lane] = s > 0.f ? p * (1.0f / s) : 0.f;
  } else {
    if (lane < topk) weights[t * topk + lane] = expf(sel - mx) * (1.0f / denom);
  }
}

// logits: scratch of T * (E + 1) floats (T * E without a shared gate vector).
TQ_API int tq_router_topk(const float* x, const void* wr, const void* shared_w, int wtype, int E, int topk,
                          int renorm, int* ids, float* weights, float* shared_gate, float* logits, int T, int H,
                          hipStream_t st) {
  if (T <= 0) return 0;
  if (topk < 1 || topk > 64 || topk > E || E > 8192) return TQ_ERR_UNSUPPORTED;
  int tg = RT;
  while (tg > 1 && (size_t)tg * H * sizeof(float) > 32 * 1024) tg /= 2;   // small enough for several workgroups per CU
  const size_t shmem = (size_t)tg * H * sizeof(float);
  if (shmem > 160 * 1024) return TQ_ERR_UNSUPPORTED;
  const int rows = E + (shared_w ? 1 : 0);
  const int groups = (T + tg - 1) / tg;
  // with few groups of tokens the rows are dealt over more workgroups
  int row_groups = 256 / groups;
  row_groups = row_groups < 1 ? 1 : (row_groups > (rows + 3) / 4 ? (rows + 3) / 4 : row_groups);
#define TQ_ROUTER(TGV)                                                                                              \
  do {                                                                                                              \
    if (shmem > 48 * 1024)                                                                                          \
      hipFuncSetAttribute((const void*)router_logits_kernel<W, TGV>, hipFuncAttributeMaxDynamicSharedMemorySize,    \
                          (int)shmem);                                                                              \
    hipLaunchKernelGGL((router_logits_kernel<W, TGV>), dim3(groups, row_groups), dim3(256), shmem, st, x,           \
                       (const W*)wr, (const W*)shared_w, rows, E, logits, T, H);                                    \
  } while (0)
  TQ_DISPATCH_W(wtype, {
    if (tg == 8) TQ_ROUTER(8);
    else if (tg == 4) TQ_ROUTER(4);
    else if (tg == 2) TQ_ROUTER(2);
    else TQ_ROUTER(1);
  });
#undef TQ_ROUTER
  TQ_LAUNCH_CHECK();
  hipLaunchKernelGGL(router_select_kernel, dim3((T + 3) / 4), dim3(256), (size_t)4 * E * sizeof(float), st, logits,
                     rows, E, topk, renorm, ids, weights, shared_gate, T);
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
// One workgroup of 16 waves does all of it.  Wave w owns the w-th sixteenth of the pairs: it goes through
// them 64 at a time, and for every expert present among the 64 (found leader by leader with ballots) gives
// the lanes of that expert their rank in order of lane and adds their number to its count of the expert.
// After a barrier the counts of all waves give every expert's first row and every wave's first row within
// the expert, and each pair's row is that plus its rank.
#define AW 16   // waves

__global__ __launch_bounds__(64 * AW) void moe_align_kernel(const int* __restrict__ ids, int n_pairs, int E,
                                                            int topk, int unit, int cap,
                                                            int* __restrict__ sorted_token,
                                                            int* __restrict__ pair_slot,
                                                            int* __restrict__ tile_expert,
                                                            int* __restrict__ n_tiles) {
  extern __shared__ int cnt[];        // [AW][E] counts, then E starts
  int* starts = cnt + AW * E;
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  for (int i = threadIdx.x; i < cap; i += blockDim.x) sorted_token[i] = -1;
  for (int i = threadIdx.x; i < AW * E; i += blockDim.x) cnt[i] = 0;
  __syncthreads();
  const int per = ((n_pairs + AW - 1) / AW + TQ_WAVE - 1) / TQ_WAVE * TQ_WAVE;   // pairs per wave, whole batches
  const int seg_beg = wave * per, seg_end = min(n_pairs, seg_beg + per);
  int* mine = cnt + wave * E;
  for (int b = seg_beg; b < seg_end; b += TQ_WAVE) {
    const int i = b + lane;
    const bool valid = i < seg_end;
    const int e = valid ? ids[i] : -1;
    int rank = 0;
    unsigned long long rest = __ballot(valid);
    while (rest) {
      const int leader = __ffsll((long long)rest) - 1;
      const int e0 = __shfl(e, leader, TQ_WAVE);
      const unsigned long long m = __ballot(valid && e == e0);
      const int base = mine[e0];
      if (e == e0 && valid) rank = base + __popcll(m & ((1ull << lane) - 1ull));
      __builtin_amdgcn_wave_barrier();
      if (lane == leader) mine[e0] = base + __popcll(m);
      __builtin_amdgcn_wave_barrier();
      rest &= ~m;
    }
    if (valid) pair_slot[i] = rank;      // rank within (wave, expert) for now
  }
  __syncthreads();
  // counts become each wave's first row within its expert; starts[e] first holds the expert's padded size
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    int total = 0;
    for (int w = 0; w < AW; ++w) {
      const int c = cnt[w * E + e];
      cnt[w * E + e] = total;
      total += c;
    }
    starts[e] = (total + unit - 1) / unit * unit;
  }
  __syncthreads();
  if (wave == 0) {      // exclusive scan of the padded sizes: each lane a contiguous run of experts
    const int chunk = (E + TQ_WAVE - 1) / TQ_WAVE;
    const int e0 = lane * chunk, e1 = min(E, e0 + chunk);
    int sum = 0;
    for (int e = e0; e < e1; ++e) sum += starts[e];
    int incl = sum;
#pragma unroll
    for (int o = 1; o < TQ_WAVE; o <<= 1) {
      const int up = __shfl_up(incl, o, TQ_WAVE);
      if (lane >= o) incl += up;
    }
    int row = incl - sum;
    for (int e = e0; e < e1; ++e) {
      const int padded = starts[e];
      starts[e] = row;
      for (int j = 0; j < padded / unit; ++j) tile_expert[row / unit + j] = e;
      row += padded;
    }
    if (lane == TQ_WAVE - 1) n_tiles[0] = incl / unit;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
    const int e = ids[i], w = i / per;
    const int r = starts[e] + cnt[w * E + e] + pair_slot[i];
    pair_slot[i] = r;
    sorted_token[r] = i / topk;
  }
}

// cap: rows that sorted_token holds, a multiple of unit and at least n_pairs + min(E, n_pairs) * (unit - 1);
// tile_expert holds cap / unit entries.
TQ_API int tq_moe_align(const int* ids, int n_pairs, int E, int topk, int unit, int cap, int* sorted_token,
                        int* pair_slot, int* tile_expert, int* n_tiles, hipStream_t st) {
  if (n_pairs <= 0) return 0;
  if (unit < 1 || cap % unit != 0 || cap < n_pairs + (E < n_pairs ? E : n_pairs) * (unit - 1)) return TQ_ERR_BAD_ARG;
  const size_t shmem = (size_t)(AW + 1) * E * sizeof(int);
  if (shmem > 160 * 1024) return TQ_ERR_UNSUPPORTED;
  if (shmem > 48 * 1024)
    hipFuncSetAttribute((const void*)moe_align_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(64 * AW), shmem, st, ids, n_pairs, E, topk, unit, cap,
                     sorted_token, pair_slot, tile_expert, n_tiles);
  TQ_LAUNCH_CHECK();
  return 0;
}
