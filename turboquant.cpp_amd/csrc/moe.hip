// Routing of tokens to experts: router logits, softmax, top-k, and the order of (token, expert)
// pairs by expert that the expert products work through.
#include "common.h"

// ---------------------------------------------------------------- router
// Two kernels.  router_logits: logit[t][e] = sum_j x[t][j] * wr[e][j] in float
// (/root/reference/src/engine/tq_moe.c:611-618), with the shared expert's gate vector as one more row.  A
// wave takes one row of wr (or a few) at a time for a group of up to 8 tokens whose activations wait in LDS; lane l sums
// a fixed share of the elements and the lanes' sums are added by a butterfly: one order for every token,
// whatever else is in the batch.  Rows are dealt over a second grid dimension when
// there are few tokens, so that decoding does not leave the chip to eight waves.
// router_select, one wave per token: top-k by logit, k rounds of a search in which >= lets the highest index
// win among equal logits, so ids come out by descending logit (tq_moe.c:626-645).  Weights:
//   renorm != 0: softmax over the selected logits (tq_moe.c:648-678);
//   renorm == 0: softmax over all experts, the selected probabilities kept as they are.
// shared_gate[t] = 1 / (1 + exp(-(x . shared_w)))  (tq_moe.c:1012-1018, with an exact exponential).
#define RT 8   // most tokens per workgroup of router_logits
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void load4(const float* p, float* w) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p);
  w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float* w) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  w[0] = __uint_as_float(v.x << 16);
  w[1] = __uint_as_float(v.x & 0xffff0000u);
  w[2] = __uint_as_float(v.y << 16);
  w[3] = __uint_as_float(v.y & 0xffff0000u);
}

// TG: tokens per workgroup (tokens beyond T are zeros in LDS and are not stored).  RW: rows of wr that a wave
// takes at a time, so that one read of the activations from LDS serves RW rows.  Neither changes the order in
// which a logit is summed: of every 512 elements lane l sums 4 l .. 4 l + 3 and 256 + 4 l .. 256 + 4 l + 3 (its
// 16-byte reads from LDS then lie side by side with its neighbours'), block after block.  In LDS a token's row is
// filled with zeros up to a multiple of 512, so the last block needs no predicate: there the weights are read
// from the row's last elements instead, and multiplied by zeros.
template <class W, int TG, int RW>
__global__ __launch_bounds__(256) void router_logits_kernel(const float* __restrict__ x, const W* __restrict__ wr,
                                                            const W* __restrict__ shared_w, int rows, int E,
                                                            float* __restrict__ logits, int T, int H) {
  extern __shared__ __attribute__((aligned(16))) float xs[];      // [TG][Hp]
  const int Hp = (H + 511) / 512 * 512;
  const int t0 = blockIdx.x * TG;
  const int nt = min(TG, T - t0);
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const bool vec = H % 4 == 0;
  if (vec) {
    const int Hp4 = Hp / 4, H4 = H / 4;
    f32x4* dst = reinterpret_cast<f32x4*>(xs);
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < TG; ++k)
      for (int j = threadIdx.x; j < Hp4; j += blockDim.x)
        dst[k * Hp4 + j] = k < nt && j < H4 ? reinterpret_cast<const f32x4*>(x + (size_t)(t0 + k) * H)[j] : zero;
  } else {
    for (int i = threadIdx.x; i < TG * Hp; i += blockDim.x) {
      const int k = i / Hp, j = i % Hp;
      xs[i] = k < nt && j < H ? x[(size_t)(t0 + k) * H + j] : 0.f;
    }
  }
  __syncthreads();
  // workgroups start at different rows, so that they do not all ask for the same row at once
  const int rot = (blockIdx.x * 5) % rows;
  for (int idx = (blockIdx.y * 4 + wave) * RW; idx < rows; idx += gridDim.y * 4 * RW) {
    const W* row[RW];
    int e[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
      const int i = min(idx + r, rows - 1) + rot;
      e[r] = i < rows ? i : i - rows;
      row[r] = e[r] < E ? wr + (size_t)e[r] * H : shared_w;
    }
    float s[RW][TG];
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
      for (int k = 0; k < TG; ++k) s[r][k] = 0.f;
    if (vec) {
      const f32x4* xv = reinterpret_cast<const f32x4*>(xs);
      const int Hp4 = Hp / 4;
      constexpr int NB = RW >= 4 ? 2 : 4;      // blocks whose weights are asked for before the first is used
      for (int b0 = 0; b0 < Hp; b0 += NB * 512) {
        float w[NB][RW][8];
#pragma unroll
        for (int u = 0; u < NB; ++u) {
          const int b = b0 + u * 512;
          const int g0 = min(b + 4 * lane, H - 4), g1 = min(b + 256 + 4 * lane, H - 4);
#pragma unroll
          for (int r = 0; r < RW; ++r) {
            load4(row[r] + g0, &w[u][r][0]);
            load4(row[r] + g1, &w[u][r][4]);
          }
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
          const int b = b0 + u * 512;
          if (b < Hp) {
#pragma unroll
            for (int k = 0; k < TG; ++k) {
              const f32x4 a = xv[k * Hp4 + b / 4 + lane];
              const f32x4 c = xv[k * Hp4 + b / 4 + 64 + lane];
#pragma unroll
              for (int r = 0; r < RW; ++r) {
                float v = s[r][k];
                v = fmaf(a.x, w[u][r][0], v);
                v = fmaf(a.y, w[u][r][1], v);
                v = fmaf(a.z, w[u][r][2], v);
                v = fmaf(a.w, w[u][r][3], v);
                v = fmaf(c.x, w[u][r][4], v);
                v = fmaf(c.y, w[u][r][5], v);
                v = fmaf(c.z, w[u][r][6], v);
                v = fmaf(c.w, w[u][r][7], v);
                s[r][k] = v;
              }
            }
          }
        }
      }
    } else {
      for (int j = lane; j < H; j += TQ_WAVE) {
#pragma unroll
        for (int r = 0; r < RW; ++r) {
          const float w = to_f32(row[r][j]);
#pragma unroll
          for (int k = 0; k < TG; ++k) s[r][k] = fmaf(xs[k * Hp + j], w, s[r][k]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
      for (int k = 0; k < TG; ++k) {
        const float v = wave_sum(s[r][k]);
        if (lane == 0 && k < nt && idx + r < rows) logits[(size_t)(t0 + k) * rows + e[r]] = v;
      }
  }
}

// One wave chooses for one token.  src: the token's `rows` logits; lg: E floats of LDS for this wave; ids,
// weights, shared_gate: where the token's results go; ids2: a second place for the ids (LDS), or null.
__device__ __forceinline__ void select_token(const float* __restrict__ src, int rows, int E, int topk, int renorm,
                                             float* lg, int* __restrict__ ids, int* ids2,
                                             float* __restrict__ weights, float* __restrict__ shared_gate) {
  const int lane = threadIdx.x % TQ_WAVE;
  for (int e = lane; e < E; e += TQ_WAVE) lg[e] = src[e];
  if (rows > E && lane == 0) shared_gate[0] = 1.0f / (1.0f + expf(-src[E]));
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
      ids[k] = bi;
      if (ids2) ids2[k] = bi;
      lg[bi] = -INFINITY;   // taken out of the later rounds
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (renorm) {
    const float m = wave_max(lane < topk ? sel : -INFINITY);
    const float p = lane < topk ? expf(sel - m) : 0.f;
    const float s = wave_sum(p);
    if (lane < topk) weights[lane] = s > 0.f ? p * (1.0f / s) : 0.f;
  } else {
    if (lane < topk) weights[lane] = expf(sel - mx) * (1.0f / denom);
  }
}

__global__ __launch_bounds__(256) void router_select_kernel(const float* __restrict__ logits, int rows, int E,
                                                            int topk, int renorm, int* __restrict__ ids,
                                                            float* __restrict__ weights,
                                                            float* __restrict__ shared_gate, int T) {
  extern __shared__ float sm[];      // [4][E]
  const int wave = threadIdx.x / TQ_WAVE;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  select_token(logits + (size_t)t * rows, rows, E, topk, renorm, sm + wave * E, ids + (size_t)t * topk, nullptr,
               weights + (size_t)t * topk, shared_gate + t);
}

static int launch_router_logits(const float* x, const void* wr, const void* shared_w, int wtype, int E,
                                float* logits, int T, int H, hipStream_t st) {
  int tg = RT;
  const size_t hp = ((size_t)H + 511) / 512 * 512;      // a token's row in LDS
  while (tg > 1 && (size_t)tg * hp * sizeof(float) > 32 * 1024) tg /= 2;   // small enough for several workgroups per CU
  const size_t shmem = (size_t)tg * hp * sizeof(float);
  if (shmem > 160 * 1024) return TQ_ERR_UNSUPPORTED;
  const int rows = E + (shared_w ? 1 : 0);
  const int groups = (T + tg - 1) / tg;
  // The rows are dealt over so many workgroups that the chip holds about 2048 of them: what a wave does is a
  // chain of loads, and only many waves hide it.  A wave takes 1, 2 or 4 rows at a time.
  int row_groups = 2048 / groups;
  row_groups = row_groups < 1 ? 1 : (row_groups > (rows + 3) / 4 ? (rows + 3) / 4 : row_groups);
  const int rows_per_wave = (rows + row_groups * 4 - 1) / (row_groups * 4);
  const int rw = rows_per_wave >= 4 ? 4 : (rows_per_wave >= 2 ? 2 : 1);
#define TQ_ROUTER(TGV, RWV)                                                                                         \
  do {                                                                                                              \
    if (shmem > 48 * 1024)                                                                                          \
      (void)hipFuncSetAttribute((const void*)router_logits_kernel<W, TGV, RWV>,                                           \
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);                                  \
    hipLaunchKernelGGL((router_logits_kernel<W, TGV, RWV>), dim3(groups, row_groups), dim3(256), shmem, st, x,      \
                       (const W*)wr, (const W*)shared_w, rows, E, logits, T, H);                                    \
  } while (0)
#define TQ_ROUTER_RW(TGV)          \
  do {                             \
    if (rw == 4) TQ_ROUTER(TGV, 4); \
    else if (rw == 2) TQ_ROUTER(TGV, 2); \
    else TQ_ROUTER(TGV, 1);        \
  } while (0)
  TQ_DISPATCH_W(wtype, {
    if (tg == 8) TQ_ROUTER_RW(8);
    else if (tg == 4) TQ_ROUTER_RW(4);
    else if (tg == 2) TQ_ROUTER_RW(2);
    else TQ_ROUTER_RW(1);
  });
#undef TQ_ROUTER_RW
#undef TQ_ROUTER
  TQ_LAUNCH_CHECK();
  return 0;
}

// logits: scratch of T * (E + 1) floats (T * E without a shared gate vector).
TQ_API int tq_router_topk(const float* x, const void* wr, const void* shared_w, int wtype, int E, int topk,
                          int renorm, int* ids, float* weights, float* shared_gate, float* logits, int T, int H,
                          hipStream_t st) {
  if (T <= 0) return 0;
  if (topk < 1 || topk > 64 || topk > E || E > 8192) return TQ_ERR_UNSUPPORTED;
  const int rc = launch_router_logits(x, wr, shared_w, wtype, E, logits, T, H, st);
  if (rc) return rc;
  const int rows = E + (shared_w ? 1 : 0);
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
//   tile_expert[cap / unit + p]   first row tile of item p, n_tiles[1] items in all: an expert's row tiles two at a
//                    time (its last one alone when their number is odd), for the product that takes two tiles of
//                    one expert per workgroup; item p ends where item p + 1 begins, the last one at n_tiles[0]
// One workgroup of 16 waves does all of it.  Wave w owns the w-th sixteenth of the pairs: it goes through
// them 64 at a time, finds for every lane the lanes that hold the same expert (a ballot per bit of the expert's
// number), gives it its rank among them in order of lane and adds their number to its count of the expert.
// After a barrier the counts of all waves give every expert's first row and every wave's first row within
// the expert, and each pair's row is that plus its rank.
#define AW 16   // waves (one where a single token is ordered: the result does not depend on their number)

// One wave goes through its pairs seg_beg .. seg_end - 1, 64 at a time: every lane finds the lanes that hold the same
// expert (a ballot per bit of the expert's number), takes its rank among the wave's pairs of that expert so far, in
// order of pair, and the expert's first lane adds the batch's number to the wave's count mine[e].  The rank goes to
// pair_slot[i], or, with one_batch (at most 64 pairs a wave), stays with the lane in my_e, my_rank.
__device__ __forceinline__ void rank_segment(const int* ids, int seg_beg, int seg_end, int E, int* mine,
                                             int* __restrict__ pair_slot, bool one_batch, int& my_e, int& my_rank) {
  const int lane = threadIdx.x % TQ_WAVE;
  for (int b = seg_beg; b < seg_end; b += TQ_WAVE) {
    const int i = b + lane;
    const bool valid = i < seg_end;
    const int e = valid ? ids[i] : -1;
    // the lanes that hold the same expert: one ballot per bit of the expert's number
    unsigned long long same = __ballot(valid);
    for (int bit = 0; (1 << bit) < E; ++bit) {
      const unsigned long long set = __ballot(valid && ((e >> bit) & 1));
      same &= ((e >> bit) & 1) ? set : ~set;
    }
    const unsigned long long lower = same & ((1ull << lane) - 1ull);
    const int base = mine[valid ? e : 0];
    const int rank = base + __popcll(lower);
    __builtin_amdgcn_wave_barrier();       // every lane has read its count before the expert's first lane adds to it
    if (valid && lower == 0) mine[e] = base + __popcll(same);
    __builtin_amdgcn_wave_barrier();
    if (one_batch) {
      my_e = e;
      my_rank = rank;
    } else if (valid) {
      pair_slot[i] = rank;      // rank within (wave, expert) for now
    }
  }
}

// Wave 0 of a workgroup turns the experts' padded sizes starts[e] into their first rows (an exclusive scan, each lane
// a contiguous run of experts) and writes the row tiles' experts, the items and their numbers.
__device__ __forceinline__ void scan_starts(int* starts, int E, int unit, int cap, int* __restrict__ tile_expert,
                                            int* __restrict__ n_tiles) {
  const int lane = threadIdx.x % TQ_WAVE;
  {
    const int chunk = (E + TQ_WAVE - 1) / TQ_WAVE;
    const int e0 = lane * chunk, e1 = min(E, e0 + chunk);
    int sum = 0, isum = 0;
    for (int e = e0; e < e1; ++e) {
      sum += starts[e];
      isum += (starts[e] / unit + 1) / 2;
    }
    int incl = sum, iincl = isum;
#pragma unroll
    for (int o = 1; o < TQ_WAVE; o <<= 1) {
      const int up = __shfl_up(incl, o, TQ_WAVE);
      const int iup = __shfl_up(iincl, o, TQ_WAVE);
      if (lane >= o) {
        incl += up;
        iincl += iup;
      }
    }
    int row = incl - sum, item = iincl - isum;
    int* items = tile_expert + cap / unit;
    for (int e = e0; e < e1; ++e) {
      const int padded = starts[e];
      starts[e] = row;
      for (int j = 0; j < padded / unit; ++j) {
        tile_expert[row / unit + j] = e;
        if (j % 2 == 0) items[item++] = row / unit + j;
      }
      row += padded;
    }
    if (lane == TQ_WAVE - 1) {
      n_tiles[0] = incl / unit;
      n_tiles[1] = iincl;
    }
  }
}

// ids may lie in LDS or in memory; cnt: (NW + 1) * E ints of LDS ([NW][E] counts, then E starts).  All NW waves
// of the workgroup call it together.
template <int NW>
__device__ __forceinline__ void align_pairs(const int* ids, int n_pairs, int E, int topk, int unit, int cap,
                                            int* __restrict__ sorted_token, int* __restrict__ pair_slot,
                                            int* __restrict__ tile_expert, int* __restrict__ n_tiles, int* cnt) {
  int* starts = cnt + NW * E;
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  for (int i = threadIdx.x; i < cap; i += blockDim.x) sorted_token[i] = -1;
  for (int i = threadIdx.x; i < NW * E; i += blockDim.x) cnt[i] = 0;
  __syncthreads();
  const int per = ((n_pairs + NW - 1) / NW + TQ_WAVE - 1) / TQ_WAVE * TQ_WAVE;   // pairs per wave, whole batches
  const int seg_beg = wave * per, seg_end = min(n_pairs, seg_beg + per);
  int* mine = cnt + wave * E;
  // with at most 64 pairs per wave a thread meets its pair again in the last loop (i == threadIdx.x both times):
  // expert and rank stay in its registers and need not go through memory
  const bool one_batch = per == TQ_WAVE;
  int my_e = -1, my_rank = 0;
  rank_segment(ids, seg_beg, seg_end, E, mine, pair_slot, one_batch, my_e, my_rank);
  __syncthreads();
  // counts become each wave's first row within its expert; starts[e] first holds the expert's padded size
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    int total = 0;
    for (int w = 0; w < NW; ++w) {
      const int c = cnt[w * E + e];
      cnt[w * E + e] = total;
      total += c;
    }
    starts[e] = (total + unit - 1) / unit * unit;
  }
  __syncthreads();
  if (wave == 0) scan_starts(starts, E, unit, cap, tile_expert, n_tiles);
  __syncthreads();
  if (one_batch) {
    if (my_e >= 0) {
      const int i = threadIdx.x;
      const int r = starts[my_e] + cnt[wave * E + my_e] + my_rank;
      pair_slot[i] = r;
      sorted_token[r] = i / topk;
    }
    return;
  }
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
    const int e = ids[i], w = i / per;
    const int r = starts[e] + cnt[w * E + e] + pair_slot[i];
    pair_slot[i] = r;
    sorted_token[r] = i / topk;
  }
}

__global__ __launch_bounds__(64 * AW) void moe_align_kernel(const int* __restrict__ ids, int n_pairs, int E,
                                                            int topk, int unit, int cap,
                                                            int* __restrict__ sorted_token,
                                                            int* __restrict__ pair_slot,
                                                            int* __restrict__ tile_expert,
                                                            int* __restrict__ n_tiles) {
  extern __shared__ int cnt[];
  align_pairs<AW>(ids, n_pairs, E, topk, unit, cap, sorted_token, pair_slot, tile_expert, n_tiles, cnt);
}

// The same order by several workgroups, for steps of many tokens (one workgroup's waves go through 32,768 pairs in
// 56 us, a compute unit's instructions being what it takes): three launches over V = 16 * workgroups waves that own
// the pairs in V contiguous runs, as the waves of the one workgroup do.  count: every wave ranks its pairs and leaves
// its counts per expert in table[v][e]; scan (one workgroup): the counts become each wave's first row within its
// expert, table[V][e] each expert's first row, and the row tiles and items are written; place: every pair's row.
// The results are those of the one workgroup: pairs in order of expert and, within an expert, of pair.
// table: (V + 1) * E ints of memory.
#define AC 8      // waves whose counts one thread of the scan adds up
__global__ __launch_bounds__(64 * AW) void align_count_kernel(const int* __restrict__ ids, int n_pairs, int E, int cap,
                                                              int* __restrict__ sorted_token,
                                                              int* __restrict__ pair_slot, int* __restrict__ table) {
  extern __shared__ int cnt[];       // [AW][E]
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int V = gridDim.x * AW, v = blockIdx.x * AW + wave;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < cap; i += gridDim.x * blockDim.x) sorted_token[i] = -1;
  for (int i = threadIdx.x; i < AW * E; i += blockDim.x) cnt[i] = 0;
  __syncthreads();
  const int per = ((n_pairs + V - 1) / V + TQ_WAVE - 1) / TQ_WAVE * TQ_WAVE;
  const int seg_beg = min(n_pairs, v * per), seg_end = min(n_pairs, seg_beg + per);
  int my_e = -1, my_rank = 0;
  rank_segment(ids, seg_beg, seg_end, E, cnt + wave * E, pair_slot, false, my_e, my_rank);
  __builtin_amdgcn_wave_barrier();
  for (int e = lane; e < E; e += TQ_WAVE) table[(size_t)v * E + e] = cnt[wave * E + e];
}

__global__ __launch_bounds__(64 * AW) void align_scan_kernel(int* __restrict__ table, int V, int E, int unit, int cap,
                                                             int* __restrict__ tile_expert, int* __restrict__ n_tiles) {
  extern __shared__ int sm_a[];        // [chunks][E] sums of AC waves' counts, then E starts
  const int chunks = (V + AC - 1) / AC;
  int* starts = sm_a + chunks * E;
  // thread (chunk c, expert e): the counts of waves AC c .. AC c + AC - 1, all asked for at once
  for (int idx = threadIdx.x; idx < chunks * E; idx += blockDim.x) {
    const int c = idx / E, e = idx % E;
    int sum = 0;
#pragma unroll
    for (int u = 0; u < AC; ++u) sum += AC * c + u < V ? table[(size_t)(AC * c + u) * E + e] : 0;
    sm_a[idx] = sum;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    int total = 0;
    for (int c = 0; c < chunks; ++c) {
      const int t = sm_a[c * E + e];
      sm_a[c * E + e] = total;
      total += t;
    }
    starts[e] = (total + unit - 1) / unit * unit;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < chunks * E; idx += blockDim.x) {
    const int c = idx / E, e = idx % E;
    int cv[AC];
#pragma unroll
    for (int u = 0; u < AC; ++u) cv[u] = AC * c + u < V ? table[(size_t)(AC * c + u) * E + e] : 0;
    int total = sm_a[idx];
#pragma unroll
    for (int u = 0; u < AC; ++u)
      if (AC * c + u < V) {
        table[(size_t)(AC * c + u) * E + e] = total;
        total += cv[u];
      }
  }
  if (threadIdx.x / TQ_WAVE == 0) scan_starts(starts, E, unit, cap, tile_expert, n_tiles);
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) table[(size_t)V * E + e] = starts[e];
}

__global__ __launch_bounds__(64 * AW) void align_place_kernel(const int* __restrict__ ids, int n_pairs, int E, int topk,
                                                              const int* __restrict__ table,
                                                              int* __restrict__ pair_slot,
                                                              int* __restrict__ sorted_token) {
  extern __shared__ int sm_a[];        // [AW][E] first rows of this workgroup's waves within the experts, then E starts
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int V = gridDim.x * AW, v = blockIdx.x * AW + wave;
  for (int i = threadIdx.x; i < AW * E; i += blockDim.x) sm_a[i] = table[(size_t)blockIdx.x * AW * E + i];
  for (int e = threadIdx.x; e < E; e += blockDim.x) sm_a[AW * E + e] = table[(size_t)V * E + e];
  __syncthreads();
  const int* off = sm_a + wave * E;
  const int* starts = sm_a + AW * E;
  const int per = ((n_pairs + V - 1) / V + TQ_WAVE - 1) / TQ_WAVE * TQ_WAVE;
  const int seg_beg = min(n_pairs, v * per), seg_end = min(n_pairs, seg_beg + per);
  for (int i0 = seg_beg + lane; i0 < seg_end; i0 += 4 * TQ_WAVE) {
    int e[4], rk[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * TQ_WAVE;
      e[u] = i < seg_end ? ids[i] : 0;
      rk[u] = i < seg_end ? pair_slot[i] : 0;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * TQ_WAVE;
      if (i < seg_end) {
        const int r = starts[e[u]] + off[e[u]] + rk[u];
        pair_slot[i] = r;
        sorted_token[r] = i / topk;
      }
    }
  }
}

// Workgroups for the order of n_pairs pairs by several workgroups, or 0: the one workgroup does it (few pairs, or
// more experts than the scan's LDS holds, or a table too small).  Measured with 60 experts, 4 per token: 8,192 pairs
// 12 us against 17, 32,768 pairs 15 against 56, 131,072 pairs 40 against 225; 4,096 pairs 9 against 8.
#define ALIGN_MULTI_FROM 8192
static int align_workgroups(int n_pairs, int E, size_t table_ints) {
  if (n_pairs < ALIGN_MULTI_FROM) return 0;
  int g = n_pairs / 1024;
  g = g < 2 ? 2 : (g > 16 ? 16 : g);
  const int V = g * AW, chunks = (V + AC - 1) / AC;
  if ((size_t)(V + 1) * E > table_ints) return 0;
  if (((size_t)(chunks + 1) * E + 0) * sizeof(int) > 64 * 1024 || (size_t)(AW + 1) * E * sizeof(int) > 64 * 1024) return 0;
  return g;
}

static int launch_align_multi(const int* ids, int n_pairs, int E, int topk, int unit, int cap, int* sorted_token,
                              int* pair_slot, int* tile_expert, int* n_tiles, int* table, int g, hipStream_t st) {
  const int V = g * AW, chunks = (V + AC - 1) / AC;
  const size_t lds_count = (size_t)AW * E * sizeof(int), lds_scan = (size_t)(chunks + 1) * E * sizeof(int),
               lds_place = (size_t)(AW + 1) * E * sizeof(int);
  if (lds_scan > 48 * 1024)
    (void)hipFuncSetAttribute((const void*)align_scan_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_scan);
  if (lds_place > 48 * 1024) {
    (void)hipFuncSetAttribute((const void*)align_count_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_place);
    (void)hipFuncSetAttribute((const void*)align_place_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_place);
  }
  hipLaunchKernelGGL(align_count_kernel, dim3(g), dim3(64 * AW), lds_count, st, ids, n_pairs, E, cap, sorted_token,
                     pair_slot, table);
  hipLaunchKernelGGL(align_scan_kernel, dim3(1), dim3(64 * AW), lds_scan, st, table, V, E, unit, cap, tile_expert,
                     n_tiles);
  hipLaunchKernelGGL(align_place_kernel, dim3(g), dim3(64 * AW), lds_place, st, ids, n_pairs, E, topk, table, pair_slot,
                     sorted_token);
  TQ_LAUNCH_CHECK();
  return 0;
}

// The choice and the order of pairs in one workgroup of NW waves, for up to NW tokens (decoding): wave w chooses for token w,
// then all waves order the pairs; the same device functions and so the same results as the two kernels.
template <int NW>
__global__ __launch_bounds__(64 * NW) void select_align_kernel(const float* __restrict__ logits, int rows, int E,
                                                               int topk, int renorm, int* __restrict__ ids,
                                                               float* __restrict__ weights,
                                                               float* __restrict__ shared_gate, int T, int unit,
                                                               int cap, int* __restrict__ sorted_token,
                                                               int* __restrict__ pair_slot,
                                                               int* __restrict__ tile_expert,
                                                               int* __restrict__ n_tiles) {
  extern __shared__ int sm_i[];       // (NW + 1) * E ints for the order, NW * topk ids, NW * E floats for the choice
  int* cnt = sm_i;
  int* ids_l = cnt + (NW + 1) * E;
  float* lg = (float*)(ids_l + NW * topk);
  const int wave = threadIdx.x / TQ_WAVE;
  if (wave < T)
    select_token(logits + (size_t)wave * rows, rows, E, topk, renorm, lg + wave * E, ids + (size_t)wave * topk,
                 ids_l + wave * topk, weights + (size_t)wave * topk, shared_gate + wave);
  __syncthreads();
  align_pairs<NW>(ids_l, T * topk, E, topk, unit, cap, sorted_token, pair_slot, tile_expert, n_tiles, cnt);
}

// cap: rows that sorted_token holds, a multiple of unit and at least n_pairs + min(E, n_pairs) * (unit - 1);
// tile_expert holds 2 * cap / unit entries (row tiles, then items), n_tiles two.
TQ_API int tq_moe_align(const int* ids, int n_pairs, int E, int topk, int unit, int cap, int* sorted_token,
                        int* pair_slot, int* tile_expert, int* n_tiles, hipStream_t st) {
  if (n_pairs <= 0) return 0;
  if (unit < 1 || cap % unit != 0 || cap < n_pairs + (E < n_pairs ? E : n_pairs) * (unit - 1)) return TQ_ERR_BAD_ARG;
  const size_t shmem = (size_t)(AW + 1) * E * sizeof(int);
  if (shmem > 160 * 1024) return TQ_ERR_UNSUPPORTED;
  if (shmem > 48 * 1024)
    (void)hipFuncSetAttribute((const void*)moe_align_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(64 * AW), shmem, st, ids, n_pairs, E, topk, unit, cap,
                     sorted_token, pair_slot, tile_expert, n_tiles);
  TQ_LAUNCH_CHECK();
  return 0;
}

// tq_router_topk followed by tq_moe_align; up to 16 tokens take two kernels instead of three, and from 8,192 pairs on
// several workgroups order the pairs (the same order).  logits: scratch of T * (E + 1) floats (T * E without a shared
// gate vector); what it holds afterwards means nothing.
TQ_API int tq_route(const float* x, const void* wr, const void* shared_w, int wtype, int E, int topk, int renorm,
                    int* ids, float* weights, float* shared_gate, float* logits, int unit, int cap, int* sorted_token,
                    int* pair_slot, int* tile_expert, int* n_tiles, int T, int H, hipStream_t st) {
  if (T <= 0) return 0;
  const size_t shmem = ((size_t)(AW + 1) * E + (size_t)AW * topk + (size_t)AW * E) * 4;
  if (T > AW || shmem > 64 * 1024) {
    const int rc = tq_router_topk(x, wr, shared_w, wtype, E, topk, renorm, ids, weights, shared_gate, logits, T, H, st);
    if (rc) return rc;
    // once the experts are chosen the logits are done with: the order by several workgroups keeps its table there
    const int n = T * topk;
    const int g = align_workgroups(n, E, (size_t)T * (E + (shared_w ? 1 : 0)));
    if (g == 0) return tq_moe_align(ids, n, E, topk, unit, cap, sorted_token, pair_slot, tile_expert, n_tiles, st);
    if (unit < 1 || cap % unit != 0 || cap < n + (E < n ? E : n) * (unit - 1)) return TQ_ERR_BAD_ARG;
    return launch_align_multi(ids, n, E, topk, unit, cap, sorted_token, pair_slot, tile_expert, n_tiles, (int*)logits, g,
                              st);
  }
  if (topk < 1 || topk > 64 || topk > E || E > 8192) return TQ_ERR_UNSUPPORTED;
  const int n_pairs = T * topk;
  if (unit < 1 || cap % unit != 0 || cap < n_pairs + (E < n_pairs ? E : n_pairs) * (unit - 1)) return TQ_ERR_BAD_ARG;
  const int rc = launch_router_logits(x, wr, shared_w, wtype, E, logits, T, H, st);
  if (rc) return rc;
  if (T == 1) {      // one wave: its barriers cost nothing
    const size_t shmem1 = ((size_t)2 * E + topk + E) * 4;
    hipLaunchKernelGGL(select_align_kernel<1>, dim3(1), dim3(64), shmem1, st, logits, E + (shared_w ? 1 : 0), E, topk,
                       renorm, ids, weights, shared_gate, T, unit, cap, sorted_token, pair_slot, tile_expert, n_tiles);
    TQ_LAUNCH_CHECK();
    return 0;
  }
  if (shmem > 48 * 1024)
    (void)hipFuncSetAttribute((const void*)select_align_kernel<AW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  hipLaunchKernelGGL(select_align_kernel<AW>, dim3(1), dim3(64 * AW), shmem, st, logits, E + (shared_w ? 1 : 0), E, topk,
                     renorm, ids, weights, shared_gate, T, unit, cap, sorted_token, pair_slot, tile_expert, n_tiles);
  TQ_LAUNCH_CHECK();
  return 0;
}
