// Row-wise kernels: embedding rows, residual sum + RMS norm, rotary position encoding with
// the write of keys and values into cache pages, and the weighted sum of expert outputs.
// All of them are bound by memory traffic; each fuses what would otherwise be a second pass.
#include "common.h"

// ---------------------------------------------------------------- embedding
// x[t, :] = table[tokens[t], :] widened to float; no scaling for this architecture
// (/root/reference/src/engine/tq_transformer.c:2297-2329); `scale` other than 1 multiplies the row, for the
// architectures that scale their embeddings (tq_transformer.c:2332).
template <class W>
__global__ void embed_kernel(const int* __restrict__ tokens, const W* __restrict__ table,
                             float* __restrict__ x, int H, float scale) {
  const int t = blockIdx.x;
  const W* row = table + (size_t)tokens[t] * H;
  float* out = x + (size_t)t * H;
  if (scale == 1.0f) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = to_f32(row[i]);
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = to_f32(row[i]) * scale;
  }
}

TQ_API int tq_embed(const int* tokens, const void* table, int wtype, float* x, int T, int H, float scale, hipStream_t st) {
  if (T <= 0) return 0;
  TQ_DISPATCH_W(wtype, { hipLaunchKernelGGL(embed_kernel<W>, dim3(T), dim3(256), 0, st, tokens, (const W*)table, x, H, scale); });
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- a soft cap on logits
// x <- cap * tanh(x / cap), in place: what a model plan may ask for between the vocabulary product and sampling.
__global__ void softcap_kernel(float* __restrict__ x, int64_t n, float cap) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

TQ_API int tq_softcap(float* x, int64_t n, float cap, hipStream_t st) {
  if (n <= 0) return 0;
  if (!(cap > 0.f)) return TQ_ERR_BAD_ARG;
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, x, n, cap);
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- rows by index
// The rows of a sequence's fixed-size state lie at its slot; a step works on the rows of its own sequences.
// gather: dst[i] = src[idx[i]];  scatter: dst[idx[i]] = src[i];  rows of `words` 32-bit words.  grid (rows, chunks).
__global__ void move_rows_kernel(const uint32_t* __restrict__ src, const int* __restrict__ idx, uint32_t* __restrict__ dst,
                                 int64_t words, int scatter) {
  const int64_t row = blockIdx.x, at = idx[row];
  const uint32_t* from = src + (scatter ? row : at) * words;
  uint32_t* to = dst + (scatter ? at : row) * words;
  for (int64_t w = (int64_t)blockIdx.y * blockDim.x + threadIdx.x; w < words; w += (int64_t)gridDim.y * blockDim.x) to[w] = from[w];
}

// src, dst: rows of row_bytes bytes (a multiple of 4); idx [n]: for gather the row of src behind each row of dst, for
// scatter the row of dst that each row of src goes to (every index once).
TQ_API int tq_move_rows(const void* src, const int* idx, void* dst, int n, int64_t row_bytes, int scatter, hipStream_t st) {
  if (n <= 0 || row_bytes <= 0) return 0;
  if (row_bytes % 4 != 0 || n > 65535 * 32768) return TQ_ERR_UNSUPPORTED;
  const int64_t words = row_bytes / 4;
  const int chunks = (int)((words + 1023) / 1024 < 1024 ? (words + 1023) / 1024 : 1024);
  hipLaunchKernelGGL(move_rows_kernel, dim3(n, chunks), dim3(256), 0, st, (const uint32_t*)src, idx, (uint32_t*)dst, words, scatter);
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- residual sum + RMS norm
// For row r (token rows[r], or r itself when rows is null):
//   v = x[row] + d[row]                         (the residual sum, in float)
//   x[row] = v                                  (only when rows is null)
//   ss = sum v^2 / H + eps ; out = (v * (1/sqrt(ss))) * w
// Formula and product order of /root/reference/src/engine/tq_ops.c:1373-1410.  What is added, d, is either
//   the partial sums delta[s][row] one after the other, s ascending (each added to v in turn), or, with y set,
//   the experts' outputs that nobody has summed yet, as moe_combine below would:
//   d = sum_j weights[row][j] * y[pair_slot[row][j]] (j ascending) + gate[row] * sum_s delta[s][row].
// The sum of squares is taken in a fixed order that does not depend on the number of rows.
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 load4f(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 load4f(const bf16_t* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return f32x4{__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
               __uint_as_float(u.y & 0xffff0000u)};
}
__device__ __forceinline__ void store4(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, f32x4 v) {
  uint2 u;
  u.x = (uint32_t)f32_to_bf16(v.x).bits | ((uint32_t)f32_to_bf16(v.y).bits << 16);
  u.y = (uint32_t)f32_to_bf16(v.z).bits | ((uint32_t)f32_to_bf16(v.w).bits << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

// A thread takes four consecutive elements at a time when H is a multiple of four (every load is 16 bytes and
// all of a thread's loads can be on their way at once), else one element at a time; what is computed per
// element is the same.
template <class W>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ delta, int S,
                                   size_t delta_stride, const float* __restrict__ y,
                                   const int* __restrict__ pair_slot, const float* __restrict__ weights, int topk,
                                   const float* __restrict__ gate, const W* __restrict__ w, float eps,
                                   const int* __restrict__ rows, act_t* __restrict__ out,
                                   float* __restrict__ out32, int H) {
  extern __shared__ __attribute__((aligned(16))) float v[];       // H floats, then one float per wave
  __shared__ int slot[64];
  __shared__ float wgt[64];
  float* red = v + (H + 3) / 4 * 4;
  const int r = blockIdx.x;
  const int row = rows ? rows[r] : r;
  float* xr = x + (size_t)row * H;
  const float* dr = delta + (size_t)row * H;
  float g = 1.0f;
  if (y) {
    if (threadIdx.x < topk) {      // the token's rows and weights once, not once per element
      slot[threadIdx.x] = pair_slot[(size_t)row * topk + threadIdx.x];
      wgt[threadIdx.x] = weights[(size_t)row * topk + threadIdx.x];
    }
    if (gate) g = gate[row];
    __syncthreads();
  }
  const bool vec = H % 4 == 0;
  float ss = 0.f;
  if (vec) {
#pragma unroll 2
    for (int i = threadIdx.x * 4; i < H; i += blockDim.x * 4) {
      // the terms are fetched four at a time and added in their order: the loads of a group are on their way
      // together instead of one after the other
      f32x4 a = load4f(xr + i);
      if (y) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < topk; j += 4) {
          f32x4 t[4];
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (j + u < topk) t[u] = load4f(y + (size_t)slot[j + u] * H + i);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (j + u < topk) acc += wgt[j + u] * t[u];
        }
        if (S > 0) {
          f32x4 sh = {0.f, 0.f, 0.f, 0.f};
          for (int s = 0; s < S; s += 4) {
            f32x4 t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
              if (s + u < S) t[u] = load4f(dr + (s + u) * delta_stride + i);
#pragma unroll
            for (int u = 0; u < 4; ++u)
              if (s + u < S) sh += t[u];
          }
          acc += g * sh;
        }
        a += acc;
      } else {
        for (int s = 0; s < S; s += 4) {
          f32x4 t[4];
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (s + u < S) t[u] = load4f(dr + (s + u) * delta_stride + i);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (s + u < S) a += t[u];
        }
      }
      store4(v + i, a);
      if (!rows) store4(xr + i, a);
      ss += a.x * a.x;
      ss += a.y * a.y;
      ss += a.z * a.z;
      ss += a.w * a.w;
    }
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      float a = xr[i];
      if (y) {
        float acc = 0.f;
        for (int j = 0; j < topk; ++j) acc += wgt[j] * y[(size_t)slot[j] * H + i];
        if (S > 0) {
          float sh = 0.f;
          for (int s = 0; s < S; ++s) sh += dr[s * delta_stride + i];
          acc += g * sh;
        }
        a += acc;
      } else {
        for (int s = 0; s < S; ++s) a += dr[s * delta_stride + i];
      }
      v[i] = a;
      if (!rows) xr[i] = a;
      ss += a * a;
    }
  }
  ss = block_sum(ss, red);
  ss = ss / (float)H + eps;
  const float rs = 1.0f / sqrtf(ss);
  if (vec) {
#pragma unroll 2
    for (int i = threadIdx.x * 4; i < H; i += blockDim.x * 4) {
      const f32x4 o = load4f(v + i) * rs * load4f(w + i);
      if (out) store4(out + (size_t)r * H + i, o);
      if (out32) store4(out32 + (size_t)r * H + i, o);
    }
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float o = v[i] * rs * to_f32(w[i]);
      if (out) out[(size_t)r * H + i] = from_f32<act_t>(o);
      if (out32) out32[(size_t)r * H + i] = o;
    }
  }
}

TQ_API int tq_add_rmsnorm(float* x, const float* delta, int S, int64_t delta_stride, const float* y,
                          const int* pair_slot, const float* weights, int topk, const float* gate, const void* w,
                          int wtype, float eps, const int* rows, int R, void* out, float* out32, int H,
                          hipStream_t st) {
  if (R <= 0) return 0;
  if (y && (topk < 1 || topk > 64 || !pair_slot || !weights)) return TQ_ERR_BAD_ARG;
  // a row of 2,048 and more by 512 threads, so that each takes its four elements in one go and all of a row's loads
  // are on their way at once (a function of H alone: a row's sums do not depend on what else the step holds)
  const int threads = (H % 4 == 0 && H >= 2048) ? 512 : 256;
  const size_t shmem = (size_t)((H + 3) / 4 * 4 + threads / TQ_WAVE) * sizeof(float);
  if (shmem > 150 * 1024) return TQ_ERR_UNSUPPORTED;
  TQ_DISPATCH_W(wtype, {
    if (shmem > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)add_rmsnorm_kernel<W>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    hipLaunchKernelGGL(add_rmsnorm_kernel<W>, dim3(R), dim3(threads), shmem, st, x, delta, S, (size_t)delta_stride, y,
                       pair_slot, weights, topk, gate, (const W*)w, eps, rows, (act_t*)out, out32, H);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- the gate of a gated pair, applied afterwards
// out[m][n] = f(gu[m][n]) * gu[m][N + n]: for a pair of products that came out of one plain product over the two
// matrices laid one behind the other (a library's, which has no such epilogue).  gu is float32 with row stride ld.
template <bool VEC>
__global__ __launch_bounds__(256) void gated_act_kernel(const float* __restrict__ gu, int64_t ld, act_t* __restrict__ out,
                                                        int N, int gate) {
  const float* row = gu + (size_t)blockIdx.y * ld;
  act_t* dst = out + (size_t)blockIdx.y * N;
  if (VEC) {
    const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (n >= N) return;
    const f32x4 g = load4f(row + n), u = load4f(row + N + n);
    store4(dst + n, f32x4{gate_fn(g.x, gate) * u.x, gate_fn(g.y, gate) * u.y, gate_fn(g.z, gate) * u.z,
                          gate_fn(g.w, gate) * u.w});
  } else {
    const int n = blockIdx.x * 256 + threadIdx.x;
    if (n < N) dst[n] = from_f32<act_t>(gate_fn(row[n], gate) * row[N + n]);
  }
}

TQ_API int tq_gated_act(const float* gu, int64_t ld, void* out, int M, int N, int gate, hipStream_t st) {
  if (M <= 0 || N <= 0) return 0;
  if (gate < 0 || gate >= TQ_GATE_COUNT || ld < 2 * (int64_t)N) return TQ_ERR_BAD_ARG;
  if (M > 65535) return TQ_ERR_UNSUPPORTED;
  const bool vec = N % 4 == 0 && ld % 4 == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % 16) == 0;
  if (vec)
    hipLaunchKernelGGL(gated_act_kernel<true>, dim3((N / 4 + 255) / 256, M), dim3(256), 0, st, gu, ld, (act_t*)out, N, gate);
  else
    hipLaunchKernelGGL(gated_act_kernel<false>, dim3((N + 255) / 256, M), dim3(256), 0, st, gu, ld, (act_t*)out, N, gate);
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- RMS norm of every head of q and k
// qkv[t] holds, in float, nh query heads, then nkv key heads, then nkv value heads of hd each.  Every query head is
// normed over its hd values with the weights wq[hd], every key head with wk[hd] (a null pointer leaves those heads
// as they are), in place: the per-head norm between the product and the rotation of
// /root/reference/src/engine/tq_transformer.c:1111-1124, with the formula of tq_ops.c:1373-1410.  A wave per head.
template <class W>
__global__ __launch_bounds__(256) void head_rmsnorm_kernel(float* __restrict__ qkv, const W* __restrict__ wq,
                                                           const W* __restrict__ wk, float eps, int nh, int nkv, int hd) {
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int head = blockIdx.y * 4 + wave;
  if (head >= nh + nkv) return;
  const W* w = head < nh ? wq : wk;
  if (!w) return;
  float* x = qkv + ((size_t)blockIdx.x * (nh + 2 * nkv) + head) * hd;
  float ss = 0.f;
  for (int i = lane; i < hd; i += TQ_WAVE) ss = fmaf(x[i], x[i], ss);
  ss = wave_sum(ss) / (float)hd + eps;
  const float rs = 1.0f / sqrtf(ss);
  for (int i = lane; i < hd; i += TQ_WAVE) x[i] = x[i] * rs * to_f32(w[i]);
}

TQ_API int tq_head_rmsnorm(float* qkv, const void* wq, const void* wk, int wtype, float eps, int T, int nh, int nkv,
                           int hd, hipStream_t st) {
  if (T <= 0 || (!wq && !wk)) return 0;
  if (nh < 0 || nkv < 0 || hd < 1 || (nh + nkv + 3) / 4 > 65535) return TQ_ERR_BAD_ARG;
  TQ_DISPATCH_W(wtype, {
    hipLaunchKernelGGL(head_rmsnorm_kernel<W>, dim3(T, (nh + nkv + 3) / 4), dim3(256), 0, st, qkv, (const W*)wq,
                       (const W*)wk, eps, nh, nkv, hd);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- rotary encoding + cache write
// qkv[t] holds, in float, nh query heads, then nkv key heads, then nkv value heads of hd each.
// Queries and keys are rotated by angle pos * inv_freq[i] (float) on the pair
//   pairing 0 ("half"):        (x[i], x[i + rot/2])   (/root/reference/src/engine/tq_transformer.c:1263-1289)
//   pairing 1 ("interleaved"): (x[2i], x[2i+1])        (/root/reference/src/engine/tq_ops.c:1418-1448)
// as (a, b) <- (a cos - b sin, a sin + b cos); dimensions from rot on pass through.  Rotated queries
// go to q_out; rotated keys and the values go into the page that holds position pos of the token's
// sequence: page = block_table[seq][pos / page_size], row pos % page_size of kv head h.  After the
// layer's own offset (already added to k_pool / v_pool) keys lie [page][kv head][row][hd] and values
// transposed, [page][kv head][hd][row].
// A workgroup of four waves takes `spb` heads of one token (grid (T, ceil(heads / spb))); a wave takes every
// fourth of them and turns pair i of all its heads with one sine and cosine.  write_kv: 0 queries only, 1 keys
// and values, 2 keys only (the values of whole runs of tokens go through v_write_tile_kernel below).
// element i of a bias that the product before did not add; BIAS: 0 none, 1 float32, 2 bfloat16 (a template
// argument, so that the loads of the bias go out beside those of the row and not behind a branch)
template <int BIAS>
__device__ __forceinline__ float bias_elem(const void* bias, size_t i) {
  if (BIAS == 0) return 0.f;
  return BIAS == 1 ? ((const float*)bias)[i] : to_f32(((const bf16_t*)bias)[i]);
}

template <int BIAS>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(const float* __restrict__ qkv, const void* __restrict__ bias,
                                     const int* __restrict__ positions,
                                     const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
                                     int bt_stride, const float* __restrict__ inv_freq, int pairing, int rot,
                                     act_t* __restrict__ q_out, act_t* __restrict__ k_pool,
                                     act_t* __restrict__ v_pool, int page_size, int64_t page_stride, int nh,
                                     int nkv, int hd, int write_kv, int spb) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int heads = nh + 2 * nkv;       // 0..nh-1 query heads, then key heads, then value heads
  const int s0 = blockIdx.y * spb + wave, s1 = min(blockIdx.y * spb + spb, heads);
  if (s0 >= s1) return;
  const int pos = positions[t];
  const float* src_t = qkv + (size_t)t * heads * hd;
  act_t* q_t = q_out + (size_t)t * nh * hd;
  act_t *k_t = nullptr, *v_t = nullptr;      // the token's row of kv head 0 in its page
  if (write_kv && s1 > nh) {
    const int page = block_table[(size_t)seq_of_token[t] * bt_stride + pos / page_size];
    const int row = pos % page_size;
    k_t = k_pool + (size_t)page * page_stride + (size_t)row * hd;
    v_t = v_pool + (size_t)page * page_stride + row;
  }
  const int rot_end = write_kv ? min(s1, nh + nkv) : min(s1, nh);     // heads below this are rotated
  const size_t kv_head_stride = (size_t)page_size * hd;
  const int half = rot / 2;
  for (int i = lane; i < half; i += TQ_WAVE) {
    const float theta = (float)pos * inv_freq[i];
    float sn, cs;
    sincosf(theta, &sn, &cs);
    const int ia = pairing == 0 ? i : 2 * i;
    const int ib = pairing == 0 ? i + half : 2 * i + 1;
    for (int s = s0; s < rot_end; s += 4) {
      const float* src = src_t + (size_t)s * hd;
      act_t* dst = s < nh ? q_t + (size_t)s * hd : k_t + (size_t)(s - nh) * kv_head_stride;
      const float a = src[ia] + bias_elem<BIAS>(bias, (size_t)s * hd + ia);
      const float b = src[ib] + bias_elem<BIAS>(bias, (size_t)s * hd + ib);
      dst[ia] = from_f32<act_t>(a * cs - b * sn);
      dst[ib] = from_f32<act_t>(a * sn + b * cs);
    }
  }
  for (int s = s0; s < rot_end; s += 4) {      // dimensions from rot on pass through
    const float* src = src_t + (size_t)s * hd;
    act_t* dst = s < nh ? q_t + (size_t)s * hd : k_t + (size_t)(s - nh) * kv_head_stride;
    for (int i = rot + lane; i < hd; i += TQ_WAVE)
      dst[i] = from_f32<act_t>(src[i] + bias_elem<BIAS>(bias, (size_t)s * hd + i));
  }
  if (write_kv != 1) return;
  for (int s = s0; s < s1; s += 4) {           // values lie transposed, [hd][row]
    if (s < nh + nkv) continue;
    const float* src = src_t + (size_t)s * hd;
    act_t* col = v_t + (size_t)(s - nh - nkv) * kv_head_stride;
    for (int i = lane; i < hd; i += TQ_WAVE)
      col[(size_t)i * page_size] = from_f32<act_t>(src[i] + bias_elem<BIAS>(bias, (size_t)s * hd + i));
  }
}

// The values of runs of tokens, one run per sequence (tokens cu_seqlens[b] .. of sequence b lie at positions
// start[b] ..): a workgroup takes 64 positions that share a page (grid (chunks, nkv, B)), turns their rows
// [position][hd] into [hd][position] in LDS and writes every dimension's positions 16 bytes at a time, where the
// token-by-token write above would touch a cache line per dimension for two bytes.
#define VT_POS 64
template <int VEC, int BIAS>      // positions per 16-byte store; the bias as in rope_kv_write_kernel
__global__ __launch_bounds__(256) void v_write_tile_kernel(const float* __restrict__ qkv,
                                                           const void* __restrict__ bias,
                                                           const int* __restrict__ cu_seqlens,
                                                           const int* __restrict__ slots,
                                                           const int* __restrict__ start,
                                                           const int* __restrict__ block_table, int bt_stride,
                                                           act_t* __restrict__ v_pool, int page_size,
                                                           int64_t page_stride, int nh, int nkv, int hd) {
  extern __shared__ __attribute__((aligned(16))) unsigned char vt_raw[];
  act_t* ts = (act_t*)vt_raw;                        // [hd][VT_POS + VEC]
  constexpr int TS = VT_POS + VEC;
  const int b = blockIdx.z, h = blockIdx.y;
  const int t0 = cu_seqlens[b], n = cu_seqlens[b + 1] - t0, st = start[b];
  const int P0 = (st / VT_POS + blockIdx.x) * VT_POS;
  const int lo = max(P0, st), hi = min(P0 + VT_POS, st + n);
  if (lo >= hi) return;
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int heads = nh + 2 * nkv;
  const float* src0 = qkv + ((size_t)(t0 + lo - st) * heads + nh + nkv + h) * hd;      // value row of position lo
  const size_t row_stride = (size_t)heads * hd;
  const size_t bias0 = (size_t)(nh + nkv + h) * hd;      // the bias of this value head
  if (hd % 4 == 0) {        // 16 bytes of a row per thread and turn, all of a thread's loads on their way at once
    const int q4 = hd / 4, total = (hi - lo) * q4;
#pragma unroll 8
    for (int idx = threadIdx.x; idx < total; idx += 256) {
      const int r = idx / q4, d = (idx % q4) * 4;
      const f32x4 v = load4f(src0 + r * row_stride + d);
      act_t* to = ts + d * TS + (lo + r - P0);
      to[0] = from_f32<act_t>(v.x + bias_elem<BIAS>(bias, bias0 + d));
      to[TS] = from_f32<act_t>(v.y + bias_elem<BIAS>(bias, bias0 + d + 1));
      to[2 * TS] = from_f32<act_t>(v.z + bias_elem<BIAS>(bias, bias0 + d + 2));
      to[3 * TS] = from_f32<act_t>(v.w + bias_elem<BIAS>(bias, bias0 + d + 3));
    }
  } else {
    for (int r = wave; r < hi - lo; r += 4)
      for (int d = lane; d < hd; d += TQ_WAVE)
        ts[d * TS + (lo + r - P0)] = from_f32<act_t>(src0[r * row_stride + d] + bias_elem<BIAS>(bias, bias0 + d));
  }
  __syncthreads();
  const int page = block_table[(size_t)slots[b] * bt_stride + P0 / page_size];
  act_t* base = v_pool + (size_t)page * page_stride + (size_t)h * page_size * hd + P0 % page_size;
  constexpr int GROUPS = VT_POS / VEC;
  for (int idx = threadIdx.x; idx < hd * GROUPS; idx += blockDim.x) {
    const int d = idx / GROUPS, g = idx % GROUPS;
    const int p0 = P0 + g * VEC;
    act_t* dst = base + (size_t)d * page_size + g * VEC;
    const act_t* from = ts + d * TS + g * VEC;
    if (p0 >= lo && p0 + VEC <= hi) {
      *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(from);
    } else {
      for (int j = max(p0, lo) - p0; j < min(p0 + VEC, hi) - p0; ++j) dst[j] = from[j];
    }
  }
}

// cu_seqlens, slots, start (null, or [B + 1], [B], [B] with max_new the longest run): the tokens as runs of
// consecutive positions, one per sequence; given for whole prompts, they let the values go by tiles.
// bias (null, or [(nh + 2 nkv) * hd] of bias_type): added to qkv as it is read, for a product that left it out.
TQ_API int tq_rope_kv_write(const float* qkv, const void* bias, int bias_type, const int* positions, const int* seq_of_token,
                            const int* block_table, int bt_stride, const float* inv_freq, int pairing, int rot,
                            void* q_out, void* k_pool, void* v_pool, int page_size, int64_t page_stride, int T,
                            int nh, int nkv, int hd, int write_kv, const int* cu_seqlens, const int* slots,
                            const int* start, int B, int max_new, hipStream_t st) {
  if (T <= 0) return 0;
  if (rot < 0 || rot > hd || (rot & 1) || (pairing != 0 && pairing != 1)) return TQ_ERR_BAD_ARG;
  if (bias && bias_type != TQ_F32 && bias_type != TQ_BF16) return TQ_ERR_BAD_ARG;
  constexpr int VEC = 16 / (int)sizeof(act_t);
  const size_t vt_shmem = (size_t)hd * (VT_POS + VEC) * sizeof(act_t);
  const bool tiles = write_kv && cu_seqlens && slots && start && B > 0 && B <= 65535 && nkv <= 65535 && max_new > 8 &&
                     page_size % VT_POS == 0 && vt_shmem <= 64 * 1024;
  if (tiles) write_kv = 2;
  const int heads = nh + 2 * nkv;
  // few tokens: a head per wave, so that the chip sees many small workgroups; many: all heads of a token in one
  int spb = 4;
  while (spb < heads && (int64_t)T * ((heads + spb - 1) / spb) > 4096) spb *= 2;
  if ((heads + spb - 1) / spb > 65535) return TQ_ERR_UNSUPPORTED;
  const int bias_kind = !bias ? 0 : bias_type == TQ_F32 ? 1 : 2;
#define TQ_ROPE_LAUNCH(BIAS)                                                                                          \
  hipLaunchKernelGGL(rope_kv_write_kernel<BIAS>, dim3(T, (heads + spb - 1) / spb), dim3(256), 0, st, qkv, bias,       \
                     positions, seq_of_token, block_table, bt_stride, inv_freq, pairing, rot, (act_t*)q_out,          \
                     (act_t*)k_pool, (act_t*)v_pool, page_size, page_stride, nh, nkv, hd, write_kv, spb)
  if (bias_kind == 0) TQ_ROPE_LAUNCH(0);
  else if (bias_kind == 1) TQ_ROPE_LAUNCH(1);
  else TQ_ROPE_LAUNCH(2);
#undef TQ_ROPE_LAUNCH
  TQ_LAUNCH_CHECK();
  if (tiles) {
#define TQ_VT_LAUNCH(BIAS)                                                                                            \
  do {                                                                                                                \
    if (vt_shmem > 48 * 1024)                                                                                         \
      (void)hipFuncSetAttribute((const void*)v_write_tile_kernel<VEC, BIAS>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                (int)vt_shmem);                                                                       \
    hipLaunchKernelGGL((v_write_tile_kernel<VEC, BIAS>), dim3((max_new + VT_POS - 1) / VT_POS + 1, nkv, B), dim3(256), \
                       vt_shmem, st, qkv, bias, cu_seqlens, slots, start, block_table, bt_stride, (act_t*)v_pool,     \
                       page_size, page_stride, nh, nkv, hd);                                                          \
  } while (0)
    if (bias_kind == 0) TQ_VT_LAUNCH(0);
    else if (bias_kind == 1) TQ_VT_LAUNCH(1);
    else TQ_VT_LAUNCH(2);
#undef TQ_VT_LAUNCH
    TQ_LAUNCH_CHECK();
  }
  return 0;
}

// ---------------------------------------------------------------- sum of expert outputs
// out[t] = sum_j weights[t][j] * y[slot[t][j]]   (j ascending: the order in which experts were selected,
//          /root/reference/src/engine/tq_moe.c:720,864-999)
//        + gate[t] * sum_s shared[s][t]           (shared expert last, tq_moe.c:1005-1058)
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ pair_slot,
                                                          const float* __restrict__ weights, int topk,
                                                          const float* __restrict__ shared, int S, size_t shared_stride,
                                                          const float* __restrict__ gate, float* __restrict__ out, int H) {
  __shared__ int slot[64];
  __shared__ float wgt[64];
  const int t = blockIdx.x;
  if (threadIdx.x < topk) {      // the token's rows and weights once, not once per element
    slot[threadIdx.x] = pair_slot[t * topk + threadIdx.x];
    wgt[threadIdx.x] = weights[t * topk + threadIdx.x];
  }
  __syncthreads();
  const float g = gate ? gate[t] : 1.0f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < topk; ++j) acc += wgt[j] * y[(size_t)slot[j] * H + i];
    if (shared) {
      float sh = 0.f;
      for (int s = 0; s < S; ++s) sh += shared[s * shared_stride + (size_t)t * H + i];
      acc += g * sh;
    }
    out[(size_t)t * H + i] = acc;
  }
}

TQ_API int tq_moe_combine(const float* y, const int* pair_slot, const float* weights, int topk,
                          const float* shared, int S, int64_t shared_stride, const float* gate, float* out, int T,
                          int H, hipStream_t st) {
  if (T <= 0) return 0;
  if (topk < 1 || topk > 64) return TQ_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, st, y, pair_slot, weights, topk, shared, S,
                     (size_t)shared_stride, gate, out, H);
  TQ_LAUNCH_CHECK();
  return 0;
}
