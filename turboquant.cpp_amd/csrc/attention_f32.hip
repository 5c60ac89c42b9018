// Attention over the cache pages in true 32-bit floating point on the matrix cores (v_mfma_f32_16x16x4_f32).
//
// The formulas are those of the plain kernel (attention_generic.hip): token at position p attends to positions
// lo..p, lo = max(0, p - window + 1) with a window (/root/reference/src/engine/tq_transformer.c:1646-1654), query
// head h reads kv head h / (nh / nkv) (:1675-1679), score = (q . k) * scale (:1908-1937), softmax with a running
// maximum (/root/reference/src/engine/tq_ops.c:1496-1519), output = sum p_j v_j (tq_transformer.c:1975-1976).
// Two kernels:
//
//  * attn_f32_prefill_kernel, for runs of tokens (prompts): a workgroup takes 64 consecutive tokens of one sequence
//    and one head, 16 tokens to a wave; keys and values are staged through LDS one tile of 64 positions at a time,
//    once for the whole block.
//  * attn_f32_decode_kernel + attn_f32_join_kernel, for one token per sequence: a wave takes one tile of 64
//    positions for all heads of a kv group (up to 16 to a pass), straight from the pages into the operand registers,
//    and leaves (maximum, sum, weighted values); the join adds the tiles up in order.
//
// Both compute S^T = K Q^T (keys are the rows, so a lane holds 4 keys of one query) and O^T += V^T P^T, so that the
// probabilities go into the second product from the registers they are born in; values lie transposed in the
// pages ([hd][row]) as that product's first operand wants them.  Tiles start at multiples of 64 positions, and a
// token's sums run over its tiles in ascending order, whatever else is in the batch.
//
// 16x16x4 operand layout (wave of 64 lanes): A lane l = row l%16, k l/16; B lane l = column l%16, k l/16; D lane l =
// column l%16, rows 4*(l/16) + v, v<4.  A lane's 16 bytes of an operand row are 4 consecutive elements of the
// contraction, used one by one by four instructions.
#include "common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));

#define AT 64            // positions per tile

struct AttnF32Args {
  const float* q;          // [T][nh][hd]
  const float* k_pool;     // the layer's keys: page p at k_pool + p * page_stride, [kv head][row][hd]
  const float* v_pool;     // values, [kv head][hd][row]
  const int* block_table;  // [slots][bt_stride]
  int bt_stride;
  const int* cu_seqlens;   // [B + 1]: first token of each sequence's run
  const int* slots;        // [B]
  const int* start;        // [B]: position of the run's first token
  int page_size;
  int64_t page_stride;
  int nh, nkv, hd, window;
  float scale;
  float* out;              // [T][nh][hd]
  float* partial;          // decode: [B][nh][tiles][hd + 2]
  int tiles_max;           // decode: tiles per sequence in `partial`
};

// Lanes l and l ^ 8 (the same quarter g = l / 16, rows r and r ^ 8 of 16) fetched whole lines: lane (r, g) chunk
// g + 4 (r / 8) of row r % 8 into t0 and of row 8 + r % 8 into t1.  Afterwards t0 is chunk g and t1 chunk g + 4 of
// the lane's own row r.
__device__ __forceinline__ void to_own_row(f32x4& t0, f32x4& t1) {
  f32x4 s0, s1;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    // row_ror:8 reads lane l ^ 8 of each row of 16 lanes; the bank mask says which lanes take it (0xc: 8..15, 0x3: 0..7)
    s0[i] = __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(t0[i]), __float_as_int(t1[i]), 0x128, 0xf, 0xc, false));
    s1[i] = __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(t1[i]), __float_as_int(t0[i]), 0x128, 0xf, 0x3, false));
  }
  t0 = s0;
  t1 = s1;
}

__device__ __forceinline__ float group_max(float v) {       // over the four lanes l, l^16, l^32, l^48
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  return fmaxf(v, __shfl_xor(v, 32, 64));
}
__device__ __forceinline__ float group_sum(float v) {
  v += __shfl_xor(v, 16, 64);
  return v + __shfl_xor(v, 32, 64);
}

// One tile of 64 keys for 16 queries: scores from `kf` (reads the key operand of subtile kt, chunk u), softmax
// update, and the product with the values from `vf` (value operand of d-tile dt, subtile kt).
template <int ND, class KF, class VF>
__device__ __forceinline__ void attend_tile(const f32x4 (&qf)[ND], KF kf, VF vf, int key0, int pos_q, int lo_q, float scale,
                                            float& m_run, float& l_run, f32x4 (&acc)[ND]) {
  const int g = (threadIdx.x % 64) / 16;
  f32x4 s[4];
#pragma unroll
  for (int kt = 0; kt < 4; ++kt) {
    s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < ND; ++u) {
      const f32x4 a = kf(kt, u);
#pragma unroll
      for (int i = 0; i < 4; ++i) s[kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], qf[u][i], s[kt], 0, 0, 0);
    }
  }
  float m_tile = -INFINITY;
#pragma unroll
  for (int kt = 0; kt < 4; ++kt)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int j = key0 + 16 * kt + 4 * g + v;
      const float x = (j <= pos_q && j >= lo_q) ? s[kt][v] * scale : -INFINITY;
      s[kt][v] = x;
      m_tile = fmaxf(m_tile, x);
    }
  m_tile = group_max(m_tile);
  // (a query that has nothing in its reach so far keeps a maximum of -inf: its probabilities and its factor for what
  // came before are 0 below, never exp(-inf + inf); all lanes stay together for the matrix instructions)
  const float m_new = fmaxf(m_run, m_tile);
  float l_tile = 0.f;
#pragma unroll
  for (int kt = 0; kt < 4; ++kt)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const float p = s[kt][v] == -INFINITY ? 0.f : expf(s[kt][v] - m_new);
      s[kt][v] = p;
      l_tile += p;
    }
  l_tile = group_sum(l_tile);
  const float alpha = m_run == -INFINITY ? 0.f : expf(m_run - m_new);
  l_run = l_run * alpha + l_tile;
  m_run = m_new;
#pragma unroll
  for (int dt = 0; dt < ND; ++dt) {
    acc[dt] *= alpha;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      const f32x4 a = vf(dt, kt);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], s[kt][i], acc[dt], 0, 0, 0);
    }
  }
}

// ------------------------------------------------------------------------------------------ runs of tokens
template <int ND>
__global__ __launch_bounds__(256) void attn_f32_prefill_kernel(AttnF32Args p, int blocks_per_seq) {
  extern __shared__ __align__(16) float lds[];
  constexpr int HDP = 16 * ND, KLD = HDP + 4, VLD = AT + 4;
  float* Ks = lds;                    // [AT][KLD]
  float* Vt = lds + AT * KLD;         // [HDP][VLD]
  const int seq = blockIdx.x / blocks_per_seq, blk = blockIdx.x % blocks_per_seq;
  const int h = blockIdx.y, kvh = h / (p.nh / p.nkv);
  const int t0 = p.cu_seqlens[seq], n_new = p.cu_seqlens[seq + 1] - t0;
  if (blk * 64 >= n_new) return;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, r = lane % 16, g = lane / 16;
  // head sizes that do not fill their last 16: the padding is multiplied by zeros of the queries, so it must hold numbers
  for (int i = tid; i < AT * KLD + HDP * VLD; i += 256) lds[i] = 0.f;
  const int start = p.start[seq];
  const int* table = p.block_table + (size_t)p.slots[seq] * p.bt_stride;
  const int hd = p.hd;

  // this lane's query: token blk * 64 + wave * 16 + r of the run
  const int qi = blk * 64 + wave * 16 + r;
  const bool q_ok = qi < n_new;
  const int pos_q = q_ok ? start + qi : -1;
  const int lo_q = p.window > 0 ? max(0, pos_q - p.window + 1) : 0;
  f32x4 qf[ND];
  const float* qrow = p.q + ((size_t)(t0 + (q_ok ? qi : 0)) * p.nh + h) * hd;
#pragma unroll
  for (int u = 0; u < ND; ++u) {
    const int d = 16 * u + 4 * g;
    qf[u] = q_ok && d < hd ? *reinterpret_cast<const f32x4*>(qrow + d) : f32x4{0.f, 0.f, 0.f, 0.f};
  }
  f32x4 acc[ND];
#pragma unroll
  for (int dt = 0; dt < ND; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

  // what the block as a whole can reach, and what this wave can
  const int blk_first = start + blk * 64, blk_last = start + min(n_new, blk * 64 + 64) - 1;
  const int blk_lo = p.window > 0 ? max(0, blk_first - p.window + 1) : 0;
  const int wave_first = start + blk * 64 + wave * 16, wave_last = min(blk_last, wave_first + 15);
  const int wave_lo = p.window > 0 ? max(0, wave_first - p.window + 1) : 0;

  for (int tile = blk_lo / AT; tile * AT <= blk_last; ++tile) {
    const int key0 = tile * AT;
    const int page = table[key0 / p.page_size];
    __syncthreads();          // the tile before has been used by every wave
    if (page >= 0) {
      const float* kp = p.k_pool + (size_t)page * p.page_stride + ((size_t)kvh * p.page_size + key0 % p.page_size) * hd;
      const int per_row = hd / 4;
      for (int idx = tid; idx < AT * per_row; idx += 256) {
        const int row = idx / per_row, c = idx % per_row;
        *reinterpret_cast<f32x4*>(&Ks[row * KLD + 4 * c]) = *reinterpret_cast<const f32x4*>(kp + (size_t)row * hd + 4 * c);
      }
      const float* vp = p.v_pool + (size_t)page * p.page_stride + (size_t)kvh * p.page_size * hd + key0 % p.page_size;
      for (int idx = tid; idx < hd * (AT / 4); idx += 256) {
        const int d = idx / (AT / 4), c = idx % (AT / 4);
        *reinterpret_cast<f32x4*>(&Vt[d * VLD + 4 * c]) = *reinterpret_cast<const f32x4*>(vp + (size_t)d * p.page_size + 4 * c);
      }
    }
    __syncthreads();
    if (page < 0) continue;             // a page that its group has given back: nothing of it is in anyone's reach
    if (key0 > wave_last || key0 + AT <= wave_lo) continue;
    attend_tile<ND>(
        qf, [&](int kt, int u) { return *reinterpret_cast<const f32x4*>(&Ks[(16 * kt + r) * KLD + 16 * u + 4 * g]); },
        [&](int dt, int kt) { return *reinterpret_cast<const f32x4*>(&Vt[(16 * dt + r) * VLD + 16 * kt + 4 * g]); },
        key0, pos_q, lo_q, p.scale, m_run, l_run, acc);
  }
  if (!q_ok) return;
  const float inv = 1.0f / l_run;
  float* orow = p.out + ((size_t)(t0 + qi) * p.nh + h) * hd;
#pragma unroll
  for (int dt = 0; dt < ND; ++dt) {
    const int d = 16 * dt + 4 * g;
    if (d < hd) *reinterpret_cast<f32x4*>(orow + d) = acc[dt] * inv;
  }
}

// ------------------------------------------------------------------------------------------ one token per sequence
// grid (B, nkv * passes, tiles), one wave each: wave z of a sequence takes the z-th tile of its reach for up to 16
// heads of one kv group; what it finds goes to partial[b][head][tile] = (maximum, sum, weighted values[hd]).
// Keys and values go from the pages straight into the operand registers as the products come to them, by whole
// lines of 128 bytes where the head size allows (a multiple of 32): lanes l and l ^ 8 fetch for each other and
// exchange (to_own_row).  Four or five waves share a SIMD, and while some wait for memory others multiply.
// Measured at 64 sequences of 1,071 positions on average, 16 heads of 128, a layer: 414 us with half lines per
// instruction, a tile per wave and four waves to a workgroup; 286 with whole lines; 277 with one wave to a
// workgroup.  Asking for a whole tile before the first product leaves one or two waves to a SIMD, whose loads and
// products then take turns instead of overlapping: 474 to 512 us.  A wave that takes two or three tiles in turn
// (half or a third as many waves, fewer of them empty) needs 118 registers instead of 90 and gains nothing: 302 to 306 us.
template <int ND, bool LINES>
__global__ __launch_bounds__(64) void attn_f32_decode_kernel(AttnF32Args p, int passes) {
  const int b = blockIdx.x, kvh = blockIdx.y / passes, pass = blockIdx.y % passes;
  const int lane = threadIdx.x, r = lane % 16, g = lane / 16;
  const int pos = p.start[b];                       // the token's position: it attends to lo..pos
  const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  const int first = lo / AT, last = pos / AT;
  const int tile = first + blockIdx.z;
  if (tile > last) return;
  const int* table = p.block_table + (size_t)p.slots[b] * p.bt_stride;
  const int hd = p.hd, group = p.nh / p.nkv;
  const int hq = pass * 16 + r;                     // this lane's query: head hq of the group
  const bool q_ok = hq < group;
  const int h = kvh * group + (q_ok ? hq : 0);
  const int t = p.cu_seqlens[b];
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  f32x4 qf[ND];
  const float* qrow = p.q + ((size_t)t * p.nh + h) * hd;
#pragma unroll
  for (int u = 0; u < ND; ++u) {
    const int d = 16 * u + 4 * g;
    qf[u] = *reinterpret_cast<const f32x4*>(d < hd ? qrow + d : qrow);
    qf[u] = q_ok && d < hd ? qf[u] : zero;
  }
  {
    const int key0 = tile * AT;
    const int page = table[key0 / p.page_size];
    f32x4 acc[ND];
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) acc[dt] = zero;
    float m_run = -INFINITY, l_run = 0.f;
    const float* kp = p.k_pool + (size_t)page * p.page_stride + ((size_t)kvh * p.page_size + key0 % p.page_size) * hd;
    const float* vp = p.v_pool + (size_t)page * p.page_stride + (size_t)kvh * p.page_size * hd + key0 % p.page_size;
    if (LINES) {
      const int r8 = r % 8, ch = 4 * (g + 4 * (r / 8));
      f32x4 k_next, v_next;
      attend_tile<ND>(
          qf,
          [&](int kt, int u) {
            if (u % 2) return k_next;
            const float* base = kp + (size_t)(16 * kt + r8) * hd + 16 * u + ch;
            f32x4 t0 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(base));
            f32x4 t1 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(base + (size_t)8 * hd));
            to_own_row(t0, t1);
            k_next = t1;
            return t0;
          },
          [&](int dt, int kt) {
            if (kt % 2) return v_next;
            const float* base = vp + (size_t)(16 * dt + r8) * p.page_size + 16 * kt + ch;
            f32x4 t0 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(base));
            f32x4 t1 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(base + (size_t)8 * p.page_size));
            to_own_row(t0, t1);
            v_next = t1;
            return t0;
          },
          key0, q_ok ? pos : -1, lo, p.scale, m_run, l_run, acc);
    } else {
      // (what lies beyond the head size is asked for at the tile's first address instead and replaced by zeros:
      // every lane loads, so that no load waits behind a branch)
      attend_tile<ND>(
          qf,
          [&](int kt, int u) {
            const int d = 16 * u + 4 * g;
            const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(d < hd ? kp + (size_t)(16 * kt + r) * hd + d : kp));
            return d < hd ? x : zero;
          },
          [&](int dt, int kt) {
            const int d = 16 * dt + r;
            const f32x4 x = __builtin_nontemporal_load(
                reinterpret_cast<const f32x4*>(d < hd ? vp + (size_t)d * p.page_size + 16 * kt + 4 * g : vp));
            return d < hd ? x : zero;
          },
          key0, q_ok ? pos : -1, lo, p.scale, m_run, l_run, acc);
    }
    if (!q_ok) return;
    float* out = p.partial + (((size_t)b * p.nh + h) * p.tiles_max + tile) * (hd + 2);
    if (g == 0) {
      out[0] = m_run;
      out[1] = l_run;
    }
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) {
      const int d = 16 * dt + 4 * g;
      if (d < hd) {
#pragma unroll
        for (int v = 0; v < 4; ++v) out[2 + d + v] = acc[dt][v];
      }
    }
  }
}

// out[b][h] = sum over the tiles in reach, in ascending order, of exp(m_tile - m) * values / sum of exp(m_tile - m) * sums.
// grid (B, nh), one wave: the tiles' weights exp(m_tile - m) are worked out once, a lane per tile, and kept in LDS;
// the denominators are added 64 tiles at a time in tile order; then every lane sums its dimensions over the tiles in order.
#define F32_JOIN_TILES 4096
__global__ __launch_bounds__(64) void attn_f32_join_kernel(AttnF32Args p) {
  __shared__ float wgt[F32_JOIN_TILES];
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int pos = p.start[b];
  const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  const int first = lo / AT, last = pos / AT;
  const int stride = p.hd + 2;
  const float* part = p.partial + ((size_t)b * p.nh + h) * p.tiles_max * stride;
  float m = -INFINITY;
  for (int tile = first + lane; tile <= last; tile += 64) m = fmaxf(m, part[(size_t)tile * stride]);
  m = wave_max(m);
  float l = 0.f;
  for (int t0 = first; t0 <= last; t0 += 64) {
    const int tile = t0 + lane;
    float w = 0.f, wl = 0.f;
    if (tile <= last) {
      const float* q = part + (size_t)tile * stride;
      w = expf(q[0] - m);
      wl = w * q[1];
      wgt[tile - first] = w;
    }
    l += wave_sum(wl);
  }
  __builtin_amdgcn_wave_barrier();
  const float inv = 1.0f / l;
  float* orow = p.out + ((size_t)p.cu_seqlens[b] * p.nh + h) * p.hd;
  for (int d = lane; d < p.hd; d += 64) {
    float a = 0.f;
#pragma unroll 8
    for (int tile = first; tile <= last; ++tile) a = fmaf(wgt[tile - first], part[(size_t)tile * stride + 2 + d], a);
    orow[d] = a * inv;
  }
}

// Floats of `partial` that a decode step of B sequences up to max_end positions needs.
TQ_API int64_t tq_attention_f32_scratch(int B, int nh, int hd, int max_end) {
  return (int64_t)B * nh * ((max_end + AT - 1) / AT) * (hd + 2);
}

template <int ND>
static int launch_attention_f32(const AttnF32Args& p, int B, int decode, int max_new, int max_end, hipStream_t st) {
  if (decode) {
    const int tiles = (max_end + AT - 1) / AT;
    const int group = p.nh / p.nkv, passes = (group + 15) / 16;
    // with a window a token reaches at most window positions, which lie in window / AT + 2 tiles at the most
    const int waves = p.window > 0 ? min(tiles, p.window / AT + 2) : tiles;
    if (p.nkv * passes > 65535 || waves > 65535 || tiles > F32_JOIN_TILES) return TQ_ERR_UNSUPPORTED;
    // whole lines only where the head fills its tiles of 16 (32, 64, 128, 256): the loads of that form have no
    // guard on the head size, and a head of 96 would read beyond its rows and, in the last page, beyond the pool
    if (p.hd == 16 * ND && p.hd % 32 == 0 && p.page_size % 32 == 0)
      hipLaunchKernelGGL((attn_f32_decode_kernel<ND, true>), dim3(B, p.nkv * passes, waves), dim3(64), 0, st, p, passes);
    else
      hipLaunchKernelGGL((attn_f32_decode_kernel<ND, false>), dim3(B, p.nkv * passes, waves), dim3(64), 0, st, p, passes);
    hipLaunchKernelGGL(attn_f32_join_kernel, dim3(B, p.nh), dim3(64), 0, st, p);
    return 0;
  }
  constexpr int HDP = 16 * ND;
  const size_t shmem = ((size_t)AT * (HDP + 4) + (size_t)HDP * (AT + 4)) * sizeof(float);
  if (shmem > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attn_f32_prefill_kernel<ND>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    if (e != hipSuccess) return (int)e;
  }
  const int blocks_per_seq = (max_new + 63) / 64;
  if (p.nh > 65535) return TQ_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(attn_f32_prefill_kernel<ND>, dim3((unsigned)B * blocks_per_seq, p.nh), dim3(256), shmem, st, p,
                     blocks_per_seq);
  return 0;
}

// The tokens are runs of consecutive positions, one per sequence (cu_seqlens, slots, start as in AttnF32Args);
// decode: every run is one token and `partial` holds tq_attention_f32_scratch(B, nh, hd, max_end) floats.
// hd must be a multiple of 4 and at most 256, page_size a multiple of 64, page_stride a multiple of 4.
TQ_API int tq_attention_f32(const void* q, const void* k_pool, const void* v_pool, const int* block_table, int bt_stride,
                            const int* cu_seqlens, const int* slots, const int* start, int page_size, int64_t page_stride,
                            int B, int nh, int nkv, int hd, int window, float scale, void* out, void* partial, int decode,
                            int max_new, int max_end, hipStream_t st) {
  if (B <= 0) return 0;
  if (hd <= 0 || hd % 4 != 0 || hd > 256 || nkv <= 0 || nh % nkv != 0 || page_size % AT != 0 || page_stride % 4 != 0)
    return TQ_ERR_UNSUPPORTED;
  if (((size_t)q | (size_t)k_pool | (size_t)v_pool | (size_t)out) & 15) return TQ_ERR_UNSUPPORTED;
  if (decode && !partial) return TQ_ERR_BAD_ARG;
  if (max_new <= 0 || max_end <= 0) return TQ_ERR_BAD_ARG;
  AttnF32Args p{(const float*)q, (const float*)k_pool, (const float*)v_pool, block_table, bt_stride, cu_seqlens, slots,
                start, page_size, page_stride, nh, nkv, hd, window, scale, (float*)out, (float*)partial,
                (max_end + AT - 1) / AT};
  int rc;
  if (hd <= 16) rc = launch_attention_f32<1>(p, B, decode, max_new, max_end, st);
  else if (hd <= 32) rc = launch_attention_f32<2>(p, B, decode, max_new, max_end, st);
  else if (hd <= 64) rc = launch_attention_f32<4>(p, B, decode, max_new, max_end, st);
  else if (hd <= 128) rc = launch_attention_f32<8>(p, B, decode, max_new, max_end, st);
  else rc = launch_attention_f32<16>(p, B, decode, max_new, max_end, st);
  if (rc) return rc;
  TQ_LAUNCH_CHECK();
  return 0;
}
