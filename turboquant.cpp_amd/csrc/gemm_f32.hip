// Matrix products out[m, n] = sum_k a[m, k] * w[n, k] in true 32-bit floating point on the matrix cores.
//
// v_mfma_f32_32x32x2_f32 and v_mfma_f32_16x16x4_f32 multiply and add float operands as they are (no reduced-precision
// inputs), at twice the rate that the vector unit reaches without packed instructions.  Same contract as the plain
// product (gemm_generic.hip): optional bias, optional gated pair gate(a w^T) * (a w2^T), optional row gather and
// per-row-tile matrices for experts; the reference's counterpart is its float matvec
// (/root/reference/src/engine/tq_ops.c:296-343).  Two kernels:
//
//  * gemm_f32_tile_kernel, for many rows (prompts): tiles of 64 or 128 rows by 128 columns by four waves, 16 of k
//    at a time through two LDS buffers (rows padded to 20 floats, so that the 16-byte operand reads of eight
//    neighbouring rows fall on all banks); while one buffer is multiplied the next tile is on its way from memory.
//  * gemm_f32_stream_kernel, for few rows (decoding; experts that few tokens chose): the work is reading w once.
//    A workgroup owns 16 rows of w, its four waves split k and add their sums in wave order through LDS; the
//    rows of w go from memory straight into the operand registers, with the hint that they are read once.
//
// A lane's 16 bytes of an operand row are 4 consecutive k, and the four multiply-adds that use them take them one
// by one, so a product sums k in the order (0, 4), (1, 5), (2, 6), (3, 7), (8, 12), ... within each 16 (32x32x2:
// 8 and 16x16x4: 16 elements of k per pass of four instructions); the order depends on k alone, never on the
// row, the number of rows or the tile.
//
// Operand layouts (wave of 64 lanes): 32x32x2: A lane l = row l%32, k l/32; B lane l = column l%32, k l/32; D lane l =
// column l%32, rows 8*(v/4) + 4*(l/32) + v%4, v<16.  16x16x4: A lane l = row l%16, k l/16; B alike; D lane l = column
// l%16, rows 4*(l/16) + v, v<4.
#include "common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct F32GemmArgs {
  const float* a;
  int64_t lda;
  const int* a_rows;       // row of `a` that feeds output row m (-1: none), or null for m itself
  int a_gather;            // 0: a_rows only marks live rows (>= 0) and row m itself is read
  const float* w;          // [groups][N][K]
  const float* w2;         // second matrix of the gated pair, or null
  int64_t group_stride;
  const int* tile_group;   // group of each row tile, or null (group 0)
  const int* n_tiles;      // number of live row tiles on the device, or null (all)
  const void* bias;
  int bias_type;
  float* out;
  int64_t ldc;
  int M, N, K;
  int gate;                // activation of the gated pair
};

__device__ __forceinline__ float f32_bias_at(const F32GemmArgs& g, int n) {
  if (!g.bias) return 0.f;
  return g.bias_type == TQ_F32 ? ((const float*)g.bias)[n] : to_f32(((const bf16_t*)g.bias)[n]);
}

// Row of `a` behind output row m, or null.
__device__ __forceinline__ const float* f32_row_of(const F32GemmArgs& g, int m) {
  if (m >= g.M) return nullptr;
  int src = m;
  if (g.a_rows) {
    src = g.a_rows[m];
    if (src < 0) return nullptr;
    if (!g.a_gather) src = m;
  }
  return g.a + (size_t)src * g.lda;
}

// ------------------------------------------------------------------------------------------ many rows
#define TBK 16
#define TLD (TBK + 4)

template <int MI, bool DUAL>
__global__ __launch_bounds__(256) void gemm_f32_tile_kernel(F32GemmArgs g) {
  constexpr int NI = 2, BM = 64 * MI, BN = 64 * NI;
  __shared__ __align__(16) float As[2][BM * TLD];
  __shared__ __align__(16) float Ws[2][BN * TLD];
  __shared__ __align__(16) float Vs[2][DUAL ? BN * TLD : 4];
  const int tile_m = blockIdx.x, tile_n = blockIdx.y;
  if (g.n_tiles && tile_m >= g.n_tiles[0]) return;
  const int group = g.tile_group ? g.tile_group[tile_m] : 0;
  const float* w = g.w + (size_t)group * g.group_stride;
  const float* w2 = DUAL ? g.w2 + (size_t)group * g.group_stride : nullptr;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wave_m = wave / 2, wave_n = wave % 2;
  const int lrow = tid / 4, lchunk = tid % 4;      // what this thread fetches of a tile: rows lrow + 64 j, 4 of k

  const float* arow[MI];
  const float* wrow[NI];
  const float* vrow[DUAL ? NI : 1];
#pragma unroll
  for (int j = 0; j < MI; ++j) arow[j] = f32_row_of(g, m0 + lrow + 64 * j);
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const int n = n0 + lrow + 64 * j;
    wrow[j] = n < g.N ? w + (size_t)n * g.K : nullptr;
    if (DUAL) vrow[j] = n < g.N ? w2 + (size_t)n * g.K : nullptr;
  }

  f32x16 acc[MI][NI], acc2[DUAL ? MI : 1][DUAL ? NI : 1];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        acc[i][j][v] = 0.f;
        if (DUAL) acc2[i][j][v] = 0.f;
      }
    }

  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  f32x4 ra[MI], rw[NI], rv[DUAL ? NI : 1];
  auto fetch = [&](int k0) {
    const int k = k0 + 4 * lchunk;
    const bool in = k < g.K;          // K is a multiple of 4: a chunk lies inside or outside as a whole
#pragma unroll
    for (int j = 0; j < MI; ++j) ra[j] = in && arow[j] ? *reinterpret_cast<const f32x4*>(arow[j] + k) : zero;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      rw[j] = in && wrow[j] ? *reinterpret_cast<const f32x4*>(wrow[j] + k) : zero;
      if (DUAL) rv[j] = in && vrow[j] ? *reinterpret_cast<const f32x4*>(vrow[j] + k) : zero;
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int j = 0; j < MI; ++j) *reinterpret_cast<f32x4*>(&As[buf][(lrow + 64 * j) * TLD + 4 * lchunk]) = ra[j];
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      *reinterpret_cast<f32x4*>(&Ws[buf][(lrow + 64 * j) * TLD + 4 * lchunk]) = rw[j];
      if (DUAL) *reinterpret_cast<f32x4*>(&Vs[buf][(lrow + 64 * j) * TLD + 4 * lchunk]) = rv[j];
    }
  };

  const int nk = (g.K + TBK - 1) / TBK;
  fetch(0);
  stage(0);
  __syncthreads();
  const int r32 = lane % 32, kk = lane / 32;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) fetch((kt + 1) * TBK);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      f32x4 af[MI], wf[NI], vf[DUAL ? NI : 1];
#pragma unroll
      for (int i = 0; i < MI; ++i)
        af[i] = *reinterpret_cast<const f32x4*>(&As[buf][(wave_m * 32 * MI + i * 32 + r32) * TLD + 8 * h + 4 * kk]);
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        wf[j] = *reinterpret_cast<const f32x4*>(&Ws[buf][(wave_n * 32 * NI + j * 32 + r32) * TLD + 8 * h + 4 * kk]);
        if (DUAL) vf[j] = *reinterpret_cast<const f32x4*>(&Vs[buf][(wave_n * 32 * NI + j * 32 + r32) * TLD + 8 * h + 4 * kk]);
      }
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j) {
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][s], wf[j][s], acc[i][j], 0, 0, 0);
            if (DUAL) acc2[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][s], vf[j][s], acc2[i][j], 0, 0, 0);
          }
    }
    if (kt + 1 < nk) stage(buf ^ 1);
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + wave_m * 32 * MI + i * 32 + 8 * (v / 4) + 4 * kk + v % 4;
      if (m >= g.M) continue;
      if (g.a_rows && g.a_rows[m] < 0) continue;
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        const int n = n0 + wave_n * 32 * NI + j * 32 + r32;
        if (n >= g.N) continue;
        float x = acc[i][j][v] + f32_bias_at(g, n);
        if (DUAL) x = gate_fn(x, g.gate) * acc2[i][j][v];
        g.out[(size_t)m * g.ldc + n] = x;
      }
    }
}

// ------------------------------------------------------------------------------------------ few rows
__device__ __forceinline__ f32x4 load4_once(const float* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
}

// MT tiles of 16 rows of `a` per workgroup (a row tile of the grid is 16 * MT rows).
template <int MT, bool DUAL>
__global__ __launch_bounds__(256) void gemm_f32_stream_kernel(F32GemmArgs g, int k_per_wave) {
  __shared__ __align__(16) float join[3][DUAL ? 2 : 1][MT][64 * 4];
  const int tile_m = blockIdx.x, tile_n = blockIdx.y;
  if (g.n_tiles && tile_m >= g.n_tiles[0]) return;
  const int group = g.tile_group ? g.tile_group[tile_m] : 0;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int r = lane % 16, q = lane / 16;
  const int m0 = tile_m * 16 * MT, n0 = tile_n * 16;
  const int n = n0 + r;
  // a row of w that does not exist reads row 0 instead (what it produces is never stored)
  const float* wrow = g.w + (size_t)group * g.group_stride + (size_t)(n < g.N ? n : 0) * g.K;
  const float* vrow = DUAL ? g.w2 + (size_t)group * g.group_stride + (size_t)(n < g.N ? n : 0) * g.K : nullptr;
  const float* arow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) arow[t] = f32_row_of(g, m0 + 16 * t + r);

  f32x4 acc[MT], acc2[DUAL ? MT : 1];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (DUAL) acc2[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int k_beg = wave * k_per_wave, k_end = min(g.K, k_beg + k_per_wave);
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  constexpr int U = DUAL ? 4 : 8;      // passes of 16 of k whose loads are all issued before the first product
  for (int k = k_beg; k < k_end; k += 16 * U) {
    f32x4 wf[U], vf[DUAL ? U : 1], af[MT][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kc = k + 16 * u + 4 * q;
      const bool in = kc < k_end;
      wf[u] = in ? load4_once(wrow + kc) : zero;
      if (DUAL) vf[u] = in ? load4_once(vrow + kc) : zero;
#pragma unroll
      for (int t = 0; t < MT; ++t) af[t][u] = in && arow[t] ? *reinterpret_cast<const f32x4*>(arow[t] + kc) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(wf[u][s], af[t][u][s], acc[t], 0, 0, 0);
          if (DUAL) acc2[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[u][s], af[t][u][s], acc2[t], 0, 0, 0);
        }
  }
  // the waves' sums are added in wave order
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      *reinterpret_cast<f32x4*>(&join[wave - 1][0][t][lane * 4]) = acc[t];
      if (DUAL) *reinterpret_cast<f32x4*>(&join[wave - 1][DUAL ? 1 : 0][t][lane * 4]) = acc2[t];
    }
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
#pragma unroll
    for (int ww = 0; ww < 3; ++ww) {
      const f32x4 p = *reinterpret_cast<const f32x4*>(&join[ww][0][t][lane * 4]);
      acc[t] += p;
      if (DUAL) acc2[t] += *reinterpret_cast<const f32x4*>(&join[ww][DUAL ? 1 : 0][t][lane * 4]);
    }
    // D: lane = column (row of `a`) r, rows (rows of w) 4 q + v
    const int m = m0 + 16 * t + r;
    if (m >= g.M) continue;
    if (g.a_rows && g.a_rows[m] < 0) continue;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int nn = n0 + 4 * q + v;
      if (nn >= g.N) continue;
      float x = acc[t][v] + f32_bias_at(g, nn);
      if (DUAL) x = gate_fn(x, g.gate) * acc2[t][v];
      g.out[(size_t)m * g.ldc + nn] = x;
    }
  }
}

// tile_rows: 16 or 64 rows of output per row tile; with tile_group set it is the padding unit that the row order
// was built with.  K must be a multiple of 4 and every row of a, w and w2 must start at a multiple of 16 bytes.
TQ_API int tq_gemm_f32(const void* a, int64_t lda, const int* a_rows, int a_gather, const void* w, const void* w2,
                       int64_t group_stride, const int* tile_group, const int* n_tiles, const void* bias, int bias_type,
                       void* out, int64_t ldc, int M, int N, int K, int tile_rows, int gate, hipStream_t st) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (tile_rows != 16 && tile_rows != 64)) return TQ_ERR_BAD_ARG;
  if (K % 4 != 0 || lda % 4 != 0 || group_stride % 4 != 0 || ((size_t)a & 15) || ((size_t)w & 15) || ((size_t)w2 & 15))
    return TQ_ERR_UNSUPPORTED;
  if (gate < 0 || gate >= TQ_GATE_COUNT) return TQ_ERR_BAD_ARG;
  F32GemmArgs g{(const float*)a, lda, a_rows, a_gather, (const float*)w, (const float*)w2, group_stride, tile_group,
                n_tiles, bias, bias_type, (float*)out, ldc, M, N, K, gate};
  const bool dual = w2 != nullptr;
  const bool grouped = tile_group != nullptr;
  if ((grouped && tile_rows == 16) || (!grouped && M <= 64)) {
    // few rows: every wave of a workgroup takes a quarter of k, in whole passes of 16
    const int k_per_wave = ((K + 3) / 4 + 15) / 16 * 16;
    const int mt = grouped ? 1 : (M <= 16 ? 1 : M <= 32 ? 2 : 4);
    const dim3 grid((M + 16 * mt - 1) / (16 * mt), (N + 15) / 16);
    if (grid.y > 65535) return TQ_ERR_UNSUPPORTED;
#define TQ_STREAM(MT_)                                                                                         \
  do {                                                                                                         \
    if (dual)                                                                                                  \
      hipLaunchKernelGGL((gemm_f32_stream_kernel<MT_, true>), grid, dim3(256), 0, st, g, k_per_wave);          \
    else                                                                                                       \
      hipLaunchKernelGGL((gemm_f32_stream_kernel<MT_, false>), grid, dim3(256), 0, st, g, k_per_wave);         \
  } while (0)
    if (mt == 1) TQ_STREAM(1);
    else if (mt == 2) TQ_STREAM(2);
    else TQ_STREAM(4);
#undef TQ_STREAM
  } else {
    const int mi = (grouped || M <= 64) ? 1 : 2;
    const dim3 grid((M + 64 * mi - 1) / (64 * mi), (N + 127) / 128);
    if (grid.y > 65535) return TQ_ERR_UNSUPPORTED;
    if (mi == 1) {
      if (dual) hipLaunchKernelGGL((gemm_f32_tile_kernel<1, true>), grid, dim3(256), 0, st, g);
      else hipLaunchKernelGGL((gemm_f32_tile_kernel<1, false>), grid, dim3(256), 0, st, g);
    } else {
      if (dual) hipLaunchKernelGGL((gemm_f32_tile_kernel<2, true>), grid, dim3(256), 0, st, g);
      else hipLaunchKernelGGL((gemm_f32_tile_kernel<2, false>), grid, dim3(256), 0, st, g);
    }
  }
  TQ_LAUNCH_CHECK();
  return 0;
}
