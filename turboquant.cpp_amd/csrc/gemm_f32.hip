// Matrix products out[m, n] = sum_k a[m, k] * w[n, k] in true 32-bit floating point on the matrix cores.
//
// v_mfma_f32_32x32x2_f32 and v_mfma_f32_16x16x4_f32 multiply and add float operands as they are (no reduced-precision
// inputs), at twice the rate that the vector unit reaches without packed instructions.  Same contract as the plain
// product (gemm_generic.hip): optional bias, optional gated pair gate(a w^T) * (a w2^T), optional row gather and
// per-row-tile matrices for experts; the reference's counterpart is its float matvec
// (/root/reference/src/engine/tq_ops.c:296-343).  Two kernels:
//
//  * gemm_f32_tile_kernel, for more than 16 rows: tiles of 64 or 128 rows by 128 columns by four waves, 16 of k
//    at a time through two LDS buffers (rows padded to 20 floats, so that the 16-byte operand reads of eight
//    neighbouring rows fall on all banks); while one buffer is multiplied the next tile is on its way from memory.
//    17 to 64 rows (a decode step of many sequences) are one row of tiles, at which multiply-adds and bytes of w
//    are in balance; a narrow matrix is cut into runs of k so that the chip has enough workgroups.
//  * gemm_f32_stream_kernel, for few rows (decoding; experts that few tokens chose): the work is reading w once.
//    A workgroup owns 32 rows of w (every row of `a` that a wave fetches multiplies all of them), its four waves split k
//    and add their sums in wave order through LDS; the rows of w go from memory straight into the operand
//    registers, by whole lines of 128 bytes and with the hint that they are read once.
//  Runs of k of a narrow matrix leave their sums apart; a second kernel adds them up in order and finishes them.
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

// With `part` set the grid's z cuts k into runs of k_per_split and the sums of run z go to part[z] ([run][M][N], the
// gated pair's second product behind all the first ones) as they are: gemm_f32_reduce_kernel finishes them.
template <int MI, bool DUAL>
__global__ __launch_bounds__(256) void gemm_f32_tile_kernel(F32GemmArgs g, int k_per_split, float* part) {
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
  const int k_first = blockIdx.z * k_per_split, k_last = min(g.K, k_first + k_per_split);
  auto fetch = [&](int k0) {
    const int k = k0 + 4 * lchunk;
    const bool in = k < k_last;       // K and the runs are multiples of 4: a chunk lies inside or outside as a whole
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

  const int nk = (k_last - k_first + TBK - 1) / TBK;
  fetch(k_first);
  stage(0);
  __syncthreads();
  const int r32 = lane % 32, kk = lane / 32;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) fetch(k_first + (kt + 1) * TBK);
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
        if (part) {
          part[((size_t)blockIdx.z * g.M + m) * g.N + n] = acc[i][j][v];
          if (DUAL) part[((size_t)(gridDim.z + blockIdx.z) * g.M + m) * g.N + n] = acc2[i][j][v];
          continue;
        }
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
// Lanes l and l ^ 8 (the same quarter q = l / 16, rows r and r ^ 8 of a tile of 16 rows) fetched whole lines of 128
// bytes: lane (r, q) chunk q + 4 (r / 8) of row r % 8 into t0 and of row 8 + r % 8 into t1 (a chunk is 4 floats).
// Afterwards t0 is chunk q and t1 chunk q + 4 of the lane's own row r: the operands of two consecutive passes of 16.
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

// A workgroup owns 16 * MT rows of `a` (a row tile of the grid), 16 * NT rows of w (blockIdx.y) and one run of k
// (blockIdx.z, k_per_split long); its four waves take a quarter of the run each.  Every row of `a` that a wave has
// fetched multiplies all 16 * NT rows of w.  With more than one run the sums go to `part` ([run][M][N], the gated
// pair's second product behind all the first ones) as they are, and gemm_f32_reduce_kernel adds the runs up in
// order and finishes them.
template <int MT, int NT, bool DUAL>
__global__ __launch_bounds__(256) void gemm_f32_stream_kernel(F32GemmArgs g, int k_per_split, int k_per_wave, float* part) {
  __shared__ __align__(16) float join[DUAL ? 2 : 1][NT * MT][64 * 4];
  const int tile_m = blockIdx.x, tile_n = blockIdx.y, z = blockIdx.z;
  if (g.n_tiles && tile_m >= g.n_tiles[0]) return;
  const int group = g.tile_group ? g.tile_group[tile_m] : 0;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int r = lane % 16, q = lane / 16;
  const int m0 = tile_m * 16 * MT, n0 = tile_n * 16 * NT;
  // w is fetched by whole lines: for every 32 of k one instruction takes rows 0..7 of a tile of 16 and the next rows
  // 8..15, eight lanes to a row; lanes r and r ^ 8 then exchange what belongs to the other's row.  A row of w that
  // does not exist reads row 0 instead (what it produces is never stored).
  const int chunk = 4 * (q + 4 * (r / 8));           // this lane's 4 of every 32 of k
  const float* wlo[NT];
  const float* whi[NT];
  const float* vlo[DUAL ? NT : 1];
  const float* vhi[DUAL ? NT : 1];
#pragma unroll
  for (int c = 0; c < NT; ++c) {
    const int n_lo = n0 + 16 * c + r % 8, n_hi = n_lo + 8;
    const size_t o_lo = (size_t)group * g.group_stride + (size_t)(n_lo < g.N ? n_lo : 0) * g.K + chunk;
    const size_t o_hi = (size_t)group * g.group_stride + (size_t)(n_hi < g.N ? n_hi : 0) * g.K + chunk;
    wlo[c] = g.w + o_lo;
    whi[c] = g.w + o_hi;
    if (DUAL) {
      vlo[c] = g.w2 + o_lo;
      vhi[c] = g.w2 + o_hi;
    }
  }
  const float* arow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) arow[t] = f32_row_of(g, m0 + 16 * t + r);

  f32x4 acc[NT][MT], acc2[DUAL ? NT : 1][DUAL ? MT : 1];
#pragma unroll
  for (int c = 0; c < NT; ++c)
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      acc[c][t] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (DUAL) acc2[c][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  const int run_end = min(g.K, (z + 1) * k_per_split);
  const int k_beg = z * k_per_split + wave * k_per_wave, k_end = min(run_end, k_beg + k_per_wave);
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  // P lines of 32 of k whose loads are all issued before the first product
  constexpr int P = (NT * (DUAL ? 2 : 1) * 2 + MT * 2) <= 10 ? 4 : 2;
  for (int k = k_beg; k < k_end; k += 32 * P) {
    f32x4 w0[NT][P], w1[NT][P], v0[DUAL ? NT : 1][DUAL ? P : 1], v1[DUAL ? NT : 1][DUAL ? P : 1], a0[MT][P], a1[MT][P];
    // (a chunk beyond the wave's share is asked for at the matrix's first address instead and replaced by zeros below:
    // every lane loads, so that no load waits behind a branch)
#pragma unroll
    for (int p = 0; p < P; ++p) {
      const int kl = k + 32 * p;
      const bool in = kl + chunk < k_end;              // (k_end is a multiple of 4: a chunk lies inside or outside as a whole)
#pragma unroll
      for (int c = 0; c < NT; ++c) {
        w0[c][p] = load4_once(in ? wlo[c] + kl : g.w);
        w1[c][p] = load4_once(in ? whi[c] + kl : g.w);
        if (DUAL) {
          v0[c][p] = load4_once(in ? vlo[c] + kl : g.w2);
          v1[c][p] = load4_once(in ? vhi[c] + kl : g.w2);
        }
      }
      // the rows of `a` stay in cache; they are fetched as the products want them: 4 of k at 4 q of each 16
      const int ka = kl + 4 * q;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        a0[t][p] = *reinterpret_cast<const f32x4*>(ka < k_end && arow[t] ? arow[t] + ka : g.a);
        a1[t][p] = *reinterpret_cast<const f32x4*>(ka + 16 < k_end && arow[t] ? arow[t] + ka + 16 : g.a);
      }
    }
#pragma unroll
    for (int p = 0; p < P; ++p) {
      const int kl = k + 32 * p;
      const bool in = kl + chunk < k_end;
      const int ka = kl + 4 * q;
#pragma unroll
      for (int c = 0; c < NT; ++c) {
        w0[c][p] = in ? w0[c][p] : zero;
        w1[c][p] = in ? w1[c][p] : zero;
        if (DUAL) {
          v0[c][p] = in ? v0[c][p] : zero;
          v1[c][p] = in ? v1[c][p] : zero;
        }
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        a0[t][p] = ka < k_end && arow[t] ? a0[t][p] : zero;
        a1[t][p] = ka + 16 < k_end && arow[t] ? a1[t][p] : zero;
      }
    }
#pragma unroll
    for (int p = 0; p < P; ++p) {
#pragma unroll
      for (int c = 0; c < NT; ++c) {
        to_own_row(w0[c][p], w1[c][p]);
        if (DUAL) to_own_row(v0[c][p], v1[c][p]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int c = 0; c < NT; ++c)
#pragma unroll
          for (int t = 0; t < MT; ++t) {
            acc[c][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(w0[c][p][i], a0[t][p][i], acc[c][t], 0, 0, 0);
            if (DUAL) acc2[c][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(v0[c][p][i], a0[t][p][i], acc2[c][t], 0, 0, 0);
          }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int c = 0; c < NT; ++c)
#pragma unroll
          for (int t = 0; t < MT; ++t) {
            acc[c][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(w1[c][p][i], a1[t][p][i], acc[c][t], 0, 0, 0);
            if (DUAL) acc2[c][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(v1[c][p][i], a1[t][p][i], acc2[c][t], 0, 0, 0);
          }
    }
  }
  // the waves' sums are added in wave order: waves 1, 2, 3 hand theirs to wave 0 one after the other
  for (int ww = 1; ww < 4; ++ww) {
    if (wave == ww) {
#pragma unroll
      for (int c = 0; c < NT; ++c)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          *reinterpret_cast<f32x4*>(&join[0][c * MT + t][lane * 4]) = acc[c][t];
          if (DUAL) *reinterpret_cast<f32x4*>(&join[DUAL ? 1 : 0][c * MT + t][lane * 4]) = acc2[c][t];
        }
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int c = 0; c < NT; ++c)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          acc[c][t] += *reinterpret_cast<const f32x4*>(&join[0][c * MT + t][lane * 4]);
          if (DUAL) acc2[c][t] += *reinterpret_cast<const f32x4*>(&join[DUAL ? 1 : 0][c * MT + t][lane * 4]);
        }
    }
    __syncthreads();
  }
  if (wave != 0) return;
  const bool raw = part != nullptr;       // several runs of k: leave the sums as they are
  float* dst = raw ? part + (size_t)z * g.M * g.N : g.out;
  const int64_t ld = raw ? g.N : g.ldc;
#pragma unroll
  for (int c = 0; c < NT; ++c)
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      // D: lane = column (row of `a`) r, rows (rows of w) 4 q + v
      const int m = m0 + 16 * t + r;
      if (m >= g.M) continue;
      if (g.a_rows && g.a_rows[m] < 0) continue;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int nn = n0 + 16 * c + 4 * q + v;
        if (nn >= g.N) continue;
        if (raw) {
          dst[(size_t)m * ld + nn] = acc[c][t][v];
          if (DUAL) dst[(size_t)gridDim.z * g.M * g.N + (size_t)m * ld + nn] = acc2[c][t][v];
        } else {
          float x = acc[c][t][v] + f32_bias_at(g, nn);
          if (DUAL) x = gate_fn(x, g.gate) * acc2[c][t][v];
          dst[(size_t)m * ld + nn] = x;
        }
      }
    }
}

// out[m][n] = sum over the runs, in order, of part[run][m][n] (+ bias; the gated pair: gate(that) * the same sum of
// the second product's runs).  With `keep_runs` the runs stay apart and only the bias is added, to run 0.
__global__ void gemm_f32_reduce_kernel(F32GemmArgs g, const float* __restrict__ part, int S, int dual) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)g.M * g.N) return;
  const int m = (int)(i / g.N), n = (int)(i % g.N);
  float x = 0.f, y = 0.f;
  for (int z = 0; z < S; ++z) {
    x += part[(size_t)z * g.M * g.N + i];
    if (dual) y += part[(size_t)(S + z) * g.M * g.N + i];
  }
  x += f32_bias_at(g, n);
  if (dual) x = gate_fn(x, g.gate) * y;
  g.out[(size_t)m * g.ldc + n] = x;
}
__global__ void gemm_f32_bias_kernel(F32GemmArgs g) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)g.M * g.N) return;
  g.out[i] += f32_bias_at(g, (int)(i % g.N));
}

// Into how many runs k is cut for a plain product (one matrix, up to 64 rows): enough that a narrow matrix still
// gives every compute unit two workgroups (of 128 columns for 17 to 64 rows, of 32 for fewer), each run keeping at
// least 256 of k.  A function of N and K alone, so that a row's sums do not depend on how many rows there are.
// Tiles of 16 rows of w per workgroup of the few-row kernel.  Measured on the experts' gated product at 64, 128 and 240
// tokens (60 experts of 1,408 x 2,048, 4 per token): 290, 299 and 412 us with 2; 315, 317 and 436 with 4; 272, 289 and 423 with 1.
#define SNT 2
static int f32_runs_of_k(int N, int K, int* k_per_split) {
  const int groups = (N + 127) / 128;
  int runs = 1;
  while (runs < 32 && groups * runs < 512 && K / (runs * 2 * 4 * 16) >= 2) runs *= 2;
  int per = ((K + runs - 1) / runs + 127) / 128 * 128;    // a multiple of 128: a quarter for each wave, in whole lines
  if (per < 128) per = 128;
  *k_per_split = per;
  return (K + per - 1) / per;
}
TQ_API int tq_gemm_f32_runs(int M, int N, int K, int grouped) {
  int per;
  return (grouped || M > 64) ? 1 : f32_runs_of_k(N, K, &per);      // (grouped: also a product whose rows are gathered)
}

// tile_rows: 16 or 64 rows of output per row tile; with tile_group set it is the padding unit that the row order
// was built with.  K must be a multiple of 4 and every row of a, w and w2 must start at a multiple of 16 bytes.
// scratch: for a plain product of up to 64 rows, tq_gemm_f32_runs(M, N, K, 0) * M * N floats (twice that for a gated
// pair), unless that number is 1.  keep_runs (plain products into which no second matrix goes): `out` is
// [runs][M][N] and receives the runs apart, the bias in run 0; the caller adds them up in order.
TQ_API int tq_gemm_f32(const void* a, int64_t lda, const int* a_rows, int a_gather, const void* w, const void* w2,
                       int64_t group_stride, const int* tile_group, const int* n_tiles, const void* bias, int bias_type,
                       void* out, int64_t ldc, int M, int N, int K, int tile_rows, int gate, void* scratch, int keep_runs,
                       hipStream_t st) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (tile_rows != 16 && tile_rows != 64)) return TQ_ERR_BAD_ARG;
  if (K % 4 != 0 || lda % 4 != 0 || group_stride % 4 != 0 || ((size_t)a & 15) || ((size_t)w & 15) || ((size_t)w2 & 15))
    return TQ_ERR_UNSUPPORTED;
  if (gate < 0 || gate >= TQ_GATE_COUNT) return TQ_ERR_BAD_ARG;
  F32GemmArgs g{(const float*)a, lda, a_rows, a_gather, (const float*)w, (const float*)w2, group_stride, tile_group,
                n_tiles, bias, bias_type, (float*)out, ldc, M, N, K, gate};
  const bool dual = w2 != nullptr;
  const bool grouped = tile_group != nullptr;
  if (keep_runs && (dual || grouped || a_rows || ldc != N)) return TQ_ERR_BAD_ARG;
  int k_per_split = (K + 127) / 128 * 128;
  const int runs = (grouped || a_rows || M > 64) ? 1 : f32_runs_of_k(N, K, &k_per_split);
  float* part = nullptr;
  if (runs > 1) {
    part = keep_runs ? (float*)out : (float*)scratch;
    if (!part) return TQ_ERR_BAD_ARG;
  }
  if ((grouped && tile_rows == 16) || (!grouped && M <= 16)) {
    // few rows: the work is reading w once
    const int k_per_wave = k_per_split / 4;
    const dim3 grid((M + 15) / 16, (N + 16 * SNT - 1) / (16 * SNT), runs);
    if (grid.y > 65535) return TQ_ERR_UNSUPPORTED;
    if (dual)
      hipLaunchKernelGGL((gemm_f32_stream_kernel<1, SNT, true>), grid, dim3(256), 0, st, g, k_per_split, k_per_wave, part);
    else
      hipLaunchKernelGGL((gemm_f32_stream_kernel<1, SNT, false>), grid, dim3(256), 0, st, g, k_per_split, k_per_wave, part);
  } else {
    // tiles; 17 to 64 rows of one matrix are a single row of tiles, cut into runs of k where the matrix is narrow
    const int mi = (grouped || M <= 64) ? 1 : 2;
    const dim3 grid((M + 64 * mi - 1) / (64 * mi), (N + 127) / 128, runs);
    if (grid.y > 65535) return TQ_ERR_UNSUPPORTED;
    if (mi == 1) {
      if (dual) hipLaunchKernelGGL((gemm_f32_tile_kernel<1, true>), grid, dim3(256), 0, st, g, k_per_split, part);
      else hipLaunchKernelGGL((gemm_f32_tile_kernel<1, false>), grid, dim3(256), 0, st, g, k_per_split, part);
    } else {
      if (dual) hipLaunchKernelGGL((gemm_f32_tile_kernel<2, true>), grid, dim3(256), 0, st, g, k_per_split, part);
      else hipLaunchKernelGGL((gemm_f32_tile_kernel<2, false>), grid, dim3(256), 0, st, g, k_per_split, part);
    }
  }
  if (runs > 1) {
    const unsigned blocks = (unsigned)(((int64_t)M * N + 255) / 256);
    if (!keep_runs)
      hipLaunchKernelGGL(gemm_f32_reduce_kernel, dim3(blocks), dim3(256), 0, st, g, part, runs, dual ? 1 : 0);
    else if (bias)
      hipLaunchKernelGGL(gemm_f32_bias_kernel, dim3(blocks), dim3(256), 0, st, g);
  }
  TQ_LAUNCH_CHECK();
  return 0;
}
