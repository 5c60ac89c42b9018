// Matrix products out[m, n] = sum_k a[m, k] * w[n, k] with plain float multiply-adds.
//
// Weights are row-major [out, in] as the reference keeps them
// (/root/reference/src/engine/tq_ops.c:287-343).  This kernel serves the whole 32-bit path and
// every weight type the matrix-core kernels do not take; each output element is summed over k in
// ascending order by one thread, so a row's result does not depend on which other rows are in
// the product.  One kernel covers the plain product, the product with bias, the gated pair
// gate(a w_gate) * (a w_up), gate being silu or another activation (/root/reference/src/engine/tq_transformer.c:2770-2794), and the
// same over groups of rows that each use their own matrix (experts,
// /root/reference/src/engine/tq_moe.c:864-999): rows are then taken from `a` through a_rows and
// row tile i uses matrix tile_group[i].
#include "common.h"

#define BN 64
#define BK 16

struct GemmArgs {
  const act_t* a;
  int64_t lda;
  const int* a_rows;       // row of `a` that feeds output row m (-1: none), or null for m itself
  int a_gather;            // 0: a_rows only marks live rows (>= 0) and row m itself is read
  const void* w;           // [groups][N][K]
  const void* w2;          // second matrix of the gated pair, or null
  int64_t group_stride;    // elements between the matrices of two groups
  const int* tile_group;   // group of each row tile, or null (group 0)
  const int* n_tiles;      // number of live row tiles on the device, or null (all)
  const void* bias;        // [N] or null
  int bias_type;
  void* out;               // [M][N] float, or act_t when OUT_ACT
  int64_t ldc;
  int M, N, K;
  int gate;                // activation of the gated pair
};

template <class W, int TM, bool DUAL, bool OUT_ACT>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GemmArgs g) {
  constexpr int BM = 16 * TM;
  __shared__ float As[BK][BM + 1];
  __shared__ float Ws[BK][BN + 1];
  __shared__ float Vs[DUAL ? BK : 1][BN + 1];
  const int tile_m = blockIdx.x, tile_n = blockIdx.y;
  if (g.n_tiles && tile_m >= g.n_tiles[0]) return;
  const int group = g.tile_group ? g.tile_group[tile_m] : 0;
  const W* w = (const W*)g.w + (size_t)group * g.group_stride;
  const W* w2 = DUAL ? (const W*)g.w2 + (size_t)group * g.group_stride : nullptr;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;

  float acc[TM][4], acc2[DUAL ? TM : 1][4];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[i][j] = 0.f;
      if (DUAL) acc2[i][j] = 0.f;
    }

  for (int k0 = 0; k0 < g.K; k0 += BK) {
    for (int idx = threadIdx.x; idx < BM * BK; idx += 256) {
      const int r = idx / BK, kk = idx % BK;
      const int m = m0 + r;
      float v = 0.f;
      if (m < g.M && k0 + kk < g.K) {
        int src = g.a_rows ? g.a_rows[m] : m;
        if (src >= 0 && !g.a_gather) src = m;
        if (src >= 0) v = to_f32(g.a[(size_t)src * g.lda + k0 + kk]);
      }
      As[kk][r] = v;
    }
    for (int idx = threadIdx.x; idx < BN * BK; idx += 256) {
      const int r = idx / BK, kk = idx % BK;
      const int n = n0 + r;
      const bool ok = n < g.N && k0 + kk < g.K;
      Ws[kk][r] = ok ? to_f32(w[(size_t)n * g.K + k0 + kk]) : 0.f;
      if (DUAL) Vs[kk][r] = ok ? to_f32(w2[(size_t)n * g.K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float av[TM], wv[4], vv[4];
#pragma unroll
      for (int i = 0; i < TM; ++i) av[i] = As[kk][ty + 16 * i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        wv[j] = Ws[kk][tx + 16 * j];
        if (DUAL) vv[j] = Vs[kk][tx + 16 * j];
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
          if (DUAL) acc2[i][j] = fmaf(av[i], vv[j], acc2[i][j]);
        }
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + ty + 16 * i;
    if (m >= g.M) continue;
    if (g.a_rows && g.a_rows[m] < 0) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= g.N) continue;
      float v = acc[i][j];
      if (g.bias) v += g.bias_type == TQ_F32 ? ((const float*)g.bias)[n] : to_f32(((const bf16_t*)g.bias)[n]);
      if (DUAL) v = gate_fn(v, g.gate) * acc2[i][j];
      if (OUT_ACT)
        ((act_t*)g.out)[(size_t)m * g.ldc + n] = from_f32<act_t>(v);
      else
        ((float*)g.out)[(size_t)m * g.ldc + n] = v;
    }
  }
}

template <class W, int TM>
static void launch(const GemmArgs& g, bool dual, bool out_act, hipStream_t st) {
  const dim3 grid((g.M + 16 * TM - 1) / (16 * TM), (g.N + BN - 1) / BN);
  if (dual && out_act)
    hipLaunchKernelGGL((gemm_generic_kernel<W, TM, true, true>), grid, dim3(256), 0, st, g);
  else if (dual)
    hipLaunchKernelGGL((gemm_generic_kernel<W, TM, true, false>), grid, dim3(256), 0, st, g);
  else if (out_act)
    hipLaunchKernelGGL((gemm_generic_kernel<W, TM, false, true>), grid, dim3(256), 0, st, g);
  else
    hipLaunchKernelGGL((gemm_generic_kernel<W, TM, false, false>), grid, dim3(256), 0, st, g);
}

// tile_rows: 16 or 64 rows of output per workgroup.  With tile_group set it must be the padding
// unit that the row order was built with.
TQ_API int tq_gemm_generic(const void* a, int64_t lda, const int* a_rows, int a_gather, const void* w, const void* w2, int wtype,
                           int64_t group_stride, const int* tile_group, const int* n_tiles, const void* bias,
                           int bias_type, void* out, int64_t ldc, int out_is_act, int M, int N, int K, int tile_rows,
                           int gate, hipStream_t st) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (tile_rows != 16 && tile_rows != 64)) return TQ_ERR_BAD_ARG;
  if ((N + BN - 1) / BN > 65535) return TQ_ERR_UNSUPPORTED;
  if (gate < 0 || gate >= TQ_GATE_COUNT) return TQ_ERR_BAD_ARG;
  GemmArgs g{(const act_t*)a, lda, a_rows, a_gather, w, w2, group_stride, tile_group, n_tiles, bias, bias_type, out, ldc, M, N, K, gate};
  TQ_DISPATCH_W(wtype, {
    if (tile_rows == 16)
      launch<W, 1>(g, w2 != nullptr, out_is_act != 0, st);
    else
      launch<W, 4>(g, w2 != nullptr, out_is_act != 0, st);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}
