// What the bfloat16 matrix-core products share: the arguments of a product, the loads that take whole lines with
// the read-once hint, the exchange between pairs of lanes that turns such lines into operands, and the epilogue's
// pieces.
#pragma once
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct MfmaGemmArgs {
  const bf16_t* a;
  int64_t lda;
  const int* a_rows;
  int a_gather;
  const bf16_t* w;
  const bf16_t* w2;
  int64_t group_stride;
  const int* tile_group;
  const int* n_tiles;
  const void* bias;
  int bias_type;
  void* out;
  int64_t ldc;
  int M, N, K;
  int k_per;                // k is split into runs of k_per, run z going to out + z * split_stride (float)
  int64_t split_stride;
  int gate;                 // activation of the gated pair
  int group_ratio;          // tile kernel: row tiles per entry of tile_group and unit of n_tiles (0 or 1: one)
};

// For bytes that are read once (a matrix streamed past a few rows): a load that tells the caches so.  Measured on
// a plain read of 1 GiB whose instructions take whole lines of 128 bytes: 6.8 TB/s with this hint, 4.7 without; with
// half lines per instruction (16 rows x 64 bytes, the operand layout of the 16x16x32 product) 5.7.
__device__ __forceinline__ u32x4 load16_once(const bf16_t* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
// Lanes l and l ^ 8 (the same quarter c = l / 16, rows r and r ^ 8 of a tile of 16 rows) fetched whole lines: lane
// (r, c) chunk c + 4 (r / 8) of row r % 8 into t0 and of row 8 + r % 8 into t1.  Afterwards t0 is chunk c and t1
// chunk c + 4 of the lane's own row r: the operands of two consecutive 16x16x32 products.
__device__ __forceinline__ void to_own_row(u32x4& t0, u32x4& t1) {
  u32x4 s0, s1;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    // row_ror:8 reads lane l ^ 8 of each row of 16 lanes; the bank mask says which lanes take it (0xc: 8..15, 0x3: 0..7)
    s0[i] = __builtin_amdgcn_update_dpp(t0[i], t1[i], 0x128, 0xf, 0xc, false);
    s1[i] = __builtin_amdgcn_update_dpp(t1[i], t0[i], 0x128, 0xf, 0x3, false);
  }
  t0 = s0;
  t1 = s1;
}

__device__ __forceinline__ float bias_at(const MfmaGemmArgs& g, int n) {
  if (!g.bias) return 0.f;
  return g.bias_type == TQ_F32 ? ((const float*)g.bias)[n] : to_f32(((const bf16_t*)g.bias)[n]);
}

template <bool OUT_ACT>
__device__ __forceinline__ void store_out(const MfmaGemmArgs& g, int m, int n, float v) {
  if (OUT_ACT)
    ((bf16_t*)g.out)[(size_t)m * g.ldc + n] = f32_to_bf16(v);
  else
    ((float*)g.out)[(size_t)m * g.ldc + n] = v;
}

