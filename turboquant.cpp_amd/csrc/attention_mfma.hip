// Attention over the paged cache on the matrix cores (bfloat16 in, float softmax and sums).
//
// Formulas as in attention_generic.hip (/root/reference/src/engine/tq_transformer.c:1646-1654 window,
// :1675-1679 head mapping, :1908-1976 scores, softmax, value sum).  A wave works on 16 "columns" that
// share keys and values and runs over tiles of 64 cache positions (a page, or a quarter of one):
//
//   S^T = K Q^T     v_mfma_f32_16x16x32_bf16 with A = 16 keys x 32 of hd (16 bytes per lane straight from the
//                   page, keys lie [row][hd]) and B = the columns' queries, kept in registers.  The 16 rows of
//                   block jt are not 16 consecutive keys: row i is key 32 (jt / 2) + 8 (i / 4) + 4 (jt % 2) + i % 4,
//                   so that lane l, which holds rows 4 (l / 16) + v of every block for column l % 16, holds 8
//                   consecutive keys across the two blocks of a pair.
//   softmax         per column, that is per lane: maxima and sums over a lane's registers and over the four
//                   lanes l % 16 + 16 c; all in float, running maximum across tiles.
//   O^T += V^T P^T  A = 16 of hd x 32 keys (values lie transposed in the page, [hd][row], so a lane reads its 8
//                   consecutive keys of one dimension with 16 bytes) and B = the probabilities exactly as the
//                   lane already holds them.  No transpose through LDS anywhere.
//
// Two entry points share this: whole prompts (columns = 16 consecutive tokens of a sequence, one head; four
// waves per workgroup) and decoding (columns = the query heads that share one kv head, one token; the cache is
// split into runs of 1 or 3 tiles, one wave each, and a second kernel joins the runs in order).  Tiles start at
// multiples of 64 positions and runs at multiples of the run length, so the order of every sum depends only on
// the token's own position.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define TILE 64
#define LOG2E 1.4426950408889634f
// Tiles per run when decoding a token at position p: short sequences are cut finer, so that a small batch still
// gives the chip hundreds of waves; a function of the token's own position only.  Measured with 16 kv heads: at
// position 8191, 3 tiles per run beat 4 by 15 % at 8 sequences and lose 2 to 4 % from 16 on, 2 lose 9 % and 1 loses
// 22 %; at positions 3000 and 4000, 1 tile per run beats 2 by 25 % and 9 % at 8 sequences (4 % and -2 % at 64).
__host__ __device__ __forceinline__ int tiles_per_run(int p) { return p >= 2 * 2048 ? 3 : 1; }
__host__ __device__ __forceinline__ int runs_at(int p) { return p / TILE / tiles_per_run(p) + 1; }
// Most runs that a token at a position below max_end can have.
static int most_runs(int max_end) {
  const int tiles = (max_end + 63) / 64;
  const int short_runs = tiles < 64 ? tiles : 64;          // below position 4096 no token has more than 64
  const int long_runs = (tiles + 2) / 3;
  return short_runs > long_runs ? short_runs : long_runs;
}

struct AttnArgs {
  const bf16_t* q;              // [T][nh][hd]
  const bf16_t* k_pool;         // layer's offset already added
  const bf16_t* v_pool;
  const int* block_table;
  int bt_stride;
  const int* cu_seqlens;        // [B + 1]
  const int* slots;             // [B]
  const int* start;             // [B] position of each sequence's first new token
  int page_size;
  int64_t page_stride;
  int nh, nkv, hd, window;
  float scale;
  bf16_t* out;                  // [T][nh][hd]
  float* partial;               // decoding: [B][nh][max_runs][hd + 2]
  int max_runs;
};

__device__ __forceinline__ bf16x8 ld16(const bf16_t* p) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(bf16x8, v);
}
// For the pages that decoding reads once: a load that tells the caches so.  Measured on a plain read of 1 GiB
// whose instructions take whole lines of 128 bytes: 6.8 TB/s with this hint, 4.7 without.
__device__ __forceinline__ u32x4 ld16_once(const bf16_t* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
// Lanes l and l ^ 8 (the same quarter c = l / 16, rows r and r ^ 8 of a block of 16 rows) fetched whole lines: lane
// (r, c) chunk c + 4 (r / 8) of the block's row r % 8 into t0 and of row 8 + r % 8 into t1.  Afterwards t0 is chunk c
// and t1 chunk c + 4 of the lane's own row r: the operands of two consecutive 16x16x32 products.
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
__device__ __forceinline__ bf16x8 zero16() {
  const uint4 v = make_uint4(0, 0, 0, 0);
  return __builtin_bit_cast(bf16x8, v);
}
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2(float a, float b) {      // round to nearest even, one instruction for the pair
  const bf16x2 v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ float group_max(float v) {     // over the four lanes that share l % 16
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  return fmaxf(v, __shfl_xor(v, 32, 64));
}
__device__ __forceinline__ float group_sum(float v) {
  v += __shfl_xor(v, 16, 64);
  return v + __shfl_xor(v, 32, 64);
}


// Where the workgroup's tiles lie in LDS when the head size is 64, 128 or 256 (rows of 8, 16 or 32 chunks of 16
// bytes, no padding): chunk ch of key row `row` at chunk ch ^ g(row), where g numbers the 16 rows that one
// operand read touches (rows r % 4 + 8 (r / 4) + const) 0..15, or 0..7 twice for rows of 8 chunks; chunk ch of value
// row d (64 positions, 8 chunks) at chunk ch ^ (d & 7).  Measured: such reads run at about 210 bytes per clock
// and compute unit, rows padded by 16 bytes at about 120.
template <int DT>
__device__ __forceinline__ int k_swz(int row, int ch) {
  const int g = DT == 4 ? (((row >> 1) & 1) | (((row >> 3) & 3) << 1)) : ((row & 3) | (((row >> 3) & 3) << 2));
  return row * (16 * DT) + ((ch ^ g) << 3);
}
__device__ __forceinline__ int v_swz(int d, int ch) { return d * TILE + ((ch ^ (d & 7)) << 3); }

// The part of a tile between its two products, for QG groups of 16 columns: s holds the tile's scores (rows of
// block jt as tile_step says); afterwards m_run, l_run and o are brought to the new running maximum and pf holds the
// probabilities 2^(s * scale2 - m) as the operand of the second product.
template <int DT, int QG>
__device__ __forceinline__ void softmax_tile(f32x4 (&s)[QG][4], f32x4 (&o)[QG][DT], float (&m_run)[QG], float (&l_run)[QG],
                                             int pos0, const int (&p_q)[QG], const int (&lo_q)[QG], float scale2,
                                             bool masked, bf16x8 (&pf)[2][QG]) {
  const int c = (threadIdx.x % 64) / 16;
  // mask, running maximum, probabilities
#pragma unroll
  for (int g = 0; g < QG; ++g) {
    float m_tile = -INFINITY;
    if (masked) {
#pragma unroll
      for (int jt = 0; jt < 4; ++jt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int key = pos0 + 32 * (jt / 2) + 8 * c + 4 * (jt % 2) + v;
          const bool ok = key <= p_q[g] && key >= lo_q[g];
          s[g][jt][v] = ok ? s[g][jt][v] : -INFINITY;
          m_tile = fmaxf(m_tile, s[g][jt][v]);
        }
    } else {
#pragma unroll
      for (int jt = 0; jt < 4; ++jt)
#pragma unroll
        for (int v = 0; v < 4; ++v) m_tile = fmaxf(m_tile, s[g][jt][v]);
    }
    m_tile = group_max(m_tile) * scale2;
    const float m_new = fmaxf(m_run[g], m_tile);
    const bool any = m_new != -INFINITY;
    const float alpha = any && m_run[g] != -INFINITY ? __builtin_amdgcn_exp2f(m_run[g] - m_new) : (any ? 0.f : 1.f);
    const float m_use = any ? m_new : 0.f;       // 2^(-inf - 0) = 0 for masked keys, also when all are masked
    float l_tile = 0.f;
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[g][jt][v], scale2, -m_use));
        s[g][jt][v] = p;
        l_tile += p;
      }
    l_run[g] = l_run[g] * alpha + group_sum(l_tile);
    m_run[g] = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int v = 0; v < 4; ++v) o[g][dt][v] *= alpha;
  }
  // the probabilities as the second product's operand: what the lane holds already
#pragma unroll
  for (int pr = 0; pr < 2; ++pr)
#pragma unroll
    for (int g = 0; g < QG; ++g) {
      const u32x4 pw = {pack2(s[g][2 * pr][0], s[g][2 * pr][1]), pack2(s[g][2 * pr][2], s[g][2 * pr][3]),
                        pack2(s[g][2 * pr + 1][0], s[g][2 * pr + 1][1]), pack2(s[g][2 * pr + 1][2], s[g][2 * pr + 1][3])};
      pf[pr][g] = __builtin_bit_cast(bf16x8, pw);
    }
}

// One tile of 64 positions for QG groups of 16 columns that share the tile's keys and values.  kt: the tile's
// keys, row i at kt + i * k_stride; vt: the tile's values transposed, dimension d at vt + d * v_stride (memory or
// LDS).  DT: number of 16-wide blocks of hd held in registers (hd <= 16 * DT).  p_q: position of this lane's
// column in each group (-1: no such column), lo_q: first position it may see; masked: whether any column of the
// wave has a key in this tile that it may not see (if not, the comparisons are left out).  qf: the columns'
// queries, 8 values of hd per 32-wide step at 8 * (l / 16).  Every operand read from kt and vt serves all QG
// groups.  EXACT: hd is exactly 16 DT and DT is even.  SWZ: kt and vt are tiles in LDS laid out by k_swz, v_swz.
// ONCE (with EXACT, tiles in memory that nothing else reads): keys and values are fetched by whole lines of 128
// bytes, eight lanes to a row, and lanes l and l ^ 8 exchange what belongs to the other's row.
// scale2 = scale * log2(e) > 0: maxima are kept in that unit and probabilities are 2^(s * scale2 - m), which is
// exp(s * scale - max) with one instruction for the power.
template <int DT, int QG, bool EXACT, bool SWZ = false, bool ONCE = false>
__device__ __forceinline__ void tile_step(f32x4 (&o)[QG][DT], float (&m_run)[QG], float (&l_run)[QG],
                                          const bf16x8 (&qf)[QG][(DT + 1) / 2], const bf16_t* kt, int k_stride,
                                          const bf16_t* vt, int v_stride, int hd, int pos0, const int (&p_q)[QG],
                                          const int (&lo_q)[QG], float scale2, bool masked) {
  constexpr int KS = (DT + 1) / 2;
  const int lane = threadIdx.x % 64, r = lane % 16, c = lane / 16;
  // EXACT: hd == 16 DT with DT even, so nothing below depends on hd and every product is unconditional
  const int n_dt = EXACT ? DT : hd / 16, n_ks = EXACT ? KS : (hd + 31) / 32;
  static_assert(!ONCE || (EXACT && !SWZ), "whole lines need rows of whole lines, in memory");
  const int r8 = r % 8, q8 = (c + 4 * (r / 8)) * 8;      // ONCE: this lane fetches chunk q8 / 8 of rows r8 and 8 + r8
  f32x4 s[QG][4];
#pragma unroll
  for (int jt = 0; jt < 4; ++jt) {
#pragma unroll
    for (int g = 0; g < QG; ++g) s[g][jt] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (ONCE) {
      const int row_a = 32 * (jt / 2) + 8 * (r8 / 4) + 4 * (jt % 2) + r8 % 4, row_b = row_a + 16;
      u32x4 kf[KS];
#pragma unroll
      for (int p = 0; p < KS / 2; ++p) {
        kf[2 * p] = ld16_once(kt + row_a * k_stride + 64 * p + q8);
        kf[2 * p + 1] = ld16_once(kt + row_b * k_stride + 64 * p + q8);
      }
#pragma unroll
      for (int p = 0; p < KS / 2; ++p) to_own_row(kf[2 * p], kf[2 * p + 1]);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int g = 0; g < QG; ++g)
          s[g][jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf[ks]), qf[g][ks], s[g][jt], 0, 0, 0);
      continue;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks < n_ks) {
        const int d0 = 32 * ks + 8 * c;
        const int krow = 32 * (jt / 2) + 8 * (r / 4) + 4 * (jt % 2) + r % 4;
        const bf16x8 kf = SWZ ? ld16(kt + k_swz<DT>(krow, 4 * ks + c))
                              : (EXACT || d0 < hd ? ld16(kt + krow * k_stride + d0) : zero16());
#pragma unroll
        for (int g = 0; g < QG; ++g) s[g][jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[g][ks], s[g][jt], 0, 0, 0);
      }
    }
  }
  bf16x8 pf[2][QG];
  softmax_tile<DT, QG>(s, o, m_run, l_run, pos0, p_q, lo_q, scale2, masked, pf);
  if (ONCE) {
    // a row of values (64 positions of one dimension) is one line: both halves of the tile come with it
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      u32x4 v0 = ld16_once(vt + (16 * dt + r8) * v_stride + q8), v1 = ld16_once(vt + (16 * dt + 8 + r8) * v_stride + q8);
      to_own_row(v0, v1);
#pragma unroll
      for (int g = 0; g < QG; ++g) {
        o[g][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, v0), pf[0][g], o[g][dt], 0, 0, 0);
        o[g][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, v1), pf[1][g], o[g][dt], 0, 0, 0);
      }
    }
    return;
  }
#pragma unroll
  for (int pr = 0; pr < 2; ++pr) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      if (dt < n_dt) {
        const bf16x8 vf = SWZ ? ld16(vt + v_swz(16 * dt + r, 4 * pr + c)) : ld16(vt + (16 * dt + r) * v_stride + 32 * pr + 8 * c);
#pragma unroll
        for (int g = 0; g < QG; ++g) o[g][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[pr][g], o[g][dt], 0, 0, 0);
      }
    }
  }
}

// Runs the wave's 16 columns over tiles [tile_beg, tile_end) straight from the cache pages.
template <int DT, bool EXACT>
__device__ __forceinline__ void attend(f32x4 (&o)[1][DT], float (&m_run)[1], float (&l_run)[1],
                                       const bf16x8 (&qf)[1][(DT + 1) / 2], const bf16_t* kh, const bf16_t* vh,
                                       const int* table, int page_size, int64_t page_stride, int hd, int tile_beg,
                                       int tile_end, int p, bool valid, int lo_q, float scale2) {
  const int pq[1] = {valid ? p : -1}, lq[1] = {lo_q};
  for (int tile = tile_beg; tile < tile_end; ++tile) {
    const int pos0 = tile * TILE;
    const int page = table[pos0 / page_size];
    const int in_page = pos0 % page_size;
    const bf16_t* kt = kh + (int64_t)page * page_stride + (int64_t)in_page * hd;      // [row][hd]
    const bf16_t* vt = vh + (int64_t)page * page_stride + in_page;                     // [hd][row]
    const bool masked = pos0 + TILE - 1 > p || pos0 < lo_q;      // the same for all lanes
    tile_step<DT, 1, EXACT, false, EXACT>(o, m_run, l_run, qf, kt, hd, vt, page_size, hd, pos0, pq, lq, scale2, masked);
  }
}

// The same run of tiles for a step that has few waves (a handful of sequences): then a wave has a SIMD's registers
// to itself, and keeps a whole tile of keys and values in them (2 DT registers of 16 bytes each, fetched by whole
// lines as in tile_step) while it works on the tile before.  Every product and sum is the one of `attend`, in the same
// order: only the loads go out earlier.
template <int DT>
struct TileRegs {
  u32x4 k[4][DT / 2];       // block jt, step ks of hd (before the exchange between lanes)
  u32x4 v[DT][2];           // block dt of hd, the two halves of the tile's positions
};
template <int DT>
__device__ __forceinline__ void fetch_tile(TileRegs<DT>& t, const bf16_t* kt, int k_stride, const bf16_t* vt, int v_stride) {
  const int lane = threadIdx.x % 64, r = lane % 16, c = lane / 16;
  const int r8 = r % 8, q8 = (c + 4 * (r / 8)) * 8;
#pragma unroll
  for (int jt = 0; jt < 4; ++jt) {
    const int row_a = 32 * (jt / 2) + 8 * (r8 / 4) + 4 * (jt % 2) + r8 % 4, row_b = row_a + 16;
#pragma unroll
    for (int p = 0; p < DT / 4; ++p) {
      t.k[jt][2 * p] = ld16_once(kt + row_a * k_stride + 64 * p + q8);
      t.k[jt][2 * p + 1] = ld16_once(kt + row_b * k_stride + 64 * p + q8);
    }
  }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    t.v[dt][0] = ld16_once(vt + (16 * dt + r8) * v_stride + q8);
    t.v[dt][1] = ld16_once(vt + (16 * dt + 8 + r8) * v_stride + q8);
  }
}
template <int DT>
__device__ __forceinline__ void tile_step_regs(f32x4 (&o)[1][DT], float (&m_run)[1], float (&l_run)[1],
                                               const bf16x8 (&qf)[1][DT / 2], TileRegs<DT>& t, int pos0,
                                               const int (&p_q)[1], const int (&lo_q)[1], float scale2, bool masked) {
  f32x4 s[1][4];
#pragma unroll
  for (int jt = 0; jt < 4; ++jt) {
    s[0][jt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < DT / 4; ++p) to_own_row(t.k[jt][2 * p], t.k[jt][2 * p + 1]);
#pragma unroll
    for (int ks = 0; ks < DT / 2; ++ks)
      s[0][jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, t.k[jt][ks]), qf[0][ks], s[0][jt], 0, 0, 0);
  }
  bf16x8 pf[2][1];
  softmax_tile<DT, 1>(s, o, m_run, l_run, pos0, p_q, lo_q, scale2, masked, pf);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    to_own_row(t.v[dt][0], t.v[dt][1]);
    o[0][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, t.v[dt][0]), pf[0][0], o[0][dt], 0, 0, 0);
    o[0][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, t.v[dt][1]), pf[1][0], o[0][dt], 0, 0, 0);
  }
}
template <int DT>
__device__ __forceinline__ void attend_ahead(f32x4 (&o)[1][DT], float (&m_run)[1], float (&l_run)[1],
                                             const bf16x8 (&qf)[1][DT / 2], const bf16_t* kh, const bf16_t* vh,
                                             const int* table, int page_size, int64_t page_stride, int tile_beg,
                                             int tile_end, int p, bool valid, int lo_q, float scale2) {
  constexpr int hd = 16 * DT;
  const int pq[1] = {valid ? p : -1}, lq[1] = {lo_q};
  TileRegs<DT> t0, t1;
#define TQ_FETCH_TILE(regs, tile)                                                                          \
  do {                                                                                                     \
    const int pos0_ = (tile) * TILE;                                                                       \
    const int64_t base_ = (int64_t)table[pos0_ / page_size] * page_stride;                                 \
    const int in_page_ = pos0_ % page_size;                                                                \
    fetch_tile<DT>(regs, kh + base_ + (int64_t)in_page_ * hd, hd, vh + base_ + in_page_, page_size);       \
  } while (0)
#define TQ_STEP_TILE(regs, tile)                                                                           \
  do {                                                                                                     \
    const int pos0_ = (tile) * TILE;                                                                       \
    const bool masked_ = pos0_ + TILE - 1 > p || pos0_ < lo_q;                                             \
    tile_step_regs<DT>(o, m_run, l_run, qf, regs, pos0_, pq, lq, scale2, masked_);                         \
  } while (0)
  TQ_FETCH_TILE(t0, tile_beg);
  for (int tile = tile_beg; tile < tile_end; tile += 2) {
    if (tile + 1 < tile_end) TQ_FETCH_TILE(t1, tile + 1);
    TQ_STEP_TILE(t0, tile);
    if (tile + 1 < tile_end) {
      if (tile + 2 < tile_end) TQ_FETCH_TILE(t0, tile + 2);
      TQ_STEP_TILE(t1, tile + 1);
    }
  }
#undef TQ_FETCH_TILE
#undef TQ_STEP_TILE
}

template <int DT>
__device__ __forceinline__ void load_query(bf16x8 (&qf)[(DT + 1) / 2], const bf16_t* qrow, int hd, bool valid) {
  const int c = (threadIdx.x % 64) / 16;
#pragma unroll
  for (int ks = 0; ks < (DT + 1) / 2; ++ks) {
    const int d0 = 32 * ks + 8 * c;
    qf[ks] = valid && d0 < hd ? ld16(qrow + d0) : zero16();
  }
}

// ------------------------------------------------------------------------------------------ whole prompts
// grid (blocks of 64 QG new tokens x heads x sequences), block 256: wave w takes tokens 16 QG w .. of its block,
// QG groups of 16.  The cache already holds the step's keys and values.  Blocks are numbered from the end of the
// sequences: a block attends to everything before it, so the longest ones start first and the short ones fill
// the gaps that they leave.  The workgroup brings each tile of keys and values into one of two LDS buffers
// (swizzled for head sizes 64, 128, 256; else key rows padded by KPAD and value rows VSTR long) while it works on
// the other, and the tile after that is on its way from memory into registers meanwhile: one barrier per tile.
#define KPAD 8
#define VSTR 72

template <int DT, int QG, bool EXACT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void attn_prefill_kernel(AttnArgs a, int n_blocks, int B) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  constexpr int QW = 16 * QG;
  constexpr int KCH = (TILE * 2 * DT + 255) / 256;      // 16-byte chunks of a key tile per thread
  constexpr int VCH = (16 * DT * 8 + 255) / 256;        // and of a value tile
  const int hd = EXACT ? 16 * DT : a.hd, kcpr = hd / 8;
  // elements of one buffer: keys [TILE][hd + KPAD], values [hd][VSTR]; swizzled instead of padded when EXACT
  const int kstr = EXACT ? hd : hd + KPAD, vstr = EXACT ? TILE : VSTR;
  const int buf = TILE * kstr + hd * vstr;
  bf16_t* Ks = (bf16_t*)smem_raw;
  bf16_t* Vs = Ks + TILE * kstr;
  const int per_block = a.nh * B;
  const int blk = n_blocks - 1 - (int)blockIdx.x / per_block;
  const int h = (int)blockIdx.x % per_block % a.nh, seq = (int)blockIdx.x % per_block / a.nh;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, r = lane % 16, c = lane / 16;
  const int t0 = a.cu_seqlens[seq], n = a.cu_seqlens[seq + 1] - t0;
  const int qb = blk * 4 * QW;
  if (qb >= n) return;
  const int start = a.start[seq];
  const int kvh = h / (a.nh / a.nkv);
  const int64_t head_off = (int64_t)kvh * a.page_size * hd;
  const int* table = a.block_table + (size_t)a.slots[seq] * a.bt_stride;

  int p_q[QG], lo_q[QG];
  bf16x8 qf[QG][(DT + 1) / 2];
  f32x4 o[QG][DT];
  float m_run[QG], l_run[QG];
#pragma unroll
  for (int g = 0; g < QG; ++g) {
    const int qi = qb + wave * QW + g * 16 + r;
    const bool valid = qi < n;
    p_q[g] = valid ? start + qi : -1;
    lo_q[g] = a.window > 0 ? max(0, p_q[g] - a.window + 1) : 0;
    load_query<DT>(qf[g], a.q + ((size_t)(t0 + (valid ? qi : 0)) * a.nh + h) * hd, hd, valid);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[g][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run[g] = -INFINITY;
    l_run[g] = 0.f;
  }
  // tiles the workgroup goes through, and those among them that this wave's tokens can see
  const int wg_first = start + qb, wg_last = start + min(qb + 4 * QW, n) - 1;
  const int tile_beg = (a.window > 0 ? max(0, wg_first - a.window + 1) : 0) / TILE, tile_end = wg_last / TILE + 1;
  const int wq0 = qb + wave * QW;
  const bool wave_has = wq0 < n;
  const int wave_first = start + wq0, wave_last = start + min(wq0 + QW, n) - 1;
  const int wave_lo_last = a.window > 0 ? max(0, wave_last - a.window + 1) : 0;     // first key of the wave's last token
  const int wave_beg = (a.window > 0 ? max(0, wave_first - a.window + 1) : 0) / TILE;
  const int wave_end = wave_has ? wave_last / TILE + 1 : 0;

  // what this thread carries of every tile: where its chunks lie in the tile in memory and in LDS (a thread
  // past the end of a small tile carries the last chunk once more)
  int k_g[KCH], k_l[KCH], v_g[VCH], v_l[VCH];
#pragma unroll
  for (int j = 0; j < KCH; ++j) {
    const int i = min(tid + j * 256, TILE * kcpr - 1), row = i / kcpr, ch = i % kcpr;
    k_g[j] = row * hd + ch * 8;
    k_l[j] = EXACT ? k_swz<DT>(row, ch) : row * kstr + ch * 8;
  }
#pragma unroll
  for (int j = 0; j < VCH; ++j) {
    const int i = min(tid + j * 256, hd * 8 - 1), d = i / 8, ch = i % 8;
    v_g[j] = d * a.page_size + ch * 8;
    v_l[j] = EXACT ? v_swz(d, ch) : d * vstr + ch * 8;
  }
  u32x4 pk[KCH], pv[VCH];
  const int tiles_per_page = a.page_size / TILE;
  int page_next = table[tile_beg / tiles_per_page];     // page of the tile that the next fetch takes
#define TQ_FETCH(tile)                                                                                      \
  do {                                                                                                      \
    const int64_t base = head_off + (int64_t)page_next * a.page_stride;                                     \
    const int in_page = ((tile) % tiles_per_page) * TILE;                                                   \
    const bf16_t* kg = a.k_pool + base + (int64_t)in_page * hd;                                             \
    const bf16_t* vg = a.v_pool + base + in_page;                                                           \
    _Pragma("unroll") for (int j = 0; j < KCH; ++j) pk[j] = *reinterpret_cast<const u32x4*>(kg + k_g[j]);   \
    _Pragma("unroll") for (int j = 0; j < VCH; ++j) pv[j] = *reinterpret_cast<const u32x4*>(vg + v_g[j]);   \
    if ((tile) + 1 < tile_end) page_next = table[((tile) + 1) / tiles_per_page];                            \
  } while (0)
#define TQ_STAGE(off)                                                                                       \
  do {                                                                                                      \
    _Pragma("unroll") for (int j = 0; j < KCH; ++j) *reinterpret_cast<u32x4*>(Ks + (off) + k_l[j]) = pk[j]; \
    _Pragma("unroll") for (int j = 0; j < VCH; ++j) *reinterpret_cast<u32x4*>(Vs + (off) + v_l[j]) = pv[j]; \
  } while (0)

  TQ_FETCH(tile_beg);
  TQ_STAGE(0);
  if (tile_beg + 1 < tile_end) TQ_FETCH(tile_beg + 1);
  __syncthreads();
  int cur = 0;
  for (int tile = tile_beg; tile < tile_end; ++tile, cur ^= buf) {
    if (tile + 1 < tile_end) {
      TQ_STAGE(cur ^ buf);
      if (tile + 2 < tile_end) TQ_FETCH(tile + 2);
    }
    if (tile >= wave_beg && tile < wave_end) {
      const int pos0 = tile * TILE;
      const bool masked = pos0 + TILE - 1 > wave_first || pos0 < wave_lo_last;
      tile_step<DT, QG, EXACT, EXACT>(o, m_run, l_run, qf, Ks + cur, kstr, Vs + cur, vstr, hd, pos0, p_q, lo_q,
                                      a.scale * LOG2E, masked);
    }
    __syncthreads();
  }
#undef TQ_FETCH
#undef TQ_STAGE
#pragma unroll
  for (int g = 0; g < QG; ++g) {
    if (p_q[g] < 0) continue;
    const float inv = 1.0f / l_run[g];
    bf16_t* orow = a.out + ((size_t)(t0 + p_q[g] - start) * a.nh + h) * hd;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      if (16 * dt < hd) {
        const u32x2 w = {pack2(o[g][dt][0] * inv, o[g][dt][1] * inv), pack2(o[g][dt][2] * inv, o[g][dt][3] * inv)};
        *reinterpret_cast<u32x2*>(orow + 16 * dt + 4 * c) = w;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------ decoding
// One new token per sequence at position start[b].  grid (runs, nkv * ceil(g / 16), B), block 64: the wave
// takes run x (tiles S x .. S x + S - 1, S = tiles_per_run(position)) for up to 16 of the g = nh / nkv heads of one kv head and
// writes their unnormalised sums with maximum and denominator.  The grid has the runs of the step's longest
// sequence, so that no wave is started for nothing where all sequences are about as long (a wave that finds no run
// costs as much to start as one that does: a third more of them made the kernel a fifth slower).  A shorter
// sequence of the same step may still have more runs than that, positions below 4096 being cut finer: its waves
// then take the further runs in turn (wave x the runs x, x + the grid's runs, ...), each into its own place, so
// that no wave has more than one or two of them (left to the last wave alone, 30 runs in a row made a step with
// one sequence beyond position 4096 and seven shorter ones a third slower).
// AHEAD (with EXACT): the form for steps of few waves, which fetches a tile ahead (attend_ahead).
template <int DT, bool EXACT, bool AHEAD = false>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(AHEAD ? 1 : (DT > 8 ? 2 : 3)))) void attn_decode_kernel(AttnArgs a) {
  const int b = blockIdx.z;
  const int g = a.nh / a.nkv, ngc = (g + 15) / 16;
  const int kvh = blockIdx.y / ngc, cg = blockIdx.y % ngc;
  const int lane = threadIdx.x, r = lane % 16, c = lane / 16;
  const int p = a.start[b];
  const int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;
  const int S = tiles_per_run(p), n_runs = runs_at(p);
  if ((int)blockIdx.x >= n_runs) return;
  const int hg = cg * 16 + r;                 // head within the group
  const bool valid = hg < g;
  const int h = kvh * g + (valid ? hg : 0);
  const int64_t head_off = (int64_t)kvh * a.page_size * a.hd;
  const int* table = a.block_table + (size_t)a.slots[b] * a.bt_stride;
  const int t = a.cu_seqlens[b];

  bf16x8 qf[1][(DT + 1) / 2];
  load_query<DT>(qf[0], a.q + ((size_t)t * a.nh + h) * a.hd, a.hd, valid);
  for (int run = blockIdx.x; run < n_runs; run += gridDim.x) {
    const int tile_beg = max(run * S, lo / TILE), tile_end = min((run + 1) * S, p / TILE + 1);
    if (tile_beg >= tile_end) continue;       // all of the run lies before the window
    f32x4 o[1][DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[0][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run[1] = {-INFINITY}, l_run[1] = {0.f};
    if constexpr (AHEAD)
      attend_ahead<DT>(o, m_run, l_run, qf, a.k_pool + head_off, a.v_pool + head_off, table, a.page_size, a.page_stride,
                       tile_beg, tile_end, p, valid, lo, a.scale * LOG2E);
    else
      attend<DT, EXACT>(o, m_run, l_run, qf, a.k_pool + head_off, a.v_pool + head_off, table, a.page_size, a.page_stride,
                        a.hd, tile_beg, tile_end, p, valid, lo, a.scale * LOG2E);
    if (!valid) continue;
    float* out = a.partial + (((size_t)b * a.nh + h) * a.max_runs + run) * (a.hd + 2);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      if (16 * dt < a.hd) {
#pragma unroll
        for (int v = 0; v < 4; ++v) out[16 * dt + 4 * c + v] = o[0][dt][v];
      }
    }
    if (c == 0) {
      out[a.hd] = m_run[0];
      out[a.hd + 1] = l_run[0];
    }
  }
}

// Joins the runs of one (sequence, head) in order of position: grid (nh, B), block 64.  The weights
// 2^(m_s - m) of the runs are worked out once, a lane per run, and kept in LDS; then every lane sums its
// dimensions over the runs in order.
#define MAX_RUNS_LDS 2048
__global__ __launch_bounds__(64) void attn_join_kernel(AttnArgs a) {
  __shared__ float wgt[MAX_RUNS_LDS];
  const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  const int p = a.start[b];
  const int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;
  const int S = tiles_per_run(p);
  const int run_beg = lo / TILE / S, run_end = p / TILE / S + 1;
  const int stride = a.hd + 2;
  const float* part = a.partial + ((size_t)b * a.nh + h) * a.max_runs * stride;
  float m = -INFINITY;
  for (int s = run_beg + lane; s < run_end; s += 64) m = fmaxf(m, part[(size_t)s * stride + a.hd]);
  m = wave_max(m);
  float l = 0.f;
  for (int s0 = run_beg; s0 < run_end; s0 += 64) {     // denominators in run order, 64 runs at a time
    const int s = s0 + lane;
    float w = 0.f, wl = 0.f;
    if (s < run_end) {
      w = __builtin_amdgcn_exp2f(part[(size_t)s * stride + a.hd] - m);      // maxima are in units of log2
      wl = w * part[(size_t)s * stride + a.hd + 1];
      wgt[s - run_beg] = w;
    }
    l += wave_sum(wl);
  }
  __builtin_amdgcn_wave_barrier();
  const float inv = 1.0f / l;
  bf16_t* orow = a.out + ((size_t)a.cu_seqlens[b] * a.nh + h) * a.hd;
  if (a.hd == 128) {          // a lane takes two neighbouring dimensions: one pass over the runs, 8 bytes at a time
    float acc0 = 0.f, acc1 = 0.f;
#pragma unroll 8
    for (int s = run_beg; s < run_end; ++s) {
      const float2 v = *reinterpret_cast<const float2*>(part + (size_t)s * stride + 2 * lane);
      acc0 = fmaf(wgt[s - run_beg], v.x, acc0);
      acc1 = fmaf(wgt[s - run_beg], v.y, acc1);
    }
    *reinterpret_cast<uint32_t*>(orow + 2 * lane) = pack2(acc0 * inv, acc1 * inv);
    return;
  }
  for (int d = lane; d < a.hd; d += 64) {
    float acc = 0.f;
#pragma unroll 8
    for (int s = run_beg; s < run_end; ++s) acc = fmaf(wgt[s - run_beg], part[(size_t)s * stride + d], acc);
    orow[d] = f32_to_bf16(acc * inv);
  }
}

// ------------------------------------------------------------------------------------------ launch
template <int DT, int QG, bool EXACT>
static int launch_prefill(const AttnArgs& a, int B, int max_new, hipStream_t st) {
  const size_t shmem = 2 * (EXACT ? (size_t)2 * TILE * a.hd : (size_t)TILE * (a.hd + KPAD) + (size_t)a.hd * VSTR) * sizeof(bf16_t);
  if (shmem > 48 * 1024)
    (void)hipFuncSetAttribute((const void*)attn_prefill_kernel<DT, QG, EXACT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  const int n_blocks = (max_new + 64 * QG - 1) / (64 * QG);
  if ((int64_t)n_blocks * a.nh * B > 0x7fffffff) return TQ_ERR_UNSUPPORTED;
  hipLaunchKernelGGL((attn_prefill_kernel<DT, QG, EXACT>), dim3(n_blocks * a.nh * B), dim3(256), shmem, st, a, n_blocks, B);
  return 0;
}
template <int DT, bool EXACT>
static void launch_decode(const AttnArgs& a, int B, int grid_runs, hipStream_t st) {
  const int g = a.nh / a.nkv;
  const dim3 grid(grid_runs, a.nkv * ((g + 15) / 16), B);
  // at most a wave to a SIMD: each has the registers to fetch a tile ahead (one sequence at position 8,191: 2.38 ms a
  // step against 2.61; with more waves than that the form is no faster, from twice as many on slower)
  if (EXACT && DT <= 8 && (int64_t)grid.x * grid.y * grid.z <= 1024)
    hipLaunchKernelGGL((attn_decode_kernel<DT, EXACT, EXACT && DT <= 8>), grid, dim3(64), 0, st, a);
  else
    hipLaunchKernelGGL((attn_decode_kernel<DT, EXACT>), grid, dim3(64), 0, st, a);
  hipLaunchKernelGGL(attn_join_kernel, dim3(a.nh, B), dim3(64), 0, st, a);
}

// Number of floats of `partial` that decoding B sequences up to position max_end needs.
TQ_API int64_t tq_attention_decode_scratch(int B, int nh, int hd, int max_end) {
  return (int64_t)B * nh * most_runs(max_end) * (hd + 2);
}

// decode != 0: every sequence brings exactly one token.  max_new: longest run of new tokens of a sequence;
// max_end: largest position + 1 that any token of the step has.
TQ_API int tq_attention_mfma(const void* q, const void* k_pool, const void* v_pool, const int* block_table,
                             int bt_stride, const int* cu_seqlens, const int* slots, const int* start, int page_size,
                             int64_t page_stride, int B, int nh, int nkv, int hd, int window, float scale, void* out,
                             float* partial, int decode, int max_new, int max_end, hipStream_t st) {
  if (B <= 0) return 0;
  if (hd % 16 != 0 || hd < 16 || hd > 256 || page_size % TILE != 0 || nkv <= 0 || nh % nkv != 0)
    return TQ_ERR_UNSUPPORTED;
  if (nh > 65535 || B > 65535 || page_stride % 8 != 0 || !(scale > 0.f)) return TQ_ERR_UNSUPPORTED;
  if (decode && most_runs(max_end) > MAX_RUNS_LDS) return TQ_ERR_UNSUPPORTED;
  AttnArgs a{(const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool, block_table, bt_stride, cu_seqlens, slots,
             start, page_size, page_stride, nh, nkv, hd, window, scale, (bf16_t*)out, partial,
             most_runs(max_end)};
  const int dt = hd / 16;
  // head sizes 64, 128 and 256 have kernels of their own in which nothing depends on hd at run time
  if (decode) {
    if (!partial) return TQ_ERR_BAD_ARG;
    const int grid_runs = runs_at(max_end > 0 ? max_end - 1 : 0);      // the runs of the step's longest sequence
    if (dt == 4) launch_decode<4, true>(a, B, grid_runs, st);
    else if (dt == 8) launch_decode<8, true>(a, B, grid_runs, st);
    else if (dt == 16) launch_decode<16, true>(a, B, grid_runs, st);
    else if (dt < 4) launch_decode<4, false>(a, B, grid_runs, st);
    else if (dt < 8) launch_decode<8, false>(a, B, grid_runs, st);
    else launch_decode<16, false>(a, B, grid_runs, st);
  } else {
    // two groups of 16 tokens per wave, which halves the reads from LDS per product, when that still leaves
    // the chip two workgroups per compute unit and registers allow; else one group
    const bool two = (int64_t)((max_new + 127) / 128) * nh * B >= 512;
    int rc;
    if (dt == 4) rc = two ? launch_prefill<4, 2, true>(a, B, max_new, st) : launch_prefill<4, 1, true>(a, B, max_new, st);
    else if (dt == 8) rc = two ? launch_prefill<8, 2, true>(a, B, max_new, st) : launch_prefill<8, 1, true>(a, B, max_new, st);
    else if (dt == 16) rc = launch_prefill<16, 1, true>(a, B, max_new, st);
    else if (dt < 4) rc = two ? launch_prefill<4, 2, false>(a, B, max_new, st) : launch_prefill<4, 1, false>(a, B, max_new, st);
    else if (dt < 8) rc = two ? launch_prefill<8, 2, false>(a, B, max_new, st) : launch_prefill<8, 1, false>(a, B, max_new, st);
    else rc = launch_prefill<16, 1, false>(a, B, max_new, st);
    if (rc) return rc;
  }
  TQ_LAUNCH_CHECK();
  return 0;
}
