// Matrix products out[m, n] = sum_k a[m, k] * w[n, k] on the matrix cores, bfloat16 in, float sums.
//
// Same contract as the plain product (gemm_generic.hip): optional bias, optional gated pair
// gate(a w^T) * (a w2^T) (gate: silu or another activation), optional row gather and per-row-tile matrices for experts.  Two kernels:
//
//  * gemm_stream_kernel, for few rows (decoding): the work is reading w once.  A wave owns 16 rows of w
//    and streams them straight from memory into the operand registers of v_mfma_f32_16x16x32_bf16 (lane
//    l holds 8 consecutive k of row l % 16).  The loads take whole lines of 128 bytes, eight lanes to a row, with
//    the hint that the bytes are read once, and pairs of lanes then exchange registers: half lines per
//    instruction, which the operand layout would give by itself, read a quarter slower.  The few rows of `a`
//    are read the same way, without the hint, and stay in cache.  The waves of a workgroup split k among them and
//    add their partial sums in wave order through LDS, so that even a narrow matrix gives the chip enough
//    waves and bytes in flight.  How k is split depends on N and K only, never on the number of rows.
//  * gemm_tile_kernel, for many rows (prompts): tiles of BM x 128 outputs by eight waves, 64 of k at a time staged
//    through two LDS buffers (16-byte chunks, XOR-swizzled by row so that the operand reads of
//    v_mfma_f32_32x32x16_bf16 do not collide); while one buffer is multiplied the next tile is written into
//    the other and the one after that is on its way from memory.
//
// Operand layouts (wave of 64 lanes): 16x16x32: A lane l = row l%16, k 8*(l/16)..+7; B lane l = column l%16,
// same k; D lane l = column l%16, rows 4*(l/16)+v, v<4.  32x32x16: A lane l = row l%32, k 8*(l/32)..+7;
// B alike; D lane l = column l%32, rows 8*(v/4) + 4*(l/32) + v%4, v<16.
#include "common.h"

#include "gemm_mfma.h"

// ------------------------------------------------------------------------------------------ few rows
// The sums of one wave: its share k_beg .. k_end of k for NTL tiles of 16 columns (tile t starts at column col0[t])
// and MT tiles of 16 rows (ap: the rows of `a` that this lane fetches, q: its chunk of 8 within each 64 of k).
template <int MT, bool DUAL, int NTL>
__device__ __forceinline__ void stream_accumulate(const MfmaGemmArgs& g, const int (&col0)[NTL], int group,
                                                  const bf16_t* const (&ap)[MT][2], int q, int k_beg, int k_end,
                                                  f32x4 (&acc)[NTL][MT], f32x4 (&acc2)[DUAL ? NTL : 1][DUAL ? MT : 1]) {
  const int r = (threadIdx.x % 64) % 16;
#pragma unroll
  for (int t = 0; t < NTL; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (DUAL) acc2[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  // U steps of 32 at a time, every load issued before the first product, so that a wave keeps U (2U with the
  // gated pair) kilobytes of w in flight per column tile.  w and a are fetched by whole lines: for each pair of
  // steps (64 of k, 128 bytes of a row) eight lanes take a row, one instruction the tile's rows 0..7 and the next
  // rows 8..15, and lanes l and l ^ 8 then exchange what belongs to the other's row.  Rows of w that do not exist
  // read row 0 instead (what they produce is never stored); rows of a that do not exist, and chunks beyond the
  // wave's share or beyond K, load nothing and multiply zeros.
  constexpr int U_ONE = (DUAL ? 4 : 8) / (MT == 4 ? 2 : 1);
  constexpr int U = U_ONE / NTL >= 2 ? U_ONE / NTL : 2;
  {
    size_t row_a[NTL], row_b[NTL];
#pragma unroll
    for (int t = 0; t < NTL; ++t) {
      const int n_a = col0[t] + r % 8, n_b = n_a + 8;
      row_a[t] = (size_t)group * g.group_stride + (size_t)(n_a < g.N ? n_a : 0) * g.K + q * 8;
      row_b[t] = (size_t)group * g.group_stride + (size_t)(n_b < g.N ? n_b : 0) * g.K + q * 8;
    }
    const u32x4 zero = {0u, 0u, 0u, 0u};
    for (int k = k_beg; k < k_end; k += 32 * U) {
      u32x4 wf[NTL][U], vf[DUAL ? NTL : 1][DUAL ? U : 1];
      u32x4 af[MT][U];
#pragma unroll
      for (int j = 0; j < U / 2; ++j) {
        const int kp = k + 64 * j;
        const bool okw = kp + q * 8 < k_end;      // k_end <= K, both multiples of 8: a chunk is in or out as a whole
#pragma unroll
        for (int t = 0; t < NTL; ++t) {
          wf[t][2 * j] = okw ? load16_once(g.w + row_a[t] + kp) : zero;
          wf[t][2 * j + 1] = okw ? load16_once(g.w + row_b[t] + kp) : zero;
          if (DUAL) {
            vf[t][2 * j] = okw ? load16_once(g.w2 + row_a[t] + kp) : zero;
            vf[t][2 * j + 1] = okw ? load16_once(g.w2 + row_b[t] + kp) : zero;
          }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int hf = 0; hf < 2; ++hf)
            af[mt][2 * j + hf] = okw && ap[mt][hf] ? *reinterpret_cast<const u32x4*>(ap[mt][hf] + kp) : zero;
      }
#pragma unroll
      for (int j = 0; j < U / 2; ++j) {
#pragma unroll
        for (int t = 0; t < NTL; ++t) {
          to_own_row(wf[t][2 * j], wf[t][2 * j + 1]);
          if (DUAL) to_own_row(vf[t][2 * j], vf[t][2 * j + 1]);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) to_own_row(af[mt][2 * j], af[mt][2 * j + 1]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const bf16x8 ax = __builtin_bit_cast(bf16x8, af[mt][u]);
#pragma unroll
          for (int t = 0; t < NTL; ++t) {
            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax, __builtin_bit_cast(bf16x8, wf[t][u]), acc[t][mt], 0, 0, 0);
            if (DUAL)
              acc2[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax, __builtin_bit_cast(bf16x8, vf[t][u]), acc2[t][mt], 0, 0, 0);
          }
        }
    }
  }
}

// A workgroup of 64 * (waves that split k) threads takes column tile `tile_n` (16 * NTL columns) of row tile
// `tile_m` (16 * MT rows) over run `z` of k (k_per long; run 0 is all of k unless the product is split into
// partial sums); red: LDS of [waves][NTL * MT * (DUAL ? 2 : 1)][4][64] floats.  What a wave reads of `a` serves
// its NTL tiles of 16 columns: with many rows the way of `a` from L2 into the compute unit is what binds, and two
// column tiles per wave halve it.
template <int MT, bool DUAL, bool OUT_ACT, int NTL = 1>
__device__ __forceinline__ void stream_body(MfmaGemmArgs g, int tile_n, int tile_m, int z, float* red) {
  if (g.n_tiles && tile_m >= g.n_tiles[0]) return;
  const int k_lo = z * g.k_per, k_hi = min(g.K, k_lo + g.k_per);
  if (z) {
    g.out = (float*)g.out + z * g.split_stride;
    g.bias = nullptr;
  }
  const int group = g.tile_group ? g.tile_group[tile_m] : 0;
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, nw = blockDim.x / 64;
  const int r = lane % 16, c = lane / 16;
  const int n0 = tile_n * 16 * NTL, m0 = tile_m * 16 * MT;
  // the rows of `a` that this lane fetches: r % 8 and 8 + r % 8 of each tile of 16 (as with w below)
  const int q = c + 4 * (r / 8);            // and the chunk of 8 within each 64 of k
  const bf16_t* ap[MT][2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const int m = m0 + mt * 16 + 8 * hf + r % 8;
      int src = -1;
      if (m < g.M) {
        src = g.a_rows ? g.a_rows[m] : m;
        if (src >= 0 && !g.a_gather) src = m;
      }
      ap[mt][hf] = src >= 0 ? g.a + (size_t)src * g.lda + q * 8 : nullptr;
    }
  // this wave's share of k, in steps of 32; an even number of them, so that every pair of steps is a line of w
  const int steps = (k_hi - k_lo + 31) / 32;
  const int per = ((steps + nw - 1) / nw + 1) & ~1;
  const int k_beg = k_lo + wave * per * 32, k_end = min(k_hi, k_lo + (wave + 1) * per * 32);

  f32x4 acc[NTL][MT], acc2[DUAL ? NTL : 1][DUAL ? MT : 1];
  int col0[NTL];
#pragma unroll
  for (int t = 0; t < NTL; ++t) col0[t] = n0 + 16 * t;
  stream_accumulate<MT, DUAL, NTL>(g, col0, group, ap, q, k_beg, k_end, acc, acc2);
  // The waves' partial sums are added in wave order, every thread of the workgroup taking some of the outputs.
  constexpr int PAIRS = NTL * MT;               // (column tile, row tile) pairs: set t * MT + mt, the gate's partner PAIRS on
  constexpr int SETS = PAIRS * (DUAL ? 2 : 1);
  if (nw > 1) {
#pragma unroll
    for (int t = 0; t < NTL; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          red[((wave * SETS + t * MT + mt) * 4 + v) * 64 + lane] = acc[t][mt][v];
          if (DUAL) red[((wave * SETS + PAIRS + t * MT + mt) * 4 + v) * 64 + lane] = acc2[t][mt][v];
        }
    __syncthreads();
    for (int i = threadIdx.x; i < PAIRS * 256; i += blockDim.x) {
      const int ol = i % 64, v = (i / 64) % 4, pair = i / 256, mt = pair % MT, t = pair / MT;
      float s = 0.f, s2 = 0.f;
      for (int w = 0; w < nw; ++w) {
        s += red[((w * SETS + pair) * 4 + v) * 64 + ol];
        if (DUAL) s2 += red[((w * SETS + PAIRS + pair) * 4 + v) * 64 + ol];
      }
      const int on = n0 + 16 * t + ol % 16, om = m0 + mt * 16 + 4 * (ol / 16) + v;
      if (on >= g.N || om >= g.M) continue;
      if (g.a_rows && g.a_rows[om] < 0) continue;
      float o = s + bias_at(g, on);
      if (DUAL) o = gate_fn(o, g.gate) * s2;
      store_out<OUT_ACT>(g, om, on, o);
    }
    return;
  }
#pragma unroll
  for (int t = 0; t < NTL; ++t) {
    const int n = n0 + 16 * t + r;
    if (n >= g.N) continue;
    const float b = bias_at(g, n);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int m = m0 + mt * 16 + 4 * c + v;
        if (m >= g.M) continue;
        if (g.a_rows && g.a_rows[m] < 0) continue;
        float o = acc[t][mt][v] + b;
        if (DUAL) o = gate_fn(o, g.gate) * acc2[t][mt][v];
        store_out<OUT_ACT>(g, m, n, o);
      }
  }
}

// grid (ceil(N / (16 NTL)), row tiles of 16 * MT rows, runs of k).  Two column tiles per wave need the registers of a
// workgroup of at most 8 waves.
template <int MT, bool DUAL, bool OUT_ACT, int NTL>
__global__ __launch_bounds__(NTL > 1 ? 512 : 1024) void gemm_stream_kernel(MfmaGemmArgs g) {
  extern __shared__ float red[];
  stream_body<MT, DUAL, OUT_ACT, NTL>(g, blockIdx.x, blockIdx.y, blockIdx.z, red);
}

// Two products that do not depend on each other in one launch (decoding: the routed experts' product beside
// the shared expert's): workgroups 0 .. n2 - 1 take the second, smaller one (column tile id % nx2 of row tile
// id / nx2 % rows2, run id / nx2 / rows2 of k), so that it is under way at once, the others the first.  Both are
// split over k by the waves of this launch; the second one, when its k is much longer than the first one's, also
// into runs whose partial sums go out apart.
template <bool DUAL, bool OUT_ACT>
__global__ __launch_bounds__(1024) void gemm_stream_pair_kernel(MfmaGemmArgs g1, int nx1, MfmaGemmArgs g2, int nx2,
                                                                 int rows2, int n2) {
  extern __shared__ float red[];
  const int id = blockIdx.x;
  if (id < n2)
    stream_body<1, DUAL, OUT_ACT>(g2, id % nx2, id / nx2 % rows2, id / nx2 / rows2, red);
  else
    stream_body<1, DUAL, OUT_ACT>(g1, (id - n2) % nx1, (id - n2) / nx1, 0, red);
}

// ------------------------------------------------------------------------------------------ q, k, v of a few tokens
// The product that makes queries, keys and values of up to 16 tokens, with what follows it in the same launch:
// bias, rotation of queries and keys (pairs (d, d + hd / 2), the whole head rotated), queries out in bfloat16,
// keys and values into their cache pages (as rope_kv_write_kernel of elementwise.hip does it from the float
// product; same formulas, same float arithmetic).  A workgroup takes the two tiles of 16 columns that hold the
// partners of 16 pairs of one head: columns head * hd + 16 j .. and the same + hd / 2; grid (heads * hd / 32), the
// waves split k.
struct RopeWriteArgs {
  const int* positions;        // [T]
  const int* seq_of_token;     // [T]
  const int* block_table;
  int bt_stride;
  const float* inv_freq;       // [hd / 2]
  bf16_t* q_out;               // [T][nh * hd]
  bf16_t* k_pool;              // the layer's offset already added; null: keys and values are not written
  bf16_t* v_pool;
  int page_size;
  int64_t page_stride;
  int nh, nkv, hd;
};

__global__ __launch_bounds__(512) void qkv_rope_write_kernel(MfmaGemmArgs g, RopeWriteArgs p) {
  extern __shared__ float red[];       // [waves][2][4][64]
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, nw = blockDim.x / 64;
  const int r = lane % 16, c = lane / 16;
  const int per_head = p.hd / 32;
  const int head = blockIdx.x / per_head, j = blockIdx.x % per_head;
  const int col0[2] = {head * p.hd + 16 * j, head * p.hd + p.hd / 2 + 16 * j};
  const int q = c + 4 * (r / 8);
  const bf16_t* ap[1][2];
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    const int m = 8 * hf + r % 8;
    ap[0][hf] = m < g.M ? g.a + (size_t)m * g.lda + q * 8 : nullptr;
  }
  const int steps = (g.K + 31) / 32;
  const int per = ((steps + nw - 1) / nw + 1) & ~1;
  const int k_beg = wave * per * 32, k_end = min(g.K, (wave + 1) * per * 32);
  f32x4 acc[2][1], acc2[1][1];
  stream_accumulate<1, false, 2>(g, col0, 0, ap, q, k_beg, k_end, acc, acc2);
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int v = 0; v < 4; ++v) red[((wave * 2 + t) * 4 + v) * 64 + lane] = acc[t][0][v];
  __syncthreads();
  for (int i = threadIdx.x; i < 256; i += blockDim.x) {
    const int ol = i % 64, v = i / 64;
    const int m = 4 * (ol / 16) + v, d = 16 * j + ol % 16;      // token and dimension (of the pair's first half)
    if (m >= g.M) continue;
    float a = 0.f, b = 0.f;
    for (int w = 0; w < nw; ++w) {      // in wave order, as the product alone adds them
      a += red[((w * 2 + 0) * 4 + v) * 64 + ol];
      b += red[((w * 2 + 1) * 4 + v) * 64 + ol];
    }
    a += bias_at(g, col0[0] + ol % 16);
    b += bias_at(g, col0[1] + ol % 16);
    const int pos = p.positions[m];
    if (head < p.nh + p.nkv) {
      const float theta = (float)pos * p.inv_freq[d];
      float sn, cs;
      sincosf(theta, &sn, &cs);
      const float ra = a * cs - b * sn, rb = a * sn + b * cs;
      a = ra;
      b = rb;
    }
    if (head < p.nh) {
      bf16_t* dst = p.q_out + ((size_t)m * p.nh + head) * p.hd;
      dst[d] = f32_to_bf16(a);
      dst[d + p.hd / 2] = f32_to_bf16(b);
      continue;
    }
    if (!p.k_pool) continue;
    const int page = p.block_table[(size_t)p.seq_of_token[m] * p.bt_stride + pos / p.page_size];
    const int row = pos % p.page_size;
    const size_t kv_head_stride = (size_t)p.page_size * p.hd;
    if (head < p.nh + p.nkv) {         // keys lie [row][hd]
      bf16_t* dst = p.k_pool + (size_t)page * p.page_stride + (size_t)(head - p.nh) * kv_head_stride + (size_t)row * p.hd;
      dst[d] = f32_to_bf16(a);
      dst[d + p.hd / 2] = f32_to_bf16(b);
    } else {                           // values lie transposed, [hd][row]
      bf16_t* dst = p.v_pool + (size_t)page * p.page_stride + (size_t)(head - p.nh - p.nkv) * kv_head_stride + row;
      dst[(size_t)d * p.page_size] = f32_to_bf16(a);
      dst[(size_t)(d + p.hd / 2) * p.page_size] = f32_to_bf16(b);
    }
  }
}

// ------------------------------------------------------------------------------------------ many rows
// grid (row tiles of BM, ceil(N / BN)); block of 8 waves laid WM x WN over the tile of BM x BN outputs (BN = 128
// unless said): BM = 128 as 4 x 2 (a wave owns 32 x 64 outputs, or 32 x 96 with BN = 192; the experts' gated pair as
// 2 x 4, 64 x 32 of each of its two products), BM = 256 as 4 x 2 (64 x 64 or 64 x 96), BM = 64 as 2 x 4 (32 x 32).  Eight waves beat four here: twice the waves hide twice the latency.
#define TBN 128
// Most LDS for the sums of the waves that split k: 128 KB lets the gated pair of 64 rows have 8 waves (22.7 us for the
// shared expert at 64 rows against 25.1 with 4).
#define TQ_STREAM_LDS (128 * 1024)
#define TBK 64

// Where 16-byte chunk `chunk` of row `row` lies in a tile: rows of 128 bytes, the chunk index XOR-ed with bits 1..3
// of the row.  Measured with ds_read_b128 in the operand layout (lane l reads row l % 32): this runs at the full
// 128 bytes per clock; XOR with bits 0..2 at 107, no swizzle at 31.
__device__ __forceinline__ int swz(int row, int chunk) { return row * TBK + ((chunk ^ ((row >> 1) & 7)) << 3); }

template <int BM, int WM, int WN, bool DUAL, bool OUT_ACT, int BN = TBN>
__global__ __launch_bounds__(64 * WM * WN) void gemm_tile_kernel(MfmaGemmArgs g) {
  constexpr int NT = 64 * WM * WN;
  constexpr int MI = BM / WM / 32;               // 32-high row tiles per wave
  constexpr int NI = BN / WN / 32;              // 32-wide column tiles per wave
  constexpr int A_CH = BM * 8 / NT;              // 16-byte chunks of the a tile per thread
  constexpr int W_CH = BN * 8 / NT;
  static_assert(MI >= 1 && NI >= 1 && A_CH >= 1 && W_CH >= 1 && BM * 8 % NT == 0 && BN * 8 % NT == 0, "tile layout");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // two buffers, each a tile of `a`, one of `w` and (gated pair) one of `w2`
  constexpr int BUF = (BM + BN * (DUAL ? 2 : 1)) * TBK;
  bf16_t* As = (bf16_t*)smem;
  bf16_t* Ws = As + BM * TBK;
  bf16_t* Vs = Ws + BN * TBK;
  // Which tile this workgroup takes.  Workgroups are dealt to the chip's 8 dies in turn (id % 8), and each die
  // has its own L2: so the tiles are numbered such that one die gets a contiguous run of them.  One matrix: a
  // run goes through bands of 8 row tiles, down a band's column of row tiles first, so that workgroups that run
  // at the same time on a die share their tiles of `a` and of `w` in that die's L2.  A matrix per expert: a run
  // goes expert by expert, so that an expert's matrix is read by one die (by two where a run ends), and within an
  // expert column by column with the expert's row tiles side by side (measured against row tile by row tile: 6 to
  // 12 % faster, the more the more row tiles an expert has); only the row tiles in use are dealt.
  int tile_m, tile_n;
  {
    // an entry of tile_group (and a unit of n_tiles) stands for `ratio` row tiles of this kernel where the row
    // order was padded to a multiple of the tile's height
    const int ratio = g.group_ratio > 1 ? g.group_ratio : 1;
    const int gx = g.tile_group && g.n_tiles ? min(g.n_tiles[0] * ratio, (int)gridDim.x) : (int)gridDim.x;
    const int gy = gridDim.y, total = gx * gy;
    const int id = blockIdx.y * gridDim.x + blockIdx.x;
    const int die = id % 8, q = total / 8, rem = total % 8;
    if (id / 8 >= q + (die < rem ? 1 : 0)) return;
    const int logical = die * q + min(die, rem) + id / 8;
    if (g.tile_group) {
      // the expert whose row tiles [lo, hi) hold row tile logical / gy; within it column by column, the expert's
      // row tiles of a column one after the other, so that they read that column's rows of w at the same time
      const int u = logical / gy / ratio, e = g.tile_group[u], gu = gx / ratio;
      int lo = u, hi = u + 1;
      while (lo > 0 && g.tile_group[lo - 1] == e) --lo;
      while (hi < gu && g.tile_group[hi] == e) ++hi;
      lo *= ratio;
      hi *= ratio;
      const int local = logical - lo * gy, n_e = hi - lo;
      tile_n = local / n_e;
      tile_m = lo + local % n_e;
    } else {
      const int band = logical / (8 * gy), in_band = logical % (8 * gy);
      const int bh = min(8, gx - band * 8);
      tile_m = band * 8 + in_band % bh;
      tile_n = in_band / bh;
    }
  }
  const int group = g.tile_group ? g.tile_group[tile_m / (g.group_ratio > 1 ? g.group_ratio : 1)] : 0;
  const bf16_t* w = g.w + (size_t)group * g.group_stride;
  const bf16_t* w2 = DUAL ? g.w2 + (size_t)group * g.group_stride : nullptr;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  // an expert's rows stand at the head of its units: a tile that begins with a row of padding holds nothing else
  if (g.tile_group && g.a_rows && g.a_rows[min(m0, g.M - 1)] < 0) return;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / WN, wn = wave % WN;
  // A wave whose rows of an expert's tile are all padding (the expert's last tile is half empty on average) has
  // nothing to multiply: it fetches and stages its share of the tile and waits at the barriers.
  const int wave_m0 = m0 + wm * (MI * 32);
  const bool active = !(g.tile_group && g.a_rows) || (wave_m0 < g.M && g.a_rows[wave_m0] >= 0);
  // this workgroup's run of k: k_lo .. k_lo + Kl (all of k unless the product is split), and where its sums go
  const int k_lo = blockIdx.z * g.k_per;
  const int Kl = min(g.K, k_lo + g.k_per) - k_lo;
  if (blockIdx.z) {
    g.out = (float*)g.out + blockIdx.z * g.split_stride;
    g.bias = nullptr;
  }

  // What this thread fetches of each tile: chunk `ch` of row `row`.  Rows past the end of `a` or `w`, and rows
  // of padding in an expert's tile, read some valid row instead: an output depends on its own row of `a` and
  // of `w` only, and those outputs are never stored.  So the loads need no predicate.
  const bf16_t* a_src[A_CH];
  int a_dst[A_CH], w_dst[W_CH];
  const bf16_t *w_src[W_CH], *v_src[W_CH];
#pragma unroll
  for (int i = 0; i < A_CH; ++i) {
    const int idx = tid + i * NT, row = idx / 8, ch = idx % 8;
    const int m = min(m0 + row, g.M - 1);
    int src = m;
    if (g.a_rows && g.a_gather) src = max(g.a_rows[m], 0);
    a_src[i] = g.a + (size_t)src * g.lda + k_lo + ch * 8;
    a_dst[i] = swz(row, ch);
  }
#pragma unroll
  for (int i = 0; i < W_CH; ++i) {
    const int idx = tid + i * NT, row = idx / 8, ch = idx % 8;
    const int n = min(n0 + row, g.N - 1);
    w_src[i] = w + (size_t)n * g.K + k_lo + ch * 8;
    v_src[i] = DUAL ? w2 + (size_t)n * g.K + k_lo + ch * 8 : nullptr;
    w_dst[i] = swz(row, ch);
  }
  const int ch_of_thread = tid % 8;     // (tid + i * NT) % 8

  f32x16 acc[MI][NI], acc2[DUAL ? MI : 1][DUAL ? NI : 1];
#pragma unroll
  for (int mi = 0; mi < MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        acc[mi][ni][v] = 0.f;
        if (DUAL) acc2[mi][ni][v] = 0.f;
      }

  u32x4 pa[A_CH], pw[W_CH], pv[DUAL ? W_CH : 1];
  const u32x4 z = {0u, 0u, 0u, 0u};
  // FETCH: the thread's chunks of the tile at k0 into registers; only the last tile of a K that is no multiple
  // of 64 needs zeros past the end.  STAGE: registers into LDS.  (Written as macros so that the small arrays
  // above are only ever indexed by constants and stay in registers.)
#define TQ_FETCH(k0)                                                                                          \
  do {                                                                                                        \
    if ((k0) + TBK <= Kl) {                                                                                   \
      _Pragma("unroll") for (int i = 0; i < A_CH; ++i)                                                        \
          pa[i] = *reinterpret_cast<const u32x4*>(a_src[i] + (k0));                                           \
      _Pragma("unroll") for (int i = 0; i < W_CH; ++i) {                                                      \
        pw[i] = *reinterpret_cast<const u32x4*>(w_src[i] + (k0));                                             \
        if (DUAL) pv[i] = *reinterpret_cast<const u32x4*>(v_src[i] + (k0));                                   \
      }                                                                                                       \
    } else {                                                                                                  \
      const bool k_ok = (k0) + ch_of_thread * 8 < Kl;                                                         \
      _Pragma("unroll") for (int i = 0; i < A_CH; ++i)                                                        \
          pa[i] = k_ok ? *reinterpret_cast<const u32x4*>(a_src[i] + (k0)) : z;                                \
      _Pragma("unroll") for (int i = 0; i < W_CH; ++i) {                                                      \
        pw[i] = k_ok ? *reinterpret_cast<const u32x4*>(w_src[i] + (k0)) : z;                                  \
        if (DUAL) pv[i] = k_ok ? *reinterpret_cast<const u32x4*>(v_src[i] + (k0)) : z;                        \
      }                                                                                                       \
    }                                                                                                         \
  } while (0)
#define TQ_STAGE(off)                                                                                         \
  do {                                                                                                        \
    _Pragma("unroll") for (int i = 0; i < A_CH; ++i) *reinterpret_cast<u32x4*>(As + (off) + a_dst[i]) = pa[i]; \
    _Pragma("unroll") for (int i = 0; i < W_CH; ++i) {                                                        \
      *reinterpret_cast<u32x4*>(Ws + (off) + w_dst[i]) = pw[i];                                               \
      if (DUAL) *reinterpret_cast<u32x4*>(Vs + (off) + w_dst[i]) = pv[i];                                     \
    }                                                                                                         \
  } while (0)

  // Tile t is computed from buffer t % 2 while tile t + 1 goes from registers into the other buffer and tile
  // t + 2 is on its way from memory into registers: one barrier per step of 64 of k.
  TQ_FETCH(0);
  TQ_STAGE(0);
  if (TBK < Kl) TQ_FETCH(TBK);
  __syncthreads();
  const int lr = lane % 32, lc = lane / 32;
  int cur = 0;
  for (int k0 = 0; k0 < Kl; k0 += TBK, cur ^= BUF) {
    if (k0 + TBK < Kl) {
      TQ_STAGE(cur ^ BUF);
      if (k0 + 2 * TBK < Kl) TQ_FETCH(k0 + 2 * TBK);
    }
    const bf16_t* Ac = As + cur;
    const bf16_t* Wc = Ws + cur;
    const bf16_t* Vc = Vs + cur;
    if (active)
#pragma unroll
    for (int j = 0; j < TBK / 16; ++j) {
      bf16x8 af[MI], wf[NI], vf[DUAL ? NI : 1];
#pragma unroll
      for (int mi = 0; mi < MI; ++mi) {
        const int row = wm * (MI * 32) + mi * 32 + lr;
        af[mi] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(Ac + swz(row, 2 * j + lc)));
      }
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) {
        const int row = wn * (NI * 32) + ni * 32 + lr;
        wf[ni] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(Wc + swz(row, 2 * j + lc)));
        if (DUAL) vf[ni] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(Vc + swz(row, 2 * j + lc)));
      }
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mi], wf[ni], acc[mi][ni], 0, 0, 0);
          if (DUAL) acc2[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mi], vf[ni], acc2[mi][ni], 0, 0, 0);
        }
    }
    __syncthreads();
  }
#undef TQ_FETCH
#undef TQ_STAGE

  if (!active) return;
#pragma unroll
  for (int ni = 0; ni < NI; ++ni) {
    const int n = n0 + wn * (NI * 32) + ni * 32 + lr;
    if (n >= g.N) continue;
    const float b = bias_at(g, n);
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * (MI * 32) + mi * 32 + 8 * (v / 4) + 4 * lc + (v % 4);
        if (m >= g.M) continue;
        if (g.a_rows && g.a_rows[m] < 0) continue;
        float o = acc[mi][ni][v] + b;
        if (DUAL) o = gate_fn(o, g.gate) * acc2[mi][ni][v];
        store_out<OUT_ACT>(g, m, n, o);
      }
  }
}

// ------------------------------------------------------------------------------------------ experts with many rows
// A matrix per expert whose rows are ordered in units of 64: a workgroup of 16 waves takes an item of the row order,
// two units of one expert (or the expert's last one alone), and 256 columns: 128 of each matrix of a gated pair, or
// 256 of one matrix.  What binds such a product is the bytes that a compute unit has on their way: every tile of 64
// rows asks for its expert's matrices again, and a tile's bytes travel for the time of a miss whoever holds them,
// since a wave's loads come back in the order it asked.  With the tile kernel's loads, stores into LDS and products
// taken out one at a time, 2,048 tokens over 60 experts of 1,408 x 2,048 took 215 us without the products, 225
// without the reads from LDS, 155 without the loads (248 whole); reads that hit in a die's L2 alone run at 31 TB/s,
// three times what the tile kernel moves.  So two units per workgroup, for which an expert's matrices pass two
// thirds as often, and the tiles straight from memory into a ring of three LDS stages (global_load_lds_dwordx4: no
// registers in between, no stores into LDS by the waves), two of them on their way while the third is multiplied
// (with one on its way the tiles alone took 205 us, with two 153).  A load instruction of a wave fills eight rows
// of 128 bytes in LDS, lane l the l-th chunk of 16 bytes: the XOR swizzle of the tile kernel is therefore applied
// to what a lane asks for, not to where it lands.  The ring leaves one workgroup to a compute unit; its barrier
// is a bare s_barrier behind a wait for the wave's own loads of the tile that is due (a __syncthreads would wait
// for the loads of the later tiles too).  Tried and slower: all reads of a step from LDS before its first product
// (230 us against 209), a ring of four stages for w with the tiles of a asked for by waves of their own one step
// ahead (247), the same with the tiles of a through registers (the compiler waits for every load before each store).
// The sums of an output run over k in the same order as in the tile kernel: same bits.
#define RING_STAGES 3
__device__ __forceinline__ void load_to_lds16(const bf16_t* src, bf16_t* wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)wave_base, 16, 0, 0);
}

template <bool DUAL, bool OUT_ACT>
__global__ __launch_bounds__(1024) void gemm_ring_kernel(MfmaGemmArgs g) {
  constexpr int BM = 128, BH = 128;                  // rows of a; columns per half of the tile of w
  constexpr int STAGE = (BM + 2 * BH) * TBK;         // elements of one stage
  constexpr int L = 3;                               // loads per thread and stage: its chunk of a, of either half of w
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16_t* ring = (bf16_t*)smem;
  const int units_all = g.M / 64;
  const int* items = g.tile_group + units_all;
  const int n_units = min(g.n_tiles[0], units_all);
  const int n_items = min(g.n_tiles[1], units_all);
  // the items are dealt to the dies as the tile kernel deals an expert's row tiles: a die gets a contiguous run,
  // expert by expert, within an expert column by column with the expert's items of a column side by side
  int item, tile_n;
  {
    const int gy = gridDim.y, total = n_items * gy;
    const int id = blockIdx.y * gridDim.x + blockIdx.x;
    const int die = id % 8, q = total / 8, rem = total % 8;
    if (id / 8 >= q + (die < rem ? 1 : 0)) return;
    const int logical = die * q + min(die, rem) + id / 8;
    const int p = logical / gy, e = g.tile_group[items[p]];
    int lo = p, hi = p + 1;
    while (lo > 0 && g.tile_group[items[lo - 1]] == e) --lo;
    while (hi < n_items && g.tile_group[items[hi]] == e) ++hi;
    const int local = logical - lo * gy, n_e = hi - lo;
    tile_n = local / n_e;
    item = lo + local % n_e;
  }
  const int u0 = items[item];
  const int units = (item + 1 < n_items ? items[item + 1] : n_units) - u0 >= 2 ? 2 : 1;
  const int group = g.tile_group[u0];
  const bf16_t* w = g.w + (size_t)group * g.group_stride;
  const bf16_t* w2 = DUAL ? g.w2 + (size_t)group * g.group_stride : w;
  const int m0 = u0 * 64;
  const int n0 = tile_n * (DUAL ? BH : 2 * BH);      // first column of the first half
  const int n1 = DUAL ? n0 : n0 + BH;                // and of the second (the other matrix's same columns, or the next 128)
  const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wm = wave / 4, wn = wave % 4;            // 4 x 4 waves, each 32 rows x 32 columns of either half
  const int wave_m0 = m0 + wm * 32;
  const bool active = wm < 2 * units && wave_m0 < g.M && (!g.a_rows || g.a_rows[wave_m0] >= 0);

  // What this thread asks for of each stage: the chunk that belongs at place tid % 8 of row tid / 8 of the tile of a
  // and of either half of w.  Rows past the end, rows of padding and the second unit's rows of an item of one read
  // some valid row instead: those outputs are never stored.
  const int row = tid / 8;
  const int chunk = (tid % 8) ^ ((row >> 1) & 7);
  const bf16_t *a_src, *w_src, *v_src;
  {
    const int m = min(m0 + (units == 2 ? row : row % 64), g.M - 1);
    int src = m;
    if (g.a_rows && g.a_gather) src = max(g.a_rows[m], 0);
    a_src = g.a + (size_t)src * g.lda + chunk * 8;
    w_src = w + (size_t)min(n0 + row, g.N - 1) * g.K + chunk * 8;
    v_src = w2 + (size_t)min(n1 + row, g.N - 1) * g.K + chunk * 8;
  }
  const int wave_off = wave * 8 * TBK;               // the eight rows that a load of this wave fills
#define TQ_ISSUE(stage, k0)                                                  \
  do {                                                                       \
    bf16_t* base = ring + (stage) * STAGE + wave_off;                        \
    load_to_lds16(a_src + (k0), base);                                       \
    load_to_lds16(w_src + (k0), base + BM * TBK);                            \
    load_to_lds16(v_src + (k0), base + (BM + BH) * TBK);                     \
  } while (0)

  f32x16 acc, acc2;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f, acc2[v] = 0.f;
  const int steps = g.K / TBK;
  for (int s = 0; s < RING_STAGES - 1 && s < steps; ++s) TQ_ISSUE(s, s * TBK);
  const int lr = lane % 32, lc = lane / 32;
  int cur = 0;
  for (int t = 0; t < steps; ++t) {
    // tile t is in LDS once no more loads of this wave are on their way than those of the tiles behind it
    // (s_waitcnt: vmcnt in bits 3..0, nothing asked of the other counters)
    if (t + 1 < steps) __builtin_amdgcn_s_waitcnt(0x0F70 | L);
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    // every wave's share of tile t has landed and every wave is through with tile t - 1, whose stage tile t + 2 takes
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (t + RING_STAGES - 1 < steps) {
      int nxt = cur + RING_STAGES - 1;
      if (nxt >= RING_STAGES) nxt -= RING_STAGES;
      TQ_ISSUE(nxt, (t + RING_STAGES - 1) * TBK);
    }
    if (active) {
      const bf16_t* Ac = ring + cur * STAGE;
      const bf16_t* Wc = Ac + BM * TBK;
      const bf16_t* Vc = Wc + BH * TBK;
#pragma unroll
      for (int j = 0; j < TBK / 16; ++j) {
        const bf16x8 af = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(Ac + swz(wm * 32 + lr, 2 * j + lc)));
        const bf16x8 wf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(Wc + swz(wn * 32 + lr, 2 * j + lc)));
        const bf16x8 vf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(Vc + swz(wn * 32 + lr, 2 * j + lc)));
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, wf, acc, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, vf, acc2, 0, 0, 0);
      }
    }
    if (++cur == RING_STAGES) cur = 0;
  }
#undef TQ_ISSUE
  if (!active) return;
  const int na = n0 + wn * 32 + lr, nb = n1 + wn * 32 + lr;
  const float ba = na < g.N ? bias_at(g, na) : 0.f, bb = !DUAL && nb < g.N ? bias_at(g, nb) : 0.f;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int m = m0 + wm * 32 + 8 * (v / 4) + 4 * lc + (v % 4);
    if (m >= g.M) continue;
    if (g.a_rows && g.a_rows[m] < 0) continue;
    if (DUAL) {
      if (na < g.N) store_out<OUT_ACT>(g, m, na, gate_fn(acc[v] + ba, g.gate) * acc2[v]);
    } else {
      if (na < g.N) store_out<OUT_ACT>(g, m, na, acc[v] + ba);
      if (nb < g.N) store_out<OUT_ACT>(g, m, nb, acc2[v] + bb);
    }
  }
}

// ------------------------------------------------------------------------------------------ launch
// Waves that split k in the streaming kernel: a power of two, enough for about 2048 waves on the chip when one
// matrix is multiplied and for about 256 per matrix when there is one per expert, each wave keeping at least 256 of
// k.  A function of N, K and of whether the product is over experts, never of the number of rows.
static int split_k_waves(int N, int K, bool grouped) {
  const int n_tiles = (N + 15) / 16;
  const int want = grouped ? 256 : 2048;
  int s = 1;
  while (s < 16 && n_tiles * s < want && K / (s * 2) >= 256) s *= 2;
  return s;
}

// MT row tiles of 16; more than one (17 to 64 rows of one matrix) go with two column tiles per wave.
template <int MT>
static int launch_stream(MfmaGemmArgs g, bool dual, bool out_act, int row_tiles, hipStream_t st, int splits = 1) {
  constexpr int NTL = MT > 1 ? 2 : 1;
  if (splits > 1) {        // runs of k, each a multiple of 64 so that it starts at a whole line
    g.k_per = ((g.K + 63) / 64 + splits - 1) / splits * 64;
    if ((int64_t)(splits - 1) * g.k_per >= g.K) return TQ_ERR_BAD_ARG;
  }
  int nw = split_k_waves((g.N + NTL - 1) / NTL, splits > 1 ? g.k_per : g.K, g.tile_group != nullptr);
  const size_t per_wave = (size_t)NTL * MT * (dual ? 2 : 1) * 4 * 64 * sizeof(float);
  while (nw > 1 && (nw * per_wave > TQ_STREAM_LDS || (NTL > 1 && nw > 8))) nw /= 2;
  const dim3 grid((g.N + 16 * NTL - 1) / (16 * NTL), row_tiles, splits);
  const size_t shmem = nw > 1 ? nw * per_wave : 0;
  if (shmem > TQ_STREAM_LDS) return TQ_ERR_UNSUPPORTED;
#define TQ_STREAM(D, O)                                                                                       \
  do {                                                                                                        \
    if (shmem > 48 * 1024)                                                                                    \
      (void)hipFuncSetAttribute((const void*)gemm_stream_kernel<MT, D, O, NTL>,                               \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);                      \
    hipLaunchKernelGGL((gemm_stream_kernel<MT, D, O, NTL>), grid, dim3(64 * nw), shmem, st, g);               \
  } while (0)
  if (dual && out_act) TQ_STREAM(true, true);
  else if (dual) TQ_STREAM(true, false);
  else if (out_act) TQ_STREAM(false, true);
  else TQ_STREAM(false, false);
#undef TQ_STREAM
  return 0;
}

template <int BM, int WM, int WN, int BN = TBN>
static int launch_tile(const MfmaGemmArgs& g, bool dual, bool out_act, int splits, hipStream_t st) {
  const dim3 grid((g.M + BM - 1) / BM, (g.N + BN - 1) / BN, splits);
  const size_t shmem = (size_t)2 * (BM + BN * (dual ? 2 : 1)) * TBK * sizeof(bf16_t);
#define TQ_TILE(D, O)                                                                                  \
  do {                                                                                                 \
    if (shmem > 48 * 1024)                                                                             \
      (void)hipFuncSetAttribute((const void*)gemm_tile_kernel<BM, WM, WN, D, O, BN>,                         \
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);                     \
    hipLaunchKernelGGL((gemm_tile_kernel<BM, WM, WN, D, O, BN>), grid, dim3(64 * WM * WN), shmem, st,  \
                       g);                                                                             \
  } while (0)
  if (dual && out_act)
    TQ_TILE(true, true);
  else if (dual)
    TQ_TILE(true, false);
  else if (out_act)
    TQ_TILE(false, true);
  else
    TQ_TILE(false, false);
#undef TQ_TILE
  return 0;
}

// grid (units of 64 rows: at most so many items, tiles of 256 columns: 128 of a gated pair)
static int launch_ring(const MfmaGemmArgs& g, bool dual, bool out_act, hipStream_t st) {
  const int cols = dual ? 128 : 256;
  const dim3 grid(g.M / 64, (g.N + cols - 1) / cols);
  const size_t shmem = (size_t)RING_STAGES * (128 + 256) * TBK * sizeof(bf16_t);
#define TQ_RING(D, O)                                                                                              \
  do {                                                                                                             \
    if (hipFuncSetAttribute((const void*)gemm_ring_kernel<D, O>, hipFuncAttributeMaxDynamicSharedMemorySize,       \
                            (int)shmem) != hipSuccess)                                                             \
      return TQ_ERR_UNSUPPORTED;                                                                                   \
    hipLaunchKernelGGL((gemm_ring_kernel<D, O>), grid, dim3(1024), shmem, st, g);                                  \
  } while (0)
  if (dual && out_act) TQ_RING(true, true);
  else if (dual) TQ_RING(true, false);
  else if (out_act) TQ_RING(false, true);
  else TQ_RING(false, false);
#undef TQ_RING
  return 0;
}

// Whether a product of 17 to 64 rows takes the tiled kernel: a matrix wide enough to give every compute unit two
// tiles of 128 columns (a vocabulary).  The tiles read `a` through LDS once per 128 columns, the streaming kernel
// once per 32 (measured at 151,936 x 2,048 and 64 rows: 159 us against 466 with 16 columns a wave).
static bool wide_enough_for_tiles(int N) { return (N + TBN - 1) / TBN >= 512 && (N + TBN - 1) / TBN <= 65535; }

// Which tile a plain product of many rows takes: 128 x 128, 128 x 192, 256 x 128 or 256 x 192 outputs (0..3).  The
// larger the tile, the fewer bytes pass through LDS per multiply-add (measured on products that fill the chip
// evenly: 1.06, 1.05 and 1.12 times the rate of 128 x 128); against that stand the compute units left idle when
// the tiles do not divide evenly among the 256 of them, and the rows and columns of padding at the edges.  2,048
// rows by 6,144 columns are 768, 512, 384 or 256 tiles: three, two, one and a half, or one to a compute unit.
static int plain_tile_choice(int M, int N, int splits) {
  static const int bm[4] = {128, 128, 256, 256}, bn[4] = {128, 192, 128, 192};
  static const double rate[4] = {1.0, 1.06, 1.05, 1.12};
  int best = 0;
  double best_score = 0.0;
  for (int c = 0; c < 4; ++c) {
    const double rows = (M + bm[c] - 1) / bm[c], cols = (N + bn[c] - 1) / bn[c];
    const double per_cu = rows * cols * splits / 256.0;
    const double even = per_cu / (double)(int64_t)(per_cu + 0.999999);
    const double useful = ((double)M * N) / (rows * bm[c] * cols * bn[c]);
    const double score = rate[c] * even * useful;
    if (score > best_score * 1.0001) {
      best = c;
      best_score = score;
    }
  }
  return best;
}

// Whether a gated pair of a few hundred rows with one matrix goes in tiles of 64 rows rather than 128.  With so few
// rows a workgroup's time is its steps over k, 1.0 us a step in the lower tile against 1.35 in the taller, as long as
// it has its compute unit to itself; of the lower tiles two fit on a compute unit (80 KB of LDS each), of the
// taller one.  So: the lower tile where it needs no more than one workgroup to a compute unit, or where the
// taller one would need a second round and the lower fits in one (320 rows by 2 x 5,632 x 2,048: 34 us against
// 46; 384 rows: 47 against 46; 192 rows by 2 x 20,480 x 3,584: 103 against 149; 128 rows: 110 against 92).
static bool gated_pair_in_tiles_of_64(int M, int N) {
  const int64_t cols = (N + TBN - 1) / TBN;
  const int64_t lower = (int64_t)((M + 63) / 64) * cols, taller = (int64_t)((M + 127) / 128) * cols;
  return lower <= 256 || (taller > 256 && lower <= 512);
}

// Into how many runs of k a plain product of M rows may be split when its partial sums are wanted apart.  Many
// rows: a product whose tiles do not fill the chip twice, and that has k enough, goes faster in 2 to 4 runs, each
// at least 1024 long, and up to 1,024 rows as tile_runs says.  17 to 64 rows of a narrow matrix with a long k in the
// streaming kernel (at most 8 waves over k): as many runs as bring about 4096 waves, each wave keeping 128 of k
// (64 rows by 2,048 x 2,048: 13.4 us in two runs against 15.2 in one; by 2,048 x 5,632: 17.3 in four against 20.7
// in two); from 33 rows on the tile kernel with its runs instead, where it may split k.  1 for up to 16 rows.
// Runs of k for a product that goes in tiles of 64 rows (up to 1,024 rows): a workgroup's time is its steps over k
// (about 0.6 us each, whatever the memory does), so up to 8 runs, each at least 256 long, while the workgroups stay
// within two to a compute unit and the partial sums within 8 MB, which the kernel behind has to read (128 rows by
// 2,048 x 2,048: 8.7 us in eight runs against 14.6 in two; by 2,048 x 5,632: 13.7 against 19.3 in four).
static int tile_runs(int M, int N, int K) {
  const int64_t tiles64 = (int64_t)((M + 63) / 64) * ((N + TBN - 1) / TBN);
  int t = 1;
  while (t < 8 && tiles64 * t * 2 <= 512 && K / (t * 2) >= 256 && (int64_t)t * 2 * M * N * 4 <= (8 << 20)) t *= 2;
  // every run must begin before the end of k (runs are whole tiles of 64)
  while (t > 1 && (int64_t)(t - 1) * (((K + TBK - 1) / TBK + t - 1) / t * TBK) >= K) t /= 2;
  return t;
}

// Whether partial sums of 33 to 64 rows come from the tile kernel rather than the streaming one: where the tile
// kernel may split k at all.  Its one row tile then has up to eight runs of k to the streaming kernel's two to four
// (64 rows by 2,048 x 2,048: 7.9 us against 13.1; by 2,048 x 5,632: 12.9 against 17.0; by 3,584 x 20,480: 46 against
// 62).
// From 17 to 32 rows it is level (2,048 x 2,048: 6.7 to 7.6 us against 7.8 to 8.7; 2,048 x 5,632: 11.9 to 12.7 against
// 10.6 to 11.8), and the streaming kernel's fewer runs are less for the next kernel to add.
static bool few_rows_in_tiles(int M, int N, int K) {
  return M > 32 && M <= 64 && !wide_enough_for_tiles(N) && tile_runs(M, N, K) > 1;
}

TQ_API int tq_gemm_mfma_splits(int M, int N, int K) {
  if (M <= 16) return 1;
  if (M <= 64) {
    if (wide_enough_for_tiles(N)) return 1;
    if (few_rows_in_tiles(M, N, K)) return tile_runs(M, N, K);
    const int64_t waves = (int64_t)((N + 31) / 32) * 8;
    int s = 1;
    while (s < 8 && waves * s < 4096 && K / (16 * s) >= 128) s *= 2;
    return s;
  }
  const int64_t tiles = (int64_t)((M + 127) / 128) * ((N + TBN - 1) / TBN);
  int s = 1;
  while (s < 4 && tiles * s < 512 && K / (s * 2) >= 1024) s *= 2;
  if (M <= 64 * 16) {      // tiles of 64 rows: more and shorter runs
    const int t = tile_runs(M, N, K);
    if (t > s) s = t;
  }
  return s;
}

// a: bfloat16 [.., K] with row stride lda (a multiple of 8, as K must be); w, w2: bfloat16.
// tile_rows: with tile_group set, the padding unit of the row order (16, 32, 64, 128 or 256); else a hint that is
// ignored.  64 + TQ_TILE_PAIRS: units of 64 taken two at a time, by the items that the row order lists behind its
// row tiles (tile_group[M / 64 ..], n_tiles[1]).
// splits > 1 (as tq_gemm_mfma_splits says, for a plain product into float): run z of k goes to out + z * M * ldc,
// the bias to run 0; the sum over the runs is the caller's.
TQ_API int tq_gemm_mfma(const void* a, int64_t lda, const int* a_rows, int a_gather, const void* w, const void* w2,
                        int64_t group_stride, const int* tile_group, const int* n_tiles, const void* bias,
                        int bias_type, void* out, int64_t ldc, int out_is_act, int M, int N, int K, int tile_rows,
                        int splits, int gate, hipStream_t st) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 8 != 0 || lda % 8 != 0) return TQ_ERR_BAD_ARG;
  if (((uintptr_t)a | (uintptr_t)w | (uintptr_t)w2) % 16 != 0 || (group_stride % 8) != 0) return TQ_ERR_BAD_ARG;
  const bool dual = w2 != nullptr, out_act = out_is_act != 0;
  if (splits < 1 || splits > 64 || gate < 0 || gate >= TQ_GATE_COUNT) return TQ_ERR_BAD_ARG;
  if (splits > 1 && (dual || out_act || tile_group || a_rows || splits != tq_gemm_mfma_splits(M, N, K))) return TQ_ERR_BAD_ARG;
  const int k_per = ((K + TBK - 1) / TBK + splits - 1) / splits * TBK;
  if (splits > 1 && (int64_t)(splits - 1) * k_per >= K) return TQ_ERR_BAD_ARG;
  MfmaGemmArgs g{(const bf16_t*)a, lda, a_rows, a_gather, (const bf16_t*)w, (const bf16_t*)w2, group_stride,
                 tile_group, n_tiles, bias, bias_type, out, ldc, M, N, K, splits > 1 ? k_per : K, (int64_t)M * ldc, gate, 1};
  int rc = 0;
  if (tile_group) {
    if (tile_rows == 16) {
      if (M % 16) return TQ_ERR_BAD_ARG;
      rc = launch_stream<1>(g, dual, out_act, M / 16, st);
    } else if (tile_rows == 32) {      // the streaming kernel with two row tiles and two column tiles to a wave
      if (M % 32) return TQ_ERR_BAD_ARG;
      rc = launch_stream<2>(g, dual, out_act, M / 32, st);
    } else if (tile_rows == 64 || tile_rows == 64 + TQ_TILE_PAIRS) {
      if ((N + TBN - 1) / TBN > 65535 || M % 64) return TQ_ERR_UNSUPPORTED;
      if (tile_rows != 64 && K % TBK == 0 && K >= 2 * TBK)
        rc = launch_ring(g, dual, out_act, st);
      else
        rc = launch_tile<64, 2, 4>(g, dual, out_act, 1, st);
    } else if (tile_rows == 128) {     // experts with hundreds of rows each: the taller tile's rate for little padding
      if ((N + TBN - 1) / TBN > 65535 || M % 128) return TQ_ERR_UNSUPPORTED;
      // the gated pair as 2 x 4 waves of 64 x 32 outputs (and as many of w2): 3 to 4 % faster than 4 x 2 of 32 x 64
      if (dual)
        rc = launch_tile<128, 2, 4>(g, dual, out_act, 1, st);
      else
        rc = launch_tile<128, 4, 2>(g, dual, out_act, 1, st);
    } else if (tile_rows == 256) {
      // A thousand rows and more each.  The gated pair takes tiles as tall as the unit, a wave's 64 x 64 outputs per
      // pass over its operands (13,199 tokens x 8 of 64 experts of 2,560 x 3,584: 4.37 ms against 5.09 in tiles of 128
      // rows); the plain product, whose k is the shorter one, stays with two tiles of 128 to a unit (2.85 ms; 3.00 as
      // tiles of 256), of which one that holds padding only ends at once.
      if ((N + TBN - 1) / TBN > 65535 || M % 256) return TQ_ERR_UNSUPPORTED;
      if (dual) {
        rc = launch_tile<256, 4, 2>(g, dual, out_act, 1, st);
      } else {
        g.group_ratio = 2;
        rc = launch_tile<128, 4, 2>(g, dual, out_act, 1, st);
      }
    } else {
      return TQ_ERR_BAD_ARG;
    }
  } else if (M <= 16) {
    rc = launch_stream<1>(g, dual, out_act, 1, st);
  } else if (M <= 64 && wide_enough_for_tiles(N)) {
    rc = launch_tile<64, 2, 4>(g, dual, out_act, splits, st);
  } else if (M <= 64 && splits > 1 && few_rows_in_tiles(M, N, K)) {
    rc = launch_tile<64, 2, 4>(g, dual, out_act, splits, st);
  } else if (M <= 32) {
    rc = launch_stream<2>(g, dual, out_act, 1, st, splits);
  } else if (M <= 64) {
    rc = launch_stream<4>(g, dual, out_act, 1, st, splits);
  } else {
    if ((N + TBN - 1) / TBN > 65535) return TQ_ERR_UNSUPPORTED;
    if (M <= 64 * 16 && !dual)
      rc = launch_tile<64, 2, 4>(g, dual, out_act, splits, st);
    else if (dual && gated_pair_in_tiles_of_64(M, N))
      rc = launch_tile<64, 2, 4>(g, dual, out_act, splits, st);
    else if (dual)
      rc = launch_tile<128, 4, 2>(g, dual, out_act, splits, st);
    else
      switch (plain_tile_choice(M, N, splits)) {
        case 1: rc = launch_tile<128, 4, 2, 192>(g, dual, out_act, splits, st); break;
        case 2: rc = launch_tile<256, 4, 2, 128>(g, dual, out_act, splits, st); break;
        case 3: rc = launch_tile<256, 4, 2, 192>(g, dual, out_act, splits, st); break;
        default: rc = launch_tile<128, 4, 2>(g, dual, out_act, splits, st);
      }
  }
  if (rc) return rc;
  TQ_LAUNCH_CHECK();
  return 0;
}

// Into how many runs of k the second product of a pair is split when its partial sums are wanted apart: the
// workgroups of a pair have the waves that suit the first product, so a second product that alone would have s
// times as many waves over its k gets s runs instead.  A function of the two products' N and K and of whether each
// has a matrix per expert.
static int pair_run_of_k(int N1, int K1, bool grouped1, int N2, int K2, bool grouped2) {
  const int nw = split_k_waves(N1, K1, grouped1), nw2 = split_k_waves(N2, K2, grouped2);
  if (nw2 <= nw) return K2;
  return ((K2 + 63) / 64 + nw2 / nw - 1) / (nw2 / nw) * 64;      // a multiple of 64: runs start at whole lines
}
TQ_API int tq_gemm_mfma_pair_splits(int N1, int K1, int grouped1, int N2, int K2, int grouped2) {
  const int k_per = pair_run_of_k(N1, K1, grouped1 != 0, N2, K2, grouped2 != 0);
  return (K2 + k_per - 1) / k_per;
}

// Two products of few rows in one launch.  d1, d2: 19 numbers each, in the order of tq_gemm_mfma's arguments from
// `a` to `tile_rows`, then the gate's activation.  Both must be products that the streaming kernel takes 16 rows at a time (a matrix per
// expert with tile_rows 16, or one matrix with M <= 16), both gated or both not, both into the same type.  The
// waves that split k are those of the first product (the larger one by convention).  splits2 > 1 (as
// tq_gemm_mfma_pair_splits says, for a plain second product into float): run z of its k goes to
// out + z * M * ldc, the bias to run 0.
TQ_API int tq_gemm_mfma_pair(const int64_t* d1, const int64_t* d2, int splits2, hipStream_t st) {
  MfmaGemmArgs g[2];
  int row_tiles[2];
  bool dual[2], out_act[2];
  const int64_t* d[2] = {d1, d2};
  for (int i = 0; i < 2; ++i) {
    const int64_t* p = d[i];
    const int M = (int)p[14], N = (int)p[15], K = (int)p[16], tile_rows = (int)p[17];
    if (M <= 0 || N <= 0 || K <= 0 || K % 8 != 0 || p[1] % 8 != 0 || p[6] % 8 != 0) return TQ_ERR_BAD_ARG;
    if (((uintptr_t)p[0] | (uintptr_t)p[4] | (uintptr_t)p[5]) % 16 != 0) return TQ_ERR_BAD_ARG;
    g[i] = MfmaGemmArgs{(const bf16_t*)p[0], p[1], (const int*)p[2], (int)p[3], (const bf16_t*)p[4], (const bf16_t*)p[5],
                        p[6], (const int*)p[7], (const int*)p[8], (const void*)p[9], (int)p[10], (void*)p[11], p[12],
                        M, N, K, K, 0, (int)p[18], 1};
    if (g[i].gate < 0 || g[i].gate >= TQ_GATE_COUNT) return TQ_ERR_BAD_ARG;
    dual[i] = p[5] != 0;
    out_act[i] = p[13] != 0;
    if (g[i].tile_group) {
      if (tile_rows != 16 || M % 16) return TQ_ERR_BAD_ARG;
      row_tiles[i] = M / 16;
    } else {
      if (M > 16) return TQ_ERR_BAD_ARG;
      row_tiles[i] = 1;
    }
  }
  if (dual[0] != dual[1] || out_act[0] != out_act[1]) return TQ_ERR_BAD_ARG;
  if (splits2 < 1) return TQ_ERR_BAD_ARG;
  if (splits2 > 1) {
    if (dual[1] || out_act[1] || g[1].a_rows || g[1].tile_group) return TQ_ERR_BAD_ARG;
    g[1].k_per = pair_run_of_k(g[0].N, g[0].K, g[0].tile_group != nullptr, g[1].N, g[1].K, false);
    if (splits2 != (g[1].K + g[1].k_per - 1) / g[1].k_per) return TQ_ERR_BAD_ARG;
    g[1].split_stride = (int64_t)g[1].M * g[1].ldc;
  }
  const int nw = split_k_waves(g[0].N, g[0].K, g[0].tile_group != nullptr);
  const size_t shmem = nw > 1 ? (size_t)nw * (dual[0] ? 2 : 1) * 4 * 64 * sizeof(float) : 0;
  const int nx1 = (g[0].N + 15) / 16, nx2 = (g[1].N + 15) / 16;
  const int64_t n1 = (int64_t)nx1 * row_tiles[0], n2 = (int64_t)nx2 * row_tiles[1] * splits2;
  if (n1 + n2 > 0x7fffffff) return TQ_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)(n1 + n2));
#define TQ_PAIR(D, O) \
  hipLaunchKernelGGL((gemm_stream_pair_kernel<D, O>), grid, dim3(64 * nw), shmem, st, g[0], nx1, g[1], nx2, row_tiles[1], (int)n2)
  if (dual[0] && out_act[0]) TQ_PAIR(true, true);
  else if (dual[0]) TQ_PAIR(true, false);
  else if (out_act[0]) TQ_PAIR(false, true);
  else TQ_PAIR(false, false);
#undef TQ_PAIR
  TQ_LAUNCH_CHECK();
  return 0;
}

// Queries, keys and values of T <= 16 tokens in one launch: a [T][K] bfloat16 (row stride lda) times w [(nh + 2 nkv)
// hd][K] plus bias, queries and keys rotated by positions[t] * inv_freq[d] on the pairs (d, d + hd / 2), queries to
// q_out [T][nh hd], keys and values into the pages (k_pool / v_pool with the layer's offset added; null: only the
// queries are made).  hd must be a multiple of 32 and the rotation span the whole head.
TQ_API int tq_qkv_rope_write(const void* a, int64_t lda, const void* w, const void* bias, int bias_type, int T, int K,
                             const int* positions, const int* seq_of_token, const int* block_table, int bt_stride,
                             const float* inv_freq, void* q_out, void* k_pool, void* v_pool, int page_size,
                             int64_t page_stride, int nh, int nkv, int hd, hipStream_t st) {
  if (T <= 0) return 0;
  if (T > 16 || hd % 32 != 0 || hd <= 0 || nh <= 0 || nkv <= 0) return TQ_ERR_UNSUPPORTED;
  if (K <= 0 || K % 8 != 0 || lda % 8 != 0 || ((uintptr_t)a | (uintptr_t)w) % 16 != 0) return TQ_ERR_BAD_ARG;
  if ((k_pool == nullptr) != (v_pool == nullptr) || page_size <= 0) return TQ_ERR_BAD_ARG;
  const int heads = k_pool ? nh + 2 * nkv : nh;
  const int N = (nh + 2 * nkv) * hd;
  MfmaGemmArgs g{(const bf16_t*)a, lda, nullptr, 1, (const bf16_t*)w, nullptr, 0, nullptr, nullptr, bias, bias_type,
                 nullptr, 0, T, N, K, K, 0, 0, 1};
  RopeWriteArgs p{positions, seq_of_token, block_table, bt_stride, inv_freq, (bf16_t*)q_out, (bf16_t*)k_pool,
                  (bf16_t*)v_pool, page_size, page_stride, nh, nkv, hd};
  int nw = split_k_waves(heads * hd / 2, K, false);
  if (nw > 8) nw = 8;
  const size_t shmem = (size_t)nw * 2 * 4 * 64 * sizeof(float);
  hipLaunchKernelGGL(qkv_rope_write_kernel, dim3(heads * (hd / 32)), dim3(64 * nw), shmem, st, g, p);
  TQ_LAUNCH_CHECK();
  return 0;
}
