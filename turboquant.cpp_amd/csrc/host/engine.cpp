// The step executor: see engine.h.  Host code only; every kernel it runs is reached through the entry points that
// turboquant_kernels.h declares, with the arguments that the Python face of the kernels (ops.py) would give them for
// the same step, so that a step gives the same bits whichever of the two issues it.
//
// Memory: the caller brings one workspace per step.  A first pass over the step works out, without launching, what
// every kernel's result needs (the same code as the pass that launches, with an arena that only counts); the
// workspace then holds what lives for the whole step (the residual stream, the vendor library's scratch) and two
// halves that the schedule entries take in turn: what an entry leaves for the next norm to add lies in its half
// while the next entry works in the other.
#include "engine.h"

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "../turboquant_kernels.h"
#include "host_common.h"
#include "vendor.h"

namespace {

thread_local char g_error[512] = "";
thread_local int64_t g_launches = 0;
thread_local int64_t g_vendor_products = 0;

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code ? code : TQ_ERR_BAD_ARG;
}

const char* code_text(int code) {
  if (code == TQ_ERR_BAD_ARG) return "arguments rejected by the launcher";
  if (code == TQ_ERR_UNSUPPORTED) return "size not supported by this kernel";
  return "error at launch";
}

struct Arena {
  char* base = nullptr;
  size_t cap = 0, used = 0, peak = 0;
  bool dry = true, overflow = false;
  void* take(size_t bytes) {
    const size_t at = (used + 255) & ~(size_t)255;
    used = at + bytes;
    if (used > peak) peak = used;
    if (dry) return reinterpret_cast<void*>(256);      // never dereferenced, never handed to a kernel
    if (used > cap) {
      overflow = true;
      return nullptr;
    }
    return base + at;
  }
};

// What a part leaves for the next norm to add into the residual stream.
struct Pending {
  const float* delta = nullptr;   // [S][T][H] partial sums, added in order
  int S = 0;
  const float* y = nullptr;       // rows of the experts' outputs, summed per token with `weights` through `pair_slot`
  const int* pair_slot = nullptr;
  const float* weights = nullptr;
  int topk = 0;
  const float* gate = nullptr;    // scales the partial sums in `delta` (the shared expert's)
};

struct Ctx {
  const tq_model_desc* m;
  const tq_step_desc* s;
  Arena arena;          // the running entry's half
  Arena whole;          // what lives for the whole step
  bool dry;
  hipStream_t stream;
  hipEvent_t forked = nullptr, joined = nullptr;
  void* vendor_ws[2] = {nullptr, nullptr};   // main and side stream
  int T, B, H;
};

#define RUN(c, name, call)                                                            \
  do {                                                                                \
    if (!(c).dry) {                                                                   \
      const int rc__ = (call);                                                        \
      ++g_launches;                                                                   \
      if (rc__ != 0) return fail(rc__, "%s: %s (%d)", name, code_text(rc__), rc__);   \
    }                                                                                 \
  } while (0)

bool bf16_path() { return TQ_ACT_TYPE == TQ_BF16; }

bool use_mfma(const tq_weight& w, int64_t K) {
#if defined(TQ_ACT_BF16)
  return w.wtype == TQ_BF16 && K % 8 == 0;
#else
  (void)w;
  (void)K;
  return false;
#endif
}

// One product, as ops.gemm sees it.
struct Product {
  const void* a = nullptr;
  int64_t lda = 0;
  const int* a_rows = nullptr;
  int gather = 1;
  tq_weight w{nullptr, 0};
  const void* w2 = nullptr;
  int64_t gstride = 0;
  const int* tile_group = nullptr;
  const int* n_tiles = nullptr;
  tq_weight bias{nullptr, 0};
  int out_act = 0;
  int M = 0, N = 0, K = 0;
  int tile_rows = 0;
  int gate = 0;
  bool partial = false;
  void* dest = nullptr;      // where the result goes, if not into the arena (never with partial sums)
};

// Whether a plain product goes to the vendor's library: the caller's bound on the rows, not under capture, and the
// library has a kernel for the shapes that would be asked of it (the product itself, or a gated pair's product over
// both matrices in chunks of rows); the same answer in the pass that counts and in the pass that launches.
bool vendor_product(const Ctx& c, const Product& p) {
  const tq_step_desc& s = *c.s;
  if (!(bf16_path() && s.vendor_min_rows > 0 && p.M >= s.vendor_min_rows && (p.K < 16384 || p.M >= 8192) &&
        p.w.wtype == TQ_BF16 && !s.capturing && !s.decode && tq_vendor_available()))
    return false;
  if (!p.w2) return tq_vendor_takes(p.M, p.N, p.K, p.lda, p.out_act) != 0;
  const int64_t chunk = s.vendor_gated_rows > 0 ? s.vendor_gated_rows : 4096;
  const int rows = (int)(p.M < chunk ? p.M : chunk), last = (int)(p.M % chunk);
  return tq_vendor_takes(rows, 2 * p.N, p.K, p.lda, 0) != 0 && (last == 0 || tq_vendor_takes(last, 2 * p.N, p.K, p.lda, 0) != 0);
}

int gated_act(Ctx& c, const float* gu, int64_t ld, void* out, int M, int N, int gate) {
  RUN(c, "gated_act", tq_gated_act(gu, ld, out, M, N, gate, c.stream));
  return 0;
}

// out (and, for partial sums, how many there are) of one product; mirrors ops.gemm.
int product(Ctx& c, const Product& p, void** out, int* splits, int side = 0) {
  const bool grouped = p.tile_group != nullptr;
  const size_t esz = p.out_act ? TQ_ACT_BYTES : 4;
  const int tile_rows = p.tile_rows ? p.tile_rows : (p.M <= 32 ? 16 : 64);
  const int unit_rows = tile_rows % TQ_TILE_PAIRS;      // pairs of units are the matrix-core product's alone
  *splits = 1;
  auto result = [&](size_t bytes) { return p.dest ? p.dest : c.arena.take(bytes); };
  if (!grouped && !p.a_rows && !p.bias.ptr && vendor_product(c, p)) {
    if (!p.w2) {
      *out = result((size_t)p.M * p.N * esz);
      RUN(c, "vendor product",
          tq_vendor_product(p.a, p.lda, p.w.ptr, *out, p.out_act, p.M, p.N, p.K, c.vendor_ws[side], c.stream));
      if (!c.dry) ++g_vendor_products;
      return 0;
    }
    const bool behind = (const char*)p.w2 == (const char*)p.w.ptr + (size_t)p.N * p.K * 2;
    if (p.out_act && behind) {
      // f(a w^T) * (a w2^T) with w2 behind w: one product over both matrices into float, some thousand rows at a
      // time, and the gate's activation in a pass of its own
      *out = result((size_t)p.M * p.N * esz);
      const int64_t chunk = c.s->vendor_gated_rows > 0 ? c.s->vendor_gated_rows : 4096;
      float* gu = (float*)c.arena.take((size_t)(p.M < chunk ? p.M : chunk) * 2 * p.N * 4);
      for (int64_t r = 0; r < p.M; r += chunk) {
        const int rows = (int)(p.M - r < chunk ? p.M - r : chunk);
        RUN(c, "vendor product",
            tq_vendor_product((const char*)p.a + r * p.lda * 2, p.lda, p.w.ptr, gu, 0, rows, 2 * p.N, p.K,
                              c.vendor_ws[side], c.stream));
        if (!c.dry) ++g_vendor_products;
        if (int rc = gated_act(c, gu, 2 * p.N, (char*)*out + r * p.N * TQ_ACT_BYTES, rows, p.N, p.gate)) return rc;
      }
      return 0;
    }
  }
#if defined(TQ_ACT_BF16)
  if (use_mfma(p.w, p.K)) {
    if (p.partial) *splits = tq_gemm_mfma_splits(p.M, p.N, p.K);
    *out = result((size_t)*splits * p.M * p.N * esz);
    RUN(c, "gemm_mfma",
        tq_gemm_mfma(p.a, p.lda, p.a_rows, p.gather, p.w.ptr, p.w2, p.gstride, p.tile_group, p.n_tiles, p.bias.ptr,
                     (int)p.bias.wtype, *out, p.N, p.out_act, p.M, p.N, p.K, tile_rows, *splits, p.gate, c.stream));
    return 0;
  }
#else
  if (p.w.wtype == TQ_F32 && p.K % 4 == 0 && p.lda % 4 == 0 && p.gstride % 4 == 0 && ((uintptr_t)p.w.ptr & 15) == 0 &&
      ((uintptr_t)p.w2 & 15) == 0 && (unit_rows == 16 || unit_rows == 64)) {
    const int runs = tq_gemm_f32_runs(p.M, p.N, p.K, grouped || p.a_rows != nullptr);
    if (p.partial) *splits = runs;
    *out = result((size_t)*splits * p.M * p.N * 4);
    void* scratch = nullptr;
    if (runs > 1 && !p.partial) scratch = c.arena.take((size_t)runs * (p.w2 ? 2 : 1) * p.M * p.N * 4);
    RUN(c, "gemm_f32",
        tq_gemm_f32(p.a, p.lda, p.a_rows, p.gather, p.w.ptr, p.w2, p.gstride, p.tile_group, p.n_tiles, p.bias.ptr,
                    (int)p.bias.wtype, *out, p.N, p.M, p.N, p.K, unit_rows, p.gate, scratch, p.partial && runs > 1,
                    c.stream));
    return 0;
  }
#endif
  *out = result((size_t)p.M * p.N * esz);
  RUN(c, "gemm",
      tq_gemm_generic(p.a, p.lda, p.a_rows, p.gather, p.w.ptr, p.w2, (int)p.w.wtype, p.gstride, p.tile_group, p.n_tiles,
                      p.bias.ptr, (int)p.bias.wtype, *out, p.N, p.out_act, p.M, p.N, p.K, unit_rows, p.gate, c.stream));
  return 0;
}

#if defined(TQ_ACT_BF16)
void pair_desc(const Product& p, void* out, int tile_rows, int64_t* d) {
  const int64_t v[19] = {(int64_t)(uintptr_t)p.a, p.lda, (int64_t)(uintptr_t)p.a_rows, p.gather, (int64_t)(uintptr_t)p.w.ptr,
                         (int64_t)(uintptr_t)p.w2, p.gstride, (int64_t)(uintptr_t)p.tile_group, (int64_t)(uintptr_t)p.n_tiles,
                         (int64_t)(uintptr_t)p.bias.ptr, p.bias.ptr ? p.bias.wtype : 0, (int64_t)(uintptr_t)out, p.N, p.out_act,
                         p.M, p.N, p.K, tile_rows, p.gate};
  memcpy(d, v, sizeof(v));
}
#endif

// Two products that do not depend on each other; mirrors ops.gemm_pair (only the second may leave partial sums).
int product_pair(Ctx& c, const Product& p1, const Product& p2, void** out1, void** out2, int* splits2) {
  *splits2 = 1;
#if defined(TQ_ACT_BF16)
  const Product* ps[2] = {&p1, &p2};
  bool fused = true;
  int tile_rows[2];
  for (int i = 0; i < 2; ++i) {
    const Product& p = *ps[i];
    tile_rows[i] = p.tile_rows ? p.tile_rows : (p.M <= 32 ? 16 : 64);
    const bool few = p.tile_group ? tile_rows[i] == 16 : p.M <= 16;
    fused = fused && few && use_mfma(p.w, p.K);
  }
  fused = fused && (p1.w2 == nullptr) == (p2.w2 == nullptr) && p1.out_act == p2.out_act;
  if (fused) {
    if (p2.partial) *splits2 = tq_gemm_mfma_pair_splits(p1.N, p1.K, p1.tile_group != nullptr, p2.N, p2.K, 0);
    *out1 = c.arena.take((size_t)p1.M * p1.N * (p1.out_act ? TQ_ACT_BYTES : 4));
    *out2 = c.arena.take((size_t)*splits2 * p2.M * p2.N * (p2.out_act ? TQ_ACT_BYTES : 4));
    int64_t d1[19], d2[19];
    pair_desc(p1, *out1, tile_rows[0], d1);
    pair_desc(p2, *out2, tile_rows[1], d2);
    RUN(c, "gemm_pair", tq_gemm_mfma_pair(d1, d2, *splits2, c.stream));
    return 0;
  }
#endif
  int s1;
  if (int rc = product(c, p1, out1, &s1)) return rc;
  return product(c, p2, out2, splits2);
}

int norm(Ctx& c, const tq_norm_desc& n, float* x, const Pending& p, const int* rows, int R, void** out, float** out32,
         bool want32) {
  *out = c.arena.take((size_t)R * c.H * TQ_ACT_BYTES);
  *out32 = want32 ? (float*)c.arena.take((size_t)R * c.H * 4) : nullptr;
  RUN(c, "add_rmsnorm",
      tq_add_rmsnorm(x, p.delta, p.S, (int64_t)c.T * c.H, p.y, p.pair_slot, p.weights, p.topk, p.gate, n.weight.ptr,
                     (int)n.weight.wtype, (float)n.eps, rows, R, *out, *out32, c.H, c.stream));
  return 0;
}

// mirrors parts/attention.py (without a norm of the heads) over ops.qkv_rope_write, ops.attention and ops.gemm
int attention(Ctx& c, const tq_attention_desc& a, const tq_entry_desc& e, const void* normed, Pending* pending) {
  const tq_step_desc& s = *c.s;
  const int T = c.T, nh = (int)a.num_heads, nkv = (int)a.num_kv_heads, hd = (int)a.head_dim, K = (int)a.hidden;
  const int width = (nh + 2 * nkv) * hd;
  if (e.layer_offset + (int64_t)nkv * e.page_size * hd > e.page_stride) return fail(TQ_ERR_BAD_ARG, "attention: layer does not fit in a page");
  if (s.max_end > e.table_width * e.page_size) return fail(TQ_ERR_BAD_ARG, "attention: positions reach beyond the page table");
  char* kp = e.k_pages ? (char*)e.k_pages + e.layer_offset * TQ_ACT_BYTES : nullptr;
  char* vp = e.v_pages ? (char*)e.v_pages + e.layer_offset * TQ_ACT_BYTES : nullptr;
  void* kw = e.owns ? kp : nullptr;
  void* vw = e.owns ? vp : nullptr;
  void* q = nullptr;
  bool fused = false;
#if defined(TQ_ACT_BF16)
  fused = T <= 16 && a.pairing == 0 && a.rotary_dim == hd && hd % 32 == 0 && use_mfma(a.qkv_weight, K);
  if (fused) {
    q = c.arena.take((size_t)T * nh * hd * TQ_ACT_BYTES);
    RUN(c, "qkv_rope_write",
        tq_qkv_rope_write(normed, K, a.qkv_weight.ptr, a.qkv_bias.ptr, (int)a.qkv_bias.wtype, T, K, s.positions,
                          s.slot_of_token, e.table, (int)e.table_width, a.inv_freq, q, kw, vw, (int)e.page_size,
                          e.page_stride, nh, nkv, hd, c.stream));
  }
#endif
  if (!fused) {
    Product p;
    p.a = normed, p.lda = K, p.w = a.qkv_weight, p.M = T, p.N = width, p.K = K;
    // the vendor library's product has no bias of its own that costs nothing: the rotation adds it as it reads
    const bool late = a.qkv_bias.ptr && vendor_product(c, p);
    if (!late) p.bias = a.qkv_bias;
    void* qkv;
    int one;
    if (int rc = product(c, p, &qkv, &one)) return rc;
    q = c.arena.take((size_t)T * nh * hd * TQ_ACT_BYTES);
    const bool by_runs = e.owns && !s.decode;
    RUN(c, "rope_kv_write",
        tq_rope_kv_write((const float*)qkv, late ? a.qkv_bias.ptr : nullptr, late ? (int)a.qkv_bias.wtype : 0, s.positions,
                         s.slot_of_token, e.table, (int)e.table_width, a.inv_freq, (int)a.pairing, (int)a.rotary_dim, q, kw,
                         vw, (int)e.page_size, e.page_stride, T, nh, nkv, hd, e.owns ? 1 : 0, by_runs ? s.cu_seqlens : nullptr,
                         by_runs ? s.slots : nullptr, by_runs ? s.start : nullptr, by_runs ? (int)s.B : 0,
                         by_runs ? (int)s.max_new : 0, c.stream));
  }
  void* o = c.arena.take((size_t)T * nh * hd * TQ_ACT_BYTES);
  bool done = false;
#if defined(TQ_ACT_BF16)
  if (hd % 16 == 0 && hd <= 256 && e.page_size % 64 == 0 && e.page_stride % 8 == 0 && a.scale > 0) {
    float* partial = nullptr;
    if (s.decode) partial = (float*)c.arena.take((size_t)tq_attention_decode_scratch((int)s.B, nh, hd, (int)s.max_end) * 4);
    RUN(c, "attention_mfma",
        tq_attention_mfma(q, kp, vp, e.table, (int)e.table_width, s.cu_seqlens, s.slots, s.start, (int)e.page_size,
                          e.page_stride, (int)s.B, nh, nkv, hd, (int)a.window, (float)a.scale, o, partial, (int)s.decode,
                          (int)s.max_new, (int)s.max_end, c.stream));
    done = true;
  }
#else
  if (hd % 4 == 0 && hd <= 256 && e.page_size % 64 == 0 && e.page_stride % 4 == 0 && e.layer_offset % 4 == 0) {
    void* partial = nullptr;
    if (s.decode) partial = c.arena.take((size_t)tq_attention_f32_scratch((int)s.B, nh, hd, (int)s.max_end) * 4);
    RUN(c, "attention_f32",
        tq_attention_f32(q, kp, vp, e.table, (int)e.table_width, s.cu_seqlens, s.slots, s.start, (int)e.page_size,
                         e.page_stride, (int)s.B, nh, nkv, hd, (int)a.window, (float)a.scale, o, partial, (int)s.decode,
                         (int)s.max_new, (int)s.max_end, c.stream));
    done = true;
  }
#endif
  if (!done) {
    if (hd > 512) return fail(TQ_ERR_UNSUPPORTED, "attention: head size %d is beyond the 512 this kernel takes", hd);
    RUN(c, "attention",
        tq_attention_generic(q, kp, vp, s.positions, s.slot_of_token, e.table, (int)e.table_width, (int)e.page_size,
                             e.page_stride, T, nh, nkv, hd, (int)a.window, (float)a.scale, o, c.stream));
  }
  Product p;
  p.a = o, p.lda = (int64_t)nh * hd, p.w = a.out_weight, p.bias = a.out_bias, p.M = T, p.N = K, p.K = nh * hd, p.partial = true;
  void* out;
  int splits;
  if (int rc = product(c, p, &out, &splits)) return rc;
  *pending = Pending();
  pending->delta = (const float*)out, pending->S = splits;
  return 0;
}

int dense_ffn(Ctx& c, const tq_dense_ffn_desc& f, const void* normed, Pending* pending, int side = 0) {
  Product g;
  g.a = normed, g.lda = f.hidden, g.w = f.gate_w, g.w2 = f.up_w.ptr, g.out_act = 1, g.M = c.T, g.N = (int)f.inner,
  g.K = (int)f.hidden, g.gate = (int)f.gate;
  void* h;
  int one;
  if (int rc = product(c, g, &h, &one, side)) return rc;
  Product d;
  d.a = h, d.lda = f.inner, d.w = f.down_w, d.M = c.T, d.N = (int)f.hidden, d.K = (int)f.inner, d.partial = true;
  void* out;
  int splits;
  if (int rc = product(c, d, &out, &splits, side)) return rc;
  *pending = Pending();
  pending->delta = (const float*)out, pending->S = splits;
  return 0;
}

// Rows per tile that suit a product over experts, by the pairs per expert on average; mirrors ops.expert_tile_rows.
int expert_tile_rows(const Ctx& c, int64_t n_pairs, int64_t E, bool mfma) {
  if (n_pairs <= (mfma ? 5 : 12) * E) return 16;
  if (mfma && n_pairs <= 10 * E) return 32;
  if (mfma && n_pairs >= c.s->expert_128_from * E) return n_pairs >= c.s->expert_256_from * E ? 256 : 128;
  return 64;
}

// mirrors parts/ffn.py SparseMoE.forward
int moe_ffn(Ctx& c, const tq_moe_ffn_desc& f, const void* normed, const float* normed32, Pending* pending) {
  const tq_step_desc& s = *c.s;
  const int T = c.T, H = (int)f.hidden, E = (int)f.num_experts, k = (int)f.top_k, I = (int)f.inner, Is = (int)f.shared_inner;
  if (k < 1 || k > 64 || k > E) return fail(TQ_ERR_UNSUPPORTED, "route: top_k %d must be within 1..min(E, 64)", k);
  const bool gated = Is > 0 && f.shared_scale.ptr != nullptr;
  if (gated && f.shared_scale.wtype != f.router.wtype) return fail(TQ_ERR_BAD_ARG, "route: shared_scale must have the router's type");
  const int64_t n_pairs = (int64_t)T * k;
  const int unit = expert_tile_rows(c, n_pairs, E, use_mfma(f.expert_gate, H));
  int64_t cap = n_pairs + (E < n_pairs ? E : n_pairs) * (unit - 1);
  cap = (cap + unit - 1) / unit * unit;
  // outputs of the routing
  int* ids = (int*)c.arena.take((size_t)n_pairs * 4);
  float* weights = (float*)c.arena.take((size_t)n_pairs * 4);
  float* gate = gated ? (float*)c.arena.take((size_t)T * 4) : nullptr;
  float* logits = (float*)c.arena.take((size_t)T * (E + (gated ? 1 : 0)) * 4);
  int* sorted_token = (int*)c.arena.take((size_t)cap * 4);
  int* pair_slot = (int*)c.arena.take((size_t)n_pairs * 4);
  int* tile_expert = (int*)c.arena.take((size_t)(cap / unit) * 2 * 4);      // row tiles, then items of two
  int* n_tiles = (int*)c.arena.take(2 * 4);
  auto route = [&]() -> int {
    RUN(c, "route",
        tq_route(normed32, f.router.ptr, gated ? f.shared_scale.ptr : nullptr, (int)f.router.wtype, E, k, (int)f.renormalize,
                 ids, weights, gate, logits, unit, (int)cap, sorted_token, pair_slot, tile_expert, n_tiles, T, H, c.stream));
    return 0;
  };
  // what the products are told: units of 64 two at a time where experts have that many rows (ops.expert_product_rows)
  const int rows = unit == 64 && n_pairs >= s.expert_pairs_from * E ? 64 + TQ_TILE_PAIRS : unit;
  Product eg;       // the experts' gated pair over the gathered rows
  eg.a = normed, eg.lda = H, eg.a_rows = sorted_token, eg.w = f.expert_gate, eg.w2 = f.expert_up.ptr, eg.gstride = (int64_t)I * H,
  eg.tile_group = tile_expert, eg.n_tiles = n_tiles, eg.out_act = 1, eg.M = (int)cap, eg.N = I, eg.K = H, eg.tile_rows = rows,
  eg.gate = (int)f.gate;
  Product ed;       // their down product, row for row
  ed.lda = I, ed.a_rows = sorted_token, ed.gather = 0, ed.w = f.expert_down, ed.gstride = (int64_t)H * I, ed.tile_group = tile_expert,
  ed.n_tiles = n_tiles, ed.M = (int)cap, ed.N = H, ed.K = I, ed.tile_rows = rows;
  Product sg;       // the shared expert
  sg.a = normed, sg.lda = H, sg.w = f.shared_gate, sg.w2 = f.shared_up.ptr, sg.out_act = 1, sg.M = T, sg.N = Is, sg.K = H,
  sg.gate = (int)f.gate;
  Product sd;
  sd.lda = Is, sd.w = f.shared_down, sd.M = T, sd.N = H, sd.K = Is, sd.partial = true;
  *pending = Pending();
  pending->pair_slot = pair_slot, pending->weights = weights, pending->topk = k, pending->gate = gate;
  if (Is > 0 && T <= 16 && unit == 16) {
    // a handful of tokens: the shared expert's two products ride in the launches of the routed experts'
    if (int rc = route()) return rc;
    void *h, *hs, *y, *shared;
    int one, splits;
    if (int rc = product_pair(c, eg, sg, &h, &hs, &one)) return rc;
    ed.a = h, sd.a = hs;
    if (int rc = product_pair(c, ed, sd, &y, &shared, &splits)) return rc;
    pending->y = (const float*)y, pending->delta = (const float*)shared, pending->S = splits;
    return 0;
  }
  // The shared expert needs nothing from the router: beside the routed experts on a second stream, where that pays
  // (a few passes of tiles over the chip, and a step long enough on the chip for the host's forking to vanish)
  bool side = false;
  if (Is > 0) {
    const int64_t tiles = (int64_t)((T + 127) / 128) * ((Is + 127) / 128);
    const bool worth = T >= s.side_from || s.capturing;
    side = s.side_stream != nullptr && worth && tiles < 8 * 256;
    hipStream_t main_stream = c.stream;
    if (side && !c.dry) {
      if (hipEventRecord(c.forked, main_stream) != hipSuccess || hipStreamWaitEvent(s.side_stream, c.forked, 0) != hipSuccess)
        return fail(TQ_ERR_BAD_ARG, "the side stream cannot wait for the main stream");
      c.stream = s.side_stream;
    }
    void* hs;
    int one, splits;
    int rc = product(c, sg, &hs, &one, side ? 1 : 0);
    sd.a = hs;
    void* shared = nullptr;
    if (!rc) rc = product(c, sd, &shared, &splits, side ? 1 : 0);
    c.stream = main_stream;
    if (rc) return rc;
    pending->delta = (const float*)shared, pending->S = splits;
  }
  if (int rc = route()) return rc;
  void *h, *y;
  int one;
  if (int rc = product(c, eg, &h, &one)) return rc;
  ed.a = h;
  if (int rc = product(c, ed, &y, &one)) return rc;
  pending->y = (const float*)y;
  if (side && !c.dry) {
    if (hipEventRecord(c.joined, s.side_stream) != hipSuccess || hipStreamWaitEvent(c.stream, c.joined, 0) != hipSuccess)
      return fail(TQ_ERR_BAD_ARG, "the main stream cannot wait for the side stream");
  }
  return 0;
}

struct Events {
  hipEvent_t forked = nullptr, joined = nullptr;
};
thread_local Events g_events[16];

int events_for_device(Ctx& c) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return fail(TQ_ERR_BAD_ARG, "no current device");
  Events& e = g_events[dev];
  if (!e.forked) {
    if (hipEventCreateWithFlags(&e.forked, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&e.joined, hipEventDisableTiming) != hipSuccess)
      return fail(TQ_ERR_BAD_ARG, "cannot create events");
  }
  c.forked = e.forked, c.joined = e.joined;
  return 0;
}

int check_model(const tq_model_desc& m, const tq_step_desc& s) {
  if (s.T <= 0 || s.B <= 0 || s.n_want < 0 || s.B > s.T) return fail(TQ_ERR_BAD_ARG, "a step needs tokens and sequences");
  if (m.n_layers <= 0 || m.n_entries <= 0 || !m.layers || !m.entries) return fail(TQ_ERR_BAD_ARG, "a model needs layers and a schedule");
  for (int64_t i = 0; i < m.n_entries; ++i) {
    const tq_entry_desc& e = m.entries[i];
    if (e.layer < 0 || e.layer >= m.n_layers) return fail(TQ_ERR_BAD_ARG, "schedule entry %d names layer %d", (int)i, (int)e.layer);
    const tq_layer_desc& l = m.layers[e.layer];
    if (l.attention.hidden != m.hidden) return fail(TQ_ERR_BAD_ARG, "layer %d has another width than the model", (int)e.layer);
    if (l.attention.num_kv_heads <= 0 || l.attention.num_heads % l.attention.num_kv_heads)
      return fail(TQ_ERR_BAD_ARG, "layer %d: heads must be a multiple of kv heads", (int)e.layer);
    if (l.attention.rotary_dim % 2 || l.attention.rotary_dim > l.attention.head_dim)
      return fail(TQ_ERR_BAD_ARG, "layer %d: the rotation must span an even number of dimensions within the head", (int)e.layer);
    if (l.ffn_kind != TQ_FFN_DENSE && l.ffn_kind != TQ_FFN_MOE) return fail(TQ_ERR_BAD_ARG, "layer %d: unknown feed-forward kind", (int)e.layer);
    if (!e.k_pages || !e.v_pages || !e.table) return fail(TQ_ERR_BAD_ARG, "schedule entry %d has no cache", (int)i);
  }
  return 0;
}

// One pass over the step: dry (counting) or launching.
int walk(Ctx& c, size_t* entry_bytes) {
  const tq_model_desc& m = *c.m;
  const tq_step_desc& s = *c.s;
  const int T = c.T, H = c.H;
  float* x = (float*)c.whole.take((size_t)T * H * 4);
  if (bf16_path() && s.vendor_min_rows > 0 && T >= s.vendor_min_rows && !s.capturing && !s.decode && tq_vendor_available()) {
    c.vendor_ws[0] = c.whole.take(TQ_VENDOR_WORKSPACE);
    c.vendor_ws[1] = s.side_stream ? c.whole.take(TQ_VENDOR_WORKSPACE) : c.vendor_ws[0];
  }
  const size_t whole_bytes = (c.whole.used + 255) & ~(size_t)255;
  char* halves[2] = {nullptr, nullptr};
  if (!c.dry) {
    halves[0] = c.whole.base + whole_bytes;
    halves[1] = halves[0] + *entry_bytes;
  }
  size_t most = 0;
  auto next_half = [&](int64_t i) {
    if (c.arena.peak > most) most = c.arena.peak;
    c.arena = Arena();
    c.arena.dry = c.dry;
    c.arena.base = halves[i & 1];
    c.arena.cap = c.dry ? 0 : *entry_bytes;
  };
  RUN(c, "embed", tq_embed(s.tokens, m.embedding.ptr, (int)m.embedding.wtype, x, T, H, (float)m.embedding_scale, c.stream));
  Pending pending;
  for (int64_t i = 0; i < m.n_entries; ++i) {
    next_half(i);
    const tq_entry_desc& e = m.entries[i];
    const tq_layer_desc& l = m.layers[e.layer];
    void* normed;
    float* normed32;
    if (int rc = norm(c, l.mixer_norm, x, pending, nullptr, T, &normed, &normed32, false)) return rc;
    if (int rc = attention(c, l.attention, e, normed, &pending)) return rc;
    const bool moe = l.ffn_kind == TQ_FFN_MOE;
    if (int rc = norm(c, l.ffn_norm, x, pending, nullptr, T, &normed, &normed32, moe)) return rc;
    if (int rc = moe ? moe_ffn(c, l.moe, normed, normed32, &pending) : dense_ffn(c, l.dense, normed, &pending)) return rc;
    if (c.arena.overflow) return fail(TQ_ERR_BAD_ARG, "the workspace is too small for schedule entry %d", (int)i);
  }
  next_half(m.n_entries);
  if (s.n_want > 0) {
    void* normed;
    float* normed32;
    if (int rc = norm(c, m.final_norm, x, pending, s.want_rows, (int)s.n_want, &normed, &normed32, false)) return rc;
    // the vocabulary's product: a plain product into float that writes the caller's logits
    Product p;
    p.a = normed, p.lda = H, p.w = m.lm_head, p.M = (int)s.n_want, p.N = (int)m.vocab, p.K = H, p.dest = s.logits;
    void* got;
    int one;
    if (int rc = product(c, p, &got, &one)) return rc;
    if (m.logit_softcap > 0) RUN(c, "softcap", tq_softcap(s.logits, (int64_t)s.n_want * m.vocab, (float)m.logit_softcap, c.stream));
  }
  if (c.arena.peak > most) most = c.arena.peak;
  if (c.arena.overflow || c.whole.overflow) return fail(TQ_ERR_BAD_ARG, "the workspace is too small");
  *entry_bytes = (most + 255) & ~(size_t)255;
  return 0;
}

int run(const tq_model_desc* m, const tq_step_desc* s, bool launch, int64_t* bytes) {
  if (!m || !s) return fail(TQ_ERR_BAD_ARG, "no model or no step");
  if (int rc = check_model(*m, *s)) return rc;
  Ctx c{};
  c.m = m, c.s = s, c.stream = s->stream, c.T = (int)s->T, c.B = (int)s->B, c.H = (int)m->hidden;
  c.dry = true;
  c.whole.dry = true;
  size_t entry_bytes = 0;
  if (int rc = walk(c, &entry_bytes)) return rc;
  const size_t whole_bytes = (c.whole.used + 255) & ~(size_t)255;
  const size_t need = whole_bytes + 2 * entry_bytes;
  if (bytes) *bytes = (int64_t)need;
  if (!launch) return 0;
  if (!s->workspace || ((uintptr_t)s->workspace & 255) || (size_t)s->workspace_bytes < need)
    return fail(TQ_ERR_BAD_ARG, "the step needs %zu bytes of workspace aligned to 256, the caller brought %lld", need,
                (long long)s->workspace_bytes);
  if (s->n_want > 0 && !s->logits) return fail(TQ_ERR_BAD_ARG, "logits are wanted and there is nowhere to put them");
  Ctx r{};
  r.m = m, r.s = s, r.stream = s->stream, r.T = c.T, r.B = c.B, r.H = c.H;
  r.dry = false;
  r.whole.dry = false;
  r.whole.base = (char*)s->workspace;
  r.whole.cap = whole_bytes;
  if (s->side_stream)
    if (int rc = events_for_device(r)) return rc;
  g_launches = 0;
  g_vendor_products = 0;
  return walk(r, &entry_bytes);
}

}  // namespace

extern "C" {

int64_t tq_step_workspace(const tq_model_desc* model, const tq_step_desc* step) {
  int64_t bytes = 0;
  const int rc = run(model, step, false, &bytes);
  return rc ? (rc < 0 ? rc : -rc) : bytes;
}

int tq_step_forward(const tq_model_desc* model, const tq_step_desc* step) { return run(model, step, true, nullptr); }

const char* tq_engine_last_error(void) { return g_error; }

int64_t tq_engine_last_launches(void) { return g_launches; }

int64_t tq_engine_last_vendor_products(void) { return g_vendor_products; }

void tq_engine_struct_sizes(int64_t* out) {
  out[0] = sizeof(tq_weight), out[1] = sizeof(tq_norm_desc), out[2] = sizeof(tq_attention_desc);
  out[3] = sizeof(tq_dense_ffn_desc), out[4] = sizeof(tq_moe_ffn_desc), out[5] = sizeof(tq_layer_desc);
  out[6] = sizeof(tq_entry_desc), out[7] = sizeof(tq_model_desc), out[8] = sizeof(tq_step_desc);
}

}  // extern "C"
