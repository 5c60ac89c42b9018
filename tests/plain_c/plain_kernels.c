/* Plain C twins of the GPU kernels: one function beside each kernel entry point of the library, with the same data
 * contract (packed rows, cache pages behind a table of pages per slot, pairs ordered by expert in units of rows),
 * whole arrays in host memory, one loop nest each, every sum in double and in ascending order.  Values are float
 * (a test that checks a bfloat16 kernel widens its operands first).  The formulas are the reference's; each function
 * cites where.  Nothing of the library calls, includes or links this file: tests compile it and compare every
 * kernel with its twin, and the twins with the plain model in Python. */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* x[t] = table[tokens[t]] * scale  (/root/reference/src/engine/tq_transformer.c:2297-2337: the token's row, scaled
 * for models that scale it) */
void pc_embed(const int* tokens, const float* table, float* x, int T, int H, float scale) {
  for (int t = 0; t < T; ++t)
    for (int i = 0; i < H; ++i) x[(size_t)t * H + i] = table[(size_t)tokens[t] * H + i] * scale;
}

/* x = cap * tanh(x / cap)  (/root/reference/src/engine/tq_transformer.c:2980-2986, for models that cap their logits) */
void pc_softcap(float* x, int64_t n, float cap) {
  for (int64_t i = 0; i < n; ++i) x[i] = cap * tanhf(x[i] / cap);
}

/* dst[i] = src[idx[i]] (gather) or dst[idx[i]] = src[i] (scatter), rows of `row_floats` floats */
void pc_move_rows(const float* src, const int* idx, float* dst, int n, int row_floats, int scatter) {
  for (int i = 0; i < n; ++i) {
    const float* s = src + (size_t)(scatter ? i : idx[i]) * row_floats;
    float* d = dst + (size_t)(scatter ? idx[i] : i) * row_floats;
    memcpy(d, s, (size_t)row_floats * sizeof(float));
  }
}

/* The sum that experts leave to the next norm: d[t] = sum_j weights[t][j] * y[pair_slot[t][j]] + gate[t] * sum_s
 * shared[s][t]  (/root/reference/src/engine/tq_moe.c:994-999: output += weight * expert output, in selection order;
 * :1011-1018, 1057-1058: + sigmoid gate * shared expert).  Any of y, shared, gate may be null. */
void pc_moe_combine(const float* y, const int* pair_slot, const float* weights, int topk, const float* shared, int S,
                    const float* gate, float* out, int T, int H) {
  for (int t = 0; t < T; ++t)
    for (int i = 0; i < H; ++i) {
      double acc = 0.0;
      if (y)
        for (int j = 0; j < topk; ++j)
          acc += (double)weights[(size_t)t * topk + j] * y[(size_t)pair_slot[(size_t)t * topk + j] * H + i];
      double sh = 0.0;
      for (int s = 0; s < S; ++s) sh += shared[((size_t)s * T + t) * H + i];
      acc += (gate ? (double)gate[t] : 1.0) * sh;
      out[(size_t)t * H + i] = (float)acc;
    }
}

/* v = x[row] + d[row]; x[row] = v (when rows is null); out = v / sqrt(mean(v^2) + eps) * w
 * (/root/reference/src/engine/tq_ops.c:1373-1410: eps inside the root, the weight multiplied last).  d: S partial sums
 * [S][T][H] added in order, or null.  rows: which tokens to norm (R of them), or null for all T. */
void pc_add_rmsnorm(float* x, const float* delta, int S, const float* w, float eps, const int* rows, int R, float* out,
                    int T, int H) {
  const int n = rows ? R : T;
  for (int r = 0; r < n; ++r) {
    const int t = rows ? rows[r] : r;
    double ss = 0.0;
    for (int i = 0; i < H; ++i) {
      float v = x[(size_t)t * H + i];
      for (int s = 0; s < S; ++s) v += delta[((size_t)s * T + t) * H + i];
      if (!rows) x[(size_t)t * H + i] = v;
      out[(size_t)r * H + i] = v;
      ss += (double)v * v;
    }
    const double rs = 1.0 / sqrt(ss / H + (double)eps);
    for (int i = 0; i < H; ++i) out[(size_t)r * H + i] = (float)(out[(size_t)r * H + i] * rs * w[i]);
  }
}

/* The same norm over each head of q and k within a row of [q | k | v]  (/root/reference/src/engine/tq_transformer.c:
 * 1111-1123: per-head norm of queries and keys before the rotation, for models that have it). */
void pc_head_rmsnorm(float* qkv, const float* wq, const float* wk, float eps, int T, int nh, int nkv, int hd) {
  const int width = (nh + 2 * nkv) * hd;
  for (int t = 0; t < T; ++t)
    for (int h = 0; h < nh + nkv; ++h) {
      const float* w = h < nh ? wq : wk;
      if (!w) continue;
      float* v = qkv + (size_t)t * width + (size_t)h * hd;
      double ss = 0.0;
      for (int i = 0; i < hd; ++i) ss += (double)v[i] * v[i];
      const double rs = 1.0 / sqrt(ss / hd + (double)eps);
      for (int i = 0; i < hd; ++i) v[i] = (float)(v[i] * rs * w[i]);
    }
}

static double gate_fn(double v, int gate) {
  if (gate == 0) return v / (1.0 + exp(-v));                    /* silu, /root/reference/src/engine/tq_ops.c:1473-1476 */
  if (gate == 1) return 0.5 * v * (1.0 + tanh(0.7978845608028654 * (v + 0.044715 * v * v * v)));   /* gelu_tanh */
  const double r = v > 0.0 ? v : 0.0;                           /* relu squared */
  return r * r;
}

/* out[m][n] = f(gu[m][n]) * gu[m][N + n]: the gate of a pair that came out of one product over both matrices */
void pc_gated_act(const float* gu, int64_t ld, float* out, int M, int N, int gate) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) out[(size_t)m * N + n] = (float)(gate_fn(gu[m * ld + n], gate) * gu[m * ld + N + n]);
}

/* out[m][n] = sum_k a[row(m)][k] * w[g(m)][n][k] (+ bias[n]), or with w2 the gated pair f(a w^T + bias) * (a w2^T)
 * (/root/reference/src/engine/tq_ops.c:296-343: rows of w times the vector; the pair:
 * /root/reference/src/engine/tq_transformer.c:2770-2806).  a_rows: the row of `a` behind each output row, -1 for
 * none (then the output row is left alone); with gather 0 a live output row m reads row m.  tile_group: the matrix
 * of each unit of tile_rows output rows (n_units of them in use), or null for one matrix. */
void pc_gemm(const float* a, int64_t lda, const int* a_rows, int gather, const float* w, const float* w2,
             int64_t group_stride, const int* tile_group, int n_units, int tile_rows, const float* bias, int gate,
             float* out, int M, int N, int K) {
  for (int m = 0; m < M; ++m) {
    if (tile_group && m / tile_rows >= n_units) continue;
    int src = m;
    if (a_rows) {
      if (a_rows[m] < 0) continue;
      if (gather) src = a_rows[m];
    }
    const int64_t g = tile_group ? tile_group[m / tile_rows] : 0;
    const float* ar = a + src * lda;
    for (int n = 0; n < N; ++n) {
      const float* wr = w + g * group_stride + (size_t)n * K;
      double s = 0.0;
      for (int k = 0; k < K; ++k) s += (double)ar[k] * wr[k];
      if (bias) s += bias[n];
      if (w2) {
        const float* vr = w2 + g * group_stride + (size_t)n * K;
        double u = 0.0;
        for (int k = 0; k < K; ++k) u += (double)ar[k] * vr[k];
        s = gate_fn(s, gate) * u;
      }
      out[(size_t)m * N + n] = (float)s;
    }
  }
}

/* Rotation of queries and keys and the write of keys and values into their pages.  Angle of pair i: position *
 * inv_freq[i] (/root/reference/src/engine/tq_ops.c:1424-1425); pairing 0 ("half") rotates (x[i], x[i + rotary/2]),
 * pairing 1 (x[2i], x[2i+1]) (/root/reference/src/engine/tq_transformer.c:1263-1289); (a, b) -> (a cos - b sin,
 * a sin + b cos).  qkv: [T][(nh + 2 nkv) hd] float, bias added first if given.  q_out [T][nh hd].  Pages: a page holds
 * every layer's keys [kv head][row][hd] (values transposed [kv head][hd][row]) at layer_offset; token t's row is
 * position % page_size of page table[slot_of_token[t]][position / page_size]. */
void pc_rope_kv_write(const float* qkv, const float* bias, const int* positions, const int* slot_of_token,
                      const int* table, int table_width, const float* inv_freq, int pairing, int rotary_dim,
                      float* q_out, float* k_pages, float* v_pages, int64_t layer_offset, int page_size,
                      int64_t page_stride, int T, int nh, int nkv, int hd) {
  const int width = (nh + 2 * nkv) * hd, half = rotary_dim / 2;
  float* row = (float*)malloc(sizeof(float) * (size_t)width);
  for (int t = 0; t < T; ++t) {
    for (int i = 0; i < width; ++i) row[i] = qkv[(size_t)t * width + i] + (bias ? bias[i] : 0.f);
    for (int h = 0; h < nh + nkv; ++h) {
      float* x = row + (size_t)h * hd;
      for (int i = 0; i < half; ++i) {
        const float ang = (float)positions[t] * inv_freq[i];
        const double c = cos((double)ang), s = sin((double)ang);
        const int ia = pairing == 0 ? i : 2 * i, ib = pairing == 0 ? i + half : 2 * i + 1;
        const double xa = x[ia], xb = x[ib];
        x[ia] = (float)(xa * c - xb * s);
        x[ib] = (float)(xa * s + xb * c);
      }
    }
    memcpy(q_out + (size_t)t * nh * hd, row, sizeof(float) * (size_t)nh * hd);
    if (!k_pages) continue;
    const int p = positions[t];
    const int64_t page = table[(size_t)slot_of_token[t] * table_width + p / page_size];
    for (int h = 0; h < nkv; ++h)
      for (int i = 0; i < hd; ++i) {
        k_pages[page * page_stride + layer_offset + ((size_t)h * page_size + p % page_size) * hd + i] =
            row[(size_t)(nh + h) * hd + i];
        v_pages[page * page_stride + layer_offset + ((size_t)h * hd + i) * page_size + p % page_size] =
            row[(size_t)(nh + nkv + h) * hd + i];
      }
  }
}

/* Attention of token t over positions max(0, p - window + 1) .. p of its own sequence, read from the pages
 * (/root/reference/src/engine/tq_transformer.c:1646-1654: the window holds the last `window` positions, the current
 * one among them; :1675-1679: score = q . k * scale; /root/reference/src/engine/tq_ops.c:1496-1519: softmax with the
 * maximum taken out; the sum over values in order of position).  window 0: all positions.  Query head h reads key
 * and value head h / (nh / nkv). */
void pc_attention(const float* q, const float* k_pages, const float* v_pages, const int* positions,
                  const int* slot_of_token, const int* table, int table_width, int64_t layer_offset, int page_size,
                  int64_t page_stride, int T, int nh, int nkv, int hd, int window, float scale, float* out) {
  for (int t = 0; t < T; ++t) {
    const int p = positions[t], slot = slot_of_token[t];
    const int lo = window > 0 && p - window + 1 > 0 ? p - window + 1 : 0;
    const int n = p - lo + 1;
    double* s = (double*)malloc(sizeof(double) * (size_t)n);
    for (int h = 0; h < nh; ++h) {
      const int kvh = h / (nh / nkv);
      const float* qh = q + ((size_t)t * nh + h) * hd;
      double mx = -INFINITY;
      for (int j = lo; j <= p; ++j) {
        const int64_t page = table[(size_t)slot * table_width + j / page_size];
        const float* kr = k_pages + page * page_stride + layer_offset + ((size_t)kvh * page_size + j % page_size) * hd;
        double d = 0.0;
        for (int i = 0; i < hd; ++i) d += (double)qh[i] * kr[i];
        s[j - lo] = d * scale;
        if (s[j - lo] > mx) mx = s[j - lo];
      }
      double denom = 0.0;
      for (int j = 0; j < n; ++j) {
        s[j] = exp(s[j] - mx);
        denom += s[j];
      }
      for (int i = 0; i < hd; ++i) {
        double o = 0.0;
        for (int j = lo; j <= p; ++j) {
          const int64_t page = table[(size_t)slot * table_width + j / page_size];
          o += s[j - lo] * v_pages[page * page_stride + layer_offset + ((size_t)kvh * hd + i) * page_size + j % page_size];
        }
        out[((size_t)t * nh + h) * hd + i] = (float)(o / denom);
      }
    }
    free(s);
  }
}

/* Router: logits in float order-free double sums, top-k with >= so that among equal logits the highest index wins
 * and ids come out by descending logit (/root/reference/src/engine/tq_moe.c:611-645); weights: softmax over the
 * selected logits (renorm, :648-678) or over all experts with the selected probabilities kept; shared_gate =
 * 1 / (1 + exp(-(x . shared_w))) (:1012-1018).  logits_out [T][E] may be null. */
void pc_router_topk(const float* x, const float* wr, const float* shared_w, int E, int topk, int renorm, int* ids,
                    float* weights, float* shared_gate, float* logits_out, int T, int H) {
  double* lg = (double*)malloc(sizeof(double) * (size_t)E);
  char* taken = (char*)malloc((size_t)E);
  for (int t = 0; t < T; ++t) {
    const float* xr = x + (size_t)t * H;
    for (int e = 0; e < E; ++e) {
      double s = 0.0;
      for (int i = 0; i < H; ++i) s += (double)xr[i] * wr[(size_t)e * H + i];
      lg[e] = (double)(float)s;
      if (logits_out) logits_out[(size_t)t * E + e] = (float)s;
    }
    if (shared_w) {
      double s = 0.0;
      for (int i = 0; i < H; ++i) s += (double)xr[i] * shared_w[i];
      shared_gate[t] = (float)(1.0 / (1.0 + exp(-s)));
    }
    double mx = -INFINITY, denom = 0.0;
    for (int e = 0; e < E; ++e) mx = lg[e] > mx ? lg[e] : mx;
    for (int e = 0; e < E; ++e) denom += exp(lg[e] - mx);
    memset(taken, 0, (size_t)E);
    double sel[64];
    for (int k = 0; k < topk; ++k) {
      int best = -1;
      for (int e = 0; e < E; ++e)
        if (!taken[e] && (best < 0 || lg[e] >= lg[best])) best = e;
      taken[best] = 1;
      ids[(size_t)t * topk + k] = best;
      sel[k] = lg[best];
    }
    if (renorm) {
      double s = 0.0;
      for (int k = 0; k < topk; ++k) s += exp(sel[k] - sel[0]);
      for (int k = 0; k < topk; ++k) weights[(size_t)t * topk + k] = (float)(exp(sel[k] - sel[0]) / s);
    } else {
      for (int k = 0; k < topk; ++k) weights[(size_t)t * topk + k] = (float)(exp(sel[k] - mx) / denom);
    }
  }
  free(lg);
  free(taken);
}

/* The order of pairs by expert: pair i = (token i / topk, expert ids[i]); an expert's pairs lie together in order
 * of i, each expert's run starts at a multiple of `unit` rows, the rows between are -1.  sorted_token [cap],
 * pair_slot [n_pairs], tile_expert [2 cap / unit]: the expert of each unit in use, then (from cap / unit on) the
 * first unit of each item, an expert's units two at a time; counts: units and items in use.  (The reference takes one token at a
 * time and its experts one after the other, /root/reference/src/engine/tq_moe.c:864-999, and needs no such order; that
 * a token's experts are summed in selection order is kept by pc_moe_combine.) */
void pc_moe_align(const int* ids, int n_pairs, int E, int topk, int unit, int cap, int* sorted_token, int* pair_slot,
                  int* tile_expert, int* counts) {
  for (int r = 0; r < cap; ++r) sorted_token[r] = -1;
  int row = 0, units = 0, items = 0;
  for (int e = 0; e < E; ++e) {
    int n = 0;
    for (int i = 0; i < n_pairs; ++i)
      if (ids[i] == e) {
        sorted_token[row + n] = i / topk;
        pair_slot[i] = row + n;
        ++n;
      }
    const int nu = (n + unit - 1) / unit;
    for (int u = 0; u < nu; ++u) {
      tile_expert[units + u] = e;
      if (u % 2 == 0) tile_expert[cap / unit + items++] = units + u;
    }
    units += nu;
    row += nu * unit;
  }
  counts[0] = units;
  counts[1] = items;
}

/* First maximum wins (/root/reference/src/engine/tq_generate.c:30-40) */
void pc_argmax(const float* logits, int rows, int V, int* out) {
  for (int r = 0; r < rows; ++r) {
    int best = 0;
    for (int i = 1; i < V; ++i)
      if (logits[(size_t)r * V + i] > logits[(size_t)r * V + best]) best = i;
    out[r] = best;
  }
}

/* -log softmax(logits[r])[target[r]], the sum in double  (/root/reference/tools/quant.c:577-592) */
void pc_nll(const float* logits, const int* target, int rows, int V, double* out) {
  for (int r = 0; r < rows; ++r) {
    const float* l = logits + (size_t)r * V;
    float mx = l[0];
    double s = 0.0;
    for (int i = 1; i < V; ++i) mx = l[i] > mx ? l[i] : mx;
    for (int i = 0; i < V; ++i) s += exp((double)(l[i] - mx));
    out[r] = -((double)(l[target[r]] - mx) - log(s));
  }
}

/* Over the counts[r] recent tokens of row r, once per occurrence: a positive logit is divided by the penalty, any
 * other multiplied (/root/reference/src/engine/tq_generate.c:387-400).  recent: [rows][window], the live entries first. */
void pc_rep_penalty(float* logits, const int* recent, const int* counts, int window, float penalty, int rows, int V) {
  for (int r = 0; r < rows; ++r)
    for (int j = 0; j < counts[r]; ++j) {
      const int tok = recent[(size_t)r * window + j];
      if (tok < 0 || tok >= V) continue;
      float* l = logits + (size_t)r * V + tok;
      *l = *l > 0.f ? *l / penalty : *l * penalty;
    }
}

/* xorshift64* to a float in [0, 1]  (/root/reference/src/engine/tq_generate.c:53-58) */
static float next_uniform(uint64_t* state) {
  *state ^= *state >> 12;
  *state ^= *state << 25;
  *state ^= *state >> 27;
  return (float)((*state * 0x2545F4914F6CDD1DULL) >> 33) / (float)(1u << 31);
}

typedef struct {
  float p;
  int id;
} pc_prob;

static int by_probability(const void* a, const void* b) {      /* descending; equal probabilities by index */
  const pc_prob *x = (const pc_prob*)a, *y = (const pc_prob*)b;
  if (x->p != y->p) return x->p < y->p ? 1 : -1;
  return x->id - y->id;
}

/* Temperature and top-p sampling of one row (/root/reference/src/engine/tq_generate.c:81-156, float arithmetic in
 * the reference's order): greedy if temperature or top_p is not positive; candidates are the logits >= max - 16 T;
 * p = exp((l - max) / T), normalised by the candidates' sum; sorted descending (the reference's qsort leaves equal
 * probabilities in no stated order: here by index); the prefix whose running sum first reaches top_p is kept;
 * r = uniform * that sum; the first candidate whose running sum reaches r is the token.  state: the generator's,
 * which moves on by one draw. */
int pc_sample_topp_u(const float* logits, int V, float temperature, float top_p, float uniform);
int pc_sample_topp(const float* logits, int V, float temperature, float top_p, uint64_t* state) {
  if (temperature <= 0.f || top_p <= 0.f) return pc_sample_topp_u(logits, V, temperature, top_p, 0.f);
  return pc_sample_topp_u(logits, V, temperature, top_p, next_uniform(state));
}

/* The same with the uniform number given (the kernels take one per row from the host's generator) */
int pc_sample_topp_u(const float* logits, int V, float temperature, float top_p, float uniform) {
  if (temperature <= 0.f || top_p <= 0.f) {
    int best;
    pc_argmax(logits, 1, V, &best);
    return best;
  }
  float mx = logits[0];
  for (int i = 1; i < V; ++i) mx = logits[i] > mx ? logits[i] : mx;
  const float threshold = mx - 16.0f * temperature, inv_t = 1.0f / temperature;
  pc_prob* cand = (pc_prob*)malloc(sizeof(pc_prob) * (size_t)V);
  int n = 0;
  float sum = 0.f;
  for (int i = 0; i < V; ++i)
    if (logits[i] >= threshold) {
      cand[n].p = expf((logits[i] - mx) * inv_t);
      cand[n].id = i;
      sum += cand[n].p;
      ++n;
    }
  const float inv_sum = 1.0f / sum;
  for (int i = 0; i < n; ++i) cand[i].p *= inv_sum;
  qsort(cand, (size_t)n, sizeof(pc_prob), by_probability);
  float cumulative = 0.f;
  int n_top = 0;
  for (int i = 0; i < n; ++i) {
    cumulative += cand[i].p;
    n_top = i + 1;
    if (cumulative >= top_p) break;
  }
  const float r = uniform * cumulative;
  float cdf = 0.f;
  int token = cand[0].id;
  for (int i = 0; i < n_top; ++i) {
    cdf += cand[i].p;
    if (cdf >= r) {
      token = cand[i].id;
      break;
    }
  }
  free(cand);
  return token;
}

float pc_next_uniform(uint64_t* state) { return next_uniform(state); }
