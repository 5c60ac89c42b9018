// The step executor: one call runs a whole step (embedding, every schedule entry's layer, final norm, vocabulary
// product) by issuing this library's kernels one after the other from C, with no interpreter between two launches.
//
// The reference's host is C: one function walks the layers of a step (tq_forward,
// /root/reference/src/engine/tq_transformer.c:2281-3029) over a model structure that its loader filled
// (/root/reference/include/turboquant/tq_engine.h).  Here the model structure is the set of descriptors below, which
// say, layer by layer, which part runs with which sizes, constants and weights; a host in any language fills them
// (the Python package does, from the model's plan and its loaded parameters) and
// hands them to tq_step_forward together with the step's packed tokens.  The executor knows the parts (norm,
// attention, dense and sparse feed-forward, the pre-norm arrangement) and nothing of any architecture.
//
// Every field of every structure is 8 bytes wide (int64_t, double or a pointer), so a host lays them out without
// knowing the compiler's padding rules.  Pointers in tq_weight and in the step are device pointers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
  const void* ptr;        // NULL: the parameter is absent
  int64_t wtype;          // TQ_F32 (0) or TQ_BF16 (1)
} tq_weight;

typedef struct {
  tq_weight weight;       // [hidden]
  double eps;
} tq_norm_desc;

typedef struct {
  int64_t hidden, num_heads, num_kv_heads, head_dim;
  int64_t window;         // 0: every earlier position is in reach
  int64_t pairing;        // 0: pairs (i, i + rotary_dim / 2); 1: pairs (2i, 2i + 1)
  int64_t rotary_dim;
  double scale;           // of the scores
  tq_weight qkv_weight;   // [(heads + 2 kv heads) * head_dim, hidden]
  tq_weight qkv_bias;     // [(heads + 2 kv heads) * head_dim] or absent
  tq_weight out_weight;   // [hidden, heads * head_dim]
  tq_weight out_bias;     // [hidden] or absent
  const float* inv_freq;  // [rotary_dim / 2]: the angle of pair i at position p is p * inv_freq[i]
} tq_attention_desc;

typedef struct {
  int64_t hidden, inner;
  int64_t gate;           // activation of the gate, numbered by its line in gates.def
  tq_weight gate_w, up_w; // [inner, hidden] each; up_w right behind gate_w in memory lets long prompts take one product
  tq_weight down_w;       // [hidden, inner]
} tq_dense_ffn_desc;

typedef struct {
  int64_t hidden, num_experts, top_k, inner;
  int64_t shared_inner;   // 0: no shared expert
  int64_t renormalize;    // softmax over the chosen logits (1) or over all, kept as it is for the chosen (0)
  int64_t gate;
  tq_weight router;       // [experts, hidden]
  tq_weight shared_scale; // [hidden] or absent: the shared expert is scaled by sigmoid(x . shared_scale)
  tq_weight expert_gate, expert_up;     // [experts, inner, hidden]
  tq_weight expert_down;                // [experts, hidden, inner]
  tq_weight shared_gate, shared_up;     // [shared_inner, hidden]
  tq_weight shared_down;                // [hidden, shared_inner]
} tq_moe_ffn_desc;

#define TQ_FFN_DENSE 1
#define TQ_FFN_MOE 2

// A layer in the pre-norm arrangement: x += attention(norm(x)); x += ffn(norm(x)).
typedef struct {
  tq_norm_desc mixer_norm;
  tq_attention_desc attention;
  tq_norm_desc ffn_norm;
  int64_t ffn_kind;       // TQ_FFN_DENSE or TQ_FFN_MOE: which of the two below is filled
  tq_dense_ffn_desc dense;
  tq_moe_ffn_desc moe;
} tq_layer_desc;

// One schedule entry: which layer runs, and where its keys and values live (its own, or an earlier entry's).
typedef struct {
  int64_t layer;
  void* k_pages;          // flat pool of key pages of the entry's cache group
  void* v_pages;
  const int* table;       // [slots, table_width]: logical page -> page, -1: none
  int64_t table_width;
  int64_t layer_offset;   // of this entry's rows inside a page, in elements
  int64_t page_size;      // positions per page
  int64_t page_stride;    // elements per page
  int64_t owns;           // 0: the entry reads another entry's keys and values and writes none
} tq_entry_desc;

typedef struct {
  int64_t vocab, hidden, n_layers, n_entries;
  const tq_layer_desc* layers;      // host memory
  const tq_entry_desc* entries;     // host memory: the order in which layers run
  tq_weight embedding;    // [vocab, hidden]
  tq_weight lm_head;      // [vocab, hidden] (the embedding when tied)
  tq_norm_desc final_norm;
  double embedding_scale;
  double logit_softcap;   // 0: none; else logits <- cap * tanh(logits / cap)
} tq_model_desc;

// The packed tokens of one step (as engine/batch.py packs them) and where the step may work.
typedef struct {
  int64_t T;              // tokens of the step
  int64_t B;              // sequences of the step
  int64_t n_want;         // rows whose logits are wanted
  int64_t max_new;        // the most tokens one sequence brings
  int64_t max_end;        // the furthest position + 1 that the step reaches (decode steps under capture: the bucket's)
  int64_t decode;         // every sequence brings one token
  int64_t capturing;      // the step is being recorded into a graph
  // tuning that the caller owns: plain products of vendor_min_rows rows and more may go to the vendor's matrix
  // library (0: never); gated pairs go there vendor_gated_rows at a time; experts take units of 128 rows from
  // expert_128_from rows per expert on average, of 256 from expert_256_from, and units of 64 two at a time from
  // expert_pairs_from; an eager step of side_from tokens and more runs the shared expert on the side stream
  int64_t vendor_min_rows, vendor_gated_rows, expert_128_from, expert_256_from, expert_pairs_from, side_from;
  const int* tokens;          // [T]
  const int* positions;       // [T]
  const int* slot_of_token;   // [T]
  const int* cu_seqlens;      // [B + 1]
  const int* slots;           // [B]
  const int* start;           // [B]
  const int* want_rows;       // [n_want]
  void* workspace;            // tq_step_workspace bytes of device memory, aligned to 256
  int64_t workspace_bytes;
  float* logits;              // [n_want, vocab]: the result
  hipStream_t stream;
  hipStream_t side_stream;    // NULL: everything runs in line
} tq_step_desc;

// Bytes of workspace that tq_step_forward needs for this step (a function of the model's sizes and of T, B,
// n_want, max_end, decode and the tuning fields), or a negative error.
int64_t tq_step_workspace(const tq_model_desc* model, const tq_step_desc* step);
// Runs the step: 0, or an error whose text tq_engine_last_error gives.  Allocates nothing and does not synchronise.
int tq_step_forward(const tq_model_desc* model, const tq_step_desc* step);
const char* tq_engine_last_error(void);
// sizeof of the structures above, in the order tq_weight, tq_norm_desc, tq_attention_desc, tq_dense_ffn_desc,
// tq_moe_ffn_desc, tq_layer_desc, tq_entry_desc, tq_model_desc, tq_step_desc: for a host to check its own layout.
void tq_engine_struct_sizes(int64_t* out9);
// How many kernels the last tq_step_forward of this thread launched (vendor products included).
int64_t tq_engine_last_launches(void);
// How many of them were products of the vendor's matrix library.
int64_t tq_engine_last_vendor_products(void);

#ifdef __cplusplus
}
#endif
