// The entry points of the kernel libraries (libtq_bfloat16-<hash>.so, libtq_float32-<hash>.so), as a host in C or C++
// would call them: plain C functions that take device pointers, sizes and a stream, launch on that stream and return
// 0, TQ_ERR_BAD_ARG (-1: the arguments contradict each other), TQ_ERR_UNSUPPORTED (-2: a size this kernel does not
// take; nothing was launched) or a hipError_t of the launch.  None of them allocates, frees or synchronises; scratch
// memory, where a kernel needs it, is an argument whose size a *_scratch / *_runs / *_splits function gives.  The
// comment in front of each definition in the .hip file named here says what the arguments mean; the Python face
// (ops.py) checks shapes, types and strides before every call and is the reference for how to call them.
// Weight types: TQ_F32 0, TQ_BF16 1.  Activations are bfloat16 in the bfloat16 library and float in the float32
// library (written `void*` here).  Gate activations: numbered by their lines in gates.def (0 silu, 1 gelu_tanh, 2 relu2).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "no_alloc.h"

#define TQ_ERR_BAD_ARG (-1)
#define TQ_ERR_UNSUPPORTED (-2)
// added to a tile_rows of 64 of a product over experts: two units of one expert per workgroup (see tq_gemm_mfma)
#define TQ_TILE_PAIRS 1024

#ifdef __cplusplus
extern "C" {
#endif
// elementwise.hip: embedding, soft cap, residual sum + RMS norm, per-head norm, rotation + cache write, weighted sum of expert rows (both libraries)
int tq_embed(const int* tokens, const void* table, int wtype, float* x, int T, int H, float scale, hipStream_t st);
int tq_softcap(float* x, int64_t n, float cap, hipStream_t st);
int tq_move_rows(const void* src, const int* idx, void* dst, int n, int64_t row_bytes, int scatter, hipStream_t st);
int tq_add_rmsnorm(float* x, const float* delta, int S, int64_t delta_stride, const float* y, const int* pair_slot,
        const float* weights, int topk, const float* gate, const void* w, int wtype, float eps, const int* rows,
        int R, void* out, float* out32, int H, hipStream_t st);
int tq_head_rmsnorm(float* qkv, const void* wq, const void* wk, int wtype, float eps, int T, int nh, int nkv,
        int hd, hipStream_t st);
int tq_gated_act(const float* gu, int64_t ld, void* out, int M, int N, int gate, hipStream_t st);
int tq_rope_kv_write(const float* qkv, const void* bias, int bias_type, const int* positions,
        const int* seq_of_token, const int* block_table, int bt_stride, const float* inv_freq, int pairing,
        int rot, void* q_out, void* k_pool, void* v_pool, int page_size, int64_t page_stride, int T, int nh, int nkv,
        int hd, int write_kv, const int* cu_seqlens, const int* slots, const int* start, int B, int max_new,
        hipStream_t st);
int tq_moe_combine(const float* y, const int* pair_slot, const float* weights, int topk, const float* shared,
        int S, int64_t shared_stride, const float* gate, float* out, int T, int H, hipStream_t st);
// gemm_generic.hip: the plain multiply-add product (both libraries)
int tq_gemm_generic(const void* a, int64_t lda, const int* a_rows, int a_gather, const void* w, const void* w2,
        int wtype, int64_t group_stride, const int* tile_group, const int* n_tiles, const void* bias,
        int bias_type, void* out, int64_t ldc, int out_is_act, int M, int N, int K, int tile_rows, int gate,
        hipStream_t st);
// gemm_mfma.hip: bfloat16 products on the matrix cores (bfloat16 library)
int tq_gemm_mfma_splits(int M, int N, int K);
int tq_gemm_mfma(const void* a, int64_t lda, const int* a_rows, int a_gather, const void* w, const void* w2,
        int64_t group_stride, const int* tile_group, const int* n_tiles, const void* bias, int bias_type,
        void* out, int64_t ldc, int out_is_act, int M, int N, int K, int tile_rows, int splits, int gate,
        hipStream_t st);
int tq_gemm_mfma_pair_splits(int N1, int K1, int grouped1, int N2, int K2, int grouped2);
int tq_gemm_mfma_pair(const int64_t* d1, const int64_t* d2, int splits2, hipStream_t st);
int tq_qkv_rope_write(const void* a, int64_t lda, const void* w, const void* bias, int bias_type, int T, int K,
        const int* positions, const int* seq_of_token, const int* block_table, int bt_stride,
        const float* inv_freq, void* q_out, void* k_pool, void* v_pool, int page_size, int64_t page_stride, int nh,
        int nkv, int hd, hipStream_t st);
// gemm_f32.hip: float32 products on the matrix cores (float32 library)
int tq_gemm_f32_runs(int M, int N, int K, int grouped);
int tq_gemm_f32(const void* a, int64_t lda, const int* a_rows, int a_gather, const void* w, const void* w2,
        int64_t group_stride, const int* tile_group, const int* n_tiles, const void* bias, int bias_type,
        void* out, int64_t ldc, int M, int N, int K, int tile_rows, int gate, void* scratch, int keep_runs,
        hipStream_t st);
// attention_generic.hip: token-by-token attention over the pages (both libraries)
int tq_attention_generic(const void* q, const void* k_pool, const void* v_pool, const int* positions,
        const int* seq_of_token, const int* block_table, int bt_stride, int page_size, int64_t page_stride, int T,
        int nh, int nkv, int hd, int window, float scale, void* out, hipStream_t st);
// attention_mfma.hip: bfloat16 attention on the matrix cores (bfloat16 library)
int64_t tq_attention_decode_scratch(int B, int nh, int hd, int max_end);
int tq_attention_mfma(const void* q, const void* k_pool, const void* v_pool, const int* block_table, int bt_stride,
        const int* cu_seqlens, const int* slots, const int* start, int page_size, int64_t page_stride, int B,
        int nh, int nkv, int hd, int window, float scale, void* out, float* partial, int decode, int max_new,
        int max_end, hipStream_t st);
// attention_f32.hip: float32 attention on the matrix cores (float32 library)
int64_t tq_attention_f32_scratch(int B, int nh, int hd, int max_end);
int tq_attention_f32(const void* q, const void* k_pool, const void* v_pool, const int* block_table, int bt_stride,
        const int* cu_seqlens, const int* slots, const int* start, int page_size, int64_t page_stride, int B,
        int nh, int nkv, int hd, int window, float scale, void* out, void* partial, int decode, int max_new,
        int max_end, hipStream_t st);
// moe.hip: router, choice of experts, order of pairs (both libraries)
int tq_router_topk(const float* x, const void* wr, const void* shared_w, int wtype, int E, int topk, int renorm,
        int* ids, float* weights, float* shared_gate, float* logits, int T, int H, hipStream_t st);
int tq_moe_align(const int* ids, int n_pairs, int E, int topk, int unit, int cap, int* sorted_token,
        int* pair_slot, int* tile_expert, int* n_tiles, hipStream_t st);
int tq_route(const float* x, const void* wr, const void* shared_w, int wtype, int E, int topk, int renorm,
        int* ids, float* weights, float* shared_gate, float* logits, int unit, int cap, int* sorted_token,
        int* pair_slot, int* tile_expert, int* n_tiles, int T, int H, hipStream_t st);
// sampling.hip: greedy choice, negative log-likelihood, repetition penalty, temperature and top-p (both libraries; the two *_static entry points are declared in no_alloc.h)
int tq_argmax(const float* logits, int R, int V, int* out, hipStream_t st);
int tq_nll(const float* logits, int R, int V, const int* target, float* out, hipStream_t st);
int tq_probs_half(const float* logits, int R, int V, void* probs, const void* base, double* kl, hipStream_t st);
int tq_rep_penalty(float* logits, int R, int V, const int* recent, int window, const int* counts, float penalty,
        hipStream_t st);
int64_t tq_sample_topp_scratch(int R);
int tq_sample_topp(const float* logits, int R, int V, float temperature, float top_p, const float* uniforms,
        float* probs, float* scratch, int* out, hipStream_t st);
// probe.hip: what bench.py --probe times (bfloat16 library)
int tq_probe_stream(const void* buf, int64_t bytes, int once, unsigned never, unsigned* out, hipStream_t st);
int tq_probe_mfma(int shape, int workgroups, int iters, unsigned seed, float* out, hipStream_t st);

#ifdef __cplusplus
}
#endif
