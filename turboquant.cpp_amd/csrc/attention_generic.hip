// Attention of each given token over the cache pages of its sequence, with plain float arithmetic.
//
// Token t of sequence s at position p attends to positions lo..p, lo = max(0, p - window + 1)
// when a window is set (the last `window` positions, the current one included:
// /root/reference/src/engine/tq_transformer.c:1646-1654), else 0.  Query head h reads kv head
// h / (nh / nkv) (tq_transformer.c:1675-1679).  score = (q . k) / sqrt(hd) (:1908-1937), softmax
// over the scores (/root/reference/src/engine/tq_ops.c:1496-1519), output = sum p_j v_j
// (tq_transformer.c:1975-1976).  The softmax is computed chunk by chunk with a running maximum;
// chunks start at multiples of CHUNK positions, so the order of every sum depends only on the
// token's own position.  The same kernel serves whole prompts and single decoded tokens: the cache
// has been written for all tokens of the step before it runs.  In a page, keys lie [kv head][row][hd]
// and values transposed, [kv head][hd][row].
#include "common.h"

#define CHUNK 128

__global__ __launch_bounds__(CHUNK) void attention_generic_kernel(
    const act_t* __restrict__ q, const act_t* __restrict__ k_pool, const act_t* __restrict__ v_pool,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
    int bt_stride, int page_size, int64_t page_stride, int nh, int nkv, int hd, int window, float scale,
    act_t* __restrict__ out) {
  extern __shared__ float sm[];
  float* qs = sm;                       // hd
  float* ps = qs + hd;                  // CHUNK probabilities
  float* red = ps + CHUNK;              // one per wave
  int64_t* head_off = (int64_t*)(red + 4);  // per row of the chunk: offset of its page's block for this kv head
  int* row_in_page = (int*)(head_off + CHUNK);
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int kvh = h / (nh / nkv);
  const int pos = positions[t];
  const int* table = block_table + (size_t)seq_of_token[t] * bt_stride;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;

  for (int i = tid; i < hd; i += CHUNK) qs[i] = to_f32(q[((size_t)t * nh + h) * hd + i]);
  __syncthreads();

  // each thread owns the output dimensions tid, tid + CHUNK, ... (at most 4: hd <= 512)
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

  for (int base = (lo / CHUNK) * CHUNK; base <= pos; base += CHUNK) {
    const int j = base + tid;
    const bool valid = j >= lo && j <= pos;
    float sc = -INFINITY;
    int64_t off = 0;
    if (valid) {
      const int page = table[j / page_size];
      off = (int64_t)page * page_stride + (int64_t)kvh * page_size * hd;
      const act_t* kr = k_pool + off + (int64_t)(j % page_size) * hd;   // keys: [row][hd]
      float d = 0.f;
      for (int i = 0; i < hd; ++i) d = fmaf(qs[i], to_f32(kr[i]), d);
      sc = d * scale;
    }
    head_off[tid] = off;
    row_in_page[tid] = j % page_size;
    const float m_chunk = block_max(sc, red);
    const float m_new = fmaxf(m_run, m_chunk);
    const float p = valid ? expf(sc - m_new) : 0.f;
    ps[tid] = p;
    const float l_chunk = block_sum(p, red);   // has the barriers that publish ps and the offsets
    const float alpha = m_run == -INFINITY ? 0.f : expf(m_run - m_new);
    l_run = l_run * alpha + l_chunk;
    m_run = m_new;
    const int n_in_chunk = min(CHUNK, pos - base + 1);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int d = tid + c * CHUNK;
      if (d < hd) {
        float a = acc[c] * alpha;
        for (int jj = 0; jj < n_in_chunk; ++jj) {
          const float pj = ps[jj];
          // values: [hd][row]
          if (pj != 0.f) a = fmaf(pj, to_f32(v_pool[head_off[jj] + (int64_t)d * page_size + row_in_page[jj]]), a);
        }
        acc[c] = a;
      }
    }
    __syncthreads();
  }
  const float inv = 1.0f / l_run;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int d = tid + c * CHUNK;
    if (d < hd) out[((size_t)t * nh + h) * hd + d] = from_f32<act_t>(acc[c] * inv);
  }
}

TQ_API int tq_attention_generic(const void* q, const void* k_pool, const void* v_pool, const int* positions,
                                const int* seq_of_token, const int* block_table, int bt_stride, int page_size,
                                int64_t page_stride, int T, int nh, int nkv, int hd, int window, float scale,
                                void* out, hipStream_t st) {
  if (T <= 0) return 0;
  if (hd > 4 * CHUNK || nkv <= 0 || nh % nkv != 0) return TQ_ERR_UNSUPPORTED;
  if (nh > 65535) return TQ_ERR_UNSUPPORTED;
  const size_t shmem = (size_t)(hd + CHUNK + 4) * sizeof(float) + CHUNK * (sizeof(int64_t) + sizeof(int));
  hipLaunchKernelGGL(attention_generic_kernel, dim3(T, nh), dim3(CHUNK), shmem, st, (const act_t*)q,
                     (const act_t*)k_pool, (const act_t*)v_pool, positions, seq_of_token, block_table, bt_stride,
                     page_size, page_stride, nh, nkv, hd, window, scale, (act_t*)out);
  TQ_LAUNCH_CHECK();
  return 0;
}
