// What this GPU reaches on the two things that bound the model's steps, measured rather than taken from the data
// sheet: reading memory once, and the matrix instructions by themselves.  `bench.py --probe` times both.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Every workgroup reads its share of `buf` in whole lines of 128 bytes (eight lanes to a line), 8 loads per lane on
// their way at once, with or without the hint that the bytes are read once; the XOR of everything is stored only
// if it equals `never`, which the caller chooses so that it does not.
template <bool ONCE>
__global__ __launch_bounds__(256) void probe_stream_kernel(const u32x4* __restrict__ buf, int64_t n16,
                                                           unsigned never, unsigned* __restrict__ out) {
  u32x4 x = {0u, 0u, 0u, 0u};
  const int64_t per = (n16 + gridDim.x - 1) / gridDim.x;
  const int64_t b = (int64_t)blockIdx.x * per, e = b + per < n16 ? b + per : n16;
  for (int64_t i = b + threadIdx.x; i < e; i += 8 * 256) {
    u32x4 t[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t j = i + u * 256 < e ? i + u * 256 : i;
      t[u] = ONCE ? __builtin_nontemporal_load(buf + j) : buf[j];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) x ^= t[u];
  }
  const unsigned v = x.x ^ x.y ^ x.z ^ x.w;
  if (v == never) out[0] = v;
}

// bytes: a multiple of 16.  once: 1 = loads carry the read-once hint.
TQ_API int tq_probe_stream(const void* buf, int64_t bytes, int once, unsigned never, unsigned* out, hipStream_t st) {
  if (bytes <= 0 || bytes % 16 != 0 || ((size_t)buf & 15)) return TQ_ERR_BAD_ARG;
  const int grid = 256 * 8;
  if (once)
    hipLaunchKernelGGL(probe_stream_kernel<true>, dim3(grid), dim3(256), 0, st, (const u32x4*)buf, bytes / 16, never, out);
  else
    hipLaunchKernelGGL(probe_stream_kernel<false>, dim3(grid), dim3(256), 0, st, (const u32x4*)buf, bytes / 16, never, out);
  TQ_LAUNCH_CHECK();
  return 0;
}

// Eight waves per compute unit (two per SIMD), each a loop of independent matrix instructions on operands that
// differ from lane to lane (seed != 0: pseudo-random values in [-1, 1]; seed 0: the same value everywhere, which
// draws less power and runs faster).  SHAPE 32: v_mfma_f32_32x32x16_bf16, 16: v_mfma_f32_16x16x32_bf16.
template <int SHAPE>
__global__ __launch_bounds__(512) void probe_mfma_kernel(int iters, unsigned seed, float* __restrict__ out) {
  bf16x8 a, b;
  unsigned h = (blockIdx.x * 1024u + threadIdx.x) * 2654435761u + seed;
  for (int i = 0; i < 8; ++i) {
    h = h * 1664525u + 1013904223u;
    a[i] = (__bf16)(seed ? ((int)(h >> 8) % 2001 - 1000) * 0.001f : 0.5f);
    h = h * 1664525u + 1013904223u;
    b[i] = (__bf16)(seed ? ((int)(h >> 8) % 2001 - 1000) * 0.001f : 0.5f);
  }
  float s = 0.f;
  if (SHAPE == 32) {
    f32x16 acc[6];
    for (int t = 0; t < 6; ++t)
      for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int t = 0; t < 6; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[t], 0, 0, 0);
    }
    for (int t = 0; t < 6; ++t)
      for (int v = 0; v < 16; ++v) s += acc[t][v];
  } else {
    f32x4 acc[12];
    for (int t = 0; t < 12; ++t)
      for (int v = 0; v < 4; ++v) acc[t][v] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int t = 0; t < 12; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[t], 0, 0, 0);
    }
    for (int t = 0; t < 12; ++t)
      for (int v = 0; v < 4; ++v) s += acc[t][v];
  }
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// out: workgroups * 512 floats.  The launch does workgroups * 8 * iters * 196,608 floating-point operations
// (a wave's 6 instructions of 32x32x16, or 12 of 16x16x32, per iteration: 2 * 98,304 multiply-adds).
TQ_API int tq_probe_mfma(int shape, int workgroups, int iters, unsigned seed, float* out, hipStream_t st) {
  if ((shape != 16 && shape != 32) || workgroups < 1 || iters < 1) return TQ_ERR_BAD_ARG;
  if (shape == 32)
    hipLaunchKernelGGL(probe_mfma_kernel<32>, dim3(workgroups), dim3(512), 0, st, iters, seed, out);
  else
    hipLaunchKernelGGL(probe_mfma_kernel<16>, dim3(workgroups), dim3(512), 0, st, iters, seed, out);
  TQ_LAUNCH_CHECK();
  return 0;
}
