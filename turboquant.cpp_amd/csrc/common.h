// Shared definitions of the gfx950 kernels.
//
// One library is built per activation type: TQ_ACT_BF16 (activations and cache in
// bfloat16, every sum in float) or TQ_ACT_F32 (everything in float, no matrix cores
// with reduced-precision inputs).  Weights carry their own type at run time
// (TQ_F32 or TQ_BF16) because a tensor that the checkpoint stores in 32 bits stays so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TQ_F32 0
#define TQ_BF16 1

// error codes of the extern "C" entry points (0 = ok, > 0 = hipError_t)
#define TQ_ERR_BAD_ARG (-1)
#define TQ_ERR_UNSUPPORTED (-2)
// added to a tile_rows of 64 of a product over experts: two units of one expert per workgroup (see tq_gemm_mfma)
#define TQ_TILE_PAIRS 1024

struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

// round to nearest even; NaN stays NaN
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  bf16_t r;
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    r.bits = (uint16_t)((u >> 16) | 0x40);
  } else {
    u += 0x7fffu + ((u >> 16) & 1u);
    r.bits = (uint16_t)(u >> 16);
  }
  return r;
}

template <class T>
__device__ __forceinline__ T from_f32(float f);
template <>
__device__ __forceinline__ float from_f32<float>(float f) { return f; }
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float f) { return f32_to_bf16(f); }

#if defined(TQ_ACT_BF16)
typedef bf16_t act_t;
#define TQ_ACT_TYPE TQ_BF16
#elif defined(TQ_ACT_F32)
typedef float act_t;
#define TQ_ACT_TYPE TQ_F32
#else
#error "define TQ_ACT_BF16 or TQ_ACT_F32"
#endif

#define TQ_WAVE 64

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = TQ_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, TQ_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = TQ_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, TQ_WAVE));
  return v;
}

// Sum over a workgroup in a fixed order: waves reduce by butterfly, wave totals are added
// in wave order.  `red` holds one float per wave.  Every thread gets the total.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int nw = (blockDim.x + TQ_WAVE - 1) / TQ_WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int nw = (blockDim.x + TQ_WAVE - 1) / TQ_WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = red[0];
  for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
  return t;
}

// Activation of the gate in a gated pair act(a w^T) * (a w2^T); a parameter of the products' epilogues, numbered in
// the order of the list in gates.def.
enum {
#define TQ_GATE(name, expr) TQ_GATE_##name,
#include "gates.def"
#undef TQ_GATE
  TQ_GATE_COUNT
};
__device__ __forceinline__ float gate_fn(float x, int kind) {
  switch (kind) {
#define TQ_GATE(name, expr) \
  case TQ_GATE_##name:      \
    return (expr);
#include "gates.def"
#undef TQ_GATE
  }
  return x;
}

#define TQ_LAUNCH_CHECK()                        \
  do {                                           \
    hipError_t e__ = hipGetLastError();          \
    if (e__ != hipSuccess) return (int)e__;      \
  } while (0)

// Calls `body` with `W` bound to the C type of a run-time weight type.
#define TQ_DISPATCH_W(wtype, ...)                  \
  do {                                             \
    if ((wtype) == TQ_F32) {                       \
      typedef float W;                             \
      __VA_ARGS__                                  \
    } else if ((wtype) == TQ_BF16) {               \
      typedef bf16_t W;                            \
      __VA_ARGS__                                  \
    } else {                                       \
      return TQ_ERR_BAD_ARG;                       \
    }                                              \
  } while (0)

#define TQ_API extern "C" __attribute__((visibility("default")))
