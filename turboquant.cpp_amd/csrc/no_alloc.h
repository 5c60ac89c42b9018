// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc.  tq_sample_topp needs R * V floats for the
// probabilities and a few KB for its passes, which its caller has to bring; tq_sample_topp_static makes the same
// choice, with the same kernels and the same arithmetic, out of an array that is part of the library's image:
// every GPU the library runs on holds TQ_STATIC_SAMPLE_BYTES for it until the process ends.
//
// Limits: at most TQ_STATIC_SAMPLE_MAX_ROWS rows and R * V <= TQ_STATIC_SAMPLE_MAX_PROBS; beyond them the call
// returns TQ_ERR_UNSUPPORTED (-2) and launches nothing.  The call allocates and frees nothing; the first call on a
// device (or tq_sample_topp_static_init, with that device current) looks up the array's address there.
// All calls on one GPU share that GPU's array, which keeps what the last call left in it: calls that overlap on
// one GPU (two streams, two threads) race and must be ordered by the caller.  Nothing in the array needs to be
// cleared between calls.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TQ_STATIC_SAMPLE_MAX_ROWS 64
#define TQ_STATIC_SAMPLE_MAX_PROBS (1 << 21)                 /* floats: 13 rows of 151,936 logits */
#define TQ_STATIC_SAMPLE_BYTES ((1 << 23) + (1 << 19))       /* 8.5 MiB */

#ifdef __cplusplus
extern "C" {
#endif
// Looks up the array's address on the current device; 0, or a hipError_t.
int tq_sample_topp_static_init(void);
// logits [R][V], uniforms [R] and out [R] on the device; temperature > 0 and top_p > 0.
int tq_sample_topp_static(const float* logits, int R, int V, float temperature, float top_p, const float* uniforms,
                          int* out, hipStream_t stream);
#ifdef __cplusplus
}
#endif
