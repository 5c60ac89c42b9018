// Plain bfloat16 products through the vendor's matrix library; see vendor.cpp.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TQ_VENDOR_WORKSPACE (76u << 20)      /* bytes a call may use beside its operands */

#ifdef __cplusplus
extern "C" {
#endif
int tq_vendor_available(void);
int tq_vendor_takes(int M, int N, int K, int64_t lda, int out_is_bf16);
int tq_vendor_product(const void* a, int64_t lda, const void* w, void* out, int out_is_bf16, int M, int N, int K,
                      void* workspace, hipStream_t st);
#ifdef __cplusplus
}
#endif
