// What the host code shares with the kernels' sources without taking their device code in.
#pragma once
#include <stdint.h>

#define TQ_F32 0
#define TQ_BF16 1
#ifndef TQ_ERR_BAD_ARG
#define TQ_ERR_BAD_ARG (-1)
#define TQ_ERR_UNSUPPORTED (-2)
#endif

#if defined(TQ_ACT_BF16)
#define TQ_ACT_BYTES 2
#define TQ_ACT_TYPE TQ_BF16
#elif defined(TQ_ACT_F32)
#define TQ_ACT_BYTES 4
#define TQ_ACT_TYPE TQ_F32
#else
#error "define TQ_ACT_BF16 or TQ_ACT_F32"
#endif
