// Build configuration of the host-side runtime that mirrors the slice of ncnn's public API
// the int8 path touches (ncnn generates this header from src/platform.h.in with cmake; here
// the switches are fixed: strings, stdio, int8, weight quantisation and batch on, Vulkan off).
#ifndef NCNN_PLATFORM_H
#define NCNN_PLATFORM_H

#include <stdio.h>

#define NCNN_STDIO 1
#define NCNN_STRING 1
#define NCNN_INT8 1
#define NCNN_WEIGHT_QUANT 1
#define NCNN_BATCH 1
#define NCNN_VULKAN 0

#define NCNN_EXPORT __attribute__((visibility("default")))
#define NCNN_FORCEINLINE inline __attribute__((always_inline))

// same diagnostic macro name as ncnn (src/platform.h.in:466-475)
#define NCNN_LOGE(...)                \
    do                                \
    {                                 \
        fprintf(stderr, __VA_ARGS__); \
        fprintf(stderr, "\n");        \
    } while (0)

#define NCNN_MALLOC_ALIGN 64
#define NCNN_MALLOC_OVERREAD 64

#endif // NCNN_PLATFORM_H
