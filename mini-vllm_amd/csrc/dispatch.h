// Run-time dtype code -> template type. A library is built for one activation type
// (MV_WITH_F32 or MV_WITH_BF16, or both); asking it for the other is an error, never a
// silent conversion.
#pragma once
#include "common.h"

#ifdef MV_WITH_F32
#define MV_CASE_F32(...) \
    case MV_F32: {       \
        using T = float; \
        __VA_ARGS__;     \
        break;           \
    }
#else
#define MV_CASE_F32(...)
#endif

#ifdef MV_WITH_BF16
#define MV_CASE_BF16(...) \
    case MV_BF16: {       \
        using T = bf16;   \
        __VA_ARGS__;      \
        break;            \
    }
#else
#define MV_CASE_BF16(...)
#endif

// Activation type T from `dtype`.
#define MV_DISPATCH_T(dtype, what, ...)                                                        \
    switch (dtype) {                                                                           \
        MV_CASE_F32(__VA_ARGS__)                                                               \
        MV_CASE_BF16(__VA_ARGS__)                                                              \
        default:                                                                               \
            return mv_fail("%s: this library was not built for activation dtype code %d", what, \
                           (int)(dtype));                                                      \
    }

static inline bool mv_valid_dtype(int d) { return d == MV_F32 || d == MV_BF16; }
static inline size_t mv_dtype_size(int d) { return d == MV_F32 ? 4 : 2; }
