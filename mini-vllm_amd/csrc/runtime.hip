// Host-side support of the C entry points: the error channel and a few queries.
#include "common.h"
#include <string.h>

static thread_local char g_error[512] = "";

extern "C" const char* mv_last_error() { return g_error; }

int mv_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return 1;
}

int mv_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mv_fail("%s: launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

// Bit mask of the activation types this library was built for (bit 0 float, bit 1 bf16).
extern "C" int mv_built_dtypes() {
    int m = 0;
#ifdef MV_WITH_F32
    m |= 1;
#endif
#ifdef MV_WITH_BF16
    m |= 2;
#endif
    return m;
}

extern "C" int mv_abi_version() { return 1; }
