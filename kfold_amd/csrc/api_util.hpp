// Helpers shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/kfold_hip.h"

namespace kfh {

// one message buffer per thread for the whole library
inline thread_local char g_err[512] = "";

inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

// Report a launch failure of the kernels enqueued since the last check.
inline int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(KFH_EHIP, "%s: %s", what, hipGetErrorString(e));
    return KFH_OK;
}

inline size_t align_up(size_t x, size_t a = 256) { return (x + a - 1) / a * a; }
inline bool dtype_ok(int t) { return t == KFH_BF16 || t == KFH_F32; }

}  // namespace kfh
