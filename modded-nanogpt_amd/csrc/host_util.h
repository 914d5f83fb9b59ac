// Host-side helpers shared by the C-ABI entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include "../../include/ngpt_fp8.h"

namespace ngpt {

char* last_error_buf();

inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(last_error_buf(), 512, fmt, ap);
    va_end(ap);
    return code;
}

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail((int)e, "%s: %s", what, hipGetErrorString(e));
    return NGPT_OK;
}

// Compute units of the current device (cached per process; one GPU per process by design).
int num_cus();

// Allow a kernel to use `bytes` of dynamic LDS (needed above 64 KiB); cached per kernel.
template <class K>
inline int allow_lds(K kernel, int bytes) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute(%d B LDS): %s", bytes, hipGetErrorString(e));
    return NGPT_OK;
}

inline int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

}  // namespace ngpt
