// Host-side helpers shared by the C-ABI entry points: argument checks that set the thread-local
// error text, and the launch-status check.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/q8_hip.h"

namespace q8 {

char* last_error_buf();  // thread-local, 256 bytes (defined in api.hip)

inline int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(last_error_buf(), 256, fmt, ap);
    va_end(ap);
    return code;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int launch_status(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(Q8_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return Q8_OK;
}

inline int elem_size(int dt) {
    switch (dt) {
        case Q8_I8: case Q8_E4M3: return 1;
        case Q8_BF16: case Q8_F16: return 2;
        case Q8_F32: return 4;
        default: return 0;
    }
}

}  // namespace q8
