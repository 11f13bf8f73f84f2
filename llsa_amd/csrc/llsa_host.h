// Host-side helpers of the C ABI: thread-local error string and argument checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

namespace llsa {

char* error_buffer();          // thread-local, 512 bytes (defined in api.hip)

inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

inline int launch_status(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(-100, "%s: launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool stride_ok(int64_t s) { return (s % 8) == 0; }   // bf16 rows start 16-byte aligned

}  // namespace llsa

#define LLSA_REQUIRE(cond, ...)                          \
    do {                                                 \
        if (!(cond)) return llsa::fail(-1, __VA_ARGS__); \
    } while (0)
