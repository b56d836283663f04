// Shared host-side helpers of the swin3d_amd C-ABI library (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/swin3d_amd.h"

namespace s3d {

// Thread-local description of the last failure; read by s3d_last_error_string().
char *error_buffer();
constexpr int kErrorBufferBytes = 512;

inline int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), kErrorBufferBytes, fmt, ap);
    va_end(ap);
    return code;
}

inline int hip_fail(hipError_t e, const char *what)
{
    return fail(static_cast<int>(e), "%s: %s", what, hipGetErrorString(e));
}

#define S3D_HIP_CHECK(expr)                                         \
    do {                                                            \
        hipError_t _e = (expr);                                     \
        if (_e != hipSuccess) return ::s3d::hip_fail(_e, #expr);    \
    } while (0)

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline size_t align_up(size_t a, size_t b) { return (a + b - 1) / b * b; }

}  // namespace s3d
