// Host-side plumbing shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/lowp.h"

namespace lowp {

// thread-local message buffer behind lp_last_error()
char *error_buffer();
constexpr int kErrorBufferSize = 512;

inline int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), kErrorBufferSize, fmt, ap);
    va_end(ap);
    return code;
}

inline int check_launch(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(LP_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
    return LP_OK;
}

inline bool is_scale_dtype(int d) { return d == LP_F32 || d == LP_BF16 || d == LP_E8M0; }

inline int dtype_size(int d)
{
    switch (d) {
    case LP_F32: return 4;
    case LP_BF16: return 2;
    case LP_E8M0: return 1;
    case LP_E4M3: return 1;
    default: return 0;
    }
}

}  // namespace lowp

#define LP_REQUIRE(cond, ...)                                         \
    do {                                                              \
        if (!(cond)) return lowp::fail(LP_ERR_INVALID, __VA_ARGS__);  \
    } while (0)
