// Host-side helpers shared by the C-ABI entry points: status codes, the thread-local
// error message behind nq_last_error(), and launch checking.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/nqhip.h"

namespace nq {

char *error_buffer();   // thread-local, NQ_ERROR_CHARS long (defined in nq_capi.hip)
enum { NQ_ERROR_CHARS = 512 };

inline int fail(int code, const char *format, ...) {
    va_list args;
    va_start(args, format);
    vsnprintf(error_buffer(), NQ_ERROR_CHARS, format, args);
    va_end(args);
    return code;
}

inline int check_launch(const char *what) {
    hipError_t status = hipGetLastError();
    if (status != hipSuccess)
        return fail(NQ_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(status));
    return NQ_OK;
}

inline bool aligned(const void *pointer, size_t bytes) {
    return (reinterpret_cast<uintptr_t>(pointer) % bytes) == 0;
}

}  // namespace nq

#define NQ_REQUIRE(cond, code, ...) \
    do { if (!(cond)) return nq::fail(code, __VA_ARGS__); } while (0)
