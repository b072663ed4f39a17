// Internal helpers shared by the translation units that implement the thorhip C ABI.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <string>

namespace thorhip {

// Thread-local last-error slot behind thorhip_last_error().
std::string& lastError();

inline int fail(int code, const char* fmt, ...) {
    char buffer[2048];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buffer, sizeof buffer, fmt, ap);
    va_end(ap);
    lastError() = buffer;
    return code;
}

inline int hipFail(hipError_t err, const char* what, const char* file, int line) {
    // hipGetLastError clears the sticky per-thread error so one failure is not reported twice.
    (void)hipGetLastError();
    return fail(-(int)err - 1000, "%s failed: %s (%s) at %s:%d", what, hipGetErrorName(err), hipGetErrorString(err), file, line);
}

}  // namespace thorhip

#define THORHIP_TRY(expr)                                                         \
    do {                                                                          \
        hipError_t thorhip_err__ = (expr);                                        \
        if (thorhip_err__ != hipSuccess) {                                        \
            return ::thorhip::hipFail(thorhip_err__, #expr, __FILE__, __LINE__);  \
        }                                                                         \
    } while (0)

#define THORHIP_REQUIRE(cond, ...)                      \
    do {                                                \
        if (!(cond)) {                                  \
            return ::thorhip::fail(-1, __VA_ARGS__);    \
        }                                               \
    } while (0)
