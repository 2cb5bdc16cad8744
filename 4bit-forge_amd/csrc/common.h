// Shared host-side helpers for libforge_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include "../../include/forge_hip.h"

namespace forge {

// Thread-local message returned by forge_last_error().
char* error_buffer();
int fail(int code, const char* fmt, ...);

#define FORGE_REQUIRE(cond, ...)                                     \
    do {                                                             \
        if (!(cond)) return ::forge::fail(FORGE_ERR_INVALID, __VA_ARGS__); \
    } while (0)

#define FORGE_HIP_CHECK(expr)                                                          \
    do {                                                                               \
        hipError_t _e = (expr);                                                        \
        if (_e != hipSuccess)                                                          \
            return ::forge::fail(FORGE_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(_e)); \
    } while (0)

// Check for a launch-configuration error right after <<<>>>.
#define FORGE_LAUNCH_CHECK() FORGE_HIP_CHECK(hipGetLastError())

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace forge
