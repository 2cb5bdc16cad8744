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

// Library-wide settings (forge_set_option / forge_get_option in forge_hip.h).  Each starts from
// an environment variable read ONCE, when the library is loaded; after that only
// forge_set_option changes it.  Reading one is a relaxed atomic load.
enum Option {
    OPT_SWEEP_SCHEDULE = 0,    // 0 = by tile count, 1 = left-looking, 2 = right-looking
    OPT_FP32_BLOCKED_SUM = 1,  // 1 = blocked sums stay on the fp32 matrix instruction
    OPT_SWEEP_PRODUCTS = 2,    // piece products per fp32 product in the direct sweep's updates
    OPT_FACTOR_PIECES = 3,     // 0 = fp16 halves where the operand bound is known, 1 = bf16 thirds
    OPT_MSE_REFERENCE_QUANTISER = 4,   // 1 = the shrink search rounds fma(x, 1/s, zero) as the reference does
    OPT_COUNT
};
int64_t option(Option o);

// Optional per-kernel timing (forge_kernel_timing_* in forge_hip.h).  When enabled, a
// KernelTiming object brackets one launch with two HIP events on the launch stream and
// files the pair under `name` together with the launch's algorithmic work (flops or HBM
// bytes).  Disabled (the default) it does nothing.
enum WorkKind { WORK_FLOPS = 0, WORK_BYTES = 1 };
class KernelTiming {
public:
    KernelTiming(const char* name, hipStream_t st, double work, WorkKind kind);
    ~KernelTiming();
    KernelTiming(const KernelTiming&) = delete;
    KernelTiming& operator=(const KernelTiming&) = delete;
private:
    int slot_;
    hipStream_t st_;
};

}  // namespace forge
