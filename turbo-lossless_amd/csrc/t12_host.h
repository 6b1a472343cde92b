// Host-side helpers of libturbo12: error reporting and launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include "t12_abi.h"

void t12_set_error(const char* fmt, ...);

#define T12_REQUIRE(cond, ...)                                      \
    do {                                                            \
        if (!(cond)) { t12_set_error(__VA_ARGS__); return T12_EINVAL; } \
    } while (0)

// hipGetLastError after a launch: a bad configuration is reported here, not
// at the next unrelated call.
#define T12_CHECK_LAUNCH(what)                                                        \
    do {                                                                              \
        hipError_t e_ = hipGetLastError();                                            \
        if (e_ != hipSuccess) {                                                       \
            t12_set_error("%s: %s", (what), hipGetErrorString(e_));                   \
            return T12_ELAUNCH;                                                       \
        }                                                                             \
    } while (0)
