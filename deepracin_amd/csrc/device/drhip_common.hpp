// Shared plumbing of the HIP device layer: error reporting and a few device helpers.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>

#include "dr_hip.h"

namespace drhip {

// Per-thread message of the last failure, returned by drhip_last_error().
char* error_slot();

inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_slot(), 512, fmt, ap);
    va_end(ap);
    return code;
}

inline int check(hipError_t e, const char* what) {
    if (e == hipSuccess) return DRHIP_OK;
    return fail(DRHIP_EDEVICE, "%s: %s", what, hipGetErrorString(e));
}

// Reports a launch-time error (bad configuration) right after a kernel launch.
inline int launched(const char* kernel) { return check(hipGetLastError(), kernel); }

inline hipStream_t as_stream(void* s) { return (hipStream_t)s; }

constexpr int kWave = 64;   // CDNA wavefront width

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Number of compute units of the active device (cached by drhip_init; 256 on MI355X).
int num_cu();

}  // namespace drhip

#define DRHIP_REQUIRE(cond, ...)                                   \
    do {                                                           \
        if (!(cond)) return drhip::fail(DRHIP_EINVAL, __VA_ARGS__); \
    } while (0)
