// Shared plumbing of the HIP device layer: error reporting and a few device helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdio>
#include <vector>

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

// Per-thread record of kernel execution times (drhip_timing_begin / drhip_timing_end).  While it is
// on, every launch carries its own start and stop event (hipExtLaunchKernelGGL attaches them to the
// dispatch packet), so the span is the kernel alone -- no extra packets between the kernels, which
// is what events recorded between launches would put there.
struct LaunchTimer {
    bool on = false;
    size_t used = 0;                   // events handed out since drhip_timing_begin
    std::vector<hipEvent_t> events;    // [2*i] start, [2*i+1] stop of launch i
};
LaunchTimer& launch_timer();

// Every kernel of this library is launched through here.
template <typename Kernel, typename... Args>
inline void launch(Kernel kernel, dim3 grid, dim3 block, size_t ldsBytes, hipStream_t stream, Args... args) {
    LaunchTimer& t = launch_timer();
    if (!t.on) {
        hipLaunchKernelGGL(kernel, grid, block, ldsBytes, stream, args...);
        return;
    }
    while (t.events.size() < t.used + 2) {
        hipEvent_t e;
        if (hipEventCreate(&e) != hipSuccess) { hipLaunchKernelGGL(kernel, grid, block, ldsBytes, stream, args...); return; }
        t.events.push_back(e);
    }
    hipExtLaunchKernelGGL(kernel, grid, block, ldsBytes, stream, t.events[t.used], t.events[t.used + 1], 0, args...);
    t.used += 2;
}

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Division by a number known at launch time, as a multiplication (Granlund & Montgomery): with
// l = ceil(log2 d) and mul = floor(2^32 (2^l - d) / d) + 1, n / d = (mulhi(n, mul) + n) >> l for every n < 2^31.
// A hardware integer division is some 30 dependent instructions, and in the short kernels of a batch-1 pass
// those in front of a workgroup's first loads are part of every layer's latency (~0.1 us per kernel).
struct FastDiv { unsigned d, mul, shift; };
inline FastDiv make_fastdiv(int d) {                 // d >= 1
    unsigned l = 0;
    while ((1ull << l) < (unsigned long long)d) ++l;
    const unsigned long long m = ((1ull << 32) * ((1ull << l) - (unsigned long long)d)) / (unsigned long long)d + 1;
    return FastDiv{(unsigned)d, (unsigned)m, l};
}
__device__ inline int fast_div(int n, const FastDiv& f) { return (int)((__umulhi((unsigned)n, f.mul) + (unsigned)n) >> f.shift); }

// A layer's results are stored written through (system-scope store: sc0 sc1) instead of being left dirty in the
// XCD's L2: the reader is the next kernel, whose workgroups mostly sit on other XCDs and read from memory anyway,
// and what has been written during the kernel need not be written back when it ends (0.15-0.45 us per launch on
// the 14x14 layers, 1.5 us on a 12.8 MB output).
__device__ inline void store_through(float* p, float v) {
    __hip_atomic_store((unsigned*)p, __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Element `row` of an activation vector that a split GEMV left as partial sums: slices added in
// order, then bias and ReLU -- bit for bit what the GEMV's finishing kernel stores.
__device__ inline float deferred_element(const drhip_deferred_vec& d, int row) {
    const float* pp = d.partials + row;
    float s = 0.0f;
    int sl = 0;
    // 32, 16, then 8 independent loads in flight, always summed in slice order: the partial sums come
    // from other XCDs' workgroups, so every round of loads costs a trip to memory
    for (; sl + 32 <= d.slices; sl += 32) {
        float v[32];
#pragma unroll
        for (int u = 0; u < 32; ++u) v[u] = pp[(size_t)(sl + u) * d.n];
#pragma unroll
        for (int u = 0; u < 32; ++u) s += v[u];
    }
    for (; sl + 16 <= d.slices; sl += 16) {         // (a GEMV that fills the chip leaves 16 slices: one round, not two)
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) v[u] = pp[(size_t)(sl + u) * d.n];
#pragma unroll
        for (int u = 0; u < 16; ++u) s += v[u];
    }
    for (; sl < d.slices; sl += 8) {                // the ragged end too: clamped loads, zeros by select
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = pp[(size_t)min(sl + u, d.slices - 1) * d.n];
#pragma unroll
        for (int u = 0; u < 8; ++u) s = (sl + u < d.slices) ? s + v[u] : s;
    }
    if (d.bias) s += d.bias[row];
    if (d.relu) s = fmaxf(s, 0.0f);
    if (d.divisor != 0.0f) s = s / d.divisor;
    return s;
}

// Number of compute units of the active device (cached by drhip_init; 256 on MI355X).
int num_cu();

// Per-device set-up of the fully-connected kernels' built-in scratch (k_fc.hip); `device` must be current.
int fc_static_scratch_setup(int device);

}  // namespace drhip

#define DRHIP_REQUIRE(cond, ...)                                   \
    do {                                                           \
        if (!(cond)) return drhip::fail(DRHIP_EINVAL, __VA_ARGS__); \
    } while (0)
