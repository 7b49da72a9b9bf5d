// Softmax over a flat fp32 vector in ONE workgroup of sixteen waves: wavefront-level butterfly
// reductions (ds_bpermute via __shfl_xor) for max and sum, one small LDS exchange between the waves;
// vectors of up to 2048 elements are read once and kept in registers.  (Sixteen waves, not four: a lane then
// finishes one or two logits of a deferred input, and each of them is a round of dependent loads -- 1000 logits
// behind 16 slices: 4.0 against 8.8 us.)
//
// The reference computes exp(x) on the device, downloads the vector, sums it sequentially on the
// host and launches a scale kernel (src/dR_nodes_math.c:620-678).  Mathematically this kernel is
// the same function, exp(x_i)/sum_j exp(x_j); it subtracts max(x) first so that large logits do
// not overflow, and the whole node stays on the device and asynchronous.
#include "drhip_common.hpp"

#include <cfloat>

namespace drhip {

constexpr int kSoftmaxThreads = 1024;
constexpr int kSoftmaxRegs = 2;     // vectors of up to 2048 elements live in registers: one read of x

__device__ inline float wave_max(float v) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ inline float wave_sum(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Workgroup-wide maximum / sum; the result is valid in every lane.  `red` has one slot per wave.
template <bool MAX>
__device__ inline float block_reduce(float v, float* red) {
    constexpr int nwaves = kSoftmaxThreads / kWave;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    v = MAX ? wave_max(v) : wave_sum(v);
    __syncthreads();                    // red may still be read from the previous reduction
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int w = 1; w < nwaves; ++w) r = MAX ? fmaxf(r, red[w]) : r + red[w];
    return r;
}

// xdef.partials != NULL: the logits arrive as the partial sums of the GEMV in front (slices added
// in order, then its bias and ReLU); they are finished first (and stored to xdef.finished when the
// caller wants to read the logits too).
template <bool SMALL>
__global__ void __launch_bounds__(kSoftmaxThreads)
softmax_kernel(const float* x, float* y, int n, drhip_deferred_vec xdef) {     // no __restrict__: x may become y
    __shared__ float red[kSoftmaxThreads / kWave];
    const int tid = threadIdx.x;
    if (SMALL) {                                    // n <= kSoftmaxThreads * kSoftmaxRegs
        float v[kSoftmaxRegs];
#pragma unroll
        for (int u = 0; u < kSoftmaxRegs; ++u) {
            const int i = tid + u * kSoftmaxThreads;
            v[u] = -FLT_MAX;
            if (i < n) v[u] = xdef.partials ? deferred_element(xdef, i) : x[i];
        }
        if (xdef.partials && xdef.finished) {       // (behind all the loads: a store in between would order them)
#pragma unroll
            for (int u = 0; u < kSoftmaxRegs; ++u) {
                const int i = tid + u * kSoftmaxThreads;
                if (i < n) xdef.finished[i] = v[u];
            }
        }
        float m = -FLT_MAX;
#pragma unroll
        for (int u = 0; u < kSoftmaxRegs; ++u) m = fmaxf(m, v[u]);
        m = block_reduce<true>(m, red);
        float s = 0.0f;
#pragma unroll
        for (int u = 0; u < kSoftmaxRegs; ++u) {
            v[u] = (tid + u * kSoftmaxThreads < n) ? expf(v[u] - m) : 0.0f;
            s += v[u];
        }
        const float inv = 1.0f / block_reduce<false>(s, red);
#pragma unroll
        for (int u = 0; u < kSoftmaxRegs; ++u) {
            const int i = tid + u * kSoftmaxThreads;
            if (i < n) store_through(y + i, v[u] * inv);
        }
        return;
    }
    if (xdef.partials) {
        for (int i = tid; i < n; i += kSoftmaxThreads) {
            const float s = deferred_element(xdef, i);
            y[i] = s;                           // every lane re-reads only the elements it wrote itself
            if (xdef.finished) xdef.finished[i] = s;
        }
        x = y;
    }
    float m = -FLT_MAX;
    for (int i = tid; i < n; i += kSoftmaxThreads) m = fmaxf(m, x[i]);
    m = block_reduce<true>(m, red);
    float s = 0.0f;
    for (int i = tid; i < n; i += kSoftmaxThreads) s += expf(x[i] - m);
    const float inv = 1.0f / block_reduce<false>(s, red);
    for (int i = tid; i < n; i += kSoftmaxThreads) store_through(y + i, expf(x[i] - m) * inv);
}

}  // namespace drhip

using namespace drhip;

extern "C" int drhip_softmax_ex_f32(const float* x, const drhip_deferred_vec* xdef, float* y, int n, void* stream) {
    DRHIP_REQUIRE((x || xdef) && y, "drhip_softmax_f32: NULL tensor");
    DRHIP_REQUIRE(n > 0, "drhip_softmax_f32: n = %d", n);
    DRHIP_REQUIRE(!xdef || (xdef->partials && xdef->slices > 0 && xdef->n == n), "drhip_softmax_f32: deferred input must carry partial sums of a vector of length %d", n);
    DRHIP_REQUIRE(!xdef || xdef->finished != y, "drhip_softmax_f32: the finished logits and the probabilities need separate arrays");
    const drhip_deferred_vec none = {nullptr, nullptr, 0, 0, 0, nullptr, 0.0f};
    if (n <= kSoftmaxThreads * kSoftmaxRegs)
        launch(softmax_kernel<true>, dim3(1), dim3(kSoftmaxThreads), 0, as_stream(stream), x, y, n, xdef ? *xdef : none);
    else
        launch(softmax_kernel<false>, dim3(1), dim3(kSoftmaxThreads), 0, as_stream(stream), x, y, n, xdef ? *xdef : none);
    return launched("softmax_kernel");
}

extern "C" int drhip_softmax_f32(const float* x, float* y, int n, void* stream) {
    DRHIP_REQUIRE(x, "drhip_softmax_f32: NULL tensor");
    return drhip_softmax_ex_f32(x, nullptr, y, n, stream);
}
