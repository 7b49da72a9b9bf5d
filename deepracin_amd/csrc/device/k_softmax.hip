// Softmax over a flat fp32 vector in ONE workgroup: wavefront-level butterfly reductions
// (ds_bpermute via __shfl_xor) for max and sum, one small LDS exchange between the waves.
//
// The reference computes exp(x) on the device, downloads the vector, sums it sequentially on the
// host and launches a scale kernel (src/dR_nodes_math.c:620-678).  Mathematically this kernel is
// the same function, exp(x_i)/sum_j exp(x_j); it subtracts max(x) first so that large logits do
// not overflow, and the whole node stays on the device and asynchronous.
#include "drhip_common.hpp"

#include <cfloat>

namespace drhip {

constexpr int kSoftmaxThreads = 1024;

__device__ inline float wave_max(float v) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ inline float wave_sum(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// xdef.partials != NULL: the logits arrive as the partial sums of the GEMV in front (slices added
// in order, then its bias and ReLU); they are finished into y first (and into xdef.finished, when
// the caller wants to read the logits too), which then serves as x.
__global__ void __launch_bounds__(kSoftmaxThreads)
softmax_kernel(const float* x, drhip_deferred_vec xdef, float* y, int n) {     // no __restrict__: x may become y
    __shared__ float red[kSoftmaxThreads / kWave];
    __shared__ float bcast;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int nwaves = kSoftmaxThreads / kWave;
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
    m = wave_max(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
    if (wave == 0) {
        float v = lane < nwaves ? red[lane] : -FLT_MAX;
        v = wave_max(v);
        if (lane == 0) bcast = v;
    }
    __syncthreads();
    m = bcast;

    float s = 0.0f;
    for (int i = tid; i < n; i += kSoftmaxThreads) s += expf(x[i] - m);
    s = wave_sum(s);
    __syncthreads();            // everyone has read bcast / red from the first round
    if (lane == 0) red[wave] = s;
    __syncthreads();
    if (wave == 0) {
        float v = lane < nwaves ? red[lane] : 0.0f;
        v = wave_sum(v);
        if (lane == 0) bcast = 1.0f / v;
    }
    __syncthreads();
    const float inv = bcast;
    for (int i = tid; i < n; i += kSoftmaxThreads) y[i] = expf(x[i] - m) * inv;
}

}  // namespace drhip

using namespace drhip;

extern "C" int drhip_softmax_ex_f32(const float* x, const drhip_deferred_vec* xdef, float* y, int n, void* stream) {
    DRHIP_REQUIRE((x || xdef) && y, "drhip_softmax_f32: NULL tensor");
    DRHIP_REQUIRE(n > 0, "drhip_softmax_f32: n = %d", n);
    DRHIP_REQUIRE(!xdef || (xdef->partials && xdef->slices > 0 && xdef->n == n), "drhip_softmax_f32: deferred input must carry partial sums of a vector of length %d", n);
    DRHIP_REQUIRE(!xdef || xdef->finished != y, "drhip_softmax_f32: the finished logits and the probabilities need separate arrays");
    const drhip_deferred_vec none = {nullptr, nullptr, 0, 0, 0, nullptr};
    launch(softmax_kernel, dim3(1), dim3(kSoftmaxThreads), 0, as_stream(stream), x, xdef ? *xdef : none, y, n);
    return launched("softmax_kernel");
}

extern "C" int drhip_softmax_f32(const float* x, float* y, int n, void* stream) {
    DRHIP_REQUIRE(x, "drhip_softmax_f32: NULL tensor");
    return drhip_softmax_ex_f32(x, nullptr, y, n, stream);
}
