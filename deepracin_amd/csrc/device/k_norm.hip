// Normalization of a whole tensor to a target mean and/or standard deviation:
//
//   mean = sum(x) / n,   dev = sqrt(sum((x - mean)^2) / n)      over all n = W*H*C elements
//   type 0 (mean):      y = x + (targetMean - mean)
//   type 1 (dev):       y = x * (targetDev / dev)
//   type 2 (mean, dev): y = (x + (targetMean - mean)) * (targetDev / dev)
//
// Reference: src/dR_nodes_misc.c:1163-1446 -- tree reductions in 16x8 work-groups per channel
// (`getAvg`, `getSumDev`, Kernels/dR_helper.cl:315-471), repeated until one value per channel is left,
// a blocking download and a host loop over the channels after each of the two reductions, then
// `addScalar` / `mulScalar` / `addMulScalar` (Kernels/dR_math.cl:100-144).  The deviation is taken
// about the mean for type 1 as well (the reference computes the average for all three types).
//
// Here the node stays on the device and asynchronous (HBM-bound, 4n bytes read per reduction plus
// 8n for the last sweep): a grid of at most 1024 workgroups leaves one partial sum each, and the
// kernel that needs the total adds those partials itself, every workgroup in the same fixed order,
// so no host round trip, no atomics and no device-scope fence are needed and the result is
// reproducible run to run.  The summation order differs from the reference's trees (~1e-7 relative).
#include "drhip_common.hpp"

namespace drhip {

constexpr int kNormThreads = 256;
constexpr int kNormMaxBlocks = 1024;

typedef float nf32x4 __attribute__((ext_vector_type(4)));

__device__ inline float norm_wave_sum(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Sum over the workgroup; the result is valid in every lane.
__device__ inline float norm_block_sum(float v, float* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    v = norm_wave_sum(v);
    __syncthreads();                    // red may still be read from a previous call
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < kNormThreads / kWave; ++w) s += red[w];
    return s;
}

// Total of the `count` per-workgroup partials, added in index order by every caller alike.
__device__ inline float norm_total(const float* __restrict__ partials, int count, float* red) {
    float v = 0.0f;
    for (int i = threadIdx.x; i < count; i += kNormThreads) v += partials[i];
    return norm_block_sum(v, red);
}

// partialsOut[block] = sum over the block's elements of x (DEV == false) or (x - mean)^2 (DEV == true),
// mean = total(sumPartials) / n.
template <bool DEV>
__global__ void __launch_bounds__(kNormThreads)
norm_partial_kernel(const float* __restrict__ x, const float* __restrict__ sumPartials, float* __restrict__ partialsOut,
                    size_t n, int blocks) {
    __shared__ float red[kNormThreads / kWave];
    float mean = 0.0f;
    if (DEV) mean = norm_total(sumPartials, blocks, red) / (float)n;
    const size_t n4 = n / 4;
    float s = 0.0f;
    for (size_t i = (size_t)blockIdx.x * kNormThreads + threadIdx.x; i < n4; i += (size_t)gridDim.x * kNormThreads) {
        const nf32x4 v = ((const nf32x4*)x)[i];
#pragma unroll
        for (int k = 0; k < 4; ++k) { const float d = v[k] - mean; s += DEV ? d * d : v[k]; }
    }
    if (blockIdx.x == 0)
        for (size_t i = n4 * 4 + threadIdx.x; i < n; i += kNormThreads) { const float d = x[i] - mean; s += DEV ? d * d : x[i]; }
    s = norm_block_sum(s, red);
    if (threadIdx.x == 0) partialsOut[blockIdx.x] = s;
}

__global__ void __launch_bounds__(kNormThreads)
norm_apply_kernel(const float* __restrict__ x, float* __restrict__ y, const float* __restrict__ sumPartials,
                  const float* __restrict__ devPartials, size_t n, int blocks, int type, float targetMean, float targetDev) {
    __shared__ float red[kNormThreads / kWave];
    const float mean = norm_total(sumPartials, blocks, red) / (float)n;
    float add = 0.0f, mul = 1.0f;
    if (type != 1) add = -(mean - targetMean);
    if (type != 0) {
        const float dev = sqrtf(norm_total(devPartials, blocks, red) / (float)n);
        mul = 1.0f / (dev / targetDev);
    }
    const size_t n4 = n / 4;
    for (size_t i = (size_t)blockIdx.x * kNormThreads + threadIdx.x; i < n4; i += (size_t)gridDim.x * kNormThreads) {
        nf32x4 v = ((const nf32x4*)x)[i];
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = (v[k] + add) * mul;
        ((nf32x4*)y)[i] = v;
    }
    if (blockIdx.x == 0)
        for (size_t i = n4 * 4 + threadIdx.x; i < n; i += kNormThreads) y[i] = (x[i] + add) * mul;
}

static int norm_blocks(size_t n) {
    size_t b = (n / 4 + kNormThreads - 1) / kNormThreads;
    if (b < 1) b = 1;
    return (int)(b > (size_t)kNormMaxBlocks ? kNormMaxBlocks : b);
}

}  // namespace drhip

using namespace drhip;

extern "C" size_t drhip_normalize_scratch_floats(size_t n) { return n ? 2 * (size_t)norm_blocks(n) : 0; }

extern "C" int drhip_normalize_f32(const float* x, float* y, size_t n, int type, float targetMean, float targetDev,
                                   float* scratch, void* stream) {
    DRHIP_REQUIRE(x && y && scratch, "drhip_normalize_f32: NULL pointer");
    DRHIP_REQUIRE(n > 0, "drhip_normalize_f32: empty tensor");
    DRHIP_REQUIRE(type >= 0 && type <= 2, "drhip_normalize_f32: unknown normalization type %d (0 mean, 1 deviation, 2 both)", type);
    DRHIP_REQUIRE((((size_t)x | (size_t)y) & 15) == 0, "drhip_normalize_f32: tensors must be 16-byte aligned");
    const int blocks = norm_blocks(n);
    float* sums = scratch;
    float* devs = scratch + blocks;
    hipStream_t s = as_stream(stream);
    launch((norm_partial_kernel<false>), dim3(blocks), dim3(kNormThreads), 0, s, x, (const float*)sums, sums, n, blocks);
    if (int rc = launched("norm_partial_kernel")) return rc;
    if (type != 0) {
        launch((norm_partial_kernel<true>), dim3(blocks), dim3(kNormThreads), 0, s, x, (const float*)sums, devs, n, blocks);
        if (int rc = launched("norm_partial_kernel")) return rc;
    }
    launch(norm_apply_kernel, dim3(blocks), dim3(kNormThreads), 0, s, x, y, (const float*)sums, (const float*)devs, n, blocks,
           type, targetMean, targetDev);
    return launched("norm_apply_kernel");
}
