// Max / average pooling for [C][H][W] fp32 tensors (HBM/L2-bandwidth bound; 4*(in+out) bytes).
//
// Semantics of the reference's generated kernel (src/dR_nodes_pooling.c:277-401):
//   out dims = ceil(in/stride); window anchored at (x*stx, y*sty, z*stz), no leading pad;
//   a sample whose x or y lies outside the image reads 0.0f (sampleZeroPaddedFloat,
//   Kernels/dR_helper.cl:15-28); max starts from -FLT_MAX and scans z, y, x ascending;
//   average = sum / (sx*sy*sz).
// The reference does not bound-check z; a window that hangs over the last channel reads the
// neighbouring memory there.  Here such samples read 0.0f as well.
//
// Small windows (2x2, 3x3): one lane per output element, x fastest, so a wavefront reads
// stride-separated but line-local addresses and writes 256 contiguous bytes; the scan order and
// therefore every bit of the result equal the reference's.
// Large windows (64 samples and more, e.g. the 14x14 global average of SqueezeNet): one wavefront
// per output element, lanes stride over the window and a butterfly reduction combines them.  The
// maximum (and the position of its first occurrence in scan order) is still exact; an average is
// summed in a different order than the reference's sequential loop (relative difference ~1e-7).
#include "drhip_common.hpp"

#include <cfloat>

namespace drhip {

template <bool MAX, bool ARG>
__global__ void __launch_bounds__(256)
pool_kernel(const float* __restrict__ in, float* __restrict__ out, int* __restrict__ argmax,
            int W, int H, int C, int Wo, int Ho, int Co,
            int sx, int sy, int sz, int stx, int sty, int stz) {
    const int total = Wo * Ho * Co;
    for (int idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        const int xo = idx % Wo;
        const int yo = (idx / Wo) % Ho;
        const int zo = idx / (Wo * Ho);
        const int x0 = xo * stx, y0 = yo * sty, z0 = zo * stz;
        float r = MAX ? -FLT_MAX : 0.0f;
        int where = -1;
        for (int dz = 0; dz < sz; ++dz) {
            const int z = z0 + dz;
            for (int dy = 0; dy < sy; ++dy) {
                const int y = y0 + dy;
                for (int dx = 0; dx < sx; ++dx) {
                    const int x = x0 + dx;
                    const bool inside = x < W && y < H && z < C;
                    const int flat = (z * H + y) * W + x;
                    const float v = inside ? in[flat] : 0.0f;
                    if (MAX) {
                        if (v > r) { r = v; if (ARG) where = inside ? flat : -1; }
                    } else {
                        r += v;
                    }
                }
            }
        }
        out[idx] = MAX ? r : r / (float)(sx * sy * sz);
        if (MAX && ARG) argmax[idx] = where;
    }
}

template <bool MAX, bool ARG>
__global__ void __launch_bounds__(256)
pool_wave_kernel(const float* __restrict__ in, float* __restrict__ out, int* __restrict__ argmax,
                 int W, int H, int C, int Wo, int Ho, int Co,
                 int sx, int sy, int sz, int stx, int sty, int stz) {
    const int total = Wo * Ho * Co, n = sx * sy * sz;
    const int lane = threadIdx.x & 63;
    const int idx = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);     // one wavefront per output
    if (idx >= total) return;
    const int xo = idx % Wo, yo = (idx / Wo) % Ho, zo = idx / (Wo * Ho);
    const int x0 = xo * stx, y0 = yo * sty, z0 = zo * stz;
    float r = MAX ? -FLT_MAX : 0.0f;
    int pos = 0x7fffffff, where = -1;                // scan position and flat index of the running maximum
    for (int e = lane; e < n; e += 64) {
        const int dx = e % sx, dy = (e / sx) % sy, dz = e / (sx * sy);
        const int x = x0 + dx, y = y0 + dy, z = z0 + dz;
        const bool inside = x < W && y < H && z < C;
        const int flat = (z * H + y) * W + x;
        const float v = inside ? in[flat] : 0.0f;
        if (MAX) {
            if (v > r) { r = v; pos = e; where = inside ? flat : -1; }
        } else {
            r += v;
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float ro = __shfl_xor(r, m);
        if (MAX) {
            const int po = __shfl_xor(pos, m), wo = __shfl_xor(where, m);
            if (ro > r || (ro == r && po < pos)) { r = ro; pos = po; where = wo; }   // first occurrence wins ties
        } else {
            r += ro;
        }
    }
    if (lane == 0) {
        out[idx] = MAX ? r : r / (float)n;
        if (MAX && ARG) argmax[idx] = where;
    }
}

}  // namespace drhip

using namespace drhip;

extern "C" int drhip_pool_f32(const float* in, float* out, int* argmax_out,
                              int W, int H, int C, int sx, int sy, int sz, int stx, int sty, int stz,
                              int type, void* stream) {
    DRHIP_REQUIRE(in && out, "drhip_pool_f32: NULL tensor");
    DRHIP_REQUIRE(W > 0 && H > 0 && C > 0, "drhip_pool_f32: bad input shape %dx%dx%d", W, H, C);
    DRHIP_REQUIRE(sx > 0 && sy > 0 && sz > 0 && stx > 0 && sty > 0 && stz > 0, "drhip_pool_f32: window and stride must be positive");
    DRHIP_REQUIRE(type == 0 || type == 1, "drhip_pool_f32: pooling type %d not implemented (0 max, 1 average)", type);
    DRHIP_REQUIRE(!(argmax_out && type != 0), "drhip_pool_f32: argmax output only exists for max pooling");
    const int Wo = ceil_div(W, stx), Ho = ceil_div(H, sty), Co = ceil_div(C, stz);
    const long long total = (long long)Wo * Ho * Co;
    DRHIP_REQUIRE(total < (1ll << 31) && (long long)W * H * C < (1ll << 31), "drhip_pool_f32: tensor too large for 32-bit indexing");
    const int block = 256;
    int blocks = (int)((total + block - 1) / block);
    if (blocks > 16 * num_cu()) blocks = 16 * num_cu();
    hipStream_t s = as_stream(stream);
    if (sx * sy * sz >= 64) {                        // one wavefront per output element
        const int wblocks = (int)((total + 3) / 4);
        if (type == 0 && argmax_out)
            launch((pool_wave_kernel<true, true>), dim3(wblocks), dim3(block), 0, s, in, out, argmax_out, W, H, C, Wo, Ho, Co, sx, sy, sz, stx, sty, stz);
        else if (type == 0)
            launch((pool_wave_kernel<true, false>), dim3(wblocks), dim3(block), 0, s, in, out, (int*)nullptr, W, H, C, Wo, Ho, Co, sx, sy, sz, stx, sty, stz);
        else
            launch((pool_wave_kernel<false, false>), dim3(wblocks), dim3(block), 0, s, in, out, (int*)nullptr, W, H, C, Wo, Ho, Co, sx, sy, sz, stx, sty, stz);
        return launched("pool_wave_kernel");
    }
    if (type == 0 && argmax_out)
        launch((pool_kernel<true, true>), dim3(blocks), dim3(block), 0, s, in, out, argmax_out, W, H, C, Wo, Ho, Co, sx, sy, sz, stx, sty, stz);
    else if (type == 0)
        launch((pool_kernel<true, false>), dim3(blocks), dim3(block), 0, s, in, out, (int*)nullptr, W, H, C, Wo, Ho, Co, sx, sy, sz, stx, sty, stz);
    else
        launch((pool_kernel<false, false>), dim3(blocks), dim3(block), 0, s, in, out, (int*)nullptr, W, H, C, Wo, Ho, Co, sx, sy, sz, stx, sty, stz);
    return launched("pool_kernel");
}
