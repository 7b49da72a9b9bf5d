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

// 2x2 and 3x3 windows inside one channel (sz = 1): the same scan, but all samples are fetched
// first, unconditionally and from clamped positions, so a lane pays one trip to memory instead of
// one per sample; samples outside the image become 0.0f by select afterwards.
template <bool MAX, bool ARG, int SX, int SY>
__global__ void __launch_bounds__(256)
pool_small_kernel(const float* __restrict__ in, float* __restrict__ out, int* __restrict__ argmax,
                  int W, int H, int C, int Wo, int Ho, int stx, int sty, int stz) {
    const int total = Wo * Ho * ((C + stz - 1) / stz);
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int xo = idx % Wo, yo = (idx / Wo) % Ho, zo = idx / (Wo * Ho);
    const int x0 = xo * stx, y0 = yo * sty, z = zo * stz;
    const float* pc = in + (size_t)z * H * W;
    float v[SY][SX];
#pragma unroll
    for (int dy = 0; dy < SY; ++dy)
#pragma unroll
        for (int dx = 0; dx < SX; ++dx) v[dy][dx] = pc[min(y0 + dy, H - 1) * W + min(x0 + dx, W - 1)];
    float r = MAX ? -FLT_MAX : 0.0f;
    int where = -1;
#pragma unroll
    for (int dy = 0; dy < SY; ++dy)
#pragma unroll
        for (int dx = 0; dx < SX; ++dx) {
            const bool inside = x0 + dx < W && y0 + dy < H;
            const float s = inside ? v[dy][dx] : 0.0f;
            if (MAX) {
                if (s > r) { r = s; if (ARG) where = inside ? (z * H + y0 + dy) * W + x0 + dx : -1; }
            } else {
                r += s;
            }
        }
    out[idx] = MAX ? r : r / (float)(SX * SY);
    if (MAX && ARG) argmax[idx] = where;
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
    // four samples per lane and round, fetched unconditionally from clamped positions
    for (int e0 = lane; e0 < n; e0 += 256) {
        float v[4]; int flat[4]; bool inside[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int e = e0 + 64 * u;
            const int dx = e % sx, dy = (e / sx) % sy, dz = e / (sx * sy);
            const int x = x0 + dx, y = y0 + dy, z = z0 + dz;
            inside[u] = e < n && x < W && y < H && z < C;
            flat[u] = (z * H + y) * W + x;
            v[u] = in[(min(z, C - 1) * H + min(y, H - 1)) * W + min(x, W - 1)];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int e = e0 + 64 * u;
            if (e < n) {
                const float s = inside[u] ? v[u] : 0.0f;
                if (MAX) {
                    if (s > r) { r = s; pos = e; where = inside[u] ? flat[u] : -1; }
                } else {
                    r += s;
                }
            }
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
    if (sz == 1 && sx == sy && (sx == 2 || sx == 3)) {
        const dim3 g((unsigned)((total + block - 1) / block)), b(block);
        int* none = nullptr;
#define DRHIP_POOL_SMALL(MAXV, ARGV, S, ARGP) launch((pool_small_kernel<MAXV, ARGV, S, S>), g, b, 0, s, in, out, ARGP, W, H, C, Wo, Ho, stx, sty, stz)
        if (sx == 2) {
            if (type == 0 && argmax_out) DRHIP_POOL_SMALL(true, true, 2, argmax_out);
            else if (type == 0) DRHIP_POOL_SMALL(true, false, 2, none);
            else DRHIP_POOL_SMALL(false, false, 2, none);
        } else {
            if (type == 0 && argmax_out) DRHIP_POOL_SMALL(true, true, 3, argmax_out);
            else if (type == 0) DRHIP_POOL_SMALL(true, false, 3, none);
            else DRHIP_POOL_SMALL(false, false, 3, none);
        }
#undef DRHIP_POOL_SMALL
        return launched("pool_small_kernel");
    }
    if (type == 0 && argmax_out)
        launch((pool_kernel<true, true>), dim3(blocks), dim3(block), 0, s, in, out, argmax_out, W, H, C, Wo, Ho, Co, sx, sy, sz, stx, sty, stz);
    else if (type == 0)
        launch((pool_kernel<true, false>), dim3(blocks), dim3(block), 0, s, in, out, (int*)nullptr, W, H, C, Wo, Ho, Co, sx, sy, sz, stx, sty, stz);
    else
        launch((pool_kernel<false, false>), dim3(blocks), dim3(block), 0, s, in, out, (int*)nullptr, W, H, C, Wo, Ho, Co, sx, sy, sz, stx, sty, stz);
    return launched("pool_kernel");
}
