// Direct 2-D correlation for [C][H][W] fp32 tensors: any odd kw x kh, any stride, zero padding,
// fused bias + ReLU.  This is the kernel for everything that is neither 3x3/stride-1 (Winograd)
// nor 1x1 (GEMM): SqueezeNet conv1 (3x3 stride 2, I=3), and the "direct" variant of a 3x3 layer.
//
//   out[o,y,x] = act(b[o] + sum_c sum_j sum_i in[c, y*sy + j - kh/2, x*sx + i - kw/2] * w[c][o][j][i])
//
// The reference generates one OpenCL kernel per layer which accumulates every input channel into
// GLOBAL memory (read-modify-write per (c,o), src/dR_nodes_conv2d.c:574-668) and ignores the stride.
// Here the accumulators live in registers for the whole channel loop, and the stride is honoured
// as documented in the reference header (include/dR_nodes_conv2d.h:47-54).
//
// Mapping: a workgroup of 256 lanes owns a 16x16 tile of output pixels and OCT output channels;
// one lane = one pixel x OCT accumulators.  Input channels are processed CC at a time: the
// zero-padded input patch of the tile and the OCT filters of those channels are staged in LDS
// (filters re-laid [c][tap][oc] so that a lane fetches its OCT weights of a tap with 128-bit
// broadcast reads), then every lane runs kw*kh*OCT FMAs per channel out of LDS.
#include "drhip_common.hpp"

namespace drhip {

constexpr int kDirTile = 16;            // output tile edge
constexpr int kDirThreads = kDirTile * kDirTile;
constexpr int kDirMaxLdsFloats = 15 * 1024;  // 60 KiB

template <int OCT, int KW, int KH>      // KW == 0: runtime filter size
__global__ void __launch_bounds__(kDirThreads)
conv_direct_kernel(const float* __restrict__ in, const float* __restrict__ w, const float* __restrict__ bias,
                   float* __restrict__ out, int W, int H, int I, int O, int Wo, int Ho,
                   int kw_rt, int kh_rt, int sx, int sy, int CC, int tilesX, int relu) {
    extern __shared__ float lds[];
    const int kw = KW ? KW : kw_rt, kh = KH ? KH : kh_rt;
    const int taps = kw * kh;
    const int patchW = (kDirTile - 1) * sx + kw, patchH = (kDirTile - 1) * sy + kh;
    const int patchN = patchW * patchH;
    float* patch = lds;                         // [CC][patchH][patchW]
    float* filt = lds + CC * patchN;            // [CC][taps][OCT]

    const int tid = threadIdx.x, tx = tid % kDirTile, ty = tid / kDirTile;
    const int tileX = blockIdx.x % tilesX, tileY = blockIdx.x / tilesX;
    const int o0 = blockIdx.y * OCT;
    const int xo = tileX * kDirTile + tx, yo = tileY * kDirTile + ty;
    const int px0 = tileX * kDirTile * sx - kw / 2, py0 = tileY * kDirTile * sy - kh / 2;

    float acc[OCT];
#pragma unroll
    for (int k = 0; k < OCT; ++k) acc[k] = 0.0f;

    for (int c0 = 0; c0 < I; c0 += CC) {
        const int cc = min(CC, I - c0);
        __syncthreads();                        // previous chunk fully consumed
        for (int e = tid; e < cc * patchN; e += kDirThreads) {
            const int c = e / patchN, r = e % patchN;
            const int gx = px0 + r % patchW, gy = py0 + r / patchW;
            // unconditional load from the clamped position, zero padding by select: loads under a
            // per-lane branch are waited for one by one
            const bool inside = gx >= 0 && gx < W && gy >= 0 && gy < H;
            const float v = in[(size_t)(c0 + c) * H * W + (size_t)min(max(gy, 0), H - 1) * W + min(max(gx, 0), W - 1)];
            patch[e] = inside ? v : 0.0f;
        }
        for (int e = tid; e < cc * taps * OCT; e += kDirThreads) {
            const int oc = e % OCT, tap = (e / OCT) % taps, c = e / (OCT * taps);
            const int o = o0 + oc;
            const float f = w[((size_t)(c0 + c) * O + min(o, O - 1)) * taps + tap];
            filt[e] = (o < O) ? f : 0.0f;
        }
        __syncthreads();
        for (int c = 0; c < cc; ++c) {
            const float* pc = patch + c * patchN + (ty * sy) * patchW + tx * sx;
            const float* fc = filt + c * taps * OCT;
            if (KW) {
#pragma unroll
                for (int j = 0; j < (KH ? KH : 1); ++j)
#pragma unroll
                    for (int i = 0; i < (KW ? KW : 1); ++i) {
                        const float v = pc[j * patchW + i];
#pragma unroll
                        for (int k = 0; k < OCT; ++k) acc[k] = fmaf(v, fc[(j * KW + i) * OCT + k], acc[k]);
                    }
            } else {
                for (int j = 0; j < kh; ++j)
                    for (int i = 0; i < kw; ++i) {
                        const float v = pc[j * patchW + i];
#pragma unroll
                        for (int k = 0; k < OCT; ++k) acc[k] = fmaf(v, fc[(j * kw + i) * OCT + k], acc[k]);
                    }
            }
        }
    }

    if (xo < Wo && yo < Ho) {
#pragma unroll
        for (int k = 0; k < OCT; ++k) {
            const int o = o0 + k;
            if (o < O) {
                float v = acc[k] + (bias ? bias[o] : 0.0f);
                if (relu) v = fmaxf(v, 0.0f);
                out[(size_t)o * Ho * Wo + (size_t)yo * Wo + xo] = v;
            }
        }
    }
}

// First layers (I <= 4, e.g. RGB): too little work per channel to pay for staging anything in LDS.
// One lane = one output pixel x OCT channels; its kw*kh*I input samples come straight from global
// memory (unconditional loads from clamped positions, zero padding by select; neighbours share
// cache lines), and the filters are wave-uniform, so the compiler fetches them with scalar loads
// and the FMAs take them from SGPRs.
template <int OCT, int KW, int KH, int IC>
__global__ void __launch_bounds__(kDirThreads)
conv_direct_fewc_kernel(const float* __restrict__ in, const float* __restrict__ w, const float* __restrict__ bias,
                        float* __restrict__ out, int W, int H, int I, int O, int Wo, int Ho,
                        int sx, int sy, int tilesX, int relu) {
    constexpr int taps = KW * KH;
    const int tid = threadIdx.x, tx = tid % kDirTile, ty = tid / kDirTile;
    const int tileX = blockIdx.x % tilesX, tileY = blockIdx.x / tilesX;
    const int o0 = blockIdx.y * OCT;
    const int xo = tileX * kDirTile + tx, yo = tileY * kDirTile + ty;
    const int cx = min(xo, Wo - 1) * sx - KW / 2, cy = min(yo, Ho - 1) * sy - KH / 2;   // window origin (clamped lanes recompute a valid pixel)

    float acc[OCT];
#pragma unroll
    for (int k = 0; k < OCT; ++k) acc[k] = 0.0f;

    // all samples of all IC (= I, at most 4) channels first: one memory latency for the whole lane
    float v[IC][taps];
#pragma unroll
    for (int c = 0; c < IC; ++c) {
        const float* pc = in + (size_t)c * H * W;
#pragma unroll
        for (int j = 0; j < KH; ++j)
#pragma unroll
            for (int i = 0; i < KW; ++i) {
                const int gx = cx + i, gy = cy + j;
                const float raw = pc[(size_t)min(max(gy, 0), H - 1) * W + min(max(gx, 0), W - 1)];
                v[c][j * KW + i] = (gx >= 0 && gx < W && gy >= 0 && gy < H) ? raw : 0.0f;
            }
    }
#pragma unroll
    for (int c = 0; c < IC; ++c) {
#pragma unroll
        for (int k = 0; k < OCT; ++k) {
            const float* fk = w + ((size_t)c * O + min(o0 + k, O - 1)) * taps;     // wave-uniform address
#pragma unroll
            for (int t = 0; t < taps; ++t) acc[k] = fmaf(v[c][t], fk[t], acc[k]);
        }
    }
    if (xo < Wo && yo < Ho) {
#pragma unroll
        for (int k = 0; k < OCT; ++k) {
            const int o = o0 + k;
            if (o < O) {
                float r = acc[k] + (bias ? bias[o] : 0.0f);
                if (relu) r = fmaxf(r, 0.0f);
                out[(size_t)o * Ho * Wo + (size_t)yo * Wo + xo] = r;
            }
        }
    }
}

template <int OCT>
static int launch_direct(const float* in, const float* w, const float* bias, float* out,
                         int W, int H, int I, int O, int kw, int kh, int sx, int sy, int relu, hipStream_t s) {
    const int Wo = W / sx, Ho = H / sy;
    const int tilesX = ceil_div(Wo, kDirTile), tilesY = ceil_div(Ho, kDirTile);
    const int patchN = ((kDirTile - 1) * sx + kw) * ((kDirTile - 1) * sy + kh);
    const int perChannel = patchN + kw * kh * OCT;
    int CC = kDirMaxLdsFloats / perChannel;
    if (CC > 8) CC = 8;
    if (CC > I) CC = I;
    DRHIP_REQUIRE(CC >= 1, "drhip_conv2d_direct_f32: a %dx%d filter with stride %dx%d does not fit the LDS patch", kw, kh, sx, sy);
    const size_t ldsBytes = (size_t)CC * perChannel * sizeof(float);
    dim3 grid(tilesX * tilesY, ceil_div(O, OCT)), block(kDirThreads);
    if (kw == 3 && kh == 3)
        launch((conv_direct_kernel<OCT, 3, 3>), grid, block, ldsBytes, s, in, w, bias, out, W, H, I, O, Wo, Ho, kw, kh, sx, sy, CC, tilesX, relu);
    else
        launch((conv_direct_kernel<OCT, 0, 0>), grid, block, ldsBytes, s, in, w, bias, out, W, H, I, O, Wo, Ho, kw, kh, sx, sy, CC, tilesX, relu);
    return launched("conv_direct_kernel");
}

}  // namespace drhip

using namespace drhip;

extern "C" int drhip_conv2d_direct_f32(const float* in, const float* w, const float* bias, float* out,
                                       int W, int H, int I, int O, int kw, int kh,
                                       int strideX, int strideY, int relu, void* stream) {
    DRHIP_REQUIRE(in && w && out, "drhip_conv2d_direct_f32: NULL tensor");
    DRHIP_REQUIRE(W > 0 && H > 0 && I > 0 && O > 0, "drhip_conv2d_direct_f32: bad shape %dx%dx%d -> %d", W, H, I, O);
    DRHIP_REQUIRE(kw > 0 && kh > 0 && (kw & 1) && (kh & 1), "drhip_conv2d_direct_f32: filter %dx%d must have odd sides", kw, kh);
    DRHIP_REQUIRE(strideX > 0 && strideY > 0, "drhip_conv2d_direct_f32: stride must be positive");
    DRHIP_REQUIRE(W / strideX > 0 && H / strideY > 0, "drhip_conv2d_direct_f32: output is empty");
    DRHIP_REQUIRE((long long)W * H * I < (1ll << 31) && (long long)(W / strideX) * (H / strideY) * O < (1ll << 31),
                  "drhip_conv2d_direct_f32: tensor too large");
    hipStream_t s0 = as_stream(stream);
    if (I <= 4 && kw == 3 && kh == 3) {
        const int Wo = W / strideX, Ho = H / strideY;
        const int tilesX = ceil_div(Wo, kDirTile), tilesY = ceil_div(Ho, kDirTile);
#define DRHIP_FEWC(OCTV, ICV) launch((conv_direct_fewc_kernel<OCTV, 3, 3, ICV>), dim3(tilesX * tilesY, ceil_div(O, OCTV)), dim3(kDirThreads), 0, s0, \
                                     in, w, bias, out, W, H, I, O, Wo, Ho, strideX, strideY, tilesX, relu)
#define DRHIP_FEWC_I(OCTV) do { if (I == 1) DRHIP_FEWC(OCTV, 1); else if (I == 2) DRHIP_FEWC(OCTV, 2); else if (I == 3) DRHIP_FEWC(OCTV, 3); else DRHIP_FEWC(OCTV, 4); } while (0)
        if (O >= 8) DRHIP_FEWC_I(8);            // 16 channels per lane measured slower (8.0 vs 6.6 us on 224x224x3 -> 64)
        else DRHIP_FEWC_I(4);
#undef DRHIP_FEWC_I
#undef DRHIP_FEWC
        return launched("conv_direct_fewc_kernel");
    }
    // Few output channels per lane when the tile count alone cannot fill the CUs.
    const int tiles = ceil_div(W / strideX, kDirTile) * ceil_div(H / strideY, kDirTile);
    hipStream_t s = as_stream(stream);
    if (O >= 16 && tiles * ceil_div(O, 16) >= 2 * num_cu())
        return launch_direct<16>(in, w, bias, out, W, H, I, O, kw, kh, strideX, strideY, relu, s);
    if (O >= 8 && tiles * ceil_div(O, 8) >= num_cu())
        return launch_direct<8>(in, w, bias, out, W, H, I, O, kw, kh, strideX, strideY, relu, s);
    return launch_direct<4>(in, w, bias, out, W, H, I, O, kw, kh, strideX, strideY, relu, s);
}
