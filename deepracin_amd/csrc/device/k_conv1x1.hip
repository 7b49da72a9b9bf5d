// 1x1 convolution as an fp32 MFMA GEMM over the [C][H*W] view of the tensors:
//
//   out[o][p] = act(b[o] + sum_c w[c][o] * in[c][p]),   p = y*W + x,  P = H*W
//
// MFMA-bound in principle (2*P*I*O FLOP; bytes 4*(P*I + I*O + O + P*O)), in practice the
// SqueezeNet layers are a few MFLOP each and the launch dominates.
//
// Both operands are already laid out the way v_mfma_f32_32x32x2_f32 wants them:
//   A (32 rows x 2 k): lane -> (row = lane%32, k = lane/32).  rows = output channels, and the
//     weights arrive as [I][O] (dR_Conv2d_setVariables layout with kh=kw=1), so a wave reads
//     2 x 128 contiguous bytes per operand -- the reference's [I][O]->[O][I] transpose at
//     fillBuffers (src/dR_nodes_conv2d.c:1696-1716) is not needed;
//   B (2 k x 32 cols): lane -> (col = lane%32, k = lane/32).  cols = pixels, in[c][p] is
//     contiguous in p;
//   D: lane -> col (pixel) lane%32, register r -> row (channel) 8*(r/4) + 4*(lane/32) + r%4, so
//     every store instruction writes 2 x 128 contiguous bytes of two output-channel rows.
// No LDS: each wave owns a (32*WM channels) x (32*WN pixels) tile and streams its operands from
// L2 with a register prefetch of the next 8 input channels.
//
// Reference kernel: Kernels/dR_conv2d1x1.cl:4-53 (one work-item per (x,y,o), sequential sum over
// the input channels).
#include "drhip_common.hpp"

namespace drhip {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kC1Threads = 256;
constexpr int kC1KC = 8;            // channels per prefetch group (4 MFMA k-steps)

template <int WM, int WN>
__global__ void __launch_bounds__(kC1Threads)
conv1x1_mfma_kernel(const float* __restrict__ in, const float* __restrict__ w, const float* __restrict__ bias,
                    float* __restrict__ out, int P, int I, int O, int nPT, int nTiles, int relu) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int tile = blockIdx.x * (kC1Threads / kWave) + wave;      // one tile per wave
    if (tile >= nTiles) return;
    const int o0 = (tile / nPT) * 32 * WM;
    const int p0 = (tile % nPT) * 32 * WN;

    f32x16 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    float aCur[kC1KC / 2][WM], bCur[kC1KC / 2][WN], aNxt[kC1KC / 2][WM], bNxt[kC1KC / 2][WN];
    auto load_group = [&](float (&a)[kC1KC / 2][WM], float (&b)[kC1KC / 2][WN], int c0) {
#pragma unroll
        for (int ks = 0; ks < kC1KC / 2; ++ks) {
            const int c = c0 + 2 * ks + lhi;
#pragma unroll
            for (int i = 0; i < WM; ++i) {
                const int o = o0 + 32 * i + l32;
                a[ks][i] = (c < I && o < O) ? w[(size_t)c * O + o] : 0.0f;
            }
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                const int p = p0 + 32 * j + l32;
                b[ks][j] = (c < I && p < P) ? in[(size_t)c * P + p] : 0.0f;
            }
        }
    };

    const int nGroups = (I + kC1KC - 1) / kC1KC;
    load_group(aCur, bCur, 0);
    for (int gI = 0; gI < nGroups; ++gI) {
        const bool more = gI + 1 < nGroups;
        if (more) load_group(aNxt, bNxt, (gI + 1) * kC1KC);
#pragma unroll
        for (int ks = 0; ks < kC1KC / 2; ++ks)
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < WN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(aCur[ks][i], bCur[ks][j], acc[i][j], 0, 0, 0);
        if (more) {
#pragma unroll
            for (int ks = 0; ks < kC1KC / 2; ++ks) {
#pragma unroll
                for (int i = 0; i < WM; ++i) aCur[ks][i] = aNxt[ks][i];
#pragma unroll
                for (int j = 0; j < WN; ++j) bCur[ks][j] = bNxt[ks][j];
            }
        }
    }

#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int o = o0 + 32 * i + 8 * (r / 4) + 4 * lhi + (r % 4);
            if (o >= O) continue;
            const float bv = bias ? bias[o] : 0.0f;
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                const int p = p0 + 32 * j + l32;
                if (p >= P) continue;
                float v = acc[i][j][r] + bv;
                if (relu) v = fmaxf(v, 0.0f);
                out[(size_t)o * P + p] = v;
            }
        }
}

template <int WM, int WN>
static int launch_c1(const float* in, const float* w, const float* bias, float* out, int P, int I, int O, int relu, hipStream_t s) {
    const int nPT = ceil_div(P, 32 * WN), nOT = ceil_div(O, 32 * WM), nTiles = nPT * nOT;
    const int blocks = ceil_div(nTiles, kC1Threads / kWave);
    hipLaunchKernelGGL((conv1x1_mfma_kernel<WM, WN>), dim3(blocks), dim3(kC1Threads), 0, s, in, w, bias, out, P, I, O, nPT, nTiles, relu);
    return launched("conv1x1_mfma_kernel");
}

}  // namespace drhip

using namespace drhip;

// Register tile per wave: as large as still leaves one wave per SIMD something to do.
extern "C" int drhip_conv1x1_pick_variant(int P, int I, int O) {
    (void)I;
    const int simds = 4 * num_cu();
    auto tiles = [&](int wm, int wn) { return ceil_div(O, 32 * wm) * ceil_div(P, 32 * wn); };
    if (O > 32 && P > 32 && tiles(2, 2) >= simds) return 4;
    if (P > 32 && tiles(1, 2) >= simds) return 3;
    if (O > 32 && tiles(2, 1) >= simds) return 2;
    return 1;
}

extern "C" int drhip_conv1x1_f32(const float* in, const float* w, const float* bias, float* out,
                                 int P, int I, int O, int relu, int variant, void* stream) {
    DRHIP_REQUIRE(in && w && out, "drhip_conv1x1_f32: NULL tensor");
    DRHIP_REQUIRE(P > 0 && I > 0 && O > 0, "drhip_conv1x1_f32: bad shape P=%d I=%d O=%d", P, I, O);
    DRHIP_REQUIRE((long long)P * I < (1ll << 31) && (long long)P * O < (1ll << 31) && (long long)I * O < (1ll << 31),
                  "drhip_conv1x1_f32: tensor too large for 32-bit indexing");
    if (variant == 0) variant = drhip_conv1x1_pick_variant(P, I, O);
    hipStream_t s = as_stream(stream);
    switch (variant) {
        case 1: return launch_c1<1, 1>(in, w, bias, out, P, I, O, relu, s);
        case 2: return launch_c1<2, 1>(in, w, bias, out, P, I, O, relu, s);
        case 3: return launch_c1<1, 2>(in, w, bias, out, P, I, O, relu, s);
        case 4: return launch_c1<2, 2>(in, w, bias, out, P, I, O, relu, s);
        default: return fail(DRHIP_EINVAL, "drhip_conv1x1_f32: unknown variant %d", variant);
    }
}
