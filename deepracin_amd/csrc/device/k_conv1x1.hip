// 1x1 convolution as an fp32 MFMA GEMM over the [C][H*W] view of the tensors:
//
//   out[o][p] = act(b[o] + sum_c w[c][o] * in[c][p]),   p = y*W + x,  P = H*W
//
// MFMA-bound in principle (2*P*I*O FLOP; bytes 4*(P*I + I*O + O + P*O)); the SqueezeNet layers are
// a few MFLOP each, so what matters is latency: enough waves, loads kept in flight, no second launch.
//
// Both operands are already laid out the way v_mfma_f32_32x32x2_f32 wants them:
//   A (32 rows x 2 k): lane -> (row = lane%32, k = lane/32).  rows = output channels, and the
//     weights arrive as [I][O] (dR_Conv2d_setVariables layout with kh=kw=1), so a wave reads
//     2 x 128 contiguous bytes per operand -- the reference's [I][O]->[O][I] transpose at
//     fillBuffers (src/dR_nodes_conv2d.c:1696-1716) is not needed;
//   B (2 k x 32 cols): lane -> (col = lane%32, k = lane/32).  cols = pixels, in[c][p] is
//     contiguous in p;
//   D: lane -> col (pixel) lane%32, register r -> row (channel) 8*(r/4) + 4*(lane/32) + r%4.
//
// One workgroup = one 32-channel x 32-pixel output tile, KW waves (1, 2, 4 or 8).  The input channels
// are dealt to the waves in stages of 8 (wave w takes stages w, w+KW, ...); every wave streams its
// operands straight from L2 with the next two stages already in flight (loads are unconditional
// from clamped addresses, zero padding is a select afterwards, so the compiler can count them),
// and the KW partial tiles are added in wave order through LDS before bias, ReLU and a coalesced
// store.  Splitting the channel loop inside the workgroup gives the 14x14 layers (7 pixel tiles)
// enough waves without a second kernel or atomics, and keeps the summation order fixed.
//
// Reference kernel: Kernels/dR_conv2d1x1.cl:4-53 (one work-item per (x,y,o), sequential sum over
// the input channels).
#include "drhip_common.hpp"

namespace drhip {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kC1KC = 8;            // channels per stage (4 MFMA k-steps)
constexpr int kC1Pad = 33;          // LDS row pitch of a partial tile (floats)

__global__ void __launch_bounds__(512)
conv1x1_mfma_kernel(const float* __restrict__ in, const float* __restrict__ w, const float* __restrict__ bias,
                    float* __restrict__ out, float* __restrict__ poolPartials, int P, int I, int O, int KW, int relu) {
    extern __shared__ float part[];                 // [KW][32][kC1Pad], used only when KW > 1
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // (KW, the waves per workgroup, is a kernel argument: blockDim.x would be a load from the dispatch packet in
    // front of everything else; the 15 dwords of arguments arrive in SGPRs with the wave)
    const int l32 = lane & 31, lhi = lane >> 5;
    const int o0 = blockIdx.y * 32, p0 = blockIdx.x * 32;      // (a 2-D grid: an integer division here delays the first loads)
    const int nStages = (I + kC1KC - 1) / kC1KC;

    // The epilogue's bias values are requested now (a load issued there would add a trip to memory to the tail of
    // the workgroup): with more than one wave, thread tid finishes the elements tid + q*blockDim.x of the tile.
    float biasEarly[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const int idx = tid + q * (64 * KW);
        biasEarly[q] = (bias && idx < 32 * 32) ? bias[min(o0 + (idx >> 5), O - 1)] : 0.0f;
    }

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

    // clamped operand columns: always valid addresses; out-of-range lanes are zeroed by select
    const int oL = min(o0 + l32, O - 1), pL = min(p0 + l32, P - 1);
    const bool oOk = o0 + l32 < O, pOk = p0 + l32 < P;
    float aA[4], bA[4], aB[4], bB[4];
    auto load_stage = [&](float (&a)[4], float (&b)[4], int stage) {
        stage = min(stage, nStages - 1);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const int c = min(stage * kC1KC + 2 * ks + lhi, I - 1);
            a[ks] = w[(size_t)c * O + oL];
            b[ks] = in[(size_t)c * P + pL];
        }
    };
    auto multiply = [&](const float (&a)[4], const float (&b)[4], int stage) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const bool cOk = stage * kC1KC + 2 * ks + lhi < I;
            const float av = (cOk && oOk) ? a[ks] : 0.0f;
            const float bv = (cOk && pOk) ? b[ks] : 0.0f;
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
        }
    };
    // stages wave, wave+KW, ...; two in flight
    int st = wave;
    load_stage(aA, bA, st);
    load_stage(aB, bB, st + KW);
    for (; st + KW < nStages; st += 2 * KW) {
        multiply(aA, bA, st);
        load_stage(aA, bA, st + 2 * KW);
        multiply(aB, bB, st + KW);
        load_stage(aB, bB, st + 3 * KW);
    }
    if (st < nStages) multiply(aA, bA, st);

    if (KW == 1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int o = o0 + 8 * (r / 4) + 4 * lhi + (r % 4);
            if (o < O && pOk) {
                float v = acc[r] + (bias ? bias[o] : 0.0f);
                if (relu) v = fmaxf(v, 0.0f);
                store_through(out + (size_t)o * P + p0 + l32, v);
            }
        }
        return;
    }
    // partial tiles -> LDS, then all lanes add them in wave order
#pragma unroll
    for (int r = 0; r < 16; ++r)
        part[(wave * 32 + 8 * (r / 4) + 4 * lhi + (r % 4)) * kC1Pad + l32] = acc[r];
    __syncthreads();
#pragma unroll
    for (int q = 0; q < 8; ++q) {                   // KW >= 2 waves: at most 8 elements per thread
        const int idx = tid + q * (64 * KW);
        if (idx >= 32 * 32) break;
        const int ol = idx >> 5, pl = idx & 31;
        const int o = o0 + ol, p = p0 + pl;
        float s = 0.0f;
        for (int k = 0; k < KW; ++k) s += part[(k * 32 + ol) * kC1Pad + pl];
        s += biasEarly[q];
        if (relu) s = fmaxf(s, 0.0f);
        if (poolPartials) {
            // sum over the tile's pixels: the 32 lanes of a half wave hold one channel (the trip count
            // of this loop is the same for every lane, so all of them take part in the shuffles)
            s = p < P ? s : 0.0f;
#pragma unroll
            for (int m = 16; m >= 1; m >>= 1) s += __shfl_xor(s, m, 64);
            if (pl == 0 && o < O) store_through(poolPartials + (size_t)(p0 >> 5) * O + o, s);
        } else if (o < O && p < P) {
            store_through(out + (size_t)o * P + p, s);
        }
    }
}

// Small layers (14x14 and 28x28 maps): a 32x32 tile with 512 input channels is 256 MFMAs in a row on
// one CU while most of the chip idles.  This form works on 16-channel x 16-pixel tiles with
// v_mfma_f32_16x16x4_f32 (A: lane -> row lane%16, k = lane/16; B: lane -> col lane%16, k = lane/16;
// D: lane -> col lane%16, register r -> row 4*(lane/16) + r), four times as many workgroups and a
// quarter of the dependent MFMA chain each.  KW waves (1..16) take the 4-channel k-steps round-robin
// in chunks of 8, the next chunk always in flight; k-steps past the end are multiplied as zeros
// (32 cycles each) so that the loop has no branch and the compiler can count the loads.
typedef float f32x4v __attribute__((ext_vector_type(4)));
constexpr int kC1Chunk = 8;         // k-steps per chunk (16 in flight was measured slower)
constexpr int kC1Pad16 = 17;

// POOL: the input is the tensor IN FRONT of a 3x3 / stride-2 max pooling ([I][Hin][Win]) and the B operand of
// pixel p = (py, px) of the pooled map is taken on load as the maximum of the window anchored at (2px, 2py),
// samples outside the map counting as 0.0 (src/dR_nodes_pooling.c:277-401) -- the pooled tensor, read exactly
// once by this layer, is never written and the pooling kernel in front is not launched.  A window row is ONE
// 16-byte buffer load from its first sample (nine dword gathers per operand kept the CU's address unit busy
// for longer than the whole unpooled layer takes); the resource ends with the tensor, so the load of the
// last row may run past it and reads 0.0 there.  Chunks of 4 k-steps keep the rows in registers.
typedef float f32x4ld __attribute__((ext_vector_type(4)));
constexpr unsigned kC1BufferFlags = 0x00020000u;    // dword 3 of a gfx9 raw buffer resource (32-bit data format)

template <bool POOL>
__global__ void __launch_bounds__(POOL ? 512 : 1024)
conv1x1_mfma16_kernel(const float* __restrict__ in, const float* __restrict__ w, const float* __restrict__ bias,
                      float* __restrict__ out, int P, int I, int O, int KW, int reluAndShift, int Win, int Hin, unsigned WpMul) {
    extern __shared__ float part[];                 // [KW][16][kC1Pad16]
    const int relu = reluAndShift & 1;              // (16 dwords of arguments in all: they arrive in SGPRs with the wave)
    const FastDiv Wpd = {(unsigned)((Win + 1) >> 1), WpMul, (unsigned)(reluAndShift >> 8)};
    constexpr int CH = POOL ? 4 : kC1Chunk;         // k-steps per chunk
    constexpr int NS = POOL ? 12 : 1;               // floats loaded per B operand (3 window rows of 4)
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // (KW, the waves per workgroup, is a kernel argument: (64 * KW) would be a load from the dispatch packet
    // in front of everything else)
    const int l16 = lane & 15, lk = lane >> 4;
    const int o0 = blockIdx.y * 16, p0 = blockIdx.x * 16;    // (a 2-D grid: an integer division here delays the first loads)
    const int nK = (I + 3) / 4;                     // k-steps of 4 channels
    const int oL = min(o0 + l16, O - 1), pL = min(p0 + l16, P - 1);
    const bool oOk = o0 + l16 < O, pOk = p0 + l16 < P;
    const int plane = POOL ? Win * Hin : P;

    // POOL: element offset of each window row inside a channel plane (rows below the map repeat the last row
    // and are masked), and which of the 3x3 samples lie inside the map
    int rowOff[3] = {pL, 0, 0};
    bool colIn[3] = {true, true, true}, rowIn[3] = {true, true, true};
    __amdgpu_buffer_rsrc_t rIn;
    if constexpr (POOL) {
        const int py = fast_div(pL, Wpd), px = pL - py * (int)Wpd.d;
#pragma unroll
        for (int d = 0; d < 3; ++d) {
            rowIn[d] = 2 * py + d < Hin;
            colIn[d] = 2 * px + d < Win;
            rowOff[d] = min(2 * py + d, Hin - 1) * Win + 2 * px;
        }
        rIn = __builtin_amdgcn_make_buffer_rsrc((void*)in, 0, I * plane * 4, kC1BufferFlags);
    }

    f32x4v acc = {0.f, 0.f, 0.f, 0.f};
    float aA[CH], bA[CH][NS], aB[CH], bB[CH][NS];
    // chunk j of this wave = its k-steps wave + KW*(CH*j .. CH*j + CH-1)
    auto load_chunk = [&](float (&a)[CH], float (&b)[CH][NS], int j) {
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            const int c = min(4 * (wave + KW * (CH * j + u)) + lk, I - 1);
            a[u] = w[(size_t)c * O + oL];
            if constexpr (POOL) {
#pragma unroll
                for (int d = 0; d < 3; ++d) {
                    const f32x4ld v = __builtin_bit_cast(f32x4ld, __builtin_amdgcn_raw_buffer_load_b128(rIn, 4 * (c * plane + rowOff[d]), 0, 0));
#pragma unroll
                    for (int e = 0; e < 4; ++e) b[u][4 * d + e] = v[e];
                }
            } else {
                b[u][0] = in[(size_t)c * plane + rowOff[0]];
            }
        }
    };
    auto multiply = [&](const float (&a)[CH], const float (&b)[CH][NS], int j) {
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            const bool cOk = 4 * (wave + KW * (CH * j + u)) + lk < I;
            float bv = b[u][0];
            if constexpr (POOL) {
                bv = -3.402823466e+38f;              // the pooling kernel's start value
#pragma unroll
                for (int d = 0; d < 3; ++d)
#pragma unroll
                    for (int e = 0; e < 3; ++e) bv = fmaxf(bv, (rowIn[d] && colIn[e]) ? b[u][4 * d + e] : 0.0f);
            }
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32((cOk && oOk) ? a[u] : 0.0f, (cOk && pOk) ? bv : 0.0f, acc, 0, 0, 0);
        }
    };
    const int mine = (nK - wave + KW - 1) >> (31 - __builtin_clz(KW));     // k-steps of this wave (>= 0); KW is a power of two
    const int chunks = (mine + CH - 1) / CH;
    // Two buffers, the next chunk always on its way.  The loop leaves right after the last real
    // chunk: the loads issued beyond it (clamped addresses) are never waited for.
    load_chunk(aA, bA, 0);
    // The epilogue's bias values are requested now, behind the first operands: a load issued in the epilogue would
    // add a trip to memory to the tail of every workgroup.  Thread tid finishes the elements tid, tid + 64 KW, ...
    // of the 16x16 tile (at most 4); the loads are unconditional (clamped), a branch per load costs more.
    float biasEarly[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias) {
#pragma unroll
        for (int q = 0; q < 4; ++q) biasEarly[q] = bias[min(o0 + min((tid + q * (64 * KW)) >> 4, 15), O - 1)];
    }
    for (int j = 0; j < chunks;) {
        load_chunk(aB, bB, j + 1);
        multiply(aA, bA, j);
        if (++j >= chunks) break;
        load_chunk(aA, bA, j + 1);
        multiply(aB, bB, j);
        ++j;
    }

#pragma unroll
    for (int r = 0; r < 4; ++r) part[(wave * 16 + 4 * lk + r) * kC1Pad16 + l16] = acc[r];
    __syncthreads();
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int idx = tid + q * (64 * KW);
        if (idx >= 16 * 16) break;
        const int ol = idx >> 4, pl = idx & 15;
        const int o = o0 + ol, p = p0 + pl;
        float s = 0.0f;
        for (int k = 0; k < KW; ++k) s += part[(k * 16 + ol) * kC1Pad16 + pl];
        if (o < O && p < P) {
            s += biasEarly[q];
            if (relu) s = fmaxf(s, 0.0f);
            store_through(out + (size_t)o * P + p, s);
        }
    }
}

}  // namespace drhip

using namespace drhip;

// variant = waves per output tile (1, 2, 4, 8; 16 only with 0x100) | 0x100 for 16x16 tiles.
// 32x32 tiles: as many waves as give every wave at least two 8-channel stages, more when the layer
// has few tiles.  Layers with fewer 32x32 tiles than CUs take the 16x16 form with one wave per 8
// k-steps (one chunk, a single round of loads).
extern "C" int drhip_conv1x1_pick_variant(int P, int I, int O) {
    const int tiles = ceil_div(O, 32) * ceil_div(P, 32);
    if (tiles < num_cu() && ceil_div(O, 16) * ceil_div(P, 16) <= 2 * num_cu()) {
        const int nK = ceil_div(I, 4);
        int kw = 1;
        while (kw < 4 && nK > 8 * kw) kw *= 2;
        if (nK > 32) kw = 8;                        // more than one chunk per wave: measured better with 8 waves
        return 0x100 | kw;
    }
    const int stages = ceil_div(I, kC1KC);
    int kw = 1;
    while (kw < 8 && stages >= 4 * kw && tiles * kw < 8 * num_cu()) kw *= 2;
    return kw;
}

extern "C" int drhip_conv1x1_f32(const float* in, const float* w, const float* bias, float* out,
                                 int P, int I, int O, int relu, int variant, void* stream) {
    DRHIP_REQUIRE(in && w && out, "drhip_conv1x1_f32: NULL tensor");
    DRHIP_REQUIRE(P > 0 && I > 0 && O > 0, "drhip_conv1x1_f32: bad shape P=%d I=%d O=%d", P, I, O);
    DRHIP_REQUIRE((long long)P * I < (1ll << 31) && (long long)P * O < (1ll << 31) && (long long)I * O < (1ll << 31),
                  "drhip_conv1x1_f32: tensor too large for 32-bit indexing");
    if (variant == 0) variant = drhip_conv1x1_pick_variant(P, I, O);
    if (variant & 0x100) {
        const int kw = variant & 0xff;
        DRHIP_REQUIRE((variant >> 9) == 0, "drhip_conv1x1_f32: unknown variant %#x", variant);
        DRHIP_REQUIRE(kw == 1 || kw == 2 || kw == 4 || kw == 8 || kw == 16, "drhip_conv1x1_f32: unknown variant %#x (16x16 tiles: 1..16 waves)", variant);
        const int nPT16 = ceil_div(P, 16), nOT16 = ceil_div(O, 16);
        DRHIP_REQUIRE(nOT16 <= 65535, "drhip_conv1x1_f32: too many output channels for 16x16 tiles (%d)", O);
        launch(conv1x1_mfma16_kernel<false>, dim3(nPT16, nOT16), dim3(64 * kw), (size_t)kw * 16 * kC1Pad16 * sizeof(float), as_stream(stream),
               in, w, bias, out, P, I, O, kw, relu ? 1 : 0, 0, 0, 0u);
        return launched("conv1x1_mfma16_kernel");
    }
    DRHIP_REQUIRE(variant == 1 || variant == 2 || variant == 4 || variant == 8, "drhip_conv1x1_f32: unknown variant %d (waves per tile: 1, 2, 4, 8)", variant);
    const int nPT = ceil_div(P, 32), nOT = ceil_div(O, 32);
    DRHIP_REQUIRE(nOT <= 65535, "drhip_conv1x1_f32: too many output channels (%d)", O);
    const size_t ldsBytes = variant > 1 ? (size_t)variant * 32 * kC1Pad * sizeof(float) : 0;
    launch(conv1x1_mfma_kernel, dim3(nPT, nOT), dim3(64 * variant), ldsBytes, as_stream(stream),
                       in, w, bias, out, (float*)nullptr, P, I, O, variant, relu);
    return launched("conv1x1_mfma_kernel");
}

extern "C" int drhip_conv1x1_poolsum_slices(int P) { return P > 0 ? ceil_div(P, 32) : 0; }

extern "C" int drhip_conv1x1_poolsum_f32(const float* in, const float* w, const float* bias, float* partials,
                                         int P, int I, int O, int relu, void* stream) {
    DRHIP_REQUIRE(in && w && partials, "drhip_conv1x1_poolsum_f32: NULL tensor");
    DRHIP_REQUIRE(P > 0 && I > 0 && O > 0, "drhip_conv1x1_poolsum_f32: bad shape P=%d I=%d O=%d", P, I, O);
    DRHIP_REQUIRE((long long)P * I < (1ll << 31) && (long long)P * O < (1ll << 31) && (long long)I * O < (1ll << 31),
                  "drhip_conv1x1_poolsum_f32: tensor too large for 32-bit indexing");
    // 32x32 tiles with at least two waves: the pixel sums are taken where the waves' partial tiles meet
    const int tiles = ceil_div(O, 32) * ceil_div(P, 32), stages = ceil_div(I, kC1KC);
    int kw = 2;
    while (kw < 8 && stages >= 4 * kw && tiles * kw < 8 * num_cu()) kw *= 2;
    const int nPT = ceil_div(P, 32), nOT = ceil_div(O, 32);
    DRHIP_REQUIRE(nOT <= 65535, "drhip_conv1x1_poolsum_f32: too many output channels (%d)", O);
    launch(conv1x1_mfma_kernel, dim3(nPT, nOT), dim3(64 * kw), (size_t)kw * 32 * kC1Pad * sizeof(float), as_stream(stream),
           in, w, bias, (float*)nullptr, partials, P, I, O, kw, relu);
    return launched("conv1x1_mfma_kernel");
}

extern "C" int drhip_conv1x1_pooled3s2_f32(const float* in, const float* w, const float* bias, float* out,
                                           int Win, int Hin, int I, int O, int relu, void* stream) {
    DRHIP_REQUIRE(in && w && out, "drhip_conv1x1_pooled3s2_f32: NULL tensor");
    DRHIP_REQUIRE(Win > 0 && Hin > 0 && I > 0 && O > 0, "drhip_conv1x1_pooled3s2_f32: bad shape %dx%dx%d -> %d", Win, Hin, I, O);
    const int Wp = (Win + 1) / 2, Hp = (Hin + 1) / 2, P = Wp * Hp;
    DRHIP_REQUIRE((long long)Win * Hin * I < (1ll << 29) && (long long)P * O < (1ll << 31) && (long long)I * O < (1ll << 31),
                  "drhip_conv1x1_pooled3s2_f32: tensor too large for 32-bit indexing");
    // waves per 16x16 tile: one per chunk of 4 k-steps (a single round of loads for every wave), at most 8
    const int nK = ceil_div(I, 4);
    int kw = 1;
    while (kw < 8 && nK > 4 * kw) kw *= 2;
    const int nPT16 = ceil_div(P, 16), nOT16 = ceil_div(O, 16);
    DRHIP_REQUIRE(nOT16 <= 65535, "drhip_conv1x1_pooled3s2_f32: too many output channels (%d)", O);
    const FastDiv dWp = make_fastdiv(Wp);
    launch(conv1x1_mfma16_kernel<true>, dim3(nPT16, nOT16), dim3(64 * kw), (size_t)kw * 16 * kC1Pad16 * sizeof(float), as_stream(stream),
           in, w, bias, out, P, I, O, kw, (relu ? 1 : 0) | (int)(dWp.shift << 8), Win, Hin, dWp.mul);
    return launched("conv1x1_mfma16_kernel<pooled input>");
}
