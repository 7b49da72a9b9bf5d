// Fused Winograd F(2x2,3x3) convolution for gfx950: 3x3, stride 1, SAME zero padding, [C][H][W] fp32.
//
//   Y = A^T [ (G g G^T) (.) (B^T d B) ] A   per 2x2 output tile, summed over input channels
//
// with the reference's transform matrices (Kernels/dR_winograd2.cl:64-157,191-217;
// src/dR_nodes_conv2d.c:1173-1176):
//   B^T = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 -1 0 1]   G = [1 0 0; .5 .5 .5; .5 -.5 .5; 0 0 1]
//   A^T = [1 1 1 0; 0 1 -1 1]
// (Lavin-Gray with the sign of the 4th row of B^T and the 4th column of A^T flipped, which cancels.)
//
// What is different from the reference kernel: there the 16*I multiply-adds per output are scalar
// MADs with the transformed filters streamed from global memory by every work-item.  Here the
// element-wise products are regrouped into 16 independent GEMMs, one per transform position xi:
//
//   M_xi[o][t] = sum_c U_xi[c][o] * V_xi[c][t]        (t = 2x2 tile index)
//
// and run on the fp32 matrix cores (v_mfma_f32_32x32x2_f32, 64 FLOP/clk/SIMD, MFMA-bound:
// algorithmic work 2*9*H*W*I*O FLOP direct-equivalent, 2*16*tiles*I*O FLOP issued).
//
// Workgroup = 256 lanes = 4 waves; it owns TB = 32*MT tiles x OB = 32*NT output channels for all
// 16 xi; wave w owns xi = 4w..4w+3 (so the 4 SIMDs of a CU each run their own MFMA stream).
// Input channels are consumed 8 at a time:
//   1. every lane loads the 4x4 input window of one (tile, channel) pair straight from global
//      memory (zero padded by predication), prefetched one chunk ahead into registers;
//   2. B^T d B in registers (32 adds), result written to LDS as V[xi][c][t]  (double buffered);
//   3. per k-step of 2 channels a wave issues MFMAs with A = U_xi[c][o] (read from global memory,
//      where dR_prepare stored it so that the four k-steps of a stage are one 16-byte load per lane
//      and 1 KiB contiguous per wave; prefetched one stage ahead) and B = V_xi[c][t] (one
//      conflict-free ds_read_b32 per lane);
//   4. epilogue: accumulators go through LDS 8 output channels at a time so that one lane sees
//      all 16 xi of one (tile, o), applies A^T m A, bias, ReLU and stores the 2x2 pixels
//      (adjacent lanes = adjacent tiles, 8-byte stores, edge guarded for odd sizes).
// One barrier per chunk.  Workgroup ids are remapped so that each XCD (own L2) works on a
// contiguous range of output-channel panels and therefore touches only its share of U.
// Layers with few tiles (28x28, 14x14) cannot fill 256 CUs with panels alone: there the input
// channels are split over gridDim.y workgroups whose partial outputs are summed, in fixed order,
// by whichever of them finishes last (deterministic, no float atomics).
#include "drhip_common.hpp"

namespace drhip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int kWinoThreads = 256;
constexpr int kWinoKC = 8;          // input channels per LDS stage
constexpr int kXcds = 8;            // L2 domains of MI355X

typedef float f32x4 __attribute__((ext_vector_type(4)));

// Layout of the transformed filters:  U[xi][chunk][o][8], chunk = c / 8, and inside a chunk the
// channel c%8 sits at position (c & 1) * 4 + ((c % 8) >> 1).  The MFMA A operand of k-step ks needs
// channel 2*ks + (lane / 32), so the four k-steps of a stage are ONE aligned 16-byte load per lane
// (position 4*(lane/32) + ks) and a wavefront reads 1 KiB contiguously.  Channels >= I are zero.
__host__ __device__ inline size_t wino_u_index(int xi, int c, int o, int nChunks, int O) {
    const int cc = c & 7;
    return (((size_t)xi * nChunks + (c >> 3)) * O + o) * 8 + (cc & 1) * 4 + (cc >> 1);
}

// U = G g G^T for g = w[c][o][3][3]; one lane per (padded c, o).
__global__ void __launch_bounds__(256)
winograd_filter_transform_kernel(const float* __restrict__ w, float* __restrict__ U, int I, int O, int nChunks) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= nChunks * 8 * O) return;
    const int c = idx / O, o = idx % O;
    float u[16];
    if (c < I) {
        const float* g = w + ((size_t)c * O + o) * 9;
        float t[4][3];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const float g0 = g[j], g1 = g[3 + j], g2 = g[6 + j];
            t[0][j] = g0;
            t[1][j] = 0.5f * g0 + 0.5f * g1 + 0.5f * g2;
            t[2][j] = 0.5f * g0 - 0.5f * g1 + 0.5f * g2;
            t[3][j] = g2;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float a = t[r][0], b = t[r][1], cc = t[r][2];
            u[4 * r + 0] = a;
            u[4 * r + 1] = 0.5f * a + 0.5f * b + 0.5f * cc;
            u[4 * r + 2] = 0.5f * a - 0.5f * b + 0.5f * cc;
            u[4 * r + 3] = cc;
        }
    } else {
#pragma unroll
        for (int k = 0; k < 16; ++k) u[k] = 0.0f;
    }
#pragma unroll
    for (int k = 0; k < 16; ++k) U[wino_u_index(k, c, o, nChunks, O)] = u[k];
}

// Output transform of one (tile, o): right factor A first, then A^T (order of the reference kernel).
__device__ inline void wino_output_transform(const float (&m)[16], float& y00, float& y01, float& y10, float& y11) {
    const float s0 = m[0] + m[1] + m[2],    s1 = m[1] - m[2] + m[3];
    const float s2 = m[4] + m[5] + m[6],    s3 = m[5] - m[6] + m[7];
    const float s4 = m[8] + m[9] + m[10],   s5 = m[9] - m[10] + m[11];
    const float s6 = m[12] + m[13] + m[14], s7 = m[13] - m[14] + m[15];
    y00 = s0 + s2 + s4; y01 = s1 + s3 + s5;
    y10 = s2 - s4 + s6; y11 = s3 - s5 + s7;
}

// 2x2 store with edge guards; vec2: W even and the base 8-byte aligned.
__device__ inline void wino_store_tile(float* po, int W, int H, int ox, int oy, int vec2,
                                       float y00, float y01, float y10, float y11) {
    if (vec2) {
        f32x2 v0 = {y00, y01};
        *(f32x2*)po = v0;
        if (oy + 1 < H) { f32x2 v1 = {y10, y11}; *(f32x2*)(po + W) = v1; }
    } else {
        po[0] = y00;
        if (ox + 1 < W) po[1] = y01;
        if (oy + 1 < H) {
            po[W] = y10;
            if (ox + 1 < W) po[W + 1] = y11;
        }
    }
}

// gridDim.y = number of input-channel splits KS.  KS == 1: the workgroup finishes its outputs.
// KS > 1: every split writes its partial (pre-bias) outputs to ws[split][O][H][W]; the split that
// arrives last at the panel's counter sums the partials in split order, adds bias, applies ReLU.
template <int MT, int NT>
__global__ void __launch_bounds__(kWinoThreads)
winograd_f23_mfma_kernel(const float* __restrict__ in, const float* __restrict__ U,
                         const float* __restrict__ bias, float* __restrict__ out,
                         int* __restrict__ counters, float* __restrict__ ws,
                         int W, int H, int I, int O, int tilesX, int T, int nTB, int nBlocks,
                         int chunksPerSplit, int relu, int vec2) {
    constexpr int TB = 32 * MT, OB = 32 * NT, KC = kWinoKC;
    constexpr int CSTEP = kWinoThreads / TB;        // channel distance between a lane's pairs
    constexpr int PAIRS = TB * KC / kWinoThreads;   // (tile, channel) pairs per lane and chunk (= MT)
    constexpr int VSZ = 16 * KC * TB;               // floats per V buffer
    extern __shared__ float lds[];                  // 2 * VSZ floats
    __shared__ int amLast;

    // ---- which panel: XCD-aware remap of the linear workgroup id -----------------------------
    const int perXcd = gridDim.x / kXcds;           // grid is padded to a multiple of kXcds
    const int logical = (blockIdx.x % kXcds) * perXcd + blockIdx.x / kXcds;
    if (logical >= nBlocks) return;
    const int o0 = (logical / nTB) * OB;
    const int t0 = (logical % nTB) * TB;
    const int split = blockIdx.y, nSplits = gridDim.y;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const size_t plane = (size_t)H * W;
    const int nChunksAll = (I + KC - 1) / KC;
    const int chBegin = split * chunksPerSplit;
    const int chEnd = min(nChunksAll, chBegin + chunksPerSplit);

    // ---- geometry of this lane's tile (same tile for the transform and for the epilogue) -------
    const int tl = tid % TB;                        // tile within the panel
    const int cl = tid / TB;                        // first channel-in-chunk of this lane
    const int tg = t0 + tl;
    const bool tileOk = tg < T;
    const int ty = tileOk ? tg / tilesX : 0, tx = tileOk ? tg % tilesX : 0;
    const int x0 = 2 * tx - 1, y0 = 2 * ty - 1;
    unsigned mask = 0;                              // bit 4r+s: input sample (y0+r, x0+s) exists
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int s = 0; s < 4; ++s)
            if (tileOk && y0 + r >= 0 && y0 + r < H && x0 + s >= 0 && x0 + s < W) mask |= 1u << (4 * r + s);
    const int winOff = y0 * W + x0;                 // may be negative; only used under the mask

    // ---- accumulators: [xi of this wave][channel tile][tile tile] -------------------------------
    f32x16 acc[4][NT][MT];
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[e][nt][mt][r] = 0.0f;

    f32x4 aCur[4][NT], aNxt[4][NT];                 // component ks = A operand of k-step ks
    float d[PAIRS][16];

    auto load_filters = [&](f32x4 (&a)[4][NT], int chunk) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int xi = 4 * wave + e;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int o = o0 + 32 * nt + l32;
                f32x4 z = {0.f, 0.f, 0.f, 0.f};
                a[e][nt] = (o < O) ? *(const f32x4*)(U + (((size_t)xi * nChunksAll + chunk) * O + o) * 8 + 4 * lhi) : z;
            }
        }
    };
    auto load_windows = [&](int c0) {
#pragma unroll
        for (int q = 0; q < PAIRS; ++q) {
            const int c = c0 + cl + q * CSTEP;
            const float* p = in + (size_t)c * plane + winOff;
            const unsigned m = (c < I) ? mask : 0u;
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int s = 0; s < 4; ++s)
                    d[q][4 * r + s] = ((m >> (4 * r + s)) & 1u) ? p[r * W + s] : 0.0f;
        }
    };
    // B^T d B (left factor first, like the reference kernel), then V[xi][c][t] into LDS.
    auto transform_store = [&](float* V) {
#pragma unroll
        for (int q = 0; q < PAIRS; ++q) {
            float m[16];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                m[s]      =  d[q][s]     - d[q][8 + s];
                m[4 + s]  =  d[q][4 + s] + d[q][8 + s];
                m[8 + s]  = -d[q][4 + s] + d[q][8 + s];
                m[12 + s] = -d[q][4 + s] + d[q][12 + s];
            }
            float* dst = V + (cl + q * CSTEP) * TB + tl;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float b0 = m[4 * r], b1 = m[4 * r + 1], b2 = m[4 * r + 2], b3 = m[4 * r + 3];
                dst[(4 * r + 0) * KC * TB] =  b0 - b2;
                dst[(4 * r + 1) * KC * TB] =  b1 + b2;
                dst[(4 * r + 2) * KC * TB] = -b1 + b2;
                dst[(4 * r + 3) * KC * TB] = -b1 + b3;
            }
        }
    };

    // ---- pipeline over this split's input-channel chunks ----------------------------------------
    if (chBegin < chEnd) {
        load_filters(aCur, chBegin);
        load_windows(chBegin * KC);
        transform_store(lds);
    }
    __syncthreads();

    for (int ch = chBegin; ch < chEnd; ++ch) {
        const bool more = ch + 1 < chEnd;
        if (more) {                                 // prefetch next chunk into registers
            load_filters(aNxt, ch + 1);
            load_windows((ch + 1) * KC);
        }
        const float* V = lds + ((ch - chBegin) & 1) * VSZ;
#pragma unroll
        for (int ks = 0; ks < KC / 2; ++ks) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float* vrow = V + ((4 * wave + e) * KC + 2 * ks + lhi) * TB + l32;
                float b[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) b[mt] = vrow[32 * mt];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[e][nt][mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(aCur[e][nt][ks], b[mt], acc[e][nt][mt], 0, 0, 0);
            }
        }
        if (more) {
            transform_store(lds + ((ch + 1 - chBegin) & 1) * VSZ);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) aCur[e][nt] = aNxt[e][nt];
        }
        __syncthreads();
    }

    // ---- epilogue: A^T m A (+ bias + ReLU), 8 output channels per pass through LDS --------------
    // Accumulator layout of the 32x32 MFMA: lane -> column (tile) lane%32; register r -> row
    // (output channel) 8*(r/4) + 4*(lane/32) + r%4.
    float* Ms = lds;                                // [16 xi][8 o][TB t]
    const bool direct = nSplits == 1;
    float* dstBase = direct ? out : ws + (size_t)split * O * plane;
    const int ox = 2 * tx, oy = 2 * ty;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr)
                        Ms[((4 * wave + e) * 8 + 4 * lhi + rr) * TB + 32 * mt + l32] = acc[e][nt][mt][4 * g + rr];
            __syncthreads();
#pragma unroll
            for (int q = 0; q < PAIRS; ++q) {
                const int oo = cl + q * CSTEP;      // 0..7
                const int o = o0 + 32 * nt + 8 * g + oo;
                float m[16];
#pragma unroll
                for (int xi = 0; xi < 16; ++xi) m[xi] = Ms[(xi * 8 + oo) * TB + tl];
                if (tileOk && o < O) {
                    float y00, y01, y10, y11;
                    wino_output_transform(m, y00, y01, y10, y11);
                    if (direct) {
                        if (bias) { const float bv = bias[o]; y00 += bv; y01 += bv; y10 += bv; y11 += bv; }
                        if (relu) { y00 = fmaxf(y00, 0.f); y01 = fmaxf(y01, 0.f); y10 = fmaxf(y10, 0.f); y11 = fmaxf(y11, 0.f); }
                    }
                    wino_store_tile(dstBase + (size_t)o * plane + (size_t)oy * W + ox, W, H, ox, oy, vec2, y00, y01, y10, y11);
                }
            }
            __syncthreads();
        }
    }
    if (direct) return;

    // ---- split-K: the last split to arrive reduces the partials in split order -------------------
    __threadfence();
    __syncthreads();
    if (tid == 0) amLast = (atomicAdd(&counters[logical], 1) == nSplits - 1);
    __syncthreads();
    if (!amLast) return;
    __threadfence();
    if (tileOk) {
        for (int oo = cl; oo < OB; oo += CSTEP) {
            const int o = o0 + oo;
            if (o >= O) break;
            const size_t off = (size_t)o * plane + (size_t)oy * W + ox;
            const bool right = ox + 1 < W, below = oy + 1 < H;
            float y00 = 0.f, y01 = 0.f, y10 = 0.f, y11 = 0.f;
            for (int sp = 0; sp < nSplits; ++sp) {
                const float* p = ws + (size_t)sp * O * plane + off;
                y00 += p[0];
                if (right) y01 += p[1];
                if (below) { y10 += p[W]; if (right) y11 += p[W + 1]; }
            }
            if (bias) { const float bv = bias[o]; y00 += bv; y01 += bv; y10 += bv; y11 += bv; }
            if (relu) { y00 = fmaxf(y00, 0.f); y01 = fmaxf(y01, 0.f); y10 = fmaxf(y10, 0.f); y11 = fmaxf(y11, 0.f); }
            wino_store_tile(out + off, W, H, ox, oy, vec2, y00, y01, y10, y11);
        }
    }
    if (tid == 0) counters[logical] = 0;
}

// variant = tile configuration (1..4, low 4 bits) | log2(number of input-channel splits) << 4
struct WinoCfg { int mt, nt, splits; };

static bool wino_variant(int variant, WinoCfg* c) {
    const int lg = (variant >> 4) & 0xf;
    if (lg > 6 || (variant >> 8)) return false;
    c->splits = 1 << lg;
    switch (variant & 0xf) {
        case 1: c->mt = 1; c->nt = 1; return true;
        case 2: c->mt = 2; c->nt = 1; return true;
        case 3: c->mt = 1; c->nt = 2; return true;
        case 4: c->mt = 2; c->nt = 2; return true;
        default: return false;
    }
}

struct WinoGeom { int tilesX, T, nTB, nOB, nBlocks, nChunks, chunksPerSplit, splits; };

static WinoGeom wino_geom(int W, int H, int I, int O, const WinoCfg& c) {
    WinoGeom g;
    g.tilesX = (W + 1) / 2;
    g.T = g.tilesX * ((H + 1) / 2);
    g.nTB = ceil_div(g.T, 32 * c.mt);
    g.nOB = ceil_div(O, 32 * c.nt);
    g.nBlocks = g.nTB * g.nOB;
    g.nChunks = ceil_div(I, kWinoKC);
    int splits = c.splits < g.nChunks ? c.splits : g.nChunks;
    g.chunksPerSplit = ceil_div(g.nChunks, splits);
    g.splits = ceil_div(g.nChunks, g.chunksPerSplit);      // no empty split
    return g;
}

// Workspace: [nBlocks arrival counters, padded to 64 ints][splits x O x H x W partial outputs].
static size_t wino_ws_counter_floats(const WinoGeom& g) { return (size_t)ceil_div(g.nBlocks, 64) * 64; }

template <int MT, int NT>
static int launch_wino(const float* in, const float* U, const float* bias, float* out, float* workspace,
                       int W, int H, int I, int O, int relu, const WinoCfg& c, hipStream_t s) {
    constexpr int TB = 32 * MT;
    const WinoGeom g = wino_geom(W, H, I, O, c);
    const int gridX = ceil_div(g.nBlocks, kXcds) * kXcds;
    const size_t ldsBytes = 2 * 16 * kWinoKC * TB * sizeof(float);
    const int vec2 = ((W & 1) == 0) && (((size_t)out & 7) == 0);
    int* counters = (int*)workspace;
    float* partials = workspace ? workspace + wino_ws_counter_floats(g) : nullptr;
    hipLaunchKernelGGL((winograd_f23_mfma_kernel<MT, NT>), dim3(gridX, g.splits), dim3(kWinoThreads), ldsBytes, s,
                       in, U, bias, out, counters, partials, W, H, I, O, g.tilesX, g.T, g.nTB, g.nBlocks,
                       g.chunksPerSplit, relu, vec2);
    return launched("winograd_f23_mfma_kernel");
}

}  // namespace drhip

using namespace drhip;

// Tile configuration for one layer: the biggest panels that still give every CU a workgroup; when
// even the smallest panels leave CUs idle (14x14 and 28x28 layers), split the input channels.
extern "C" int drhip_conv3x3_winograd_pick_variant(int W, int H, int I, int O) {
    const int T = ((W + 1) / 2) * ((H + 1) / 2);
    const int cus = num_cu();
    auto blocks = [&](int mt, int nt) { return ceil_div(T, 32 * mt) * ceil_div(O, 32 * nt); };
    int tile = 1;
    if (O > 32 && T > 32 && blocks(2, 2) >= 2 * cus) tile = 4;
    else if (T > 32 && blocks(2, 1) >= cus) tile = 2;
    else if (O > 32 && blocks(1, 2) >= cus) tile = 3;
    int lg = 0;
    if (tile == 1) {
        const int nChunks = ceil_div(I, kWinoKC);
        while (lg < 2 && (blocks(1, 1) << lg) < cus / 2 && (nChunks >> (lg + 1)) >= 2) ++lg;
    }
    return tile | (lg << 4);
}

extern "C" size_t drhip_conv3x3_winograd_filter_floats(int I, int O) {
    if (I <= 0 || O <= 0) return 0;
    return (size_t)16 * ceil_div(I, kWinoKC) * kWinoKC * O;
}

extern "C" size_t drhip_conv3x3_winograd_workspace_floats(int W, int H, int I, int O, int variant) {
    WinoCfg c;
    if (W <= 0 || H <= 0 || I <= 0 || O <= 0 || !wino_variant(variant, &c)) return 0;
    const WinoGeom g = wino_geom(W, H, I, O, c);
    if (g.splits <= 1) return 0;
    return wino_ws_counter_floats(g) + (size_t)g.splits * O * H * W;
}

extern "C" int drhip_winograd_filter_transform_f32(const float* w, float* U, int I, int O, void* stream) {
    DRHIP_REQUIRE(w && U, "drhip_winograd_filter_transform_f32: NULL tensor");
    DRHIP_REQUIRE(I > 0 && O > 0 && (long long)(I + 7) * O * 16 < (1ll << 31), "drhip_winograd_filter_transform_f32: bad shape I=%d O=%d", I, O);
    const int nChunks = ceil_div(I, kWinoKC);
    hipLaunchKernelGGL(winograd_filter_transform_kernel, dim3(ceil_div(nChunks * 8 * O, 256)), dim3(256), 0, as_stream(stream), w, U, I, O, nChunks);
    return launched("winograd_filter_transform_kernel");
}

extern "C" int drhip_conv3x3_winograd_f32(const float* in, const float* U, const float* bias, float* out,
                                          int W, int H, int I, int O, int relu, int variant,
                                          float* workspace, void* stream) {
    DRHIP_REQUIRE(in && U && out, "drhip_conv3x3_winograd_f32: NULL tensor");
    DRHIP_REQUIRE(W > 0 && H > 0 && I > 0 && O > 0, "drhip_conv3x3_winograd_f32: bad shape %dx%dx%d -> %d", W, H, I, O);
    DRHIP_REQUIRE((long long)W * H * I < (1ll << 31) && (long long)W * H * O < (1ll << 31) && (long long)(I + 7) * O * 16 < (1ll << 31),
                  "drhip_conv3x3_winograd_f32: tensor too large for 32-bit indexing");
    DRHIP_REQUIRE(((size_t)U & 15) == 0, "drhip_conv3x3_winograd_f32: transformed filters must be 16-byte aligned");
    if (variant == 0) {
        variant = drhip_conv3x3_winograd_pick_variant(W, H, I, O);
        if (!workspace) variant &= 0xf;            // no workspace offered: stay unsplit
    }
    WinoCfg c;
    DRHIP_REQUIRE(wino_variant(variant, &c), "drhip_conv3x3_winograd_f32: unknown variant %d", variant);
    const WinoGeom g = wino_geom(W, H, I, O, c);
    DRHIP_REQUIRE(g.splits == 1 || workspace, "drhip_conv3x3_winograd_f32: variant %d splits the input channels and needs a workspace", variant);
    DRHIP_REQUIRE(g.splits <= 65535 && (long long)g.splits * O * H * W < (1ll << 31), "drhip_conv3x3_winograd_f32: split workspace too large");
    hipStream_t s = as_stream(stream);
    if (c.mt == 1 && c.nt == 1) return launch_wino<1, 1>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
    if (c.mt == 2 && c.nt == 1) return launch_wino<2, 1>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
    if (c.mt == 1 && c.nt == 2) return launch_wino<1, 2>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
    return launch_wino<2, 2>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
}
