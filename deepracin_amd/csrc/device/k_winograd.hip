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
// A workgroup owns TB = 32*MT tiles x OB = 32*NT output channels for all 16 xi and consumes the
// input channels 8 at a time ("stage"):
//   1. a producer lane loads the 4x4 input window of one (tile, channel) pair straight from global
//      memory (zero padded by predication) two stages ahead of its use;
//   2. B^T d B in registers (32 adds), result written to LDS as V[xi][c][t]  (double buffered);
//   3. per k-step of 2 channels a consumer wave issues MFMAs with A = U_xi[c][o] (read from global
//      memory, where dR_prepare stored it so that the four k-steps of a stage are one 16-byte load
//      per lane and 1 KiB contiguous per wave) and B = V_xi[c][t] (one conflict-free ds_read_b32);
//   4. epilogue: accumulators go through LDS 16 output channels at a time so that one lane sees
//      all 16 xi of one (tile, o), applies A^T m A, bias, ReLU and stores the 2x2 pixels
//      (adjacent lanes = adjacent tiles, 8-byte stores, edge guarded for odd sizes).
// Workgroup ids are remapped so that each XCD (own L2) works on a contiguous range of
// output-channel panels and therefore touches only its share of U.
// Layers with few tiles (28x28, 14x14) cannot fill 256 CUs with panels alone: there the input
// channels are split over gridDim.y workgroups whose partial outputs are summed, in fixed order,
// by a small second kernel (deterministic, no float atomics, no device-scope fences).
#include "drhip_common.hpp"

namespace drhip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int kWinoThreads = 512;
constexpr int kWinoKC = 8;          // input channels per LDS stage
constexpr int kXcds = 8;            // L2 domains of MI355X

typedef float f32x4 __attribute__((ext_vector_type(4)));

// Layout of the transformed filters:  U[xi][chunk][o][8], chunk = c / 8, and inside a chunk the
// channel c%8 sits at position (c & 1) * 4 + ((c % 8) >> 1).  The MFMA A operand of k-step ks needs
// channel 2*ks + (lane / 32), so the four k-steps of a stage are ONE aligned 16-byte load per lane
// (position 4*(lane/32) + ks) and a wavefront reads 1 KiB contiguously.  Input channels >= I and
// output channels >= O (o is padded to a multiple of 32) hold zeros, so the loads need no predicate.
__host__ __device__ inline size_t wino_u_index(int xi, int c, int o, int nChunks, int Opad) {
    const int cc = c & 7;
    return (((size_t)xi * nChunks + (c >> 3)) * Opad + o) * 8 + (cc & 1) * 4 + (cc >> 1);
}
__host__ __device__ inline int wino_opad(int O) { return (O + 31) / 32 * 32; }

// U = G g G^T for g = w[c][o][3][3]; one lane per (padded c, o).
__global__ void __launch_bounds__(256)
winograd_filter_transform_kernel(const float* __restrict__ w, float* __restrict__ U, int I, int O, int nChunks) {
    const int Opad = wino_opad(O);
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= nChunks * 8 * Opad) return;
    const int c = idx / Opad, o = idx % Opad;
    float u[16];
    if (c < I && o < O) {
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
    for (int k = 0; k < 16; ++k) U[wino_u_index(k, c, o, nChunks, Opad)] = u[k];
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also fences global memory, which
// on gfx9 means s_waitcnt vmcnt(0): every global load issued for a later stage would have to land
// before the barrier and the software pipeline would collapse.  Nothing in this kernel passes data
// between lanes through global memory, so the LDS-only form is sufficient.
__device__ inline void wino_lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
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

// Workgroup = 512 lanes = 8 waves, split by role (a CU places wave i on SIMD i%4, so every SIMD
// hosts one wave of each role and interleaves their instructions):
//   waves 0-3  "consumers": wave w owns xi = 4w..4w+3 of the panel; they only read operands and
//              issue MFMAs (A = transformed filters from global memory, prefetched two stages
//              ahead; B = V from LDS);
//   waves 4-7  "producers": load the 4x4 input windows (two stages ahead, in registers), apply
//              B^T d B and write V[xi][c][t] into the LDS buffer the consumers will read next.
// One barrier per 8-channel stage keeps the two roles in lock step; V is double buffered, so the
// producers fill stage s+1 while the consumers multiply stage s.  The two roles run separate loops
// behind a wave-uniform (scalar) branch and execute the same number of barriers; keeping their
// code apart lets each loop wait only for its own loads and lets the registers of one role be
// reused by the other.
//
// gridDim.y = number of input-channel splits KS.  KS == 1: the workgroup finishes its outputs.
// KS > 1: every split stores its partial (pre-bias) 2x2 tiles, tile-major, to the workspace and
// winograd_split_reduce_kernel sums them in split order, adds the bias and applies ReLU.
template <int MT, int NT>
__global__ void __launch_bounds__(kWinoThreads)
winograd_f23_mfma_kernel(const float* __restrict__ in, const float* __restrict__ U,
                         const float* __restrict__ bias, float* __restrict__ out, float* __restrict__ ws,
                         int W, int H, int I, int O, int tilesX, int T, int nTB, int nBlocks,
                         int chunksPerSplit, int relu, int vec2) {
    constexpr int TB = 32 * MT, OB = 32 * NT, KC = kWinoKC;
    constexpr int PT = kWinoThreads / 2;            // lanes per role (256)
    constexpr int CSTEP = PT / TB;                  // channel distance between a producer lane's pairs
    constexpr int PAIRS = TB * KC / PT;             // (tile, channel) pairs per producer lane and stage (= MT)
    constexpr int VSZ = 16 * KC * TB;               // floats per V buffer
    constexpr int OSTEP = kWinoThreads / TB;        // output channels covered by one sweep of all lanes
    extern __shared__ float lds[];                  // 2 * VSZ floats

    // ---- which panel: XCD-aware remap of the linear workgroup id -----------------------------
    const int perXcd = gridDim.x / kXcds;           // grid is padded to a multiple of kXcds
    const int logical = (blockIdx.x % kXcds) * perXcd + blockIdx.x / kXcds;
    if (logical >= nBlocks) return;
    const int o0 = (logical / nTB) * OB;
    const int t0 = (logical % nTB) * TB;
    const int split = blockIdx.y, nSplits = gridDim.y;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // scalar: the role branch is uniform
    const int l32 = lane & 31, lhi = lane >> 5;
    const size_t plane = (size_t)H * W;
    const int nChunksAll = (I + KC - 1) / KC;
    const int chBegin = split * chunksPerSplit;
    const int chEnd = min(nChunksAll, chBegin + chunksPerSplit);    // > chBegin: the launcher creates no empty split
    const int Opad = wino_opad(O);
    float* const V0 = lds;
    float* const V1 = lds + VSZ;

    auto tile_xy = [&](int tLocal, int& txo, int& tyo) {
        const int tg = t0 + tLocal;
        const bool okT = tg < T;
        tyo = okT ? tg / tilesX : 0;
        txo = okT ? tg % tilesX : 0;
        return okT;
    };

    // ---- epilogue helper (all 512 lanes): read the 16 xi of one (tile, o) from LDS, transform, store
    float* Ms = lds;                                // [16 xi][16 o][TB t]  == 2 * VSZ floats
    const bool direct = nSplits == 1;
    const int et = tid % TB;                        // this lane's tile in the epilogue
    const int eo = tid / TB;                        // this lane's first channel within a 16-channel pass
    int etx, ety;
    const bool eTileOk = tile_xy(et, etx, ety);
    const int ox = 2 * etx, oy = 2 * ety;
    f32x4* wsTiles = direct ? nullptr : (f32x4*)ws + ((size_t)split * nBlocks + logical) * OB * TB;
    auto emit_pass = [&](int nt, int h) {
#pragma unroll
        for (int q = 0; q < 16 / OSTEP; ++q) {
            const int oo = eo + q * OSTEP;          // 0..15
            const int ol = 32 * nt + 16 * h + oo;
            const int o = o0 + ol;
            float m[16];
#pragma unroll
            for (int xi = 0; xi < 16; ++xi) m[xi] = Ms[(xi * 16 + oo) * TB + et];
            float y00, y01, y10, y11;
            wino_output_transform(m, y00, y01, y10, y11);
            if (direct) {
                if (eTileOk && o < O) {
                    if (bias) { const float bv = bias[o]; y00 += bv; y01 += bv; y10 += bv; y11 += bv; }
                    if (relu) { y00 = fmaxf(y00, 0.f); y01 = fmaxf(y01, 0.f); y10 = fmaxf(y10, 0.f); y11 = fmaxf(y11, 0.f); }
                    wino_store_tile(out + (size_t)o * plane + (size_t)oy * W + ox, W, H, ox, oy, vec2, y00, y01, y10, y11);
                }
            } else {
                f32x4 v = {y00, y01, y10, y11};
                wsTiles[(size_t)ol * TB + et] = v;  // whole panel, padding included: 1 KiB per wave
            }
        }
    };

    if (wave < 4) {
        // =================================== consumers ===========================================
        f32x16 acc[4][NT][MT];
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[e][nt][mt][r] = 0.0f;
        f32x4 aA[4][NT], aB[4][NT];                 // filters of two stages in flight; component ks = k-step
        // Unconditional loads: stages past the end re-read the last stage and are never used.
        auto load_filters = [&](f32x4 (&a)[4][NT], int chunk) {
            chunk = min(chunk, chEnd - 1);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int xi = 4 * wave + e;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    a[e][nt] = *(const f32x4*)(U + (((size_t)xi * nChunksAll + chunk) * Opad + (o0 + 32 * nt + l32)) * 8 + 4 * lhi);
            }
        };
        auto multiply = [&](const f32x4 (&a)[4][NT], const float* V) {
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
                            acc[e][nt][mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e][nt][ks], b[mt], acc[e][nt][mt], 0, 0, 0);
                }
            }
        };
        load_filters(aA, chBegin);
        load_filters(aB, chBegin + 1);
        wino_lds_barrier();                            // V0 holds the first stage
        int ch = chBegin;
        for (; ch + 1 < chEnd; ch += 2) {           // stage pairs: register sets A/B and buffers V0/V1 alternate
            multiply(aA, V0);
            load_filters(aA, ch + 2);
            wino_lds_barrier();
            multiply(aB, V1);
            load_filters(aB, ch + 3);
            wino_lds_barrier();
        }
        if (ch < chEnd) {                           // odd stage count: one more on set A
            multiply(aA, V0);
            wino_lds_barrier();
        }
        // Accumulator layout of the 32x32 MFMA: lane -> column (tile) lane%32; register r -> row
        // (output channel) 8*(r/4) + 4*(lane/32) + r%4.  16 channels per pass go through LDS.
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                        for (int rr = 0; rr < 8; ++rr)
                            Ms[((4 * wave + e) * 16 + 8 * (rr / 4) + 4 * lhi + (rr % 4)) * TB + 32 * mt + l32] = acc[e][nt][mt][8 * h + rr];
                wino_lds_barrier();
                emit_pass(nt, h);
                wino_lds_barrier();
            }
        }
    } else {
        // =================================== producers ===========================================
        const int ptid = tid - PT;
        const int tl = ptid % TB;                   // tile within the panel
        const int cl = ptid / TB;                   // first channel-in-stage of this lane
        int ptx, pty;
        const bool pTileOk = tile_xy(tl, ptx, pty);
        const int x0 = 2 * ptx - 1, y0 = 2 * pty - 1;
        unsigned mask = 0;                          // bit 4r+s: input sample (y0+r, x0+s) exists
        int rowOff[4], colOff[4];                   // clamped into the image: always a valid address
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            rowOff[r] = min(max(y0 + r, 0), H - 1) * W;
            colOff[r] = min(max(x0 + r, 0), W - 1);
#pragma unroll
            for (int s = 0; s < 4; ++s)
                if (pTileOk && y0 + r >= 0 && y0 + r < H && x0 + s >= 0 && x0 + s < W) mask |= 1u << (4 * r + s);
        }
        float dA[PAIRS][16], dB[PAIRS][16];         // raw windows of two stages in flight
        // Unconditional loads from clamped addresses; the zero padding is applied afterwards by a
        // select.  (A load under a per-lane predicate becomes its own branch region and the compiler
        // then waits for ALL outstanding loads at the next use, which serialises the pipeline.)
        auto load_windows = [&](float (&d)[PAIRS][16], int chunk) {
            chunk = min(chunk, chEnd - 1);
#pragma unroll
            for (int q = 0; q < PAIRS; ++q) {
                const int c = chunk * KC + cl + q * CSTEP;
                const float* p = in + (size_t)min(c, I - 1) * plane;
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int s = 0; s < 4; ++s) d[q][4 * r + s] = p[rowOff[r] + colOff[s]];
            }
        };
        // B^T d B (left factor first, like the reference kernel), then V[xi][c][t] into LDS.
        auto transform_store = [&](const float (&draw)[PAIRS][16], float* V, int chunk) {
#pragma unroll
            for (int q = 0; q < PAIRS; ++q) {
                const unsigned mq = (chunk * KC + cl + q * CSTEP < I) ? mask : 0u;
                float d[16], m[16];
#pragma unroll
                for (int k = 0; k < 16; ++k) d[k] = ((mq >> k) & 1u) ? draw[q][k] : 0.0f;   // zero padding
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    m[s]      =  d[s]     - d[8 + s];
                    m[4 + s]  =  d[4 + s] + d[8 + s];
                    m[8 + s]  = -d[4 + s] + d[8 + s];
                    m[12 + s] = -d[4 + s] + d[12 + s];
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
        load_windows(dA, chBegin);
        load_windows(dB, chBegin + 1);
        transform_store(dA, V0, chBegin);
        load_windows(dA, chBegin + 2);
        wino_lds_barrier();                            // V0 holds the first stage
        // Transforms are unconditional: past the last stage they re-transform the (clamped) last
        // windows into the buffer nobody reads any more, which keeps the loop free of branches that
        // would make the compiler wait for every outstanding load.
        int ch = chBegin;
        for (; ch + 1 < chEnd; ch += 2) {
            transform_store(dB, V1, ch + 1);
            load_windows(dB, ch + 3);
            wino_lds_barrier();
            transform_store(dA, V0, ch + 2);
            load_windows(dA, ch + 4);
            wino_lds_barrier();
        }
        if (ch < chEnd) {
            transform_store(dB, V1, ch + 1);
            wino_lds_barrier();
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                wino_lds_barrier();
                emit_pass(nt, h);
                wino_lds_barrier();
            }
        }
    }
}

// out[o][2x2 tile] = act(bias[o] + sum over splits of the partial tile), splits added in order.
// One lane per (o, tile); partials are [split][panel][o in panel][tile in panel] float4.
__global__ void __launch_bounds__(256)
winograd_split_reduce_kernel(const float* __restrict__ ws, const float* __restrict__ bias, float* __restrict__ out,
                             int W, int H, int O, int tilesX, int T, int nTB, int nBlocks, int TB, int OB,
                             int nSplits, int relu, int vec2) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;      // over nBlocks * OB * TB
    if (idx >= nBlocks * OB * TB) return;
    const int tLocal = idx % TB, ol = (idx / TB) % OB, panel = idx / (TB * OB);
    const int o = (panel / nTB) * OB + ol, tg = (panel % nTB) * TB + tLocal;
    if (o >= O || tg >= T) return;
    const f32x4* p = (const f32x4*)ws + idx;
    const size_t splitStride = (size_t)nBlocks * OB * TB;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    int sp = 0;
    for (; sp + 4 <= nSplits; sp += 4) {            // 4 independent 16-byte loads in flight
        f32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = p[(size_t)(sp + u) * splitStride];
#pragma unroll
        for (int u = 0; u < 4; ++u) s += v[u];
    }
    for (; sp < nSplits; ++sp) s += p[(size_t)sp * splitStride];
    if (bias) s += bias[o];
    if (relu) { s[0] = fmaxf(s[0], 0.f); s[1] = fmaxf(s[1], 0.f); s[2] = fmaxf(s[2], 0.f); s[3] = fmaxf(s[3], 0.f); }
    const int ox = 2 * (tg % tilesX), oy = 2 * (tg / tilesX);
    wino_store_tile(out + (size_t)o * H * W + (size_t)oy * W + ox, W, H, ox, oy, vec2, s[0], s[1], s[2], s[3]);
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

// Workspace: [splits][panel][o in panel][tile in panel] partial 2x2 tiles (float4 each).

template <int MT, int NT>
static int launch_wino(const float* in, const float* U, const float* bias, float* out, float* workspace,
                       int W, int H, int I, int O, int relu, const WinoCfg& c, hipStream_t s) {
    constexpr int TB = 32 * MT, OB = 32 * NT;
    const WinoGeom g = wino_geom(W, H, I, O, c);
    const int gridX = ceil_div(g.nBlocks, kXcds) * kXcds;
    const size_t ldsBytes = 2 * 16 * kWinoKC * TB * sizeof(float);
    const int vec2 = ((W & 1) == 0) && (((size_t)out & 7) == 0);
    hipLaunchKernelGGL((winograd_f23_mfma_kernel<MT, NT>), dim3(gridX, g.splits), dim3(kWinoThreads), ldsBytes, s,
                       in, U, bias, out, workspace, W, H, I, O, g.tilesX, g.T, g.nTB, g.nBlocks,
                       g.chunksPerSplit, relu, vec2);
    if (int rc = launched("winograd_f23_mfma_kernel")) return rc;
    if (g.splits > 1) {
        const int total = g.nBlocks * OB * TB;
        hipLaunchKernelGGL(winograd_split_reduce_kernel, dim3(ceil_div(total, 256)), dim3(256), 0, s,
                           workspace, bias, out, W, H, O, g.tilesX, g.T, g.nTB, g.nBlocks, TB, OB, g.splits, relu, vec2);
        return launched("winograd_split_reduce_kernel");
    }
    return DRHIP_OK;
}

}  // namespace drhip

using namespace drhip;

// Configuration for one layer, from measurements on MI355X (256 CUs):
//   - many tiles (>= 2048, i.e. 112x112 and larger): 32 tiles x 64 channels per workgroup -- every
//     transformed input element then feeds twice the MFMAs;
//   - otherwise 32 x 32 panels, and when those give fewer than ~200 workgroups (28x28, 14x14) the
//     input channels are split until they do, keeping at least 4 stages of 8 channels per split.
extern "C" int drhip_conv3x3_winograd_pick_variant(int W, int H, int I, int O) {
    const int T = ((W + 1) / 2) * ((H + 1) / 2);
    const int cus = num_cu();
    if (T >= 2048 && O >= 64) return 3;
    const int panels = ceil_div(T, 32) * ceil_div(O, 32);
    const int nChunks = ceil_div(I, kWinoKC);
    int lg = 0;
    while (lg < 4 && (panels << lg) < (3 * cus) / 4 && (nChunks >> (lg + 1)) >= 4) ++lg;
    return 1 | (lg << 4);
}

extern "C" size_t drhip_conv3x3_winograd_filter_floats(int I, int O) {
    if (I <= 0 || O <= 0) return 0;
    return (size_t)16 * ceil_div(I, kWinoKC) * kWinoKC * wino_opad(O);
}

extern "C" size_t drhip_conv3x3_winograd_workspace_floats(int W, int H, int I, int O, int variant) {
    WinoCfg c;
    if (W <= 0 || H <= 0 || I <= 0 || O <= 0 || !wino_variant(variant, &c)) return 0;
    const WinoGeom g = wino_geom(W, H, I, O, c);
    if (g.splits <= 1) return 0;
    return (size_t)g.splits * g.nBlocks * (32 * c.nt) * (32 * c.mt) * 4;
}

extern "C" int drhip_winograd_filter_transform_f32(const float* w, float* U, int I, int O, void* stream) {
    DRHIP_REQUIRE(w && U, "drhip_winograd_filter_transform_f32: NULL tensor");
    DRHIP_REQUIRE(I > 0 && O > 0 && (long long)(I + 7) * O * 16 < (1ll << 31), "drhip_winograd_filter_transform_f32: bad shape I=%d O=%d", I, O);
    const int nChunks = ceil_div(I, kWinoKC);
    hipLaunchKernelGGL(winograd_filter_transform_kernel, dim3(ceil_div(nChunks * 8 * wino_opad(O), 256)), dim3(256), 0, as_stream(stream), w, U, I, O, nChunks);
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
    DRHIP_REQUIRE(g.splits <= 65535, "drhip_conv3x3_winograd_f32: too many input-channel splits");
    hipStream_t s = as_stream(stream);
    if (c.mt == 1 && c.nt == 1) return launch_wino<1, 1>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
    if (c.mt == 2 && c.nt == 1) return launch_wino<2, 1>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
    if (c.mt == 1 && c.nt == 2) return launch_wino<1, 2>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
    return launch_wino<2, 2>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
}
