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

#include <cfloat>
#include <cstdlib>
#include <cstring>
#include <type_traits>

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
    const int tileX = blockIdx.x, tileY = blockIdx.y;       // (a 3-D grid: no integer division in front of the first loads)
    const int o0 = blockIdx.z * OCT;
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
    const int tileX = blockIdx.x, tileY = blockIdx.y;       // (a 3-D grid: no integer division in front of the first loads)
    const int o0 = blockIdx.z * OCT;
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


// First layer and the 3x3 / stride-2 max pooling behind it in one kernel, on the matrix cores.
//
// A workgroup owns a 4x4 tile of POOLED pixels x 16*MB channels.  The pooling windows of that tile
// cover 9x9 convolution outputs (81, dealt to six wavefronts as six 16-pixel MFMA columns); each
// wavefront computes its 16 pixels for all channels as a small GEMM over k = (channel, tap), 9*I <= 36
// values = up to 9 k-steps of v_mfma_f32_16x16x4_f32 (B: gathered input samples, zero padding by
// select; A: the filters [I][O][9] as they are), adds bias, applies ReLU, and parks the pixels in
// LDS; then all lanes pool out of LDS in the pooling kernel's scan order.  Convolution outputs
// outside the map count as 0.0, exactly what the pooling kernel reads there.  The full-resolution
// tensor (3.2 MB for SqueezeNet's conv1) is never written; the halo costs (9/8)^2 = 1.27x the MFMAs.
constexpr int kFpPool = 4;                          // pooled tile edge
constexpr int kFpConv = 2 * kFpPool + 1;            // convolution tile edge
constexpr int kFpPix = kFpConv * kFpConv;           // 81
constexpr int kFpWaves = (kFpPix + 15) / 16;        // 6
constexpr int kFpThreads = 64 * kFpWaves;
constexpr int kFpPitch = 16 * kFpWaves + 1;         // LDS row pitch (floats)
typedef float f32x4d __attribute__((ext_vector_type(4)));

template <int MB, int KS>                           // KS = k-steps = ceil(9*I / 4)
__global__ void __launch_bounds__(kFpThreads)
conv3x3_fewc_pool3s2_kernel(const float* __restrict__ in, const float* __restrict__ w, const float* __restrict__ bias,
                            float* __restrict__ out, unsigned wh, unsigned io, unsigned woho, unsigned cfg) {
    // (12 dwords of arguments, which arrive in SGPRs with the wave: wh = W | H << 16, io = I | O << 16,
    // woho = Wo | Ho << 16, cfg = sx | sy << 4 | relu << 8)
    const int W = (int)(wh & 0xffffu), H = (int)(wh >> 16), I = (int)(io & 0xffffu), O = (int)(io >> 16);
    const int Wo = (int)(woho & 0xffffu), Ho = (int)(woho >> 16), Wp = (Wo + 1) >> 1, Hp = (Ho + 1) >> 1;
    const int sx = (int)(cfg & 15u), sy = (int)((cfg >> 4) & 15u), relu = (int)((cfg >> 8) & 1u);
    __shared__ float convT[16 * MB * kFpPitch];
    __shared__ float wT[4 * KS * 16 * MB];          // filters as [k = (channel, tap)][channel out], zero padded
    __shared__ float biasT[16 * MB];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, lk = lane >> 4;
    const int tileX = blockIdx.x, tileY = blockIdx.y;       // (a 3-D grid: no integer division in front of the first loads)
    const int o0 = blockIdx.z * 16 * MB;

    const int q = 16 * wave + j;                    // convolution pixel within the 9x9 tile
    const int ry = q / kFpConv, rx = q % kFpConv;
    const int cy = 2 * kFpPool * tileY + ry, cx = 2 * kFpPool * tileX + rx;
    const bool pixOk = q < kFpPix && cy < Ho && cx < Wo;

    // B operands: this lane's input samples, gathered now ...
    float b[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int kidx = 4 * ks + lk;               // (channel, tap)
        const int c = kidx / 9, tap = kidx % 9;
        const int iy = cy * sy + tap / 3 - 1, ix = cx * sx + tap % 3 - 1;
        const bool ok = pixOk && kidx < 9 * I && iy >= 0 && iy < H && ix >= 0 && ix < W;
        const float v = in[((size_t)min(c, I - 1) * H + min(max(iy, 0), H - 1)) * W + min(max(ix, 0), W - 1)];
        b[ks] = ok ? v : 0.0f;
    }
    // ... while the workgroup's filters go to LDS once, read in their own order (contiguous per
    // input channel: w[c][o0 ..][9]) and written transposed, so that an MFMA A operand is 16
    // consecutive floats.
    constexpr int OBc = 16 * MB;
    constexpr int kRounds = (4 * KS * OBc + kFpThreads - 1) / kFpThreads;
    float fv[kRounds];
    int dst[kRounds];
#pragma unroll
    for (int u = 0; u < kRounds; ++u) {             // all loads first (clamped addresses), one trip to memory
        const int e = tid + u * kFpThreads;
        // e -> (c, o local, tap) in memory order for real filter values, the zero padding after them
        const bool real = e < 9 * I * OBc;
        const int c = min(e / (9 * OBc), I - 1), rest = e % (9 * OBc);
        const int ol = real ? rest / 9 : (e - 9 * I * OBc) % OBc;
        const int kidx = real ? c * 9 + rest % 9 : 9 * I + (e - 9 * I * OBc) / OBc;
        const float f = w[((size_t)c * O + min(o0 + ol, O - 1)) * 9 + rest % 9];
        fv[u] = (real && o0 + ol < O) ? f : 0.0f;
        dst[u] = e < 4 * KS * OBc ? kidx * OBc + ol : -1;
    }
    float bv = 0.0f;                                // the bias comes along in the same trip
    if (tid < OBc && bias) bv = bias[min(o0 + tid, O - 1)];
#pragma unroll
    for (int u = 0; u < kRounds; ++u)
        if (dst[u] >= 0) wT[dst[u]] = fv[u];
    if (tid < OBc) biasT[tid] = bv;
    __syncthreads();
    float a[MB][KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int m = 0; m < MB; ++m) a[m][ks] = wT[(4 * ks + lk) * OBc + 16 * m + j];
    f32x4d acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = f32x4d{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[m][ks], b[ks], acc[m], 0, 0, 0);

    // D: lane -> pixel j, register r -> channel 4*lk + r of block m
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int ch = 16 * m + 4 * lk + r;
            float v = acc[m][r] + biasT[ch];
            if (relu) v = fmaxf(v, 0.0f);
            convT[ch * kFpPitch + q] = pixOk ? v : 0.0f;
        }
    __syncthreads();

    for (int idx = tid; idx < 16 * MB * kFpPool * kFpPool; idx += kFpThreads) {
        const int ch = idx / (kFpPool * kFpPool), pp = idx % (kFpPool * kFpPool);
        const int ppy = pp / kFpPool, ppx = pp % kFpPool;
        const int py = kFpPool * tileY + ppy, px = kFpPool * tileX + ppx;
        if (py < Hp && px < Wp && o0 + ch < O) {
            float r = -FLT_MAX;
#pragma unroll
            for (int dy = 0; dy < 3; ++dy)
#pragma unroll
                for (int dx = 0; dx < 3; ++dx) {
                    const float v = convT[ch * kFpPitch + (2 * ppy + dy) * kFpConv + 2 * ppx + dx];
                    if (v > r) r = v;
                }
            store_through(out + ((size_t)(o0 + ch) * Hp + py) * Wp + px, r);
        }
    }
}

// First layer without a pooling behind it (VGG16's conv1_1: 224x224x3 -> 64, stride 1): the same
// small GEMM over k = (channel, tap) on v_mfma_f32_16x16x4_f32.  A workgroup of four waves owns a
// 16 x 4 block of output pixels x 16*MB channels; a wave owns one row of 16 pixels (one MFMA column),
// gathers its 9*I input samples (16 consecutive x per load), takes the filters from LDS (transposed
// there once per workgroup) and stores 64-byte rows per channel.
template <int MB, int KS>
__global__ void __launch_bounds__(256)
conv3x3_fewc_mfma_kernel(const float* __restrict__ in, const float* __restrict__ w, const float* __restrict__ bias,
                         float* __restrict__ out, int W, int H, int I, int O, int Wo, int Ho,
                         int sx, int sy, int tilesX, int relu) {
    constexpr int OBc = 16 * MB;
    __shared__ float wT[4 * KS * OBc];              // filters as [k = (channel, tap)][channel out], zero padded
    __shared__ float biasT[OBc];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, lk = lane >> 4;
    const int tileX = blockIdx.x, tileY = blockIdx.y;       // (a 3-D grid: no integer division in front of the first loads)
    const int o0 = blockIdx.z * OBc;
    const int x = tileX * 16 + j, y = tileY * 4 + wave;
    const bool pixOk = x < Wo && y < Ho;

    float b[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int kidx = 4 * ks + lk;               // (channel, tap)
        const int c = kidx / 9, tap = kidx % 9;
        const int iy = y * sy + tap / 3 - 1, ix = x * sx + tap % 3 - 1;
        const bool ok = pixOk && kidx < 9 * I && iy >= 0 && iy < H && ix >= 0 && ix < W;
        const float v = in[((size_t)min(c, I - 1) * H + min(max(iy, 0), H - 1)) * W + min(max(ix, 0), W - 1)];
        b[ks] = ok ? v : 0.0f;
    }
    constexpr int kRounds = (4 * KS * OBc + 255) / 256;
    float fv[kRounds];
    int dst[kRounds];
#pragma unroll
    for (int u = 0; u < kRounds; ++u) {             // e -> (c, o local, tap) in memory order, then the zero padding
        const int e = tid + u * 256;
        const bool real = e < 9 * I * OBc;
        const int c = min(e / (9 * OBc), I - 1), rest = e % (9 * OBc);
        const int ol = real ? rest / 9 : (e - 9 * I * OBc) % OBc;
        const int kidx = real ? c * 9 + rest % 9 : 9 * I + (e - 9 * I * OBc) / OBc;
        const float f = w[((size_t)c * O + min(o0 + ol, O - 1)) * 9 + rest % 9];
        fv[u] = (real && o0 + ol < O) ? f : 0.0f;
        dst[u] = e < 4 * KS * OBc ? kidx * OBc + ol : -1;
    }
    float bv = 0.0f;
    if (tid < OBc && bias) bv = bias[min(o0 + tid, O - 1)];
#pragma unroll
    for (int u = 0; u < kRounds; ++u)
        if (dst[u] >= 0) wT[dst[u]] = fv[u];
    if (tid < OBc) biasT[tid] = bv;
    __syncthreads();

    f32x4d acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = f32x4d{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int m = 0; m < MB; ++m)
            acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(wT[(4 * ks + lk) * OBc + 16 * m + j], b[ks], acc[m], 0, 0, 0);

    // D: lane -> pixel j, register r -> channel 4*lk + r of block m
    if (pixOk) {
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int ch = 16 * m + 4 * lk + r;
                if (o0 + ch < O) {
                    float v = acc[m][r] + biasT[ch];
                    if (relu) v = fmaxf(v, 0.0f);
                    store_through(out + ((size_t)(o0 + ch) * Ho + y) * Wo + x, v);
                }
            }
    }
}

// Direct 3x3 convolution on the matrix cores (stride 1 or 2, more than 4 input channels): the
// implicit GEMM  out[o][p] = sum_{c,tap} w[c][o][tap] * in[c][pixel p shifted by tap],  K = 9*I,
// on v_mfma_f32_32x32x2_f32, with no operand staged in LDS:
//
//   * the filters are laid out once, at prepare time, as F[tap][c/8][o][8] -- the layout of the Winograd
//     kernel's transformed filters with 9 taps in place of 16 transform positions: inside a chunk of 8
//     channels channel c%8 sits at position (c&1)*4 + (c%8)/2, so the A operands of the four k-steps of a
//     stage (k-step ks needs channel 2ks + lane/32) are ONE aligned 16-byte buffer load per lane and tap;
//   * the B operands are the input itself: a lane owns one output pixel (lane%32) and one channel parity
//     (lane/32) and loads the three rows of its 3x3 window with one 16-byte buffer load each (rows outside
//     the image carry an offset beyond the resource and read 0.0; the samples left and right of the image
//     are zeroed by selects).  Neighbouring lanes load overlapping windows; the CU's L1 absorbs that.
//   * a workgroup owns 32 consecutive output pixels (row-major) x 32*NT output channels; its KW waves deal
//     the 8-channel stages round-robin (wave w takes stages w, w+KW, ...), the next stage's rows in flight
//     during the 36*NT MFMAs of the current one and the filters of a tap reloaded right behind its MFMAs;
//     the KW partial tiles meet in LDS at the end and are added in wave order (fixed summation order),
//     then bias, ReLU and 128-byte row stores.
// Per stage and wave: 12 + 9*NT loads and ~50 VALU instructions (the selects) for 36*NT MFMAs.
typedef float f32x16d __attribute__((ext_vector_type(16)));
typedef float f32x4d __attribute__((ext_vector_type(4)));
constexpr unsigned kDmBufferFlags = 0x00020000u;    // dword 3 of a gfx9 raw buffer resource (32-bit data format)
constexpr unsigned kDmOutOfRange = 0x80000000u;     // byte offset no resource of at most 2 GiB contains
constexpr int kDmKC = 8;                            // input channels per stage (4 MFMA k-steps)
constexpr int kDmPartPitch = 33;

__host__ __device__ inline int dm_opad(int O) { return (O + 31) / 32 * 32; }
__host__ __device__ inline size_t dm_filter_index(int tap, int c, int o, int nChunks, int Opad) {
    const int cc = c & 7;
    return (((size_t)tap * nChunks + (c >> 3)) * Opad + o) * 8 + (cc & 1) * 4 + (cc >> 1);
}

// F[tap][c/8][o][8] from w[c][o][3][3]; channels >= I and output channels >= O (padded to a multiple of 32) are zero.
__global__ void __launch_bounds__(256)
direct_filter_layout_kernel(const float* __restrict__ w, float* __restrict__ F, int I, int O, int nChunks) {
    const int Opad = dm_opad(O);
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= nChunks * 8 * Opad) return;
    const int c = idx / Opad, o = idx % Opad;
    const bool real = c < I && o < O;
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) F[dm_filter_index(tap, c, o, nChunks, Opad)] = real ? w[((size_t)c * O + o) * 9 + tap] : 0.0f;
}

__device__ inline f32x4d dm_buf_load4(__amdgpu_buffer_rsrc_t r, unsigned voffset, unsigned soffset) {
    return __builtin_bit_cast(f32x4d, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voffset, (int)soffset, 0));
}

template <int NT, int S>                    // 32*NT output channels per workgroup; stride (both directions) 1 or 2
__global__ void __launch_bounds__(512)
conv3x3_direct_mfma_kernel(const float* __restrict__ in, const float* __restrict__ F, const float* __restrict__ bias,
                           float* __restrict__ out, unsigned wh, unsigned io, unsigned WoMul, unsigned cfg) {
    // 12 dwords of arguments, all of which arrive in SGPRs with the wave (nothing is read from the dispatch packet:
    // a scalar load in front of the first vector loads is a round trip of its own in every workgroup):
    // wh = W | H << 16, io = I | O << 16, WoMul / cfg & 31 = multiplier / shift of the division by Wo,
    // cfg bit 5 = ReLU, cfg >> 8 = waves per workgroup.
    constexpr int OB = 32 * NT, KC = kDmKC;
    const int W = (int)(wh & 0xffffu), H = (int)(wh >> 16), I = (int)(io & 0xffffu), O = (int)(io >> 16);
    const int Wo = W / S, Ho = H / S;
    const FastDiv Wod = {(unsigned)Wo, WoMul, cfg & 31u};
    const int relu = (int)((cfg >> 5) & 1u), KW = (int)(cfg >> 8);
    constexpr int NA = NT == 1 ? 2 : 1;     // accumulators per channel block: two independent MFMA chains at least
    extern __shared__ float part[];         // [KW][OB][kDmPartPitch]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lhi = lane >> 5;
    const int o0 = blockIdx.y * OB, p0 = blockIdx.x * 32;
    const int P = Wo * Ho, plane = H * W;
    const int nChunks = (I + KC - 1) / KC, Opad = dm_opad(O);

    // this lane's output pixel and the byte offsets of its three window rows
    const int p = p0 + l32;
    const bool pOk = p < P;
    const int pc = min(p, P - 1);
    const int y = fast_div(pc, Wod), x = pc - y * Wo;
    // The window starts at column x*S - 1.  Only x = 0 starts left of the image: that lane loads from column 0
    // and shifts its samples up by one (a negative offset would zero the whole load for the first pixel).
    const bool shifted = x == 0;
    const int xLoad = x * S - 1 + (shifted ? 1 : 0);
    const bool c2ok = x * S + 1 < W;        // the third sample of the window exists
    unsigned offRow[3];
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        const int iy = y * S - 1 + d;
        offRow[d] = (pOk && iy >= 0 && iy < H) ? 4u * (unsigned)(lhi * plane + iy * W + xLoad) : kDmOutOfRange;
    }

    const __amdgpu_buffer_rsrc_t rIn = __builtin_amdgcn_make_buffer_rsrc((void*)in, 0, I * plane * 4, kDmBufferFlags);
    const __amdgpu_buffer_rsrc_t rF = __builtin_amdgcn_make_buffer_rsrc((void*)F, 0, 9 * nChunks * Opad * 8 * 4, kDmBufferFlags);
    const unsigned fOff = 4u * (unsigned)((o0 + l32) * 8 + 4 * lhi);

    // rows of channels cbase + 2ks + lhi, ks = 0..3.  Plain form: one resource for the tensor, the channel in the
    // scalar offset (chunks known to lie inside the tensor).  Ranged form: the resource starts at channel cbase and
    // ends with the tensor, so channels >= I read 0.0 (ragged last chunk, prefetch past the end).
    auto load_rows_plain = [&](f32x4d (&raw)[4][3], int cbase) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int d = 0; d < 3; ++d) raw[ks][d] = dm_buf_load4(rIn, offRow[d], 4u * (unsigned)((cbase + 2 * ks) * plane));
    };
    auto load_rows_ranged = [&](f32x4d (&raw)[4][3], int cbase) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const int c = cbase + 2 * ks, left = max(I - c, 0);
            const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)(in + (size_t)min(c, I) * plane), 0, left * plane * 4, kDmBufferFlags);
#pragma unroll
            for (int d = 0; d < 3; ++d) raw[ks][d] = dm_buf_load4(r, offRow[d], 0u);
        }
    };
    auto load_filters = [&](f32x4d (&f)[NT], int tap, int chunk) {
        const unsigned soff = 4u * (unsigned)((tap * nChunks + chunk) * Opad * 8);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) f[nt] = dm_buf_load4(rF, fOff + 4u * (unsigned)(nt * 32 * 8), soff);
    };

    // the epilogue's bias values are requested now: thread tid finishes the elements tid + q*blockDim.x of the tile
    constexpr int kMaxEpi = 8;                          // (the first 8 of them: all, from two or four waves per workgroup on)
    float biasEarly[kMaxEpi];
#pragma unroll
    for (int q = 0; q < kMaxEpi; ++q) {
        const int idx = tid + q * (64 * KW);
        biasEarly[q] = (bias && idx < OB * 32) ? bias[min(o0 + (idx >> 5), O - 1)] : 0.0f;
    }

    f32x16d acc[NT][NA];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int a = 0; a < NA; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[nt][a][r] = 0.0f;

    f32x4d raw[4][3];
    f32x4d f[9][NT];
    if (wave < nChunks) {
        load_rows_ranged(raw, wave * KC);
#pragma unroll
        for (int tap = 0; tap < 9; ++tap) load_filters(f[tap], tap, wave);
    }

    auto stage = [&](int ch, auto plainNext) {
        const int next = min(ch + KW, nChunks - 1);
        // the window samples of this stage, padding applied: b[ks][3*d + e] = in[c][y*S - 1 + d][x*S - 1 + e]
        float b[4][9];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int d = 0; d < 3; ++d) {
                const f32x4d v = raw[ks][d];
                b[ks][3 * d + 0] = shifted ? 0.0f : v[0];
                b[ks][3 * d + 1] = shifted ? v[0] : v[1];
                const float third = shifted ? v[1] : v[2];
                b[ks][3 * d + 2] = c2ok ? third : 0.0f;
            }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (decltype(plainNext)::value) load_rows_plain(raw, (ch + KW) * KC);
        else load_rows_ranged(raw, (ch + KW) * KC);
#pragma unroll
        for (int tap = 0; tap < 9; ++tap) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    acc[nt][tap % NA] = __builtin_amdgcn_mfma_f32_32x32x2f32(f[tap][nt][ks], b[ks][tap], acc[nt][tap % NA], 0, 0, 0);
            load_filters(f[tap], tap, next);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // stages whose successor (KW further on) is a complete chunk prefetch in the plain form
    // (plain form only for successor chunks in front of the one with the tensor's last channel: the scalar offset is
    // not range-checked, and the row loads of the last pixels of the last row reach up to two samples past the row)
    const int chMain = (I - 1) / KC - KW;
    int ch = wave;
    for (; ch < chMain; ch += KW) stage(ch, std::true_type{});
    for (; ch < nChunks; ch += KW) stage(ch, std::false_type{});

    // partial tiles of the KW waves -> LDS -> summed in wave order.  Accumulator layout of the 32x32 MFMA:
    // lane -> column (pixel) lane%32; register r -> row (channel) 8*(r/4) + 4*(lane/32) + r%4.
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float v = acc[nt][0][r];
            if constexpr (NA == 2) v += acc[nt][1][r];
            part[(wave * OB + 32 * nt + 8 * (r / 4) + 4 * lhi + (r % 4)) * kDmPartPitch + l32] = v;
        }
    // LDS-only barrier: __syncthreads() would also wait for the outstanding (unused) prefetches
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    auto finish = [&](int idx, float biasValue) {
        const int ol = idx >> 5, pl = idx & 31;
        const int o = o0 + ol, pp = p0 + pl;
        float v = 0.0f;
        for (int k = 0; k < KW; ++k) v += part[(k * OB + ol) * kDmPartPitch + pl];
        if (o < O && pp < P) {
            v += biasValue;
            if (relu) v = fmaxf(v, 0.0f);
            store_through(out + (size_t)o * P + pp, v);
        }
    };
#pragma unroll
    for (int q = 0; q < kMaxEpi; ++q) {
        const int idx = tid + q * (64 * KW);
        if (idx < OB * 32) finish(idx, biasEarly[q]);
    }
    for (int idx = tid + kMaxEpi * (64 * KW); idx < OB * 32; idx += 64 * KW)      // one wave per workgroup only
        finish(idx, bias ? bias[min(o0 + (idx >> 5), O - 1)] : 0.0f);
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
    if (tilesY > 65535 || ceil_div(O, OCT) > 65535) return fail(DRHIP_EINVAL, "drhip_conv2d_direct_f32: %d rows of tiles x %d channel blocks exceed the launch grid", tilesY, ceil_div(O, OCT));
    dim3 grid(tilesX, tilesY, ceil_div(O, OCT)), block(kDirThreads);
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
    const char* valuOnly = getenv("DR_DIRECT_VALU");
    const bool valu = valuOnly && strcmp(valuOnly, "1") == 0;
    if (I <= 4 && kw == 3 && kh == 3 && !valu) {
        // first layers on the matrix cores: 16 x 4 pixels x 64 (32) channels per workgroup
        const int Wo = W / strideX, Ho = H / strideY;
        const int tilesX = ceil_div(Wo, 16), tilesY = ceil_div(Ho, 4);
        const int ks = ceil_div(9 * I, 4);
        const bool wide = O > 32;
        DRHIP_REQUIRE(tilesY <= 65535 && O <= 32 * 65535, "drhip_conv2d_direct_f32: tensor exceeds the launch grid");
        const dim3 grid(tilesX, tilesY, ceil_div(O, wide ? 64 : 32)), block(256);
#define DRHIP_FM(MBV, KSV) launch((conv3x3_fewc_mfma_kernel<MBV, KSV>), grid, block, 0, s0, in, w, bias, out, W, H, I, O, Wo, Ho, strideX, strideY, tilesX, relu)
#define DRHIP_FM_K(MBV) do { if (ks == 3) DRHIP_FM(MBV, 3); else if (ks == 5) DRHIP_FM(MBV, 5); else if (ks == 7) DRHIP_FM(MBV, 7); else DRHIP_FM(MBV, 9); } while (0)
        if (wide) DRHIP_FM_K(4); else DRHIP_FM_K(2);
#undef DRHIP_FM_K
#undef DRHIP_FM
        return launched("conv3x3_fewc_mfma_kernel");
    }
    if (I <= 4 && kw == 3 && kh == 3) {
        const int Wo = W / strideX, Ho = H / strideY;
        const int tilesX = ceil_div(Wo, kDirTile), tilesY = ceil_div(Ho, kDirTile);
        DRHIP_REQUIRE(tilesY <= 65535 && O <= 65535, "drhip_conv2d_direct_f32: tensor exceeds the launch grid");
#define DRHIP_FEWC(OCTV, ICV) launch((conv_direct_fewc_kernel<OCTV, 3, 3, ICV>), dim3(tilesX, tilesY, ceil_div(O, OCTV)), dim3(kDirThreads), 0, s0, \
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

extern "C" int drhip_conv3x3_pool3s2_f32(const float* in, const float* w, const float* bias, float* out,
                                         int W, int H, int I, int O, int strideX, int strideY, int relu, void* stream) {
    DRHIP_REQUIRE(in && w && out, "drhip_conv3x3_pool3s2_f32: NULL tensor");
    DRHIP_REQUIRE(W > 0 && H > 0 && O > 0 && I >= 1 && I <= 4, "drhip_conv3x3_pool3s2_f32: bad shape %dx%dx%d -> %d (1 to 4 input channels)", W, H, I, O);
    DRHIP_REQUIRE(strideX > 0 && strideY > 0 && W / strideX > 0 && H / strideY > 0, "drhip_conv3x3_pool3s2_f32: bad stride or empty output");
    DRHIP_REQUIRE((long long)W * H * I < (1ll << 31) && (long long)W * H * O < (1ll << 31), "drhip_conv3x3_pool3s2_f32: tensor too large");
    DRHIP_REQUIRE(W <= 65535 && H <= 65535 && O <= 65535 && strideX <= 15 && strideY <= 15, "drhip_conv3x3_pool3s2_f32: W, H and O are limited to 65535, strides to 15");
    const int Wo = W / strideX, Ho = H / strideY, Wp = ceil_div(Wo, 2), Hp = ceil_div(Ho, 2);
    const int tilesX = ceil_div(Wp, kFpPool), tilesY = ceil_div(Hp, kFpPool);
    hipStream_t s = as_stream(stream);
    const int ks = ceil_div(9 * I, 4);              // 3, 5, 7 or 9
    const bool wide = O > 32;                       // 64 channels per workgroup, else 32
    DRHIP_REQUIRE(tilesY <= 65535 && O <= 32 * 65535, "drhip_conv3x3_pool3s2_f32: tensor exceeds the launch grid");
    const dim3 grid(tilesX, tilesY, ceil_div(O, wide ? 64 : 32)), block(kFpThreads);
#define DRHIP_FP(MBV, KSV) launch((conv3x3_fewc_pool3s2_kernel<MBV, KSV>), grid, block, 0, s, in, w, bias, out, (unsigned)W | (unsigned)H << 16, (unsigned)I | (unsigned)O << 16, (unsigned)Wo | (unsigned)Ho << 16, (unsigned)strideX | (unsigned)strideY << 4 | (relu ? 256u : 0u))
#define DRHIP_FP_K(MBV) do { if (ks == 3) DRHIP_FP(MBV, 3); else if (ks == 5) DRHIP_FP(MBV, 5); else if (ks == 7) DRHIP_FP(MBV, 7); else DRHIP_FP(MBV, 9); } while (0)
    if (wide) DRHIP_FP_K(4); else DRHIP_FP_K(2);
#undef DRHIP_FP_K
#undef DRHIP_FP
    return launched("conv3x3_fewc_pool3s2_kernel");
}

extern "C" size_t drhip_conv3x3_direct_filter_floats(int I, int O) {
    if (I <= 0 || O <= 0) return 0;
    return (size_t)9 * ceil_div(I, kDmKC) * kDmKC * dm_opad(O);
}

extern "C" int drhip_conv3x3_direct_filter_layout_f32(const float* w, float* F, int I, int O, void* stream) {
    DRHIP_REQUIRE(w && F, "drhip_conv3x3_direct_filter_layout_f32: NULL tensor");
    DRHIP_REQUIRE(I > 0 && O > 0 && (long long)(I + 7) * (O + 31) * 9 < (1ll << 29), "drhip_conv3x3_direct_filter_layout_f32: bad shape I=%d O=%d", I, O);
    const int nChunks = ceil_div(I, kDmKC);
    launch(direct_filter_layout_kernel, dim3(ceil_div(nChunks * 8 * dm_opad(O), 256)), dim3(256), 0, as_stream(stream), w, F, I, O, nChunks);
    return launched("direct_filter_layout_kernel");
}

// variant = waves per workgroup (1, 2, 4, 8) | 0x10 for 64 output channels per workgroup (else 32)
extern "C" int drhip_conv3x3_direct_pick_variant(int Wo, int Ho, int I, int O) {
    const int nChunks = ceil_div(I, kDmKC);
    const int tiles = ceil_div(Wo * Ho, 32);
    // 64 channels per workgroup share every window between two MFMA sets; taken once such blocks alone give every
    // CU a workgroup (56x56, 256 -> 256: 44.1 us against 46.8 us with 32-channel blocks)
    const bool wide = O >= 64 && tiles * ceil_div(O, 64) >= num_cu();
    // four waves per workgroup, fewer when that would leave a wave less than two stages; eight for layers with
    // fewer workgroups than CUs (56x56, 64 -> 64: 6.5 us against 7.4 us)
    int kw = 1;
    while (kw < 4 && nChunks >= 4 * kw) kw *= 2;
    if (tiles * ceil_div(O, wide ? 64 : 32) < num_cu() && nChunks >= 8) kw = 8;
    return kw | (wide ? 0x10 : 0);
}

extern "C" int drhip_conv3x3_direct_mfma_f32(const float* in, const float* F, const float* bias, float* out,
                                             int W, int H, int I, int O, int stride, int relu, int variant, void* stream) {
    DRHIP_REQUIRE(in && F && out, "drhip_conv3x3_direct_mfma_f32: NULL tensor");
    DRHIP_REQUIRE(W > 0 && H > 0 && I > 0 && O > 0, "drhip_conv3x3_direct_mfma_f32: bad shape %dx%dx%d -> %d", W, H, I, O);
    DRHIP_REQUIRE(stride == 1 || stride == 2, "drhip_conv3x3_direct_mfma_f32: stride %d (1 or 2)", stride);
    DRHIP_REQUIRE(W <= 65535 && H <= 65535 && I <= 65535 && O <= 65535, "drhip_conv3x3_direct_mfma_f32: W, H, I and O are limited to 65535 (got %dx%dx%d -> %d)", W, H, I, O);
    const int Wo = W / stride, Ho = H / stride;
    DRHIP_REQUIRE(Wo > 0 && Ho > 0, "drhip_conv3x3_direct_mfma_f32: output is empty");
    // byte offsets into the input and the filters are 32-bit, and 0x80000000 must lie outside both
    DRHIP_REQUIRE((long long)W * H * I < (1ll << 29) && (long long)Wo * Ho * O < (1ll << 31) && (long long)(I + 7) * (O + 31) * 9 < (1ll << 29),
                  "drhip_conv3x3_direct_mfma_f32: tensor too large for 32-bit byte offsets");
    DRHIP_REQUIRE(((size_t)F & 15) == 0, "drhip_conv3x3_direct_mfma_f32: the filter bank must be 16-byte aligned");
    if (variant == 0) variant = drhip_conv3x3_direct_pick_variant(Wo, Ho, I, O);
    const int kw = variant & 0xf, wide = (variant & 0x10) != 0;
    DRHIP_REQUIRE((variant >> 5) == 0 && (kw == 1 || kw == 2 || kw == 4 || kw == 8), "drhip_conv3x3_direct_mfma_f32: unknown variant %#x", variant);
    const int OB = wide ? 64 : 32;
    const int nPT = ceil_div(Wo * Ho, 32);
    DRHIP_REQUIRE(ceil_div(O, OB) <= 65535, "drhip_conv3x3_direct_mfma_f32: too many output channels (%d)", O);
    const dim3 grid(nPT, ceil_div(O, OB)), block(64 * kw);
    const size_t ldsBytes = (size_t)kw * OB * kDmPartPitch * sizeof(float);
    hipStream_t s = as_stream(stream);
    const FastDiv dWo = make_fastdiv(Wo);
#define DRHIP_DM(NTV, SV) launch((conv3x3_direct_mfma_kernel<NTV, SV>), grid, block, ldsBytes, s, in, F, bias, out, (unsigned)W | (unsigned)H << 16, (unsigned)I | (unsigned)O << 16, dWo.mul, dWo.shift | (relu ? 32u : 0u) | (unsigned)kw << 8)
    if (wide) { if (stride == 1) DRHIP_DM(2, 1); else DRHIP_DM(2, 2); }
    else { if (stride == 1) DRHIP_DM(1, 1); else DRHIP_DM(1, 2); }
#undef DRHIP_DM
    return launched("conv3x3_direct_mfma_kernel");
}
