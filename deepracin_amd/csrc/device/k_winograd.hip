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
// algorithmic work 2*9*H*W*I*O FLOP direct-equivalent, 2*16*tiles*I*O FLOP issued).  The input
// transform happens in registers, the output transform in registers and LDS; see the kernel.
// Workgroup ids are remapped so that each XCD (own L2) works on a contiguous range of
// output-channel panels and therefore touches only its share of U.
// Layers with few tiles cannot fill 256 CUs with panels alone: there the input channels are split
// over several workgroups whose partial outputs are summed in fixed order (deterministic, no float
// atomics, no device-scope fences) - by a small second kernel, or, when all workgroups of the launch
// are resident at once, by the splits themselves: every split finishes a slice of its panel and
// waits for the other splits' partial tiles by watching the workspace slots themselves.
#include "drhip_common.hpp"

#include <atomic>
#include <cstdlib>
#include <type_traits>
#include <utility>

namespace drhip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int kWinoThreads = 256;       // 4 waves, one per row of the 4x4 transform
constexpr int kWinoKC = 8;          // input channels per stage (4 MFMA k-steps)
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

// Output stores are written through (system-scope store: sc0 sc1) instead of being left dirty in this XCD's L2:
// the consumer is the next kernel, whose workgroups mostly sit on other XCDs and read from memory anyway, and
// what is written during the kernel need not be written back when it ends (224x224x64: 23.5 vs 25.0 us).
__device__ inline void store1_through(float* p, float a) {
    __hip_atomic_store((unsigned*)p, __float_as_uint(a), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ inline void store2_through(float* p, float a, float b) {
    const f32x2 v = {a, b};
    __hip_atomic_store((unsigned long long*)p, __builtin_bit_cast(unsigned long long, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// 2x2 store with edge guards; vec2: W even and the base 8-byte aligned.
__device__ inline void wino_store_tile(float* po, int W, int H, int ox, int oy, int vec2,
                                       float y00, float y01, float y10, float y11) {
    if (vec2) {
        store2_through(po, y00, y01);
        if (oy + 1 < H) store2_through(po + W, y10, y11);
    } else {
        po[0] = y00;
        if (ox + 1 < W) po[1] = y01;
        if (oy + 1 < H) {
            po[W] = y10;
            if (ox + 1 < W) po[W + 1] = y11;
        }
    }
}

// One wavefront per row of the 4x4 transform.
//
// On gfx950 an fp32 MFMA and an fp32 VALU instruction never overlap on one SIMD (measured: a wave
// issuing MFMAs and a second wave issuing FMAs on the same SIMD take the sum of their times), so
// every VALU instruction in the channel loop is paid for in matrix throughput.  The loop is therefore
// built to need almost none:
//
//   * wave w (0..3) of a 256-lane workgroup owns the transform positions xi = 4w..4w+3, i.e. row w
//     of B^T d B.  That row needs only TWO rows of the 4x4 input window (row w combined with row 2
//     or 1), so a lane loads two rows of 4 floats and spends 8 adds per (tile, channel) - and the
//     four results are exactly the B operands (lane -> tile lane%32, k -> channel parity lane/32)
//     of that wave's own MFMAs.  V never goes through LDS and the waves of a workgroup never
//     synchronise inside the channel loop.
//   * a window row is ONE 16-byte raw buffer load (four dword loads per row kept the CU's single
//     address unit busier than the matrix cores).  The resource covers the channels from the
//     current one to the end of the tensor: rows above or below the image carry an offset beyond
//     the resource, channels past the last one see a resource of size zero, and the hardware
//     returns 0.0 for both - vertical padding and ragged channel counts cost no instruction.
//     Samples left or right of the image are zeroed by selects after the two rows are combined.
//   * all addresses are a per-lane byte offset computed once plus scalar (SGPR) bases.
//   * operands of the next stage are loaded into the registers the current stage has just
//     finished with (input rows after their transform, filters after the MFMAs of their xi pair),
//     so every load has one full stage to land.
// A workgroup owns 32 tiles x OB = 32*NT output channels; the larger OB, the more MFMAs share the
// 8 adds of a transformed input sample.  Epilogue: each wave applies the right factor A to its row
// (in registers), the four rows meet in LDS (32 KiB) and every lane finishes A^T . for its
// (tile, channel) pairs, adds bias, applies ReLU and stores 2x2 pixels (adjacent lanes = adjacent
// tiles).
//
// gridDim.y = number of input-channel splits KS.  KS == 1: the workgroup finishes its outputs.
// KS > 1: every split stores its partial (pre-bias) 2x2 tiles, tile-major, to the workspace and
// winograd_split_reduce_kernel sums them in split order, adds the bias and applies ReLU.
// The shape arguments of the convolution kernels, packed into six dwords.  The first 14 dwords of a kernel's
// arguments arrive in SGPRs with the wave (kernel-argument preload: 16 user SGPRs, two of which hold the address
// of the argument block): the three input pointers, these six dwords and the output pointer; the workspace
// pointer, which only the epilogue of a split layer needs, comes last.  Everything else is derived; nothing is
// read from the dispatch packet (gridDim, blockDim), because every scalar load in front of the first vector loads
// is a round trip of its own at the start of every workgroup (~0.07 us each).
//   wh = W | H << 16, io = I | O << 16 (each at most 65535),
//   mulX, mulTB = multipliers of the divisions by tilesX and by the number of tile panels,
//   cfg0 = shiftX | shiftTB << 5 | epilogue flags << 10 (2 bits) | vec2 << 12 | splits << 13 (16 bits) | tiered << 30 | joined << 31,
//   cfg1 = chunks per split (16 bits) | log2 splits << 24 (joined launches)
//   tiered launches: the splits field holds log2 splits of up to four tiers (4 bits each) and cfg1 their panel
//   counts per XCD (8 bits each)
#define WINO_ARGS unsigned wh, unsigned io, unsigned mulX, unsigned mulTB, unsigned cfg0, unsigned cfg1
#define WINO_UNPACK(TBV, OBV)                                                                           \
    const int W = (int)(wh & 0xffffu), H = (int)(wh >> 16), I = (int)(io & 0xffffu), O = (int)(io >> 16); \
    const int tilesX = (W + 1) >> 1, T = tilesX * ((H + 1) >> 1);                                         \
    const int nTB = (T + (TBV) - 1) / (TBV), nBlocks = nTB * ((O + (OBV) - 1) / (OBV));                   \
    const FastDiv tilesXd = {(unsigned)tilesX, mulX, cfg0 & 31u}, nTBd = {(unsigned)nTB, mulTB, (cfg0 >> 5) & 31u}; \
    const int relu = (int)((cfg0 >> 10) & 3u), vec2 = (int)((cfg0 >> 12) & 1u), nSplits = (int)((cfg0 >> 13) & 0xffffu); \
    const bool joined = (cfg0 >> 31) != 0u, tiered = ((cfg0 >> 30) & 1u) != 0u;                          \
    const int chunksPerSplit = (int)(cfg1 & 0xffffu), lgSplits = (int)((cfg1 >> 24) & 15u);
struct WinoPackedArgs { unsigned wh, io, mulX, mulTB, cfg0, cfg1; };

constexpr unsigned kBufferFlags = 0x00020000u;      // dword 3 of a gfx9 raw buffer resource (32-bit data format)
constexpr int kEpiRelu = DRHIP_EPILOGUE_RELU, kEpiMaxPool2 = DRHIP_EPILOGUE_MAXPOOL2;   // bits of the `relu` argument
constexpr unsigned kOutOfRange = 0x80000000u;       // byte offset no resource of at most 2 GiB contains

// Joined splits (see the kernel's epilogue).
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
constexpr unsigned kWinoEmpty = 0xffa5c3e1u;        // a signalling NaN: marks a workspace slot whose partial tile has not arrived
constexpr int kWinoMaxJoin = 16;                    // most splits a joined launch can have
constexpr int kWinoJoinSpins = 1 << 18;             // bound on the wait for a partner's partial tile (some 0.2 s)
constexpr int kAuxThrough = 1 | 16;                 // cache policy of a buffer access: sc0 sc1, written through to memory
constexpr int kAuxDeviceVolatile = 16 | (int)0x80000000u;   // sc1 (device scope: not served from this CU's vector cache), reloaded every time
__device__ unsigned g_wino_join_timeouts;           // partial tiles that never arrived, over the life of the process

__device__ inline f32x4 buf_load4(__amdgpu_buffer_rsrc_t r, unsigned voffset, unsigned soffset) {
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voffset, (int)soffset, 0));
}

// KW = 2: the workgroup has eight waves; waves 4..7 repeat the roles of waves 0..3 on every second stage
// (wave set k takes the stages chBegin + k, + KW, ...), and the two sets' sums meet in LDS in the epilogue,
// set 0 first.  One wave per SIMD cannot keep the matrix pipe busy (it waits for its own transforms and
// loads); layers whose workgroup count leaves one workgroup per CU get their second wave per SIMD this way,
// without a second workgroup's share of partial tiles in memory.
// FEWC: a layer with at most four input channels (an image): one stage whose third and fourth k-step would multiply
// zeros are left out, and nothing is prefetched.
template <int NT, int KW, bool FEWC = false>
__global__ void __launch_bounds__(kWinoThreads * KW, KW == 2 ? 1 : (NT == 1 ? 3 : (NT == 2 ? 2 : 1)))
winograd_f23_mfma_kernel(const float* __restrict__ in, const float* __restrict__ U, const float* __restrict__ bias,
                         WINO_ARGS, float* __restrict__ out, float* __restrict__ ws) {
    constexpr int TB = 32, OB = 32 * NT, KC = kWinoKC;
    WINO_UNPACK(TB, OB)
    extern __shared__ float P[];                    // epilogue only: [KW sets][4 rows][2][OB o][32 t] floats

    // ---- which panel: XCD-aware remap of the linear workgroup id -----------------------------
    const int perXcd = (nBlocks + kXcds - 1) / kXcds;   // the grid is padded to a multiple of kXcds
    // Joined launch: one grid row; the splits of a panel are the workgroups j = id / 8 of one XCD with equal
    // j >> lgSplits, so they share that XCD's L2 and are dispatched within 8 * splits workgroups of each other.
    // Tiered launch: an XCD's panels come in up to four tiers, each with its own number of splits, in dispatch
    // order (finest cut first, whole panels last): one workgroup of every full tier lands on each CU, so the
    // CUs end up with equal numbers of stages although the panel count is no multiple of the CU count.
    int slot = (int)(blockIdx.x / kXcds), split = (int)blockIdx.y, nSp = nSplits, lgSp = lgSplits, chunksHere = chunksPerSplit;
    if (tiered) {
        int jj = slot, base = 0;
        bool found = false;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int n = (int)((cfg1 >> (8 * k)) & 255u), l = (int)((cfg0 >> (13 + 4 * k)) & 15u);
            if (!found) {
                if (jj < (n << l)) { found = true; slot = base + (jj >> l); split = jj & ((1 << l) - 1); lgSp = l; }
                else { jj -= n << l; base += n; }
            }
        }
        if (!found) return;
        nSp = 1 << lgSp;
        chunksHere = ((I + kWinoKC - 1) / kWinoKC) >> lgSp;     // (the launcher makes tiers of equal splits only)
    } else if (joined) {
        split = slot & (nSplits - 1);
        slot >>= lgSplits;
    }
    const int logical = (blockIdx.x % kXcds) * perXcd + slot;
    if (slot >= perXcd || logical >= nBlocks) return;
    const int oBlock = fast_div(logical, nTBd);
    const int o0 = oBlock * OB;
    const int t0 = (logical - oBlock * (int)nTBd.d) * TB;
    // The fewer stages a workgroup has, the sooner its partial tiles can be on their way: small pieces first,
    // so that the workgroups that end a CU's work are whole panels, which wait for nobody.
    if (tiered) {
        if (lgSp >= 3) __builtin_amdgcn_s_setprio(3);
        else if (lgSp == 2) __builtin_amdgcn_s_setprio(2);
        else if (lgSp == 1) __builtin_amdgcn_s_setprio(1);
    }

    // With two wave sets the rest of the kernel exists twice, chosen once per workgroup: only the block that holds image
    // tile 0 carries the three selects per k-step that move that one lane's samples (`shifted` below); in every other
    // block they are constants and vanish.  (A branch inside the stage, and two copies of the channel loop alone, both cost more
    // than they saved: the first breaks the stage's instruction order, the second made the compiler spill.)
    auto rest_of_kernel = [&](auto tile0Block) {
        const int tid = threadIdx.x, lane = tid & 63;
        const int waveId = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wave = waveId & 3;                    // = row of the transform
        const int kset = waveId >> 2;                   // which of the KW wave sets
        const int l32 = lane & 31, lhi = lane >> 5;
        const int plane = H * W;
        const int nChunksAll = (I + KC - 1) / KC;
        const int chBegin = split * chunksHere;
        const int chEnd = min(nChunksAll, chBegin + chunksHere);        // > chBegin: the launcher creates no empty split
        const int Opad = wino_opad(O);

        // ---- this lane's tile and the byte offsets of the two window rows it reads ---------------
        // Row w of B^T d:  w=0: d0 - d2,  w=1: d1 + d2,  w=2: d2 - d1,  w=3: d3 - d1.
        const int tg = t0 + l32;
        const bool tileOk = tg < T;
        const int ty = tileOk ? fast_div(tg, tilesXd) : 0, tx = tileOk ? tg - ty * tilesX : 0;
        const int x0 = 2 * tx - 1, y0 = 2 * ty - 1;
        const int rowA = wave, rowB = (wave < 2) ? 2 : 1;
        const float sgn = (wave == 1) ? 1.0f : -1.0f;
        // One 16-byte load per row from the (4-byte aligned) address of its first sample.  Rows outside
        // the image carry the out-of-range offset as a whole; samples beyond the left or right edge come
        // back as the neighbouring row's pixels and are zeroed by three selects after the rows have been
        // combined (the second sample, x = 2*tx, always exists).  A negative offset would zero the whole
        // load, and only image tile 0 has one (x = -1 in row 0): that one lane loads from x = 0 instead
        // and shifts its combined samples up by one (three more selects for everybody; a branch around
        // them costs more in register copies than it saves).
        const bool shifted = decltype(tile0Block)::value && tg == 0;
        const int xLoad = shifted ? 0 : x0;
        const int yaRow = y0 + rowA, ybRow = y0 + rowB;
        const unsigned offVA = (tileOk && yaRow >= 0 && yaRow < H) ? 4u * (unsigned)(lhi * plane + yaRow * W + xLoad) : kOutOfRange;
        const unsigned offVB = (tileOk && ybRow >= 0 && ybRow < H) ? 4u * (unsigned)(lhi * plane + ybRow * W + xLoad) : kOutOfRange;
        const bool c0ok = x0 >= 0, c2ok = x0 + 2 < W, c3ok = x0 + 3 < W;
        const float k0f = c0ok ? 1.0f : 0.0f, k3f = c3ok ? 1.0f : 0.0f;

        // Window rows of channels cbase + lhi.  "Ranged" form: the resource starts at channel cbase and
        // ends with the tensor, so channels >= I read 0 without touching memory (ragged last chunk,
        // prefetch past the end).  "Plain" form for chunks known to lie inside the tensor: one resource
        // for the whole tensor, the channel offset travels in the scalar offset (a resource that changes
        // inside the loop makes the compiler wait for all outstanding loads at the loop head).
        const __amdgpu_buffer_rsrc_t rIn = __builtin_amdgcn_make_buffer_rsrc((void*)in, 0, I * plane * 4, kBufferFlags);
        auto load_rows = [&](float (&d)[8], __amdgpu_buffer_rsrc_t r, unsigned soff) {
            const f32x4 a = buf_load4(r, offVA, soff), b = buf_load4(r, offVB, soff);
#pragma unroll
            for (int s = 0; s < 4; ++s) { d[s] = a[s]; d[4 + s] = b[s]; }
        };
        auto load_rows_plain = [&](float (&d)[8], int cbase) { load_rows(d, rIn, 4u * (unsigned)(cbase * plane)); };
        auto load_rows_ranged = [&](float (&d)[8], int cbase) {
            const int left = max(I - cbase, 0);
            const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)(in + (size_t)min(cbase, I) * plane), 0,
                                                                                 left * plane * 4, kBufferFlags);
            load_rows(d, r, 0u);
        };
        // filters of one xi for a whole stage: component ks of the 16-byte load = k-step ks
        const __amdgpu_buffer_rsrc_t rU = __builtin_amdgcn_make_buffer_rsrc((void*)U, 0, 16 * nChunksAll * Opad * 8 * 4, kBufferFlags);
        const unsigned fOff = 4u * (unsigned)((o0 + l32) * 8 + 4 * lhi);
        auto load_filters = [&](f32x4 (&f)[NT], int e, int chunk) {
            const unsigned soff = 4u * (unsigned)(((4 * wave + e) * nChunksAll + chunk) * Opad * 8);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) f[nt] = buf_load4(rU, fOff + 4u * (unsigned)(nt * 32 * 8), soff);
        };

        // The epilogue's bias values are fetched now: a load issued there would add a trip to memory
        // to the tail of every workgroup.
        constexpr bool kBiasEarly = NT <= 2;
        constexpr int EO = 8 * KW;                      // output channels finished per pass of the epilogue
        float biasEarly[kBiasEarly ? OB / EO : 1];
        if (kBiasEarly && bias && (nSp == 1 || joined)) {
#pragma unroll
            for (int q = 0; q < OB / EO; ++q) biasEarly[q] = bias[min(o0 + (tid >> 5) + EO * q, O - 1)];
        }

        f32x16 acc[4][NT];
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[e][nt][r] = 0.0f;

        constexpr int KS = FEWC ? 2 : 4;                // k-steps of a stage that carry channels
        float raw[4][8];
        f32x4 f[4][NT];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) load_rows_ranged(raw[ks], (chBegin + kset) * KC + 2 * ks);
#pragma unroll
        for (int e = 0; e < 4; ++e) load_filters(f[e], e, min(chBegin + kset, nChunksAll - 1));

        // One stage: transform the rows of chunk ch (and start loading those of chunk ch+1 into the
        // same registers), then 16*NT MFMAs, reloading the filters of each xi pair behind its MFMAs.
        auto stage = [&](int ch, auto plainNext) {
            const int next = min(ch + KW, nChunksAll - 1);
            float b[4][4];                              // [k-step][xi within the row]
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                float m[4];
#pragma unroll
                for (int s = 0; s < 4; ++s) m[s] = fmaf(sgn, raw[ks][4 + s], raw[ks][s]);   // exact: sgn is +-1
                // (the masks of the first and fourth sample ride in the combinations: k0f and k3f are 1.0 or 0.0, so
                // these are the same sums with one rounding, for two instructions less per k-step)
                const float s1 = shifted ? m[0] : m[1], s2 = shifted ? m[1] : m[2], s3 = shifted ? m[2] : m[3];
                const float t2 = c2ok ? s2 : 0.0f;
                b[ks][0] = fmaf(k0f, m[0], -t2);
                b[ks][1] = s1 + t2;
                b[ks][2] = t2 - s1;
                b[ks][3] = fmaf(k3f, s3, -s1);
            }
            __builtin_amdgcn_sched_barrier(0);
            // 8 slots of 2*NT MFMAs (two xi at a time: dependent MFMAs stay 2*NT apart).  The loads of
            // the next stage are issued behind the MFMAs of a slot, so the matrix pipe keeps running
            // while they go out: input rows in the first four slots (their registers are free since
            // the transforms above), the filters of an xi pair once its last MFMA has been issued.
#pragma unroll
            for (int eg = 0; eg < 2; ++eg) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                    for (int e = 2 * eg; e < 2 * eg + 2; ++e)
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
                            acc[e][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(f[e][nt][ks], b[ks][e], acc[e][nt], 0, 0, 0);
                    if constexpr (FEWC) continue;       // (a single stage: nothing to load for a next one)
                    if (eg == 0) {
                        if constexpr (decltype(plainNext)::value) load_rows_plain(raw[ks], (ch + KW) * KC + 2 * ks);
                        else load_rows_ranged(raw[ks], (ch + KW) * KC + 2 * ks);
                    } else if (ks < 2) {
                        load_filters(f[ks], ks, next);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if constexpr (!FEWC) {
                load_filters(f[2], 2, next);
                load_filters(f[3], 3, next);
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        // Stages whose successor chunk (KW further on) is complete (all 8 channels exist) and does not hold the
        // tensor's last channel prefetch in the plain form; the last ones of the tensor use the ranged form.  (The
        // scalar offset of a buffer access is not part of its range check, and the 16-byte row loads of the last
        // tiles of the last row reach one or two samples past the row: in the last channel that is past the tensor,
        // where only the ranged form's resource ends.)
        const int chMain = min(chEnd, (I - 1) / KC - KW);
        int ch = chBegin + kset;
        for (; ch < chMain; ch += KW) stage(ch, std::true_type{});
        for (; ch < chEnd; ch += KW) stage(ch, std::false_type{});

        // ---- epilogue -----------------------------------------------------------------------------
        // Accumulator layout of the 32x32 MFMA: lane -> column (tile) lane%32; register r -> row
        // (output channel) 8*(r/4) + 4*(lane/32) + r%4.
        // Each wave applies the right factor A to its row of M and parks the two results per
        // (tile, channel) in LDS: P[row][j][channel][tile].
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float m0 = acc[0][nt][r], m1 = acc[1][nt][r], m2 = acc[2][nt][r], m3 = acc[3][nt][r];
                const int ol = 32 * nt + 8 * (r / 4) + 4 * lhi + (r % 4);
                P[(((kset * 4 + wave) * 2 + 0) * OB + ol) * TB + l32] = m0 + m1 + m2;
                P[(((kset * 4 + wave) * 2 + 1) * OB + ol) * TB + l32] = m1 - m2 + m3;
            }
        }
        // LDS-only barrier: __syncthreads() would also wait for the outstanding (unused) prefetches.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");

        // Left factor A^T over the four rows, bias, ReLU, store: lane -> tile tid%32, channels tid/32 + EO*q.
        const bool direct = nSp == 1;
        const int et = tid & 31, eo = tid >> 5;
        const int etg = t0 + et;
        const bool eTileOk = etg < T;
        const int eTy = eTileOk ? fast_div(etg, tilesXd) : 0;
        const int ox = eTileOk ? 2 * (etg - eTy * tilesX) : 0, oy = 2 * eTy;
        f32x4* wsTiles = direct ? nullptr : (f32x4*)ws + ((size_t)split * nBlocks + logical) * OB * TB;
        // this lane's 2x2 tile of channel ol, summed over the rows of the transform (and the wave sets)
        auto tile_of = [&](int ol) {
            float p[4][2];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                p[r][0] = P[((r * 2 + 0) * OB + ol) * TB + et];
                p[r][1] = P[((r * 2 + 1) * OB + ol) * TB + et];
                if constexpr (KW == 2) {                // the second wave set's half of the channel sum
                    p[r][0] += P[(((4 + r) * 2 + 0) * OB + ol) * TB + et];
                    p[r][1] += P[(((4 + r) * 2 + 1) * OB + ol) * TB + et];
                }
            }
            return f32x4{p[0][0] + p[1][0] + p[2][0], p[0][1] + p[1][1] + p[2][1],
                         p[1][0] - p[2][0] + p[3][0], p[1][1] - p[2][1] + p[3][1]};
        };
        if (joined && nSp > 1) {
            // (the partial tiles go out and are looked for at the highest priority: the other workgroups on this CU
            // are in their channel loops, and a wave at their priority gets an issue slot only when they stall)
            if (tiered) __builtin_amdgcn_s_setprio(3);
            // Every split finishes the channels ol with ol >> lgRows == split of its panel (OB >> lgSplits channels).
            // First the partial tiles the other splits are waiting for go out, written through; then this split
            // collects theirs.  A workspace slot holds kWinoEmpty (a signalling NaN, which no addition can produce)
            // until its partial tile has been stored, so a reader sees from the slot itself whether the data has
            // arrived: no flag, no counter, no wait for the stores to complete.  The reader puts kWinoEmpty back.
            const int lgRows = __builtin_ctz(OB) - lgSp;
            const __amdgpu_buffer_rsrc_t rWs = __builtin_amdgcn_make_buffer_rsrc((void*)ws, 0, 0x7ffffff0, kBufferFlags);
            const unsigned panelFloats = (unsigned)(OB * TB * 4);
            // (tiered: a workgroup's partial tiles lie at its own index in the grid, its partners' 8 workgroups apart)
            const unsigned region0 = tiered ? blockIdx.x - (unsigned)(kXcds * split) : (unsigned)logical;
            const unsigned regionStep = tiered ? (unsigned)kXcds : (unsigned)nBlocks;
            // byte address of a slot = region of the split (scalar offset) + place of the tile in the panel (per lane)
            auto region_of = [&](int sp) { return (int)(4u * (region0 + (unsigned)sp * regionStep) * panelFloats); };
            auto place_of = [&](int ol) { return (int)(16u * (unsigned)(ol * TB + et)); };
#pragma unroll
            for (int q = 0; q < OB / EO; ++q) {
                const int ol = eo + EO * q;
                if ((ol >> lgRows) == split) continue;
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, tile_of(ol)), rWs, place_of(ol), region_of(split), kAuxThrough);
            }
            const u32x4 empty = {kWinoEmpty, kWinoEmpty, kWinoEmpty, kWinoEmpty};
            // (the number of splits as a constant: every access below is unconditional.  The slot of the own split is
            // read and reset like the others - nobody ever writes it - and its content replaced by the own tile.)
            auto collect = [&](auto nSplitsConst) {
                constexpr int S = decltype(nSplitsConst)::value;
#pragma unroll
                for (int q = 0; q < OB / EO; ++q) {
                    const int ol = eo + EO * q, o = o0 + ol;
                    if ((ol >> lgRows) != split) continue;
                    const f32x4 own = tile_of(ol);
                    u32x4 part[S];
                    bool ready = false;
                    for (int spins = 0; spins < kWinoJoinSpins && !ready; ++spins) {
                        // (the loads are invariant as far as the compiler can see: without this it issues them once,
                        // in front of the loop)
                        asm volatile("" ::: "memory");
                        ready = true;
#pragma unroll
                        for (int u = 0; u < S; ++u) part[u] = __builtin_amdgcn_raw_buffer_load_b128(rWs, place_of(ol), region_of(u), kAuxDeviceVolatile);
#pragma unroll
                        for (int u = 0; u < S; ++u)
                            ready = ready && (u == split || (part[u][0] != kWinoEmpty && part[u][1] != kWinoEmpty && part[u][2] != kWinoEmpty && part[u][3] != kWinoEmpty));
                    }
                    f32x4 s = {0.f, 0.f, 0.f, 0.f};     // splits added in order, like winograd_split_reduce_kernel
#pragma unroll
                    for (int u = 0; u < S; ++u) s += (u == split) ? own : __builtin_bit_cast(f32x4, part[u]);
#pragma unroll
                    for (int u = 0; u < S; ++u) __builtin_amdgcn_raw_buffer_store_b128(empty, rWs, place_of(ol), region_of(u), kAuxThrough);
                    if (!ready) {                       // a partner never delivered: say so in the result and in the counter
                        s = f32x4{__builtin_nanf(""), __builtin_nanf(""), __builtin_nanf(""), __builtin_nanf("")};
                        atomicAdd(&g_wino_join_timeouts, 1u);
                    }
                    if (eTileOk && o < O) {
                        if (bias) s += kBiasEarly ? biasEarly[kBiasEarly ? q : 0] : bias[o];
                        if (relu & kEpiRelu) { s[0] = fmaxf(s[0], 0.f); s[1] = fmaxf(s[1], 0.f); s[2] = fmaxf(s[2], 0.f); s[3] = fmaxf(s[3], 0.f); }
                        if (relu & kEpiMaxPool2)
                            store1_through(out + (size_t)o * (plane >> 2) + (size_t)(oy >> 1) * (W >> 1) + (ox >> 1), fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])));
                        else
                            wino_store_tile(out + (size_t)o * plane + (size_t)oy * W + ox, W, H, ox, oy, vec2, s[0], s[1], s[2], s[3]);
                    }
                }
            };
            static_assert(kWinoMaxJoin == 16, "the cases below");
            if (lgSp == 1) collect(std::integral_constant<int, 2>{});
            else if (lgSp == 2) collect(std::integral_constant<int, 4>{});
            else if (lgSp == 3) collect(std::integral_constant<int, 8>{});
            else collect(std::integral_constant<int, 16>{});
            return;
        }
#pragma unroll
        for (int q = 0; q < OB / EO; ++q) {
            const int ol = eo + EO * q, o = o0 + ol;
            const f32x4 y = tile_of(ol);
            float y00 = y[0], y01 = y[1], y10 = y[2], y11 = y[3];
            if (direct) {
                if (eTileOk && o < O) {
                    if (bias) { const float bv = kBiasEarly ? biasEarly[kBiasEarly ? q : 0] : bias[o]; y00 += bv; y01 += bv; y10 += bv; y11 += bv; }
                    if (relu & kEpiRelu) { y00 = fmaxf(y00, 0.f); y01 = fmaxf(y01, 0.f); y10 = fmaxf(y10, 0.f); y11 = fmaxf(y11, 0.f); }
                    if (relu & kEpiMaxPool2)        // W, H even: the tile is one window of a 2x2/2 max pool
                        store1_through(out + (size_t)o * (plane >> 2) + (size_t)(oy >> 1) * (W >> 1) + (ox >> 1), fmaxf(fmaxf(y00, y01), fmaxf(y10, y11)));
                    else
                        wino_store_tile(out + (size_t)o * plane + (size_t)oy * W + ox, W, H, ox, oy, vec2, y00, y01, y10, y11);
                }
            } else {
                f32x4 v = {y00, y01, y10, y11};
                wsTiles[(size_t)ol * TB + et] = v;      // whole panel, padding included: 512 B per half wave
            }
        }
    };
    // (Only the eight-wave form pays back the second copy: the first layers' kernels are so short that fetching
    // twice the code costs them more - 224x224 3->64: 7.7-8.9 against 6.9 us - and the 32-channel four-wave form
    // gained nothing.)
    if constexpr (KW == 2) {
        if (t0 == 0) rest_of_kernel(std::true_type{});
        else rest_of_kernel(std::false_type{});
    } else {
        rest_of_kernel(std::true_type{});
    }
}


// The same algorithm on 16-tile x 16-channel blocks with v_mfma_f32_16x16x4_f32, for layers with few
// tiles (28x28 and 14x14 maps): four times as many workgroups as 32x32 blocks give, a quarter of
// the dependent MFMA chain in each, so fewer (or no) input-channel splits are needed to fill the
// chip.  Lane -> (tile lane%16, channel lane/16 of a 4-channel k-step); a stage of 8 channels is
// two k-steps.  The filters keep their layout: lane/16 = k picks the 16-byte half (k & 1) and the
// component pair (k >> 1) of it.  D: lane -> tile lane%16, register r -> channel 4*(lane/16) + r.
// A workgroup owns 16 tiles x OB = 16*NB output channels.
typedef float f32x4acc __attribute__((ext_vector_type(4)));

// KW wave sets of four waves (KW = 1, 2) take the stages round-robin and meet in LDS in the epilogue, set 0 first:
// a stage is only 8*NB short MFMAs long, less than a load takes to arrive, so a single wave per SIMD waits for its
// operands in every stage; with two waves per SIMD the prefetch of a wave has two stages of matrix work to land
// (14x14, 64 -> 256: 5.1 vs 5.4 us; four sets were measured slower again).
template <int NB, int KW>
__global__ void __launch_bounds__(kWinoThreads * KW)
winograd_f23_mfma16_kernel(const float* __restrict__ in, const float* __restrict__ U, const float* __restrict__ bias,
                           WINO_ARGS, float* __restrict__ out, float* __restrict__ ws) {
    constexpr int TB = 16, OB = 16 * NB, KC = kWinoKC;
    WINO_UNPACK(TB, OB)
    (void)joined; (void)lgSplits;                   // (joined splits exist for 32-tile blocks only)
    extern __shared__ float P[];                    // epilogue only: [KW sets][4 rows][2][OB o][16 t] floats

    const int perXcd = (nBlocks + kXcds - 1) / kXcds;
    const int logical = (blockIdx.x % kXcds) * perXcd + blockIdx.x / kXcds;
    if (logical >= nBlocks) return;
    const int oBlock = fast_div(logical, nTBd);
    const int o0 = oBlock * OB;
    const int t0 = (logical - oBlock * (int)nTBd.d) * TB;
    const int split = blockIdx.y;

    const int tid = threadIdx.x, lane = tid & 63;
    const int waveId = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave = waveId & 3;                    // = row of the transform
    const int kset = waveId >> 2;                   // which of the KW wave sets
    const int l16 = lane & 15, lk = lane >> 4;
    const int plane = H * W;
    const int nChunksAll = (I + KC - 1) / KC;
    const int chBegin = split * chunksPerSplit;
    const int chEnd = min(nChunksAll, chBegin + chunksPerSplit);
    const int Opad = wino_opad(O);

    // window rows, offsets and edge masks exactly as in the 32-tile kernel
    const int tg = t0 + l16;
    const bool tileOk = tg < T;
    const int ty = tileOk ? fast_div(tg, tilesXd) : 0, tx = tileOk ? tg - ty * tilesX : 0;
    const int x0 = 2 * tx - 1, y0 = 2 * ty - 1;
    const int rowA = wave, rowB = (wave < 2) ? 2 : 1;
    const float sgn = (wave == 1) ? 1.0f : -1.0f;
    const bool shifted = tg == 0;
    const int xLoad = shifted ? 0 : x0;
    const int yaRow = y0 + rowA, ybRow = y0 + rowB;
    const unsigned offVA = (tileOk && yaRow >= 0 && yaRow < H) ? 4u * (unsigned)(lk * plane + yaRow * W + xLoad) : kOutOfRange;
    const unsigned offVB = (tileOk && ybRow >= 0 && ybRow < H) ? 4u * (unsigned)(lk * plane + ybRow * W + xLoad) : kOutOfRange;
    const bool c0ok = x0 >= 0, c2ok = x0 + 2 < W, c3ok = x0 + 3 < W;
    const float k0f = c0ok ? 1.0f : 0.0f, k3f = c3ok ? 1.0f : 0.0f;

    const __amdgpu_buffer_rsrc_t rIn = __builtin_amdgcn_make_buffer_rsrc((void*)in, 0, I * plane * 4, kBufferFlags);
    auto load_rows = [&](float (&d)[8], __amdgpu_buffer_rsrc_t r, unsigned soff) {
        const f32x4 a = buf_load4(r, offVA, soff), b = buf_load4(r, offVB, soff);
#pragma unroll
        for (int s = 0; s < 4; ++s) { d[s] = a[s]; d[4 + s] = b[s]; }
    };
    auto load_rows_plain = [&](float (&d)[8], int cbase) { load_rows(d, rIn, 4u * (unsigned)(cbase * plane)); };
    auto load_rows_ranged = [&](float (&d)[8], int cbase) {
        const int left = max(I - cbase, 0);
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)(in + (size_t)min(cbase, I) * plane), 0,
                                                                             left * plane * 4, kBufferFlags);
        load_rows(d, r, 0u);
    };
    const __amdgpu_buffer_rsrc_t rU = __builtin_amdgcn_make_buffer_rsrc((void*)U, 0, 16 * nChunksAll * Opad * 8 * 4, kBufferFlags);
    const unsigned fOff = 4u * (unsigned)((o0 + l16) * 8 + 4 * (lk & 1));
    const bool oddPair = (lk >> 1) != 0;            // which components of the 16 bytes: {0,2} or {1,3}
    auto load_filters = [&](f32x4 (&f)[NB], int e, int chunk) {
        const unsigned soff = 4u * (unsigned)(((4 * wave + e) * nChunksAll + chunk) * Opad * 8);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) f[nb] = buf_load4(rU, fOff + 4u * (unsigned)(nb * 16 * 8), soff);
    };

    constexpr int EO = 16 * KW;                     // output channels finished per pass of the epilogue
    constexpr int NQ = (OB + EO - 1) / EO;
    float biasEarly[NQ];
    if (bias && nSplits == 1) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) biasEarly[q] = bias[min(o0 + (tid >> 4) + EO * q, O - 1)];
    }

    f32x4acc acc[4][NB];
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[e][nb] = f32x4acc{0.f, 0.f, 0.f, 0.f};

    float raw[2][8];
    f32x4 f[4][NB];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) load_rows_ranged(raw[ks], (chBegin + kset) * KC + 4 * ks);
#pragma unroll
    for (int e = 0; e < 4; ++e) load_filters(f[e], e, min(chBegin + kset, nChunksAll - 1));

    auto stage = [&](int ch, auto plainNext) {
        const int next = min(ch + KW, nChunksAll - 1);
        float b[2][4];                              // [k-step][xi within the row]
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            float m[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) m[s] = fmaf(sgn, raw[ks][4 + s], raw[ks][s]);
            // (the masks of the first and fourth sample ride in the combinations: k0f and k3f are 1.0 or 0.0, so
            // these are the same sums with one rounding, for two instructions less per k-step)
            const float s1 = shifted ? m[0] : m[1], s2 = shifted ? m[1] : m[2], s3 = shifted ? m[2] : m[3];
            const float t2 = c2ok ? s2 : 0.0f;
            b[ks][0] = fmaf(k0f, m[0], -t2);
            b[ks][1] = s1 + t2;
            b[ks][2] = t2 - s1;
            b[ks][3] = fmaf(k3f, s3, -s1);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int eg = 0; eg < 2; ++eg) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
                for (int e = 2 * eg; e < 2 * eg + 2; ++e)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        const float a = oddPair ? f[e][nb][2 * ks + 1] : f[e][nb][2 * ks];
                        acc[e][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b[ks][e], acc[e][nb], 0, 0, 0);
                    }
                if (eg == 0) {
                    if constexpr (decltype(plainNext)::value) load_rows_plain(raw[ks], (ch + KW) * KC + 4 * ks);
                    else load_rows_ranged(raw[ks], (ch + KW) * KC + 4 * ks);
                } else {
                    load_filters(f[ks], ks, next);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        load_filters(f[2], 2, next);
        load_filters(f[3], 3, next);
        __builtin_amdgcn_sched_barrier(0);
    };
    const int chMain = min(chEnd, (I - 1) / KC - KW);      // (see the 32-tile kernel)
    int ch = chBegin + kset;
    for (; ch < chMain; ch += KW) stage(ch, std::true_type{});
    for (; ch < chEnd; ch += KW) stage(ch, std::false_type{});

    // ---- epilogue: right factor in registers, rows meet in LDS, left factor, bias, ReLU, store ----
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float m0 = acc[0][nb][r], m1 = acc[1][nb][r], m2 = acc[2][nb][r], m3 = acc[3][nb][r];
            const int ol = 16 * nb + 4 * lk + r;
            P[(((kset * 4 + wave) * 2 + 0) * OB + ol) * TB + l16] = m0 + m1 + m2;
            P[(((kset * 4 + wave) * 2 + 1) * OB + ol) * TB + l16] = m1 - m2 + m3;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");

    const bool direct = nSplits == 1;
    const int et = tid & 15, eo = tid >> 4;
    const int etg = t0 + et;
    const bool eTileOk = etg < T;
    const int eTy = eTileOk ? fast_div(etg, tilesXd) : 0;
    const int ox = eTileOk ? 2 * (etg - eTy * tilesX) : 0, oy = 2 * eTy;
    f32x4* wsTiles = direct ? nullptr : (f32x4*)ws + ((size_t)split * nBlocks + logical) * OB * TB;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        const int ol = eo + EO * q, o = o0 + ol;
        if (ol >= OB) break;                        // (EO can exceed OB: 16 channels, four wave sets)
        float p[4][2];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            p[r][0] = P[((r * 2 + 0) * OB + ol) * TB + et];
            p[r][1] = P[((r * 2 + 1) * OB + ol) * TB + et];
#pragma unroll
            for (int ksx = 1; ksx < KW; ++ksx) {    // the other wave sets' shares of the channel sum, in set order
                p[r][0] += P[(((ksx * 4 + r) * 2 + 0) * OB + ol) * TB + et];
                p[r][1] += P[(((ksx * 4 + r) * 2 + 1) * OB + ol) * TB + et];
            }
        }
        float y00 = p[0][0] + p[1][0] + p[2][0], y01 = p[0][1] + p[1][1] + p[2][1];
        float y10 = p[1][0] - p[2][0] + p[3][0], y11 = p[1][1] - p[2][1] + p[3][1];
        if (direct) {
            if (eTileOk && o < O) {
                if (bias) { const float bv = biasEarly[q]; y00 += bv; y01 += bv; y10 += bv; y11 += bv; }
                if (relu & kEpiRelu) { y00 = fmaxf(y00, 0.f); y01 = fmaxf(y01, 0.f); y10 = fmaxf(y10, 0.f); y11 = fmaxf(y11, 0.f); }
                if (relu & kEpiMaxPool2)
                    store1_through(out + (size_t)o * (plane >> 2) + (size_t)(oy >> 1) * (W >> 1) + (ox >> 1), fmaxf(fmaxf(y00, y01), fmaxf(y10, y11)));
                else
                    wino_store_tile(out + (size_t)o * plane + (size_t)oy * W + ox, W, H, ox, oy, vec2, y00, y01, y10, y11);
            }
        } else {
            f32x4 v = {y00, y01, y10, y11};
            wsTiles[(size_t)ol * TB + et] = v;
        }
    }
}

// out[o][2x2 tile] = act(bias[o] + sum over splits of the partial tile), splits added in order.
// One lane per (o, tile); partials are [split][panel][o in panel][tile in panel] float4.
// Workgroup b works for panel (b % 8) * perXcd + ..., i.e. on the XCD whose workgroups wrote that
// panel's partial tiles a moment ago: they are still in that XCD's L2.
__global__ void __launch_bounds__(256)
winograd_split_reduce_kernel(const float* __restrict__ ws, const float* __restrict__ bias, float* __restrict__ out, WINO_ARGS) {
    // (TB, OB and TB * OB / 256 are powers of two: shifts and masks instead of integer divisions; cfg1 carries
    // log2 TB and log2 OB above the chunk count)
    const int lgTB = (int)((cfg1 >> 16) & 15u), lgOB = (int)((cfg1 >> 20) & 15u);
    const int TB = 1 << lgTB, OB = 1 << lgOB, lgBpp = lgTB + lgOB - 8;
    const int W = (int)(wh & 0xffffu), H = (int)(wh >> 16), O = (int)(io >> 16);
    const int tilesX = (W + 1) >> 1, T = tilesX * ((H + 1) >> 1);
    const int nTB = (T + TB - 1) >> lgTB, nBlocks = nTB * ((O + OB - 1) >> lgOB);
    const FastDiv tilesXd = {(unsigned)tilesX, mulX, cfg0 & 31u}, nTBd = {(unsigned)nTB, mulTB, (cfg0 >> 5) & 31u};
    const int relu = (int)((cfg0 >> 10) & 3u), vec2 = (int)((cfg0 >> 12) & 1u), nSplits = (int)((cfg0 >> 13) & 0xffffu);
    const int perXcd = (nBlocks + kXcds - 1) / kXcds;
    const int j = blockIdx.x / kXcds, jp = j >> lgBpp;
    const int panel = (blockIdx.x % kXcds) * perXcd + jp;
    if (jp >= perXcd || panel >= nBlocks) return;
    const int within = ((j & ((1 << lgBpp) - 1)) << 8) + threadIdx.x;     // (o in panel) * TB + tile in panel
    const int tLocal = within & (TB - 1), ol = within >> lgTB;
    const int oBlock = fast_div(panel, nTBd);
    const int o = oBlock * OB + ol, tg = (panel - oBlock * (int)nTBd.d) * TB + tLocal;
    if (o >= O || tg >= T) return;
    const size_t idx = (size_t)panel * TB * OB + within;
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
    if (relu & kEpiRelu) { s[0] = fmaxf(s[0], 0.f); s[1] = fmaxf(s[1], 0.f); s[2] = fmaxf(s[2], 0.f); s[3] = fmaxf(s[3], 0.f); }
    const int ty = fast_div(tg, tilesXd);
    const int ox = 2 * (tg - ty * (int)tilesXd.d), oy = 2 * ty;
    if (relu & kEpiMaxPool2)
        store1_through(out + (size_t)o * ((H >> 1) * (W >> 1)) + (size_t)(oy >> 1) * (W >> 1) + (ox >> 1), fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])));
    else
        wino_store_tile(out + (size_t)o * H * W + (size_t)oy * W + ox, W, H, ox, oy, vec2, s[0], s[1], s[2], s[3]);
}

// variant = output channels per workgroup (low 4 bits: 1 -> 32, 2 -> 64, 3 -> 128)
//         | log2(number of input-channel splits) << 4
//         | 0x100: 16-tile blocks (then the low 4 bits mean 1 -> 16, 2 -> 32, 3 -> 64 channels)
//         | 0x400: eight waves per workgroup, two wave sets sharing the stages (32-tile blocks of 32 or 64 channels,
//                  or 16-tile blocks)
//         | 0x800: joined splits - the splits of a panel add their partial tiles up inside the one launch (32-tile
//                  blocks, 2 to 16 splits, every workgroup of the launch resident at once; the workspace must have
//                  been through drhip_conv3x3_winograd_workspace_prepare_f32)
//         | 0x1000 (with 0x800, split bits 0): tiered joined splits - the panels of an XCD are dealt out in tiers
//                  of whole panels, halves, quarters, ... so that every CU ends up with about the same number of
//                  stages (see wino_tiers)
struct WinoCfg { int nt, splits, tb, waveSets; bool joined, tiered; };

static bool wino_variant(int variant, WinoCfg* c) {
    c->waveSets = (variant & 0x400) ? 2 : 1;
    c->joined = (variant & 0x800) != 0;
    c->tiered = (variant & 0x1000) != 0;
    if (variant >> 13) return false;
    if (c->tiered && (!c->joined || c->waveSets == 2 || ((variant >> 4) & 0xf) != 0 || (variant & 0xf) > 2)) return false;
    if (c->joined && !c->tiered && ((variant & 0x100) || ((variant >> 4) & 0xf) < 1 || ((variant >> 4) & 0xf) > 4)) return false;
    if (c->joined && (variant & 0x100)) return false;
    if (c->waveSets == 2 && !(variant & 0x100) && (variant & 0xf) > 2) return false;
    variant &= ~0x1c00;
    const int lg = (variant >> 4) & 0xf;
    if (lg > 6 || (variant >> 9)) return false;
    c->splits = 1 << lg;
    c->tb = (variant & 0x100) ? 16 : 32;
    switch (variant & 0xf) {
        case 1: c->nt = 1; return true;
        case 2: c->nt = 2; return true;
        case 3: c->nt = 4; return true;
        default: return false;
    }
}

struct WinoGeom { int tilesX, T, nTB, nOB, nBlocks, nChunks, chunksPerSplit, splits; };

static WinoGeom wino_geom(int W, int H, int I, int O, const WinoCfg& c) {
    WinoGeom g;
    g.tilesX = (W + 1) / 2;
    g.T = g.tilesX * ((H + 1) / 2);
    g.nTB = ceil_div(g.T, c.tb);
    g.nOB = ceil_div(O, c.tb * c.nt);
    g.nBlocks = g.nTB * g.nOB;
    g.nChunks = ceil_div(I, kWinoKC);
    int splits = c.splits < g.nChunks ? c.splits : g.nChunks;
    g.chunksPerSplit = ceil_div(g.nChunks, splits);
    g.splits = ceil_div(g.nChunks, g.chunksPerSplit);      // no empty split
    return g;
}

// Tiers of a balanced launch, per XCD.  An XCD has P panels and `cus` CUs.  Written as P / cus = w + 1/2 + 1/4 + ...
// (binary digits), the panels fall into a tier of w * cus whole panels, a tier of cus / 2 panels cut into halves,
// one of cus / 4 panels cut into quarters, and so on: each of these tiers puts one workgroup on every CU (the
// dispatcher deals the workgroups of a launch out in order, one to each CU before any CU gets a second one), and
// what is left below the finest cut goes out in that cut.  Pieces are powers of two of stages and never less
// than one stage; at most four tiers, at most 255 panels in one.  The tiers are launched finest cut first.
struct WinoTiers { int n[4], lg[4], count, wgsPerXcd, maxLg; };

static bool wino_tiers(int nBlocks, int nChunks, int cus, WinoTiers* t) {
    *t = WinoTiers{};
    const int P = ceil_div(nBlocks, kXcds);
    int maxLg = 0;
    while (maxLg < 4 && (nChunks & ((2 << maxLg) - 1)) == 0 && (cus >> (maxLg + 1)) >= 1) ++maxLg;
    auto add = [&](int n, int lg) {
        if (n <= 0) return true;
        if (t->count && t->lg[t->count - 1] == lg) { t->n[t->count - 1] += n; return t->n[t->count - 1] <= 255; }
        if (t->count == 4 || n > 255) return false;
        t->n[t->count] = n; t->lg[t->count] = lg; ++t->count;
        return true;
    };
    int r = P;
    if (!add(r / cus * cus, 0)) return false;
    r %= cus;
    for (int lg = 1; lg <= maxLg; ++lg)
        if (r >= (cus >> lg)) { if (!add(cus >> lg, lg)) return false; r -= cus >> lg; }
    if (!add(r, maxLg)) return false;
    for (int k = 0; k < t->count / 2; ++k) { std::swap(t->n[k], t->n[t->count - 1 - k]); std::swap(t->lg[k], t->lg[t->count - 1 - k]); }
    for (int k = 0; k < t->count; ++k) { t->wgsPerXcd += t->n[k] << t->lg[k]; t->maxLg = t->lg[k] > t->maxLg ? t->lg[k] : t->maxLg; }
    return t->maxLg > 0;
}

// Workspace: [splits][panel][o in panel][tile in panel] partial 2x2 tiles (float4 each); tiered launches: one
// panel-sized region per workgroup of the grid.
template <int NT, int TB>
static int launch_wino(const float* in, const float* U, const float* bias, float* out, float* workspace,
                       int W, int H, int I, int O, int relu, const WinoCfg& c, hipStream_t s) {
    constexpr int OB = TB * NT;
    const WinoGeom g = wino_geom(W, H, I, O, c);
    const int gridX = ceil_div(g.nBlocks, kXcds) * kXcds;
    const size_t ldsBytes = 4 * 2 * OB * TB * sizeof(float);
    const int vec2 = ((W & 1) == 0) && (((size_t)out & 7) == 0);
    const FastDiv dx = make_fastdiv(g.tilesX), dtb = make_fastdiv(g.nTB);
    const bool joined = c.joined && g.splits > 1;   // (a layer with fewer stages than splits may end up unsplit)
    if constexpr (TB == 32) {
        WinoTiers t;
        if (c.tiered && wino_tiers(g.nBlocks, g.nChunks, num_cu() / kXcds, &t)) {
            unsigned lgs = 0, counts = 0;
            for (int k = 0; k < t.count; ++k) { lgs |= (unsigned)t.lg[k] << (4 * k); counts |= (unsigned)t.n[k] << (8 * k); }
            launch((winograd_f23_mfma_kernel<NT, 1>), dim3(t.wgsPerXcd * kXcds), dim3(kWinoThreads), ldsBytes, s, in, U, bias,
                   (unsigned)W | (unsigned)H << 16, (unsigned)I | (unsigned)O << 16, dx.mul, dtb.mul,
                   dx.shift | dtb.shift << 5 | (unsigned)(relu & 3) << 10 | (unsigned)vec2 << 12 | lgs << 13 | 3u << 30, counts, out, workspace);
            return launched("winograd_f23_mfma_kernel");
        }
    }
    const WinoPackedArgs pa = {(unsigned)W | (unsigned)H << 16, (unsigned)I | (unsigned)O << 16, dx.mul, dtb.mul,
                               dx.shift | dtb.shift << 5 | (unsigned)(relu & 3) << 10 | (unsigned)vec2 << 12 | (unsigned)g.splits << 13 |
                                   (joined ? 1u << 31 : 0u),
                               (unsigned)g.chunksPerSplit | (joined ? (unsigned)__builtin_ctz(g.splits) << 24 : 0u)};
    // joined: one grid row, the splits of a panel side by side on one XCD (see the kernel)
    const dim3 grid = joined ? dim3(gridX * g.splits) : dim3(gridX, g.splits);
    if constexpr (TB == 32) {
        if constexpr (NT <= 2) {
            if (c.waveSets == 2) {
                // more than 64 KiB of dynamic LDS has to be asked for once per kernel
                // (the attribute belongs to the kernel's code object on ONE device)
                // (remembered per device; graphs may be prepared and applied from several host threads)
                static std::atomic<bool> raised[64];
                int device = 0;
                if (int rc = check(hipGetDevice(&device), "hipGetDevice")) return rc;
                const bool known = device >= 0 && device < 64;
                if (2 * ldsBytes > 65536 && !(known && raised[device].load(std::memory_order_acquire))) {
                    if (int rc = check(hipFuncSetAttribute((const void*)winograd_f23_mfma_kernel<NT, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(2 * ldsBytes)),
                                       "hipFuncSetAttribute(max dynamic LDS)")) return rc;
                    if (known) raised[device].store(true, std::memory_order_release);
                }
            }
            if (c.waveSets == 2)
                launch((winograd_f23_mfma_kernel<NT, 2>), grid, dim3(2 * kWinoThreads), 2 * ldsBytes, s,
                       in, U, bias, pa.wh, pa.io, pa.mulX, pa.mulTB, pa.cfg0, pa.cfg1, out, workspace);
        }
        if (c.waveSets != 2 || NT > 2) {
            if (NT <= 2 && I <= 4 && g.splits == 1) {       // an image: the stage without its two empty k-steps
                if constexpr (NT <= 2)
                    launch((winograd_f23_mfma_kernel<NT, 1, true>), grid, dim3(kWinoThreads), ldsBytes, s,
                           in, U, bias, pa.wh, pa.io, pa.mulX, pa.mulTB, pa.cfg0, pa.cfg1, out, workspace);
            } else
                launch((winograd_f23_mfma_kernel<NT, 1>), grid, dim3(kWinoThreads), ldsBytes, s,
                       in, U, bias, pa.wh, pa.io, pa.mulX, pa.mulTB, pa.cfg0, pa.cfg1, out, workspace);
        }
    } else if (c.waveSets == 2)
        launch((winograd_f23_mfma16_kernel<NT, 2>), grid, dim3(2 * kWinoThreads), 2 * ldsBytes, s,
               in, U, bias, pa.wh, pa.io, pa.mulX, pa.mulTB, pa.cfg0, pa.cfg1, out, workspace);
    else
        launch((winograd_f23_mfma16_kernel<NT, 1>), grid, dim3(kWinoThreads), ldsBytes, s,
               in, U, bias, pa.wh, pa.io, pa.mulX, pa.mulTB, pa.cfg0, pa.cfg1, out, workspace);
    if (int rc = launched("winograd_f23_mfma_kernel")) return rc;
    if (g.splits > 1 && !joined) {
        launch(winograd_split_reduce_kernel, dim3(gridX * (OB * TB / 256)), dim3(256), 0, s,
               workspace, bias, out, pa.wh, pa.io, pa.mulX, pa.mulTB, pa.cfg0,
               pa.cfg1 | (unsigned)__builtin_ctz(TB) << 16 | (unsigned)__builtin_ctz(OB) << 20);
        return launched("winograd_split_reduce_kernel");
    }
    return DRHIP_OK;
}

}  // namespace drhip

using namespace drhip;

// Configuration for one layer, from measurements on MI355X (256 CUs):
//   - 32 output channels per workgroup; 64 only for layers with very many tiles (224x224), where
//     the panels alone give several workgroups per CU and sharing the input transform pays;
//   - the input channels are split until at least ~160 workgroups exist, keeping at least 2 stages
//     of 8 channels per split;
//   - split layers with very long channel loops trade panel width against split count;
//   - small layers take the 16-tile kernel.
// 0x800 if a split of 2^lg can be joined: 2 to 8 splits of equal length (a power of two of stages), and the
// switch DR_WINO_JOIN is not 0.
static int wino_join_flag(int lg, int nChunks) {
    static const bool enabled = [] { const char* e = getenv("DR_WINO_JOIN"); return !(e && e[0] == '0'); }();
    return (enabled && lg >= 1 && lg <= 3 && (nChunks & ((1 << lg) - 1)) == 0) ? 0x800 : 0;
}

extern "C" int drhip_conv3x3_winograd_pick_variant(int W, int H, int I, int O) {
    const int T = ((W + 1) / 2) * ((H + 1) / 2);
    const int cus = num_cu();
    // Small layers (SqueezeNet's expand convolutions: <= 8 stages, a few dozen 32x32 panels) are bound
    // by the latency of one workgroup, not by throughput: 16x16 blocks, unsplit, one launch
    // (in a replayed launch graph 4.2-5.8 us per layer against 5.1-7.1 us for the 32x32 forms).
    if (ceil_div(T, 32) * ceil_div(O, 32) < cus / 2 && ceil_div(I, kWinoKC) <= 16)
        // 6+ stages and at most one workgroup per CU (14x14 maps; 56x56 64->64: 5.3 vs 5.5 us): two wave sets
        return (ceil_div(I, kWinoKC) >= 6 && ceil_div(T, 16) * ceil_div(O, 16) <= cus) ? 0x501 : 0x101;
    // (an image layer has next to no transform work to share, and twice the workgroups of half the size spread its
    // stores better: 224x224 3->64 6.1 vs 6.7 us)
    const int code = (O > 32 && T >= 8192 && I > 4) ? 2 : 1;
    const int panels = ceil_div(T, 32) * ceil_div(O, code == 2 ? 64 : 32);
    const int nChunks = ceil_div(I, kWinoKC);
    int lg = 0;
    // (a split costs a second kernel: below 6 stages in all it does not pay)
    while (lg < 5 && nChunks >= 6 && (panels << lg) < (5 * cus) / 8 && (nChunks >> (lg + 1)) >= 2) ++lg;
    // At most one workgroup per CU and at least two stages for each wave set: eight waves per workgroup,
    // so that every SIMD still has two waves to alternate between (56x56 256->256: 23.6 vs 24.8 us;
    // 28x28 512->512 as 112 panels x 2 splits: 26.3 vs 26.9 us for 64-channel panels x 4 splits).
    // A split whose workgroups are all resident at once (one per CU) adds its partial tiles up inside the launch.
    // (joined splits of fewer than 16 stages each: four waves, 14x14 512->512 as 8 splits: 10.4 vs 11.1 us)
    if ((panels << lg) <= cus && (nChunks >> lg) >= 4) {
        const int join = wino_join_flag(lg, nChunks);
        return ((join && (nChunks >> lg) < 16) ? 0 : 0x400) | code | (lg << 4) | join;
    }
    // Unsplit layers with more 32-channel panels than CUs, but no multiple of them (112x112 128->128: 392 panels,
    // two on 136 CUs and one on 120): tiers of whole, halved, ... panels even the CUs out (in a replayed VGG16
    // pass 18.4 vs 20.2 us, of which the layer behind it gives 0.5 us back).  With 8 stages it is a tie or a loss
    // (224x224 64->64 as 32-channel panels in tiers: 20.4 vs 20.0 us for 64-channel panels).
    if (lg == 0 && wino_join_flag(1, 2)) {
        static const bool tiersOn = [] { const char* e = getenv("DR_WINO_TIERS"); return !(e && e[0] == '0'); }();
        const int cusPerXcd = cus / kXcds, P = ceil_div(ceil_div(T, 32) * ceil_div(O, 32), kXcds);
        WinoTiers t;
        if (tiersOn && cusPerXcd > 0 && P >= cusPerXcd && P % cusPerXcd != 0 && nChunks >= 16 &&
            wino_tiers(ceil_div(T, 32) * ceil_div(O, 32), nChunks, cusPerXcd, &t))
            return 0x1801;
    }
    // A split layer that still has 32 or more stages per split: the same number of workgroups as
    // 64-channel panels with twice the splits share each input transform between two MFMA sets.
    if (code == 1 && lg >= 1 && lg < 5 && O >= 64 && (nChunks >> lg) >= 32) return 2 | ((lg + 1) << 4);
    return code | (lg << 4);
}

extern "C" int drhip_conv3x3_winograd_workspace_prepare_f32(float* workspace, size_t floats, void* stream) {
    DRHIP_REQUIRE(workspace || floats == 0, "drhip_conv3x3_winograd_workspace_prepare_f32: NULL workspace");
    if (floats == 0) return DRHIP_OK;
    return drhip_fill_f32(workspace, __builtin_bit_cast(float, kWinoEmpty), floats, stream);
}

extern "C" int drhip_conv3x3_winograd_join_timeouts(unsigned* count) {
    DRHIP_REQUIRE(count, "drhip_conv3x3_winograd_join_timeouts: NULL result pointer");
    return check(hipMemcpyFromSymbol(count, HIP_SYMBOL(g_wino_join_timeouts), sizeof(unsigned)), "hipMemcpyFromSymbol(join timeouts)");
}

extern "C" size_t drhip_conv3x3_winograd_filter_floats(int I, int O) {
    if (I <= 0 || O <= 0) return 0;
    return (size_t)16 * ceil_div(I, kWinoKC) * kWinoKC * wino_opad(O);
}

extern "C" size_t drhip_conv3x3_winograd_workspace_floats(int W, int H, int I, int O, int variant) {
    WinoCfg c;
    if (W <= 0 || H <= 0 || I <= 0 || O <= 0 || !wino_variant(variant, &c)) return 0;
    const WinoGeom g = wino_geom(W, H, I, O, c);
    WinoTiers t;
    if (c.tiered) return wino_tiers(g.nBlocks, g.nChunks, num_cu() / kXcds, &t) ? (size_t)t.wgsPerXcd * kXcds * (c.tb * c.nt) * c.tb * 4 : 0;
    if (g.splits <= 1) return 0;
    return (size_t)g.splits * g.nBlocks * (c.tb * c.nt) * c.tb * 4;
}

extern "C" int drhip_winograd_filter_transform_f32(const float* w, float* U, int I, int O, void* stream) {
    DRHIP_REQUIRE(w && U, "drhip_winograd_filter_transform_f32: NULL tensor");
    DRHIP_REQUIRE(I > 0 && O > 0 && (long long)(I + 7) * (O + 31) * 16 < (1ll << 29), "drhip_winograd_filter_transform_f32: bad shape I=%d O=%d", I, O);
    const int nChunks = ceil_div(I, kWinoKC);
    launch(winograd_filter_transform_kernel, dim3(ceil_div(nChunks * 8 * wino_opad(O), 256)), dim3(256), 0, as_stream(stream), w, U, I, O, nChunks);
    return launched("winograd_filter_transform_kernel");
}

extern "C" int drhip_conv3x3_winograd_f32(const float* in, const float* U, const float* bias, float* out,
                                          int W, int H, int I, int O, int relu, int variant,
                                          float* workspace, void* stream) {
    DRHIP_REQUIRE(in && U && out, "drhip_conv3x3_winograd_f32: NULL tensor");
    DRHIP_REQUIRE(W > 0 && H > 0 && I > 0 && O > 0, "drhip_conv3x3_winograd_f32: bad shape %dx%dx%d -> %d", W, H, I, O);
    // byte offsets into the input and the filters are 32-bit, and 0x80000000 must lie outside both
    DRHIP_REQUIRE((long long)W * H * I < (1ll << 29) && (long long)W * H * O < (1ll << 31) && (long long)(I + 7) * (O + 31) * 16 < (1ll << 29),
                  "drhip_conv3x3_winograd_f32: tensor too large for 32-bit byte offsets");
    DRHIP_REQUIRE(W <= 65535 && H <= 65535 && I <= 65535 && O <= 65535, "drhip_conv3x3_winograd_f32: W, H, I and O are limited to 65535 (got %dx%dx%d -> %d)", W, H, I, O);
    DRHIP_REQUIRE(((size_t)U & 15) == 0, "drhip_conv3x3_winograd_f32: transformed filters must be 16-byte aligned");
    DRHIP_REQUIRE((relu & ~(DRHIP_EPILOGUE_RELU | DRHIP_EPILOGUE_MAXPOOL2)) == 0, "drhip_conv3x3_winograd_f32: unknown epilogue flags %d", relu);
    DRHIP_REQUIRE(!(relu & DRHIP_EPILOGUE_MAXPOOL2) || ((W | H) & 1) == 0, "drhip_conv3x3_winograd_f32: the fused 2x2 max pool needs even W and H (got %dx%d)", W, H);
    if (variant == 0) {
        variant = drhip_conv3x3_winograd_pick_variant(W, H, I, O);
        if (variant & 0x1000) variant = (variant & 0xf) == 2 ? 2 : 1;      // (joined splits need a prepared workspace: explicit variants only)
        variant &= ~0x800;
        if (!workspace) variant &= 0x50f;          // no workspace offered: stay unsplit
    }
    WinoCfg c;
    DRHIP_REQUIRE(wino_variant(variant, &c), "drhip_conv3x3_winograd_f32: unknown variant %d", variant);
    const WinoGeom g = wino_geom(W, H, I, O, c);
    DRHIP_REQUIRE(g.splits == 1 || workspace, "drhip_conv3x3_winograd_f32: variant %d splits the input channels and needs a workspace", variant);
    DRHIP_REQUIRE(g.splits <= 65535, "drhip_conv3x3_winograd_f32: too many input-channel splits");
    if (c.tiered) {
        WinoTiers t;
        if (wino_tiers(g.nBlocks, g.nChunks, num_cu() / kXcds, &t)) {
            // A workgroup waits for the other splits of its panel, which follow it in dispatch order on the same
            // XCD: as long as one XCD holds more workgroups than a panel has splits, they all get to run.
            DRHIP_REQUIRE(workspace, "drhip_conv3x3_winograd_f32: variant %#x joins splits and needs a prepared workspace", variant);
            DRHIP_REQUIRE((1 << t.maxLg) < num_cu() / kXcds, "drhip_conv3x3_winograd_f32: variant %#x cuts panels into %d pieces, an XCD holds %d workgroups", variant, 1 << t.maxLg, num_cu() / kXcds);
            DRHIP_REQUIRE((long long)t.wgsPerXcd * kXcds * c.tb * c.nt * c.tb * 16 < (1ll << 31), "drhip_conv3x3_winograd_f32: workspace beyond 2 GiB");
        }
    } else if (c.joined && g.splits > 1) {
        // every workgroup waits for its panel's other splits: all of them have to be resident together
        const int perCu = c.waveSets == 2 ? 1 : (c.nt == 1 ? 3 : (c.nt == 2 ? 2 : 1));
        DRHIP_REQUIRE((g.splits & (g.splits - 1)) == 0 && g.splits <= kWinoMaxJoin && g.splits * g.chunksPerSplit == g.nChunks,
                      "drhip_conv3x3_winograd_f32: variant %#x joins %d splits of %d stages: 2, 4, 8 or 16 equal splits only", variant, g.splits, g.chunksPerSplit);
        DRHIP_REQUIRE((long long)g.nBlocks * g.splits <= (long long)num_cu() * perCu,
                      "drhip_conv3x3_winograd_f32: variant %#x needs its %d workgroups resident at once, the device holds %d", variant,
                      g.nBlocks * g.splits, num_cu() * perCu);
        DRHIP_REQUIRE((long long)g.splits * g.nBlocks * c.tb * c.nt * c.tb * 16 < (1ll << 31), "drhip_conv3x3_winograd_f32: workspace beyond 2 GiB");
    }
    hipStream_t s = as_stream(stream);
    if (c.tb == 16) {
        if (c.nt == 1) return launch_wino<1, 16>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
        if (c.nt == 2) return launch_wino<2, 16>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
        return launch_wino<4, 16>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
    }
    if (c.nt == 1) return launch_wino<1, 32>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
    if (c.nt == 2) return launch_wino<2, 32>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
    return launch_wino<4, 32>(in, U, bias, out, workspace, W, H, I, O, relu, c, s);
}
