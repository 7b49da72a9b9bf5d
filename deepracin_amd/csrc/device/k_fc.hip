// Fully connected layer at batch 1 = GEMV y[n] = act(b[n] + sum_k x[k] * Wt[k][n]); HBM-bound:
// algorithmic bytes = 4*(K*N + K + 2N), every weight is read exactly once.
//
// Mapping for gfx950
//   - Wt is [K][N], n fastest, so one row segment is contiguous: a wavefront reads 64 x float4 =
//     1 KiB of one row per load instruction (fully coalesced, nontemporal: the matrix is streamed
//     once and must not evict activations from L2 / Infinity Cache);
//   - a workgroup (4 waves) owns a panel of CBW = 64*VEC columns and a slice of rows; its waves take
//     64-row chunks round-robin and keep 8-16 row loads (8-16 KiB per wave) in flight;
//   - x for a 64-row chunk is loaded once, one element per lane, and broadcast with v_readlane;
//   - the input vector may arrive unfinished, as the partial sums a previous GEMV left behind
//     (drhip_deferred_vec): a wave then sums the slices of its 64 rows itself, in slice order, adds
//     the bias and applies ReLU - bit for bit what the reduce kernel would have stored, without
//     the launch (a ~4 us kernel between two GEMVs of 13 and 7 us);
//   - split-K: the grid is (column panels) x (row slices), sized to a few workgroups per CU; each
//     workgroup writes one partial row and a second, tiny kernel sums the partials in slice order,
//     adds the bias and applies ReLU (the same two-step shape as the reference; no device-scope
//     fences, which on a multi-XCD part cost an L2 write-back per workgroup).  Summation order is
//     fixed, so results are reproducible run to run.
//
// Reference semantics: Kernels/dR_fcl.cl:59-120 (two kernels: partial sums over partitions of K,
// then a sequential sum of the partials + bias + clamp).  The partition size there depends on the
// OpenCL device; any partitioning gives the same sum up to fp32 rounding.
#include "drhip_common.hpp"

namespace drhip {

constexpr int kFcThreads = 256;
constexpr int kFcWaves = kFcThreads / kWave;
constexpr int kFcUnroll = 8;

template <int VEC> struct VecT;
template <> struct VecT<4> { typedef float __attribute__((ext_vector_type(4))) type; };
template <> struct VecT<2> { typedef float __attribute__((ext_vector_type(2))) type; };
template <> struct VecT<1> { typedef float type; };

template <int VEC>
__device__ inline void fma_row(float (&acc)[VEC], const typename VecT<VEC>::type& w, float xv) {
    if constexpr (VEC == 1) acc[0] = fmaf(w, xv, acc[0]);
    else {
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = fmaf(w[v], xv, acc[v]);
    }
}

struct FcPlan { int vec, cbw, panels, slices, rowsPerSlice; };

// Split of the [K][N] matrix into column panels and row slices.
static FcPlan fc_plan(int K, int N) {
    FcPlan p;
    p.vec = (N % 4 == 0) ? 4 : (N % 2 == 0) ? 2 : 1;
    while (p.vec > 1 && ceil_div(N, kWave * p.vec) < 16) p.vec /= 2;    // narrow matrices (N = 1000): more, narrower panels
    p.cbw = kWave * p.vec;
    p.panels = ceil_div(N, p.cbw);
    // One workgroup per CU is enough to keep the memory system full (25088 x 4096: 61.6 us with 256 workgroups,
    // 62.1 with 1024, 64.1 with 2048), and the fewer row slices a layer leaves behind, the shorter the start of the
    // layer that sums them while it loads its input (4096 x 4096 behind 16 instead of 56 slices: 12.2 against 13.3 us).
    const int target = num_cu();                     // workgroups wanted in flight
    int slices = ceil_div(target, p.panels);
    const int maxSlices = ceil_div(K, 4 * kWave);    // at least 256 rows per workgroup (4096 x 4096: 13.7 us with 16 slices, 14.8 with 32)
    if (slices > maxSlices) slices = maxSlices;
    if (slices < 1) slices = 1;
    p.rowsPerSlice = ceil_div(ceil_div(K, slices), kWave) * kWave;   // whole chunks
    p.slices = ceil_div(K, p.rowsPerSlice);
    return p;
}

// Partial GEMV of one (column panel, row slice).  slices == 1: writes y directly (bias, ReLU).
// Otherwise writes partials[slice][n]; fc_reduce_kernel finishes.
// CH = rows per wavefront and turn (64, 32 or 16): a wavefront fetches CH activations, one per lane,
// and streams the CH matrix rows against them.  Short slices use a small CH so that all four
// wavefronts of the workgroup have rows to stream.
template <int VEC, bool DEFERRED, int CH>
__global__ void __launch_bounds__(kFcThreads)
fc_gemv_kernel(const float* __restrict__ Wt, const float* __restrict__ x, int K, int N, int rowsPerSlice, int cfg,
               const float* __restrict__ bias, float* __restrict__ y, float* __restrict__ partials, drhip_deferred_vec xdef) {
    // The first 14 dwords of arguments arrive in SGPRs with the wave: the matrix, the shape and the output pointers;
    // the description of a deferred input follows behind them.  cfg = relu | row slices << 8 (the grid's
    // y extent: read from here, not from the dispatch packet).
    const int relu = cfg & 1;
    typedef typename VecT<VEC>::type vec_t;
    constexpr int CBW = kWave * VEC;
    __shared__ float red[kFcWaves][CBW];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int panel = blockIdx.x, slice = blockIdx.y, slices = cfg >> 8;
    // Lanes past the last column re-read the last valid vector (their sums are never stored): the
    // loads stay unconditional, so the compiler can keep a precise count of loads in flight.
    const int col = min(panel * CBW + lane * VEC, N - VEC);
    const int rowBegin = slice * rowsPerSlice;
    const int rowEnd = min(K, rowBegin + rowsPerSlice);

    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;

    for (int r0 = rowBegin + wave * CH; r0 < rowEnd; r0 += kFcWaves * CH) {
        const int rows = min(CH, rowEnd - r0);
        const float* wp = Wt + (size_t)r0 * N + col;
        // The matrix stream starts before the activation is fetched: a deferred input costs a few
        // rounds of loads of its own, and the weights must not wait behind them.
        vec_t wa[kFcUnroll], wb[kFcUnroll];
        if (rows == CH) {
#pragma unroll
            for (int u = 0; u < kFcUnroll; ++u) wa[u] = __builtin_nontemporal_load((const vec_t*)(wp + (size_t)u * N));
        }
        float xraw = 0.0f;
        if (CH == kWave || lane < CH) xraw = DEFERRED ? deferred_element(xdef, min(r0 + lane, K - 1)) : x[min(r0 + lane, K - 1)];
        const float xl = (lane < rows) ? xraw : 0.0f;
        if (DEFERRED && xdef.finished && panel == 0 && lane < rows) xdef.finished[r0 + lane] = xraw;   // each row once
        if (rows == CH) {
            // CH rows as batches of 8 row loads; two batches (16 KiB per wave) are always in flight
#pragma unroll
            for (int j0 = 0; j0 < CH; j0 += 2 * kFcUnroll) {
#pragma unroll
                for (int u = 0; u < kFcUnroll; ++u)
                    wb[u] = __builtin_nontemporal_load((const vec_t*)(wp + (size_t)(j0 + kFcUnroll + u) * N));
#pragma unroll
                for (int u = 0; u < kFcUnroll; ++u)
                    fma_row<VEC>(acc, wa[u], __int_as_float(__builtin_amdgcn_readlane(__float_as_int(xl), j0 + u)));
                if (j0 + 2 * kFcUnroll < CH) {
#pragma unroll
                    for (int u = 0; u < kFcUnroll; ++u)
                        wa[u] = __builtin_nontemporal_load((const vec_t*)(wp + (size_t)(j0 + 2 * kFcUnroll + u) * N));
                }
#pragma unroll
                for (int u = 0; u < kFcUnroll; ++u)
                    fma_row<VEC>(acc, wb[u], __int_as_float(__builtin_amdgcn_readlane(__float_as_int(xl), j0 + kFcUnroll + u)));
            }
        } else {
            for (int j = 0; j < rows; ++j) {
                const float xv = __shfl(xl, j, 64);
                vec_t w = __builtin_nontemporal_load((const vec_t*)(wp + (size_t)j * N));
                fma_row<VEC>(acc, w, xv);
            }
        }
    }

    // combine the four waves of the workgroup
#pragma unroll
    for (int v = 0; v < VEC; ++v) red[wave][lane * VEC + v] = acc[v];
    __syncthreads();
    const int ncols = min(CBW, N - panel * CBW);
    for (int c = tid; c < ncols; c += kFcThreads) {
        const int n = panel * CBW + c;
        float s = red[0][c];
#pragma unroll
        for (int w = 1; w < kFcWaves; ++w) s += red[w][c];
        if (slices == 1) {
            if (bias) s += bias[n];
            if (relu) s = fmaxf(s, 0.0f);
            store_through(y + n, s);
        } else {
            store_through(partials + (size_t)slice * N + n, s);
        }
    }
}

// y[n] = act(bias[n] + sum over slices of partials[slice][n]), slices added in order.
__global__ void __launch_bounds__(256)
fc_reduce_kernel(const float* __restrict__ partials, const float* __restrict__ bias, float* __restrict__ y,
                 int N, int slices, int relu) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= N) return;
    const float* pp = partials + n;
    float s = 0.0f;
    int sl = 0;
    for (; sl + 8 <= slices; sl += 8) {             // 8 independent loads in flight, summed in slice order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = pp[(size_t)(sl + u) * N];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
    }
    for (; sl < slices; ++sl) s += pp[(size_t)sl * N];
    if (bias) s += bias[n];
    if (relu) s = fmaxf(s, 0.0f);
    store_through(y + n, s);
}

__global__ void __launch_bounds__(256)
fc_permute_rows_kernel(const float* __restrict__ src, float* __restrict__ dst, int W, int H, int C, int N) {
    // one workgroup per destination row k_chw = (z*H + y)*W + x  <-  source row k_hwc = (y*W + x)*C + z
    const int k = blockIdx.x;
    const int x = k % W, y = (k / W) % H, z = k / (W * H);
    const size_t srow = ((size_t)(y * W + x) * C + z) * N, drow = (size_t)k * N;
    for (int n = threadIdx.x; n < N; n += blockDim.x) dst[drow + n] = src[srow + n];
}

// Partial sums of drhip_fc_noalloc_f32: device memory that exists from the moment the code object
// is loaded until the process ends (one copy per GPU), so that entry point never allocates.
constexpr size_t kFcStaticScratchFloats = 64 * 1024;       // 256 KiB: what the largest layer of VGG16 needs (16 row slices of 4096 columns)
static __device__ __align__(256) float fc_static_scratch[kFcStaticScratchFloats];

constexpr int kFcMaxDevices = 64;
static float* g_fc_static_ptr[kFcMaxDevices];              // device address of the array on each GPU, set by drhip_init

// Called by drhip_init with `device` current: looks up where this GPU holds fc_static_scratch.
// The array's name is only a host-side handle; kernels and copies must be given this address.
int fc_static_scratch_setup(int device) {
    if (device < 0 || device >= kFcMaxDevices) return fail(DRHIP_EINVAL, "device ordinal %d beyond the %d this library keeps scratch for", device, kFcMaxDevices);
    if (g_fc_static_ptr[device]) return DRHIP_OK;
    float* p = nullptr;
    if (int rc = check(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(fc_static_scratch)), "hipGetSymbolAddress(fc_static_scratch)")) return rc;
    if (!p) return fail(DRHIP_EDEVICE, "hipGetSymbolAddress(fc_static_scratch) returned a NULL address");
    g_fc_static_ptr[device] = p;
    return DRHIP_OK;
}

}  // namespace drhip

using namespace drhip;

extern "C" size_t drhip_fc_scratch_floats(int K, int N) {
    if (K <= 0 || N <= 0) return 0;
    FcPlan p = fc_plan(K, N);
    return p.slices > 1 ? (size_t)p.slices * (size_t)N : 0;
}

extern "C" int drhip_fc_slices(int K, int N) {
    if (K <= 0 || N <= 0) return 0;
    return fc_plan(K, N).slices;
}

template <int VEC, int CH>
static void launch_gemv_ch(bool deferred, dim3 grid, hipStream_t s, const float* x, const drhip_deferred_vec& xd, const float* Wt,
                           const float* bias, float* y, float* partials, int K, int N, int rowsPerSlice, int relu, int defer) {
    const int cfg = (relu ? 1 : 0) | (int)(grid.y << 8);     // (an unfinished sum is simply one whose finishing kernel is not launched)
    (void)defer;
    if (deferred) launch((fc_gemv_kernel<VEC, true, CH>), grid, dim3(kFcThreads), 0, s, Wt, x, K, N, rowsPerSlice, cfg, bias, y, partials, xd);
    else launch((fc_gemv_kernel<VEC, false, CH>), grid, dim3(kFcThreads), 0, s, Wt, x, K, N, rowsPerSlice, cfg, bias, y, partials, xd);
}

template <int VEC>
static void launch_gemv(bool deferred, dim3 grid, hipStream_t s, const float* x, const drhip_deferred_vec& xd, const float* Wt,
                        const float* bias, float* y, float* partials, int K, int N, int rowsPerSlice, int relu, int defer) {
    // rows per wavefront and turn: every wavefront of the workgroup should get at least one turn
    if (rowsPerSlice >= kFcWaves * kWave) launch_gemv_ch<VEC, 64>(deferred, grid, s, x, xd, Wt, bias, y, partials, K, N, rowsPerSlice, relu, defer);
    else if (rowsPerSlice >= kFcWaves * 32) launch_gemv_ch<VEC, 32>(deferred, grid, s, x, xd, Wt, bias, y, partials, K, N, rowsPerSlice, relu, defer);
    else launch_gemv_ch<VEC, 16>(deferred, grid, s, x, xd, Wt, bias, y, partials, K, N, rowsPerSlice, relu, defer);
}

extern "C" int drhip_fc_ex_f32(const float* x, const drhip_deferred_vec* xdef, const float* Wt, const float* bias, float* y,
                               float* partials, int K, int N, int relu, int defer, void* stream) {
    DRHIP_REQUIRE((x || xdef) && Wt && (y || defer), "drhip_fc_f32: NULL pointer");
    DRHIP_REQUIRE(K > 0 && N > 0, "drhip_fc_f32: bad shape K=%d N=%d", K, N);
    DRHIP_REQUIRE(!xdef || (xdef->partials && xdef->slices > 0 && xdef->n == K),
                  "drhip_fc_f32: deferred input must carry partial sums of a vector of length K=%d", K);
    FcPlan p = fc_plan(K, N);
    DRHIP_REQUIRE(p.slices == 1 || partials, "drhip_fc_f32: this shape is split over %d row slices and needs the partials scratch", p.slices);
    DRHIP_REQUIRE(!defer || p.slices > 1, "drhip_fc_f32: only a layer that is split over row slices can leave its sum unfinished");
    DRHIP_REQUIRE(((size_t)Wt % (4 * p.vec)) == 0, "drhip_fc_f32: weight matrix not aligned for %d-wide loads", p.vec);
    DRHIP_REQUIRE(p.slices <= 65535, "drhip_fc_f32: too many row slices");
    dim3 grid(p.panels, p.slices);
    hipStream_t s = as_stream(stream);
    const drhip_deferred_vec none = {nullptr, nullptr, 0, 0, 0, nullptr, 0.0f};
    const drhip_deferred_vec& xd = xdef ? *xdef : none;
    if (p.vec == 4) launch_gemv<4>(xdef != nullptr, grid, s, x, xd, Wt, bias, y, partials, K, N, p.rowsPerSlice, relu, defer);
    else if (p.vec == 2) launch_gemv<2>(xdef != nullptr, grid, s, x, xd, Wt, bias, y, partials, K, N, p.rowsPerSlice, relu, defer);
    else launch_gemv<1>(xdef != nullptr, grid, s, x, xd, Wt, bias, y, partials, K, N, p.rowsPerSlice, relu, defer);
    if (int rc = launched("fc_gemv_kernel")) return rc;
    if (p.slices > 1 && !defer) {
        launch(fc_reduce_kernel, dim3(ceil_div(N, 256)), dim3(256), 0, s, partials, bias, y, N, p.slices, relu);
        return launched("fc_reduce_kernel");
    }
    return DRHIP_OK;
}

extern "C" int drhip_fc_f32(const float* x, const float* Wt, const float* bias, float* y,
                            float* partials, int K, int N, int relu, void* stream) {
    DRHIP_REQUIRE(x && y, "drhip_fc_f32: NULL pointer");
    return drhip_fc_ex_f32(x, nullptr, Wt, bias, y, partials, K, N, relu, 0, stream);
}

extern "C" int drhip_fc_permute_rows_f32(const float* src, float* dst, int W, int H, int C, int N, void* stream) {
    DRHIP_REQUIRE(src && dst && src != dst, "drhip_fc_permute_rows_f32: NULL or aliased matrices");
    DRHIP_REQUIRE(W > 0 && H > 0 && C > 0 && N > 0, "drhip_fc_permute_rows_f32: bad shape");
    DRHIP_REQUIRE((long long)W * H * C < (1ll << 31), "drhip_fc_permute_rows_f32: K too large");
    launch(fc_permute_rows_kernel, dim3(W * H * C), dim3(256), 0, as_stream(stream), src, dst, W, H, C, N);
    return launched("fc_permute_rows_kernel");
}

extern "C" size_t drhip_fc_noalloc_max_scratch_floats(void) { return kFcStaticScratchFloats; }

extern "C" int drhip_fc_noalloc_f32(const float* x, const float* Wt, const float* bias, float* y,
                                    int K, int N, int relu, void* stream) {
    DRHIP_REQUIRE(x && Wt && y, "drhip_fc_noalloc_f32: NULL pointer");
    DRHIP_REQUIRE(K > 0 && N > 0, "drhip_fc_noalloc_f32: bad shape K=%d N=%d", K, N);
    const size_t need = drhip_fc_scratch_floats(K, N);
    DRHIP_REQUIRE(need <= kFcStaticScratchFloats,
                  "drhip_fc_noalloc_f32: K=%d N=%d needs %zu floats of partial sums, the built-in scratch holds %zu; use drhip_fc_f32 with a caller buffer",
                  K, N, need, kFcStaticScratchFloats);
    DRHIP_REQUIRE(!launch_timer().on, "drhip_fc_noalloc_f32: not available between drhip_timing_begin and drhip_timing_end (timing creates events)");
    int device = -1;
    if (int rc = check(hipGetDevice(&device), "hipGetDevice")) return rc;
    DRHIP_REQUIRE(device >= 0 && device < kFcMaxDevices && g_fc_static_ptr[device],
                  "drhip_fc_noalloc_f32: drhip_init has not been called for device %d", device);
    // The partial sums need no clearing: every (slice, column) the finishing kernel reads is written by this call's GEMV.
    return drhip_fc_ex_f32(x, nullptr, Wt, bias, y, need ? g_fc_static_ptr[device] : nullptr, K, N, relu, 0, stream);
}
