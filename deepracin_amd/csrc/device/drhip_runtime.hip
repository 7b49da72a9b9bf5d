// Device bring-up, streams, events and memory of the HIP device layer (see include/dr_hip.h).
#include "drhip_common.hpp"

#include <algorithm>
#include <vector>

#include <algorithm>
#include <chrono>
#include <cstdlib>
#include <cstring>

namespace drhip {

char* error_slot() {
    static thread_local char msg[512] = "no error";
    return msg;
}

static int g_num_cu = 256;
int num_cu() { return g_num_cu; }

LaunchTimer& launch_timer() {
    static thread_local LaunchTimer t;
    return t;
}

__global__ void fill_f32_kernel(float* __restrict__ dst, float value, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = value;
}

__global__ void copy_f32_kernel(float* __restrict__ dst, const float* __restrict__ src, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

// One workgroup copies n floats into host memory and then raises a flag there, so that the host can watch for
// the flag instead of waiting for the stream.  Release of the data: every lane stores with system scope (written
// through all caches), waits until its stores have completed (vmcnt(0)), the workgroup meets, and lane 0 stores
// the flag with a system-scope release (one wave's fence; measured free: 0.343 ms per VGG16 image with it and
// without).  The host reads the flag with an acquire load before it touches the data.  (__threadfence_system()
// in every lane instead made the download slower than waiting for the stream: 35 against 29 us.)
__global__ void __launch_bounds__(1024) copy_then_flag_kernel(float* __restrict__ dst, const float* __restrict__ src, size_t n,
                                                              unsigned* flag, unsigned value) {
    for (size_t i = threadIdx.x; i < n; i += blockDim.x)
        __hip_atomic_store((unsigned*)dst + i, __float_as_uint(src[i]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // this lane's stores have been accepted
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_store(flag, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// dst (device) = src (pinned host memory, mapped into the device's address space), 16 bytes per lane and turn
__global__ void __launch_bounds__(256) copy_from_host_kernel(float* __restrict__ dst, const float* __restrict__ src, size_t n4, size_t n) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride)
        ((f4*)dst)[i] = __builtin_nontemporal_load((const f4*)src + i);
    if (blockIdx.x == 0 && threadIdx.x < n - 4 * n4) dst[4 * n4 + threadIdx.x] = src[4 * n4 + threadIdx.x];
}

// Measurement aid: what the shader clock does under a stream of fp32 MFMAs.  Every wave issues `iters` rounds of 8
// independent v_mfma_f32_32x32x2_f32 and reads the shader-clock counter (s_memtime) and the constant 100 MHz
// counter (s_memrealtime) in front of and behind them; ticks[2 * wave] / ticks[2 * wave + 1] = clock / 100 MHz.
typedef float f32x16p __attribute__((ext_vector_type(16)));
__global__ void __launch_bounds__(256) mfma_clock_probe_kernel(long long* __restrict__ ticks, int iters, float seed) {
    f32x16p acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    const float a = seed + threadIdx.x, b = seed * 0.5f;
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
    }
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) sum += acc[i][0] + acc[i][9];
    const long long c1 = clock64(), w1 = wall_clock64();
    if ((threadIdx.x & 63) == 0) {
        const size_t wave = (size_t)blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
        ticks[2 * wave] = (c1 - c0) + (sum == 12345.678f ? 1 : 0);     // (keeps the arithmetic alive)
        ticks[2 * wave + 1] = w1 - w0;
    }
}

}  // namespace drhip

using namespace drhip;

extern "C" {

int drhip_mfma_clock_probe(int iters, int launches, float* mhz_median, float* microseconds, void* stream) {
    DRHIP_REQUIRE(iters > 0 && iters <= (1 << 20) && launches > 0 && launches <= (1 << 16) && mhz_median, "drhip_mfma_clock_probe: bad arguments");
    const int wgs = 2 * num_cu(), waves = wgs * 4;
    long long* d = nullptr;
    if (int rc = check(hipMalloc((void**)&d, sizeof(long long) * 2 * waves), "hipMalloc(clock probe)")) return rc;
    std::vector<long long> h(2 * (size_t)waves);
    int rc = DRHIP_OK;
    for (int rep = 0; rep < launches && rc == DRHIP_OK; ++rep) {   // back to back; the last launch is the one that is read
        launch(mfma_clock_probe_kernel, dim3(wgs), dim3(256), 0, as_stream(stream), d, iters, 1.0f);
        rc = launched("mfma_clock_probe_kernel");
    }
    if (rc == DRHIP_OK) rc = check(hipMemcpyAsync(h.data(), d, sizeof(long long) * h.size(), hipMemcpyDeviceToHost, as_stream(stream)), "hipMemcpyAsync(clock probe)");
    if (rc == DRHIP_OK) rc = check(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize(clock probe)");
    (void)hipFree(d);
    if (rc != DRHIP_OK) return rc;
    std::vector<double> mhz, us;
    for (int w = 0; w < waves; ++w)
        if (h[2 * w + 1] > 0) { mhz.push_back(100.0 * (double)h[2 * w] / (double)h[2 * w + 1]); us.push_back((double)h[2 * w + 1] / 100.0); }
    DRHIP_REQUIRE(!mhz.empty(), "drhip_mfma_clock_probe: the probe recorded nothing");
    std::sort(mhz.begin(), mhz.end());
    std::sort(us.begin(), us.end());
    *mhz_median = (float)mhz[mhz.size() / 2];
    if (microseconds) *microseconds = (float)us[us.size() / 2];
    return DRHIP_OK;
}

const char* drhip_last_error(void) { return error_slot(); }

int drhip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return 0; }
    return n;
}

int drhip_init(int device, drhip_device_info* info) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return fail(DRHIP_ENODEVICE, "no HIP device available (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    }
    DRHIP_REQUIRE(device >= 0 && device < n, "device ordinal %d out of range [0,%d)", device, n);
    if (int rc = check(hipSetDevice(device), "hipSetDevice")) return rc;
    hipDeviceProp_t p;
    if (int rc = check(hipGetDeviceProperties(&p, device), "hipGetDeviceProperties")) return rc;
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0)
        return fail(DRHIP_ENODEVICE, "device %d is %s; this library carries gfx950 code only", device, p.gcnArchName);
    g_num_cu = p.multiProcessorCount;
    if (int rc = fc_static_scratch_setup(device)) return rc;
    if (info) {
        memset(info, 0, sizeof(*info));
        strncpy(info->name, p.name, sizeof(info->name) - 1);
        strncpy(info->arch, p.gcnArchName, sizeof(info->arch) - 1);
        info->device = device;
        info->num_cu = p.multiProcessorCount;
        info->wavefront = p.warpSize;
        info->lds_bytes = (int)p.sharedMemPerBlock;
        info->clock_khz = p.clockRate;
        info->hbm_bytes = p.totalGlobalMem;
        info->l2_bytes = p.l2CacheSize;
    }
    return DRHIP_OK;
}

int drhip_stream_create(void** stream) {
    DRHIP_REQUIRE(stream, "stream out-pointer is NULL");
    hipStream_t s;
    if (int rc = check(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreate")) return rc;
    *stream = (void*)s;
    return DRHIP_OK;
}
int drhip_stream_destroy(void* stream) { return stream ? check(hipStreamDestroy(as_stream(stream)), "hipStreamDestroy") : DRHIP_OK; }
int drhip_stream_sync(void* stream) { return check(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize"); }

int drhip_event_create(void** ev) {
    DRHIP_REQUIRE(ev, "event out-pointer is NULL");
    hipEvent_t e;
    if (int rc = check(hipEventCreate(&e), "hipEventCreate")) return rc;
    *ev = (void*)e;
    return DRHIP_OK;
}
int drhip_event_destroy(void* ev) { return ev ? check(hipEventDestroy((hipEvent_t)ev), "hipEventDestroy") : DRHIP_OK; }
int drhip_event_record(void* ev, void* stream) { return check(hipEventRecord((hipEvent_t)ev, as_stream(stream)), "hipEventRecord"); }
int drhip_event_elapsed_ms(void* a, void* b, float* ms) {
    DRHIP_REQUIRE(a && b && ms, "NULL event or result pointer");
    if (int rc = check(hipEventSynchronize((hipEvent_t)b), "hipEventSynchronize")) return rc;
    return check(hipEventElapsedTime(ms, (hipEvent_t)a, (hipEvent_t)b), "hipEventElapsedTime");
}

int drhip_timing_begin(void) {
    LaunchTimer& t = launch_timer();
    t.used = 0;
    t.on = true;
    return DRHIP_OK;
}

int drhip_timing_count(void) { return (int)(launch_timer().used / 2); }

int drhip_timing_end(float* ms, int capacity, int* count) {
    LaunchTimer& t = launch_timer();
    t.on = false;
    const int n = (int)(t.used / 2);
    if (count) *count = n;
    DRHIP_REQUIRE(n == 0 || (ms && capacity >= n), "drhip_timing_end: room for %d launches needed, %d given", n, capacity);
    for (int i = 0; i < n; ++i) {
        if (int rc = check(hipEventSynchronize(t.events[2 * i + 1]), "hipEventSynchronize")) return rc;
        if (int rc = check(hipEventElapsedTime(&ms[i], t.events[2 * i], t.events[2 * i + 1]), "hipEventElapsedTime")) return rc;
    }
    return DRHIP_OK;
}

int drhip_stream_wait_event(void* stream, void* ev) {
    DRHIP_REQUIRE(ev, "drhip_stream_wait_event: NULL event");
    return check(hipStreamWaitEvent(as_stream(stream), (hipEvent_t)ev, 0), "hipStreamWaitEvent");
}

int drhip_graph_capture_begin(void* stream) {
    DRHIP_REQUIRE(stream, "drhip_graph_capture_begin: the default stream cannot be captured");
    return check(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
}

int drhip_graph_capture_end(void* stream, void** graph_exec) {
    DRHIP_REQUIRE(stream && graph_exec, "drhip_graph_capture_end: NULL argument");
    *graph_exec = nullptr;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(as_stream(stream), &graph);
    if (e != hipSuccess || !graph) {
        (void)hipGetLastError();
        if (graph) (void)hipGraphDestroy(graph);
        return fail(DRHIP_EDEVICE, "hipStreamEndCapture: %s", hipGetErrorString(e));
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(DRHIP_EDEVICE, "hipGraphInstantiate: %s", hipGetErrorString(e));
    }
    *graph_exec = (void*)exec;
    return DRHIP_OK;
}

int drhip_graph_launch(void* graph_exec, void* stream) {
    DRHIP_REQUIRE(graph_exec, "drhip_graph_launch: NULL graph");
    return check(hipGraphLaunch((hipGraphExec_t)graph_exec, as_stream(stream)), "hipGraphLaunch");
}

int drhip_graph_destroy(void* graph_exec) {
    return graph_exec ? check(hipGraphExecDestroy((hipGraphExec_t)graph_exec), "hipGraphExecDestroy") : DRHIP_OK;
}

int drhip_malloc(void** dptr, size_t bytes) {
    DRHIP_REQUIRE(dptr && bytes > 0, "drhip_malloc: NULL out-pointer or zero size");
    return check(hipMalloc(dptr, bytes), "hipMalloc");
}
int drhip_free(void* dptr) { return dptr ? check(hipFree(dptr), "hipFree") : DRHIP_OK; }

int drhip_upload(void* dst, size_t off, const void* src, size_t bytes, void* stream) {
    DRHIP_REQUIRE(dst && src, "drhip_upload: NULL pointer");
    if (bytes == 0) return DRHIP_OK;
    if (int rc = check(hipMemcpyAsync((char*)dst + off, src, bytes, hipMemcpyHostToDevice, as_stream(stream)), "hipMemcpyAsync(H2D)")) return rc;
    return check(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize(H2D)");
}
int drhip_download(void* dst, const void* src, size_t off, size_t bytes, void* stream) {
    DRHIP_REQUIRE(dst && src, "drhip_download: NULL pointer");
    if (bytes == 0) return DRHIP_OK;
    if (int rc = check(hipMemcpyAsync(dst, (const char*)src + off, bytes, hipMemcpyDeviceToHost, as_stream(stream)), "hipMemcpyAsync(D2H)")) return rc;
    return check(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize(D2H)");
}

// ---- staged transfers: pinned host memory owned by the library between the caller's pageable arrays and the device

// Uploads alternate between two areas.  An area may be written again once the upload that read it last has finished.
// In the usual loop (feed, pass, download) the download that completes in between proves that: nothing is recorded and
// nothing is waited for.  Only a caller that feeds again before any download has completed gets an event recorded
// behind its upload, for the feed after the next to wait on (an event per feed costs 3.5 us of every round otherwise).
struct UploadArea {
    char* mem = nullptr;
    hipEvent_t done = nullptr;
    bool pending = false;       // an upload out of this area has been enqueued and no later download has completed
    bool recorded = false;      // `done` was recorded behind that upload
    hipStream_t stream = nullptr;
};
struct Staging {
    UploadArea up[2];           // upload areas, `cap` bytes each
    int next = 0;
    char* down = nullptr;       // download area, kStagingDownBytes
    size_t cap = 0;
    unsigned seq = 0;           // value the next download's flag will take
    long spinUs = 1000;         // how long a download watches its flag before it waits for the stream instead
    bool uploadByKernel = true; // uploads of up to kStagingKernelUpload bytes: a kernel reads the pinned area (DR_UPLOAD_KERNEL=0: the DMA engine)
};
constexpr size_t kStagingDownBytes = 64 * 1024;    // + 64 bytes behind it for the flag
constexpr size_t kStagingKernelUpload = 4u << 20;

int drhip_staging_create(void** handle, size_t upload_bytes) {
    DRHIP_REQUIRE(handle && upload_bytes > 0, "drhip_staging_create: NULL handle or zero size");
    Staging* s = new Staging();
    s->cap = upload_bytes;
    hipError_t e = hipSuccess;
    for (int a = 0; a < 2 && e == hipSuccess; ++a) e = hipHostMalloc((void**)&s->up[a].mem, upload_bytes, hipHostMallocDefault);
    if (const char* env = getenv("DR_SPIN_US")) s->spinUs = atol(env);
    if (e == hipSuccess) {
        // The flag-watching download needs this area coherent between the device's stores and the host's loads:
        // asked for explicitly; without it the download waits for the stream instead of watching the flag.
        e = hipHostMalloc((void**)&s->down, kStagingDownBytes + 64, hipHostMallocCoherent | hipHostMallocMapped);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            s->down = nullptr;
            s->spinUs = 0;
            e = hipHostMalloc((void**)&s->down, kStagingDownBytes + 64, hipHostMallocDefault);
        }
    }
    if (e == hipSuccess) memset(s->down + kStagingDownBytes, 0, 64);
    if (const char* env = getenv("DR_UPLOAD_KERNEL")) s->uploadByKernel = env[0] != '0';
    for (int a = 0; a < 2 && e == hipSuccess; ++a) e = hipEventCreateWithFlags(&s->up[a].done, hipEventDisableTiming);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        for (int a = 0; a < 2; ++a) {
            if (s->up[a].mem) (void)hipHostFree(s->up[a].mem);
            if (s->up[a].done) (void)hipEventDestroy(s->up[a].done);
        }
        if (s->down) (void)hipHostFree(s->down);
        delete s;
        return fail(DRHIP_EDEVICE, "drhip_staging_create: %s", hipGetErrorString(e));
    }
    *handle = s;
    return DRHIP_OK;
}

int drhip_staging_destroy(void* handle) {
    Staging* s = (Staging*)handle;
    if (!s) return DRHIP_OK;
    for (int a = 0; a < 2; ++a) {
        if (s->up[a].pending) (void)hipStreamSynchronize(s->up[a].stream);
        (void)hipEventDestroy(s->up[a].done);
        (void)hipHostFree(s->up[a].mem);
    }
    (void)hipHostFree(s->down);
    delete s;
    return DRHIP_OK;
}

size_t drhip_staging_upload_capacity(void* handle) { return handle ? ((Staging*)handle)->cap : 0; }
size_t drhip_staging_download_capacity(void* handle) { return handle ? kStagingDownBytes : 0; }

// A download on `stream` has completed: every upload enqueued on that stream before it has finished.
static void upload_areas_done(Staging* s, hipStream_t stream) {
    for (int a = 0; a < 2; ++a)
        if (s->up[a].pending && s->up[a].stream == stream) s->up[a].pending = s->up[a].recorded = false;
}

int drhip_upload_staged(void* handle, void* dst, size_t off, const void* src, size_t bytes, void* stream) {
    Staging* s = (Staging*)handle;
    DRHIP_REQUIRE(s && dst && src, "drhip_upload_staged: NULL pointer");
    DRHIP_REQUIRE(bytes <= s->cap, "drhip_upload_staged: %zu bytes do not fit the staging area of %zu", bytes, s->cap);
    if (bytes == 0) return DRHIP_OK;
    UploadArea& area = s->up[s->next];
    UploadArea& other = s->up[s->next ^ 1];
    s->next ^= 1;
    if (area.pending) {         // the upload before the last may still be reading this area
        if (area.recorded) {
            if (int rc = check(hipEventSynchronize(area.done), "hipEventSynchronize(staging)")) return rc;
        } else if (other.pending && other.recorded && other.stream == area.stream) {
            // (the other area's upload was enqueued behind this one's: its event covers both)
            if (int rc = check(hipEventSynchronize(other.done), "hipEventSynchronize(staging)")) return rc;
        } else if (int rc = check(hipStreamSynchronize(area.stream), "hipStreamSynchronize(staging)")) return rc;
        area.pending = area.recorded = false;
    }
    // A few hundred KiB: a kernel that reads the pinned area over the bus starts sooner than the DMA engine
    // (602 KB image: 4 us less per pass).  From 256 KiB on in two pieces: the kernel of the first half runs while
    // the host copies the second (2 us less per 602 KB image; with five pieces moved by the DMA engine the calls cost
    // the host more than the overlap returned, 0.414 vs 0.386 ms per VGG16 image).
    if (s->uploadByKernel && bytes <= kStagingKernelUpload && ((size_t)((char*)dst + off) % 16 == 0) && bytes % 4 == 0) {
        const size_t first = bytes >= (256u << 10) ? (bytes / 2) & ~(size_t)15 : bytes;
        const size_t begins[2] = {0, first}, lens[2] = {first, bytes - first};
        for (int piece = 0; piece < 2 && lens[piece] > 0; ++piece) {
            const size_t begin = begins[piece], len = lens[piece];
            memcpy(area.mem + begin, (const char*)src + begin, len);
            const size_t n = len / 4, n4 = n / 4;
            launch(copy_from_host_kernel, dim3((unsigned)std::max<size_t>(1, std::min<size_t>((n4 + 255) / 256, 512))), dim3(256), 0, as_stream(stream),
                   (float*)((char*)dst + off + begin), (const float*)(area.mem + begin), n4, n);
            if (int rc = launched("copy_from_host_kernel")) return rc;
        }
    } else {
        memcpy(area.mem, src, bytes);
        if (int rc = check(hipMemcpyAsync((char*)dst + off, area.mem, bytes, hipMemcpyHostToDevice, as_stream(stream)), "hipMemcpyAsync(H2D, staged)")) return rc;
    }
    area.pending = true;
    area.recorded = false;
    area.stream = as_stream(stream);
    if (other.pending) {        // no download has completed since the previous feed: this caller runs ahead of the device
        if (int rc = check(hipEventRecord(area.done, as_stream(stream)), "hipEventRecord(staging)")) return rc;
        area.recorded = true;
    }
    return DRHIP_OK;
}

int drhip_download_staged(void* handle, void* dst, const void* src, size_t off, size_t bytes, void* stream) {
    Staging* s = (Staging*)handle;
    DRHIP_REQUIRE(s && dst && src, "drhip_download_staged: NULL pointer");
    DRHIP_REQUIRE(bytes <= kStagingDownBytes, "drhip_download_staged: %zu bytes do not fit the staging area of %zu", bytes, kStagingDownBytes);
    if (bytes == 0) return DRHIP_OK;
    // A few KiB: a copy kernel that stores straight into the pinned area (it is mapped into the device's address
    // space) instead of a transfer by the DMA engine, whose start-up costs more than the whole copy.
    if (((size_t)((const char*)src + off) | bytes) % 4 == 0) {
        const size_t n = bytes / 4;
        if (s->spinUs > 0) {
            // The host watches a flag the kernel raises behind the data: the stream's own completion path
            // (signal, interrupt, wake-up) takes some 20 us longer than the data needs to arrive.
            volatile unsigned* flag = (volatile unsigned*)(s->down + kStagingDownBytes);
            const unsigned want = ++s->seq ? s->seq : ++s->seq;     // never 0, the flag's initial value
            launch(copy_then_flag_kernel, dim3(1), dim3(1024), 0, as_stream(stream), (float*)s->down, (const float*)((const char*)src + off), n,
                   (unsigned*)flag, want);
            if (int rc = launched("copy_then_flag_kernel")) return rc;
            const auto t0 = std::chrono::steady_clock::now();
            bool seen = false;
            for (unsigned spins = 0;; ++spins) {
                if (__atomic_load_n((const unsigned*)flag, __ATOMIC_ACQUIRE) == want) { seen = true; break; }
                if ((spins & 255) == 255 && std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - t0).count() > s->spinUs) break;
                __builtin_ia32_pause();
            }
            if (!seen) {        // a long pass, or a failed one: wait the ordinary way (and learn of any error)
                if (int rc = check(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize(D2H, staged)")) return rc;
            }
            // (Flag seen: the stream is not asked for its status here - hipStreamQuery costs 25-30 us, more than the
            // flag saves.  A launch that failed was reported when it was enqueued; the next waiting call on the
            // stream reports anything else.)
            upload_areas_done(s, as_stream(stream));
            memcpy(dst, s->down, bytes);
            return DRHIP_OK;
        }
        launch(copy_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream), (float*)s->down, (const float*)((const char*)src + off), n);
        if (int rc = launched("copy_f32_kernel")) return rc;
    } else if (int rc = check(hipMemcpyAsync(s->down, (const char*)src + off, bytes, hipMemcpyDeviceToHost, as_stream(stream)), "hipMemcpyAsync(D2H, staged)")) return rc;
    if (int rc = check(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize(D2H, staged)")) return rc;
    upload_areas_done(s, as_stream(stream));
    memcpy(dst, s->down, bytes);
    return DRHIP_OK;
}

int drhip_fill_f32(float* dst, float value, size_t n, void* stream) {
    DRHIP_REQUIRE(dst, "drhip_fill_f32: NULL pointer");
    if (n == 0) return DRHIP_OK;
    const int block = 256;
    size_t blocks = (n + block - 1) / block;
    if (blocks > 4096) blocks = 4096;
    launch(fill_f32_kernel, dim3((unsigned)blocks), dim3(block), 0, as_stream(stream), dst, value, n);
    return launched("fill_f32_kernel");
}

}  // extern "C"
