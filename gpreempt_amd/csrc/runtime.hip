// Device, stream, event, memory, flag, gate and graph entry points of the C ABI.
#include "common.hpp"
#include <atomic>
#include <ctime>
#include <mutex>

namespace gp {

static thread_local char g_err[512] = "";
void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int static_scratch_setup(int **out);  // gemm.hip
static std::atomic<int> g_cus{0};
static std::atomic<int> g_device{-1};
int device_cus() {
    int c = g_cus.load(std::memory_order_relaxed);
    if (c > 0) return c;
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) {
        g_cus.store(prop.multiProcessorCount);
        return prop.multiProcessorCount;
    }
    return 256;
}

__global__ void fill32_kernel(uint32_t *p, uint32_t v, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// One wave polls *stop with system-scope loads; bounded so that a lost release cannot hang the
// device (the reference's gpu_block spins forever, src/block.cu:1-3).
__global__ void gate_kernel(const int *stop, unsigned long long spin_limit, int *timed_out) {
    if (threadIdx.x != 0) return;
    for (unsigned long long i = 0; i < spin_limit; ++i) {
        if (__hip_atomic_load(stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0) return;
        __builtin_amdgcn_s_sleep(8);
    }
    if (timed_out) __hip_atomic_store(timed_out, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__global__ void noop_kernel() {}

// stores the device's constant-rate clock where the host can see it
__global__ void clock_probe_kernel(unsigned long long *host_word) {
    if (threadIdx.x == 0) __hip_atomic_store(host_word, (unsigned long long)wall_clock64(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// stores a value where the host can see it: a marker that says "everything before me on this stream has left the GPU"
__global__ void store_word_kernel(int *host_word, int value) {
    if (threadIdx.x == 0) __hip_atomic_store(host_word, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

struct RelayArgs { const int *flags[8]; int *mirror; int n; const int *quit; unsigned long long spin_limit; };

// Lane i mirrors flag word i into device memory; lane 0 also watches the quit word.
__global__ void flag_relay_kernel(RelayArgs a) {
    const int lane = threadIdx.x;
    int last = 0;
    for (unsigned long long it = 0; it < a.spin_limit; ++it) {
        if (lane < a.n) {
            int v = __hip_atomic_load(a.flags[lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            if (v != last) {
                __hip_atomic_store(a.mirror + lane, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                last = v;
            }
        }
        int q = 0;
        if (lane == 0) q = __hip_atomic_load(a.quit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        if (__builtin_amdgcn_readfirstlane(q) != 0) break;
        __builtin_amdgcn_s_sleep(4);
    }
    // leave the mirror lowered so that nothing stays stopped because the relay is gone
    if (lane < a.n && last != 0) __hip_atomic_store(a.mirror + lane, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

}  // namespace gp

using namespace gp;

extern "C" const char *gp_last_error(void) { return g_err; }

extern "C" int gp_init(int device) {
    int n = 0;
    GP_HIP(hipGetDeviceCount(&n));
    GP_REQUIRE(device >= 0 && device < n, "device %d not present (%d visible)", device, n);
    GP_HIP(hipSetDevice(device));
    // address of the library's static scratch on this device (gp_launch_gemm_noalloc)
    if (int rc = static_scratch_setup(nullptr)) return rc;
    if (g_device.load() != device) {
        hipDeviceProp_t prop;
        GP_HIP(hipGetDeviceProperties(&prop, device));
        g_cus.store(prop.multiProcessorCount);
        g_device.store(device);
    }
    return GP_SUCC;
}

extern "C" int gp_device_info(int *compute_units, int *clock_khz, char *name, size_t name_len) {
    int dev = 0;
    GP_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    GP_HIP(hipGetDeviceProperties(&prop, dev));
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (name && name_len) { strncpy(name, prop.name, name_len - 1); name[name_len - 1] = 0; }
    return GP_SUCC;
}

extern "C" int gp_stream_create(int priority, gp_stream *out) {
    GP_REQUIRE(out != nullptr, "null stream out");
    hipStream_t s;
    GP_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *out = new gp_stream_s{s, priority};
    return GP_SUCC;
}
extern "C" int gp_stream_destroy(gp_stream s) {
    if (!s) return GP_SUCC;
    hipError_t e = hipStreamDestroy(s->s);
    delete s;
    if (e != hipSuccess) { set_error("hipStreamDestroy: %s", hipGetErrorString(e)); return GP_FAIL; }
    return GP_SUCC;
}
extern "C" int gp_stream_sync(gp_stream s) { GP_HIP(hipStreamSynchronize(native(s))); return GP_SUCC; }
extern "C" int gp_stream_query(gp_stream s, int *idle) {
    hipError_t e = hipStreamQuery(native(s));
    if (e == hipSuccess) { if (idle) *idle = 1; return GP_SUCC; }
    if (e == hipErrorNotReady) { if (idle) *idle = 0; return GP_SUCC; }
    set_error("hipStreamQuery: %s", hipGetErrorString(e));
    return GP_FAIL;
}
extern "C" int gp_stream_priority(gp_stream s, int *priority) {
    GP_REQUIRE(s && priority, "null stream");
    *priority = s->priority;
    return GP_SUCC;
}
extern "C" int gp_stream_set_priority(gp_stream s, int priority) {
    GP_REQUIRE(s != nullptr, "null stream");
    GP_REQUIRE(priority >= 0, "priority %d", priority);
    s->priority = priority;
    return GP_SUCC;
}
extern "C" void *gp_stream_native(gp_stream s) { return (void *)native(s); }

extern "C" int gp_event_create(gp_event *out) {
    GP_REQUIRE(out != nullptr, "null event out");
    hipEvent_t e;
    GP_HIP(hipEventCreate(&e));
    *out = new gp_event_s{e};
    return GP_SUCC;
}
extern "C" int gp_event_destroy(gp_event e) {
    if (!e) return GP_SUCC;
    hipError_t r = hipEventDestroy(e->e);
    delete e;
    if (r != hipSuccess) { set_error("hipEventDestroy: %s", hipGetErrorString(r)); return GP_FAIL; }
    return GP_SUCC;
}
extern "C" int gp_event_record(gp_event e, gp_stream s) { GP_REQUIRE(e, "null event"); GP_HIP(hipEventRecord(e->e, native(s))); return GP_SUCC; }
extern "C" int gp_event_sync(gp_event e) { GP_REQUIRE(e, "null event"); GP_HIP(hipEventSynchronize(e->e)); return GP_SUCC; }
extern "C" int gp_event_query(gp_event e, int *done) {
    GP_REQUIRE(e && done, "null event");
    hipError_t r = hipEventQuery(e->e);
    if (r == hipSuccess) { *done = 1; return GP_SUCC; }
    if (r == hipErrorNotReady) { *done = 0; return GP_SUCC; }
    set_error("hipEventQuery: %s", hipGetErrorString(r));
    return GP_FAIL;
}
extern "C" int gp_event_elapsed_ms(gp_event a, gp_event b, float *ms) {
    GP_REQUIRE(a && b && ms, "null event");
    GP_HIP(hipEventElapsedTime(ms, a->e, b->e));
    return GP_SUCC;
}

extern "C" int gp_malloc(void **dev, size_t bytes) {
    GP_REQUIRE(dev != nullptr, "null out pointer");
    GP_HIP(hipMalloc(dev, bytes ? bytes : 1));
    return GP_SUCC;
}
extern "C" int gp_free(void *dev) { if (dev) GP_HIP(hipFree(dev)); return GP_SUCC; }
extern "C" int gp_host_alloc(void **host, size_t bytes) {
    GP_REQUIRE(host != nullptr, "null out pointer");
    GP_HIP(hipHostMalloc(host, bytes ? bytes : 1, hipHostMallocDefault));
    return GP_SUCC;
}
extern "C" int gp_host_free(void *host) { if (host) GP_HIP(hipHostFree(host)); return GP_SUCC; }
extern "C" int gp_memcpy_h2d(void *dev, const void *host, size_t bytes) { GP_HIP(hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice)); return GP_SUCC; }
extern "C" int gp_memcpy_d2h(void *host, const void *dev, size_t bytes) { GP_HIP(hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost)); return GP_SUCC; }
extern "C" int gp_memcpy_h2d_async(void *dev, const void *host, size_t bytes, gp_stream s) { GP_HIP(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, native(s))); return GP_SUCC; }
extern "C" int gp_memcpy_d2h_async(void *host, const void *dev, size_t bytes, gp_stream s) { GP_HIP(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, native(s))); return GP_SUCC; }
extern "C" int gp_memcpy_d2d_async(void *dst, const void *src, size_t bytes, gp_stream s) { GP_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, native(s))); return GP_SUCC; }
extern "C" int gp_fill32_async(void *dev, uint32_t value, size_t count, gp_stream s) {
    if (count == 0) return GP_SUCC;
    GP_REQUIRE(dev && ((uintptr_t)dev & 3) == 0, "fill32 needs a 4-byte aligned device pointer");
    unsigned grid = (unsigned)((count + 255) / 256);
    hipLaunchKernelGGL(fill32_kernel, dim3(grid), dim3(256), 0, native(s), (uint32_t *)dev, value, count);
    GP_HIP(hipGetLastError());
    return GP_SUCC;
}

extern "C" int gp_flag_create(volatile int **host_ptr, void **dev_ptr) {
    GP_REQUIRE(host_ptr && dev_ptr, "null out pointer");
    void *h = nullptr;
    // Coherent (fine-grained) pinned memory: a host store becomes visible to a running kernel.
    GP_HIP(hipHostMalloc(&h, 64, hipHostMallocCoherent | hipHostMallocMapped));
    memset(h, 0, 64);
    void *d = nullptr;
    GP_HIP(hipHostGetDevicePointer(&d, h, 0));
    *host_ptr = (volatile int *)h;
    *dev_ptr = d;
    return GP_SUCC;
}
extern "C" int gp_flag_destroy(volatile int *host_ptr) { if (host_ptr) GP_HIP(hipHostFree((void *)host_ptr)); return GP_SUCC; }

extern "C" int gp_flag_relay_start(void *const *flags_dev, int *mirror, int n, const int *quit_dev,
                                   unsigned long long spin_limit, gp_stream s) {
    GP_REQUIRE(flags_dev && mirror && quit_dev && s, "relay needs flags, mirror, quit flag and an explicit stream");
    GP_REQUIRE(n >= 1 && n <= 8, "relay handles 1..8 flag words");
    GP_REQUIRE(spin_limit > 0, "relay needs a finite spin limit");
    RelayArgs a{};
    for (int i = 0; i < n; ++i) { GP_REQUIRE(flags_dev[i] != nullptr, "null flag"); a.flags[i] = (const int *)flags_dev[i]; }
    a.mirror = mirror; a.n = n; a.quit = quit_dev; a.spin_limit = spin_limit;
    hipLaunchKernelGGL(flag_relay_kernel, dim3(1), dim3(64), 0, native(s), a);
    GP_HIP(hipGetLastError());
    return GP_SUCC;
}

extern "C" int gp_launch_gate(const int *stop, unsigned long long spin_limit, int *timed_out, gp_stream s) {
    GP_REQUIRE(stop != nullptr, "null gate flag");
    GP_REQUIRE(spin_limit > 0, "gate needs a finite spin limit");
    hipLaunchKernelGGL(gate_kernel, dim3(1), dim3(64), 0, native(s), stop, spin_limit, timed_out);
    GP_HIP(hipGetLastError());
    return GP_SUCC;
}
extern "C" int gp_launch_noop(gp_stream s) {
    hipLaunchKernelGGL(noop_kernel, dim3(1), dim3(64), 0, native(s));
    GP_HIP(hipGetLastError());
    return GP_SUCC;
}

// Device clock against the host's: a kernel stores wall_clock64() into fine-grained host memory and the
// host, spinning on the word, notes its own clock when the value appears.  host - device is the offset plus
// the store's way to the host; the minimum over the rounds keeps the shortest way (1-2 us).
extern "C" int gp_device_clock(gp_stream s, int rounds, double *tick_ns, double *offset_ns, unsigned long long *ticks) {
    GP_REQUIRE(tick_ns && offset_ns, "null clock out");
    if (rounds < 1) rounds = 16;
    int dev = 0, khz = 0;
    GP_HIP(hipGetDevice(&dev));
    GP_HIP(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
    GP_REQUIRE(khz > 0, "the device reports no wall clock rate");
    const double tick = 1e6 / (double)khz;
    volatile unsigned long long *word = nullptr;
    GP_HIP(hipHostMalloc((void **)&word, 64, hipHostMallocCoherent | hipHostMallocMapped));
    void *word_dev = nullptr;
    if (hipHostGetDevicePointer(&word_dev, (void *)word, 0) != hipSuccess) { hipHostFree((void *)word); set_error("gp_device_clock: no device address for the probe word"); return GP_FAIL; }
    double best = 0;
    unsigned long long best_ticks = 0;
    bool have = false;
    for (int r = 0; r < rounds; ++r) {
        *word = 0;
        hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, native(s), (unsigned long long *)word_dev);
        hipError_t e = hipGetLastError();
        unsigned long long d = 0;
        // bounded: a kernel that never ran must not hang the caller (about two seconds of polls)
        for (long spins = 0; e == hipSuccess && (d = *word) == 0 && spins < (1L << 31); ++spins) { }
        struct timespec ts;
        clock_gettime(CLOCK_MONOTONIC, &ts);
        const double host_ns = (double)ts.tv_sec * 1e9 + (double)ts.tv_nsec;
        hipError_t e2 = hipStreamSynchronize(native(s));
        if (e != hipSuccess || e2 != hipSuccess || d == 0) {
            hipHostFree((void *)word);
            set_error("gp_device_clock: the probe kernel did not report (%s)", hipGetErrorString(e != hipSuccess ? e : e2));
            return GP_FAIL;
        }
        const double off = host_ns - (double)d * tick;
        if (!have || off < best) { best = off; best_ticks = d; have = true; }
    }
    GP_HIP(hipHostFree((void *)word));
    *tick_ns = tick;
    *offset_ns = best;
    if (ticks) *ticks = best_ticks;
    return GP_SUCC;
}

extern "C" int gp_store_word_async(gp_stream s, int *word_dev, int value) {
    GP_REQUIRE(word_dev != nullptr, "gp_store_word_async: null word");
    hipLaunchKernelGGL(store_word_kernel, dim3(1), dim3(64), 0, native(s), word_dev, value);
    GP_HIP(hipGetLastError());
    return GP_SUCC;
}

extern "C" int gp_graph_begin(gp_stream s) {
    GP_REQUIRE(s != nullptr, "graph capture needs an explicit stream");
    GP_HIP(hipStreamBeginCapture(s->s, hipStreamCaptureModeThreadLocal));
    return GP_SUCC;
}
extern "C" int gp_graph_end(gp_stream s, gp_graph *out) {
    GP_REQUIRE(s && out, "null graph out");
    hipGraph_t g;
    GP_HIP(hipStreamEndCapture(s->s, &g));
    hipGraphExec_t x;
    hipError_t e = hipGraphInstantiate(&x, g, nullptr, nullptr, 0);
    if (e != hipSuccess) { hipGraphDestroy(g); set_error("hipGraphInstantiate: %s", hipGetErrorString(e)); return GP_FAIL; }
    *out = new gp_graph_s{g, x};
    return GP_SUCC;
}
extern "C" int gp_graph_launch(gp_graph g, gp_stream s) { GP_REQUIRE(g, "null graph"); GP_HIP(hipGraphLaunch(g->x, native(s))); return GP_SUCC; }
extern "C" int gp_graph_destroy(gp_graph g) {
    if (!g) return GP_SUCC;
    hipGraphExecDestroy(g->x);
    hipGraphDestroy(g->g);
    delete g;
    return GP_SUCC;
}
