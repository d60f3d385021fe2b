// Runtime part of the C ABI: device selection, memory, stream, events.
#include "xsmi_internal.h"
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>
#include <vector>

namespace {
thread_local char g_err[512] = "";
hipStream_t g_stream = nullptr;
hipStream_t g_side = nullptr;            // second stream for work that may overlap the main stream's
hipStream_t g_current = nullptr;         // what stream() hands out: g_stream, or g_side inside a side section
hipEvent_t g_fork = nullptr, g_join = nullptr;
bool g_side_pending = false;             // the second stream holds work the main stream has not waited for yet
int g_device = -1;
int g_cus = 0;
bool g_ready = false;
bool g_profiling = false;
hipEvent_t g_prof0 = nullptr, g_prof1 = nullptr;
bool g_prof_valid = false;
// A step graph under capture: the launches of every entry point are recorded instead of run.  Calls that must
// wait for the device are refused while it lasts, and hipFree (which waits too) is put off to its end.
bool g_capturing = false;
std::vector<void *> g_free_after_capture;

// Tuning switches: the value set through xsmi_set_option, else the environment variable read at first use, else
// the default.  The order of the rows is xsmi::Option's.
struct OptionRow {
    const char *name, *env;
    long value;
    bool loaded;
};
OptionRow g_options[xsmi::OPT_COUNT] = {
    {"tap_sk", "XSMI_TAP_SK", 1, false},
    {"sk_spin_limit", "XSMI_SK_SPIN_LIMIT", 1L << 22, false},
    {"tap_stages", "XSMI_TAP_STAGES", 0, false},
    {"tap_persist", "XSMI_TAP_PERSIST", 1, false},
    {"cl_halo", "XSMI_CL_HALO", 1, false},
    {"cl_stem", "XSMI_CL_STEM", 1, false},
    {"sk_wide", "XSMI_SK_WIDE", 2, false},
    {"pool_bwd", "XSMI_POOL_BWD", 2, false},
    {"pack_lanes", "XSMI_PACK_LANES", 2, false},
};

// Streams beside the second one for runs of short independent launches (filter layouts), see side_lane().
hipStream_t g_lanes[xsmi::SIDE_LANES] = {nullptr, nullptr, nullptr, nullptr};
hipEvent_t g_lane_done[xsmi::SIDE_LANES] = {nullptr, nullptr, nullptr, nullptr};
bool g_lane_used[xsmi::SIDE_LANES] = {false, false, false, false};

// Partial tiles and flags of the even-split convolution kernels: one area per stream, owned by the library (a
// launch's partial tiles are dead when it ends, and launches of one stream run one after the other).
xsmi::SkScratch g_sk_scratch[2] = {{nullptr, nullptr}, {nullptr, nullptr}};
// A word in page-locked host memory that kernels write when a bounded wait ran out; the host reads it directly.
volatile uint32_t *g_dev_error_host = nullptr;
uint32_t *g_dev_error_dev = nullptr;
}  // namespace

namespace xsmi {
void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
hipStream_t stream() { return g_current; }
// A side section runs the launches issued between side_begin() and side_end() on the second stream, ordered
// after everything enqueued on the main stream so far; side_join() makes the main stream wait for them.  The
// caller puts independent main-stream work between side_end() and side_join().
int side_begin() {
    XSMI_HIP(hipEventRecord(g_fork, g_stream));
    XSMI_HIP(hipStreamWaitEvent(g_side, g_fork, 0));
    g_current = g_side;
    g_side_pending = true;
    return XSMI_OK;
}
int side_lane(int lane) {
    if (lane <= 0 || lane >= SIDE_LANES) {
        g_current = g_side;
        return XSMI_OK;
    }
    if (!g_lane_used[lane]) {                           // the lane starts where the second stream started
        XSMI_HIP(hipStreamWaitEvent(g_lanes[lane], g_fork, 0));
        g_lane_used[lane] = true;
    }
    g_current = g_lanes[lane];
    return XSMI_OK;
}
int side_lanes_end() {
    for (int l = 1; l < SIDE_LANES; ++l)
        if (g_lane_used[l]) {
            g_lane_used[l] = false;
            XSMI_HIP(hipEventRecord(g_lane_done[l], g_lanes[l]));
            XSMI_HIP(hipStreamWaitEvent(g_side, g_lane_done[l], 0));
        }
    g_current = g_side;
    return XSMI_OK;
}
void side_end() { g_current = g_stream; }
int side_join() {
    if (!g_side_pending) return XSMI_OK;
    XSMI_HIP(hipEventRecord(g_join, g_side));
    XSMI_HIP(hipStreamWaitEvent(g_stream, g_join, 0));
    g_side_pending = false;
    return XSMI_OK;
}
bool side_pending() { return g_side_pending; }
bool on_side_stream() { return g_current == g_side; }
bool ready() { return g_ready; }
int cu_count() { return g_cus; }
bool capturing() { return g_capturing; }
long option(Option o) {
    OptionRow &r = g_options[o];
    if (!r.loaded) {
        const char *e = getenv(r.env);
        if (e && *e) r.value = atol(e);
        r.loaded = true;
    }
    return r.value;
}
SkScratch sk_scratch() { return g_sk_scratch[g_current == g_side ? 1 : 0]; }
uint32_t *device_error_word() { return g_dev_error_dev; }
// Non-zero when a kernel has reported a wait that ran out.  Outside a capture the streams are drained, the flags
// of the even-split kernels are cleared (a late producer may have left one raised) and the word is reset, so the
// library is usable again after the caller has seen the error.
int check_device_error(const char *where) {
    if (!g_dev_error_host || *g_dev_error_host == 0) return XSMI_OK;
    const uint32_t code = *g_dev_error_host;
    if (!g_capturing) {
        (void)hipStreamSynchronize(g_side);
        (void)hipStreamSynchronize(g_stream);
        g_side_pending = false;
        for (int i = 0; i < 2; ++i)
            if (g_sk_scratch[i].flags) (void)hipMemset(g_sk_scratch[i].flags, 0, SK_SCRATCH_FLAG_BYTES);
        *g_dev_error_host = 0;
    }
    set_error("%s: an even-split convolution kernel gave up waiting for a partial tile (code %u): the output of that "
              "launch is incomplete; results since then are not valid", where, code);
    return XSMI_ERR_RUNTIME;
}
void prof_begin() {
    if (g_profiling && !g_capturing && g_current == g_stream) (void)hipEventRecord(g_prof0, g_stream);
}
void prof_end() {
    if (g_profiling && !g_capturing && g_current == g_stream) {
        (void)hipEventRecord(g_prof1, g_stream);
        g_prof_valid = true;
    }
}
}  // namespace xsmi

// One float4 per thread: of the forms tried on the box (grid-stride loops over 8 to 64 workgroups per CU, four loads
// in flight per thread, the runtime's own device-to-device copy) this one moved the most bytes per second when source
// and destination come from HBM (5.9 TB/s against 5.2-5.7 for the loops and 5.3 for hipMemcpyAsync); with
// non-temporal loads and stores it moves 6.3 TB/s (a pure read of the same size 6.6, a pure fill 6.5).
typedef float xsmi_f4v __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) xsmi_copy_f4(const xsmi_f4v *__restrict__ src, xsmi_f4v *__restrict__ dst, size_t n4) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n4) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// Byte fill as a kernel (a memset node in a captured graph is not dependable): 16-byte stores over the aligned
// middle, single bytes over the unaligned head and tail.
__global__ void __launch_bounds__(256) xsmi_memset_kernel(unsigned char *p, unsigned word, size_t head, size_t n16, size_t tail) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    typedef unsigned u4v __attribute__((ext_vector_type(4)));
    if (i < n16) reinterpret_cast<u4v *>(p + head)[i] = u4v{word, word, word, word};
    if (i < head) p[i] = (unsigned char)word;
    if (i < tail) p[head + n16 * 16 + i] = (unsigned char)word;
}

#define XSMI_NOT_WHILE_CAPTURING()                                                              \
    do {                                                                                        \
        if (g_capturing) {                                                                      \
            xsmi::set_error("%s waits for the device: not possible while a step graph is being captured", __func__); \
            return XSMI_ERR_STATE;                                                              \
        }                                                                                       \
    } while (0)

extern "C" {

const char *xsmi_last_error(void) { return g_err; }

int xsmi_is_initialized(void) { return g_ready ? 1 : 0; }

int xsmi_init(int device) {
    if (g_ready) {
        if (device != g_device) {
            xsmi::set_error("xsmi_init: already initialised on device %d", g_device);
            return XSMI_ERR_STATE;
        }
        return XSMI_OK;
    }
    int count = 0;
    XSMI_HIP(hipGetDeviceCount(&count));
    XSMI_CHECK_ARG(device >= 0 && device < count, "xsmi_init: device %d out of range (%d visible)", device, count);
    XSMI_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    XSMI_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        xsmi::set_error("xsmi_init: device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
        return XSMI_ERR_RUNTIME;
    }
    int rc = xsmi::noalloc_setup(device);                // address of this GPU's copy of the static scratch array
    if (rc) return rc;
    XSMI_HIP(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
    XSMI_HIP(hipStreamCreateWithFlags(&g_side, hipStreamNonBlocking));
    XSMI_HIP(hipEventCreateWithFlags(&g_fork, hipEventDisableTiming));
    XSMI_HIP(hipEventCreateWithFlags(&g_join, hipEventDisableTiming));
    for (int l = 1; l < xsmi::SIDE_LANES; ++l) {
        XSMI_HIP(hipStreamCreateWithFlags(&g_lanes[l], hipStreamNonBlocking));
        XSMI_HIP(hipEventCreateWithFlags(&g_lane_done[l], hipEventDisableTiming));
    }
    for (int i = 0; i < 2; ++i) {
        void *p = nullptr;
        XSMI_HIP(hipMalloc(&p, xsmi::SK_SCRATCH_FLAG_BYTES + xsmi::SK_SCRATCH_PART_BYTES));
        XSMI_HIP(hipMemset(p, 0, xsmi::SK_SCRATCH_FLAG_BYTES));
        g_sk_scratch[i].flags = (uint32_t *)p;
        g_sk_scratch[i].part = (float *)((char *)p + xsmi::SK_SCRATCH_FLAG_BYTES);
    }
    {
        void *h = nullptr, *d = nullptr;
        XSMI_HIP(hipHostMalloc(&h, 64, hipHostMallocMapped));
        memset(h, 0, 64);
        XSMI_HIP(hipHostGetDevicePointer(&d, h, 0));
        g_dev_error_host = (volatile uint32_t *)h;
        g_dev_error_dev = (uint32_t *)d;
    }
    g_current = g_stream;
    g_device = device;
    g_cus = prop.multiProcessorCount;
    g_ready = true;
    return XSMI_OK;
}

int xsmi_device_info(xsmi_device_info_t *info) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(info != nullptr, "xsmi_device_info: null argument");
    hipDeviceProp_t prop;
    XSMI_HIP(hipGetDeviceProperties(&prop, g_device));
    memset(info, 0, sizeof(*info));
    info->device = g_device;
    info->cu_count = prop.multiProcessorCount;
    info->clock_khz = prop.clockRate;
    info->lds_bytes_per_cu = (int)prop.maxSharedMemoryPerMultiProcessor;
    info->wavefront = prop.warpSize;
    info->l2_bytes = prop.l2CacheSize;
    info->hbm_bytes = prop.totalGlobalMem;
    strncpy(info->name, prop.name, sizeof(info->name) - 1);
    strncpy(info->arch, prop.gcnArchName, sizeof(info->arch) - 1);
    return XSMI_OK;
}

int xsmi_malloc(void **ptr, size_t bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(ptr != nullptr, "xsmi_malloc: null result pointer");
    *ptr = nullptr;
    if (bytes == 0) bytes = 16;
    XSMI_HIP(hipMalloc(ptr, bytes));
    return XSMI_OK;
}

int xsmi_free(void *ptr) {
    XSMI_REQUIRE_INIT();
    if (ptr == nullptr) return XSMI_OK;
    if (g_capturing) {
        g_free_after_capture.push_back(ptr);
        return XSMI_OK;
    }
    // hipFree waits for the device; work queued on the stream that still uses
    // `ptr` has completed when it returns.
    XSMI_HIP(hipFree(ptr));
    return XSMI_OK;
}

int xsmi_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_NOT_WHILE_CAPTURING();
    if (bytes == 0) return XSMI_OK;
    XSMI_CHECK_ARG(dst && src, "xsmi_memcpy_h2d: null pointer");
    XSMI_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_stream));
    XSMI_HIP(hipStreamSynchronize(g_stream));
    return XSMI_OK;
}

int xsmi_host_alloc(void **ptr, size_t bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(ptr != nullptr, "xsmi_host_alloc: null result pointer");
    *ptr = nullptr;
    if (bytes == 0) bytes = 16;
    XSMI_HIP(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
    return XSMI_OK;
}

int xsmi_host_free(void *ptr) {
    XSMI_REQUIRE_INIT();
    if (ptr == nullptr) return XSMI_OK;
    XSMI_HIP(hipHostFree(ptr));
    return XSMI_OK;
}

int xsmi_memcpy_h2d_async(void *dst, const void *pinned_src, size_t bytes) {
    XSMI_REQUIRE_INIT();
    if (bytes == 0) return XSMI_OK;
    XSMI_CHECK_ARG(dst && pinned_src, "xsmi_memcpy_h2d_async: null pointer");
    XSMI_HIP(hipMemcpyAsync(dst, pinned_src, bytes, hipMemcpyHostToDevice, g_stream));
    return XSMI_OK;
}

int xsmi_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_NOT_WHILE_CAPTURING();
    if (bytes == 0) return XSMI_OK;
    XSMI_CHECK_ARG(dst && src, "xsmi_memcpy_d2h: null pointer");
    XSMI_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
    XSMI_HIP(hipStreamSynchronize(g_stream));
    return xsmi::check_device_error("xsmi_memcpy_d2h");
}

int xsmi_memcpy_d2d(void *dst, const void *src, size_t bytes) {
    XSMI_REQUIRE_INIT();
    if (bytes == 0) return XSMI_OK;
    XSMI_CHECK_ARG(dst && src, "xsmi_memcpy_d2d: null pointer");
    XSMI_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, g_stream));
    return XSMI_OK;
}

int xsmi_memset(void *dst, int byte_value, size_t bytes) {
    XSMI_REQUIRE_INIT();
    if (bytes == 0) return XSMI_OK;
    XSMI_CHECK_ARG(dst != nullptr, "xsmi_memset: null pointer");
    size_t head = (size_t)(-(intptr_t)dst) & 15;
    if (head > bytes) head = bytes;
    size_t n16 = (bytes - head) / 16, tail = bytes - head - n16 * 16;
    size_t threads = n16 > 16 ? n16 : 16;
    size_t blocks = (threads + 255) / 256;
    XSMI_CHECK_ARG(blocks < 2147483648ull, "xsmi_memset: more than 2^31 workgroups");
    unsigned word = 0x01010101u * (unsigned)(byte_value & 0xff);
    hipLaunchKernelGGL(xsmi_memset_kernel, dim3((unsigned)blocks), dim3(256), 0, xsmi::stream(),
                       (unsigned char *)dst, word, head, n16, tail);
    XSMI_LAUNCH_CHECK("xsmi_memset_kernel");
    return XSMI_OK;
}

int xsmi_conv2d_bwd_join(void) {
    XSMI_REQUIRE_INIT();
    int rc = xsmi::side_join();
    if (rc) return rc;
    return xsmi::check_device_error("xsmi_conv2d_bwd_join");
}

size_t xsmi_scratch_bytes(void) {
    return 2 * (xsmi::SK_SCRATCH_FLAG_BYTES + xsmi::SK_SCRATCH_PART_BYTES) + (size_t)XSMI_NOALLOC_SCRATCH_BYTES;
}

int xsmi_sync(void) {
    XSMI_REQUIRE_INIT();
    XSMI_NOT_WHILE_CAPTURING();
    int rc = xsmi::side_join();                      // weight gradients still on the second stream
    if (rc) return rc;
    XSMI_HIP(hipStreamSynchronize(g_stream));
    return xsmi::check_device_error("xsmi_sync");
}

int xsmi_event_synchronize(void *event) {
    XSMI_REQUIRE_INIT();
    XSMI_NOT_WHILE_CAPTURING();
    XSMI_CHECK_ARG(event != nullptr, "xsmi_event_synchronize: null event");
    XSMI_HIP(hipEventSynchronize((hipEvent_t)event));
    return xsmi::check_device_error("xsmi_event_synchronize");
}

int xsmi_set_option(const char *name, long value) {
    XSMI_CHECK_ARG(name != nullptr, "xsmi_set_option: null name");
    for (int i = 0; i < xsmi::OPT_COUNT; ++i)
        if (strcmp(name, g_options[i].name) == 0) {
            g_options[i].value = value;
            g_options[i].loaded = true;
            return XSMI_OK;
        }
    xsmi::set_error("xsmi_set_option: no option named '%s'", name);
    return XSMI_ERR_INVALID;
}

int xsmi_get_option(const char *name, long *value) {
    XSMI_CHECK_ARG(name != nullptr && value != nullptr, "xsmi_get_option: null argument");
    for (int i = 0; i < xsmi::OPT_COUNT; ++i)
        if (strcmp(name, g_options[i].name) == 0) {
            *value = xsmi::option((xsmi::Option)i);
            return XSMI_OK;
        }
    xsmi::set_error("xsmi_get_option: no option named '%s'", name);
    return XSMI_ERR_INVALID;
}

int xsmi_event_create(void **event) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(event != nullptr, "xsmi_event_create: null result pointer");
    hipEvent_t e;
    XSMI_HIP(hipEventCreate(&e));
    *event = (void *)e;
    return XSMI_OK;
}

int xsmi_event_record(void *event) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(event != nullptr, "xsmi_event_record: null event");
    XSMI_CHECK_ARG(!g_capturing, "xsmi_event_record: a timing event cannot be recorded into a step graph");
    XSMI_HIP(hipEventRecord((hipEvent_t)event, g_stream));
    return XSMI_OK;
}

int xsmi_event_elapsed_ms(void *start, void *stop, float *ms) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(start && stop && ms, "xsmi_event_elapsed_ms: null argument");
    XSMI_NOT_WHILE_CAPTURING();
    XSMI_HIP(hipEventSynchronize((hipEvent_t)stop));
    XSMI_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return XSMI_OK;
}

int xsmi_event_destroy(void *event) {
    XSMI_REQUIRE_INIT();
    if (event == nullptr) return XSMI_OK;
    XSMI_HIP(hipEventDestroy((hipEvent_t)event));
    return XSMI_OK;
}

int xsmi_profiling(int on) {
    XSMI_REQUIRE_INIT();
    if (on && !g_prof0) {
        XSMI_HIP(hipEventCreate(&g_prof0));
        XSMI_HIP(hipEventCreate(&g_prof1));
    }
    g_profiling = on != 0;
    g_prof_valid = false;
    return XSMI_OK;
}

int xsmi_last_kernel_ms(float *ms) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(ms != nullptr, "xsmi_last_kernel_ms: null argument");
    XSMI_CHECK_ARG(g_prof_valid, "xsmi_last_kernel_ms: no op has run since xsmi_profiling(1)");
    XSMI_NOT_WHILE_CAPTURING();
    XSMI_HIP(hipEventSynchronize(g_prof1));
    XSMI_HIP(hipEventElapsedTime(ms, g_prof0, g_prof1));
    return XSMI_OK;
}

int xsmi_copy_kernel(void *dst, const void *src, size_t bytes) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(dst && src, "xsmi_copy_kernel: null pointer");
    XSMI_CHECK_ARG(bytes % 16 == 0, "xsmi_copy_kernel: size must be a multiple of 16 bytes");
    size_t n4 = bytes / 16;
    if (n4 == 0) return XSMI_OK;
    size_t blocks = (n4 + 255) / 256;
    XSMI_CHECK_ARG(blocks < 2147483648ull, "xsmi_copy_kernel: more than 2^31 workgroups");
    xsmi::prof_begin();
    hipLaunchKernelGGL(xsmi_copy_f4, dim3((unsigned)blocks), dim3(256), 0, g_stream,
                       (const xsmi_f4v *)src, (xsmi_f4v *)dst, n4);
    xsmi::prof_end();
    XSMI_LAUNCH_CHECK("xsmi_copy_f4");
    return XSMI_OK;
}

int xsmi_graph_begin(void) {
    XSMI_REQUIRE_INIT();
    if (g_capturing) {
        xsmi::set_error("xsmi_graph_begin: a capture is already open");
        return XSMI_ERR_STATE;
    }
    int rc = xsmi::side_join();
    if (rc) return rc;
    // relaxed mode: the host may still call hipMalloc (a pool miss) while the stream records
    XSMI_HIP(hipStreamBeginCapture(g_stream, hipStreamCaptureModeRelaxed));
    g_capturing = true;
    return XSMI_OK;
}

int xsmi_graph_end(void **graph, int keep) {
    XSMI_REQUIRE_INIT();
    if (graph) *graph = nullptr;
    if (!g_capturing) {
        xsmi::set_error("xsmi_graph_end: no capture is open");
        return XSMI_ERR_STATE;
    }
    // the second stream joined the capture when it first waited for the main stream; it has to come back
    // before the capture can end
    int rc = xsmi::side_join();
    g_current = g_stream;
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(g_stream, &g);
    g_capturing = false;
    for (void *p : g_free_after_capture) (void)hipFree(p);
    g_free_after_capture.clear();
    if (e != hipSuccess) {
        (void)hipGetLastError();
        xsmi::set_error("hipStreamEndCapture failed: %s", hipGetErrorString(e));
        return XSMI_ERR_RUNTIME;
    }
    if (rc || !keep || !graph) {
        if (g) (void)hipGraphDestroy(g);
        return rc;
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) {
        xsmi::set_error("hipGraphInstantiate failed: %s", hipGetErrorString(e));
        return XSMI_ERR_RUNTIME;
    }
    *graph = (void *)exec;
    return XSMI_OK;
}

int xsmi_graph_launch(void *graph) {
    XSMI_REQUIRE_INIT();
    XSMI_CHECK_ARG(graph != nullptr, "xsmi_graph_launch: null graph");
    XSMI_CHECK_ARG(!g_capturing, "xsmi_graph_launch: a capture is open");
    int rc = xsmi::side_join();
    if (rc) return rc;
    XSMI_HIP(hipGraphLaunch((hipGraphExec_t)graph, g_stream));
    return XSMI_OK;
}

int xsmi_graph_destroy(void *graph) {
    XSMI_REQUIRE_INIT();
    if (graph == nullptr) return XSMI_OK;
    XSMI_CHECK_ARG(!g_capturing, "xsmi_graph_destroy: a capture is open");
    // replays still in flight read the executable graph: wait for them first
    XSMI_HIP(hipStreamSynchronize(g_stream));
    XSMI_HIP(hipGraphExecDestroy((hipGraphExec_t)graph));
    return XSMI_OK;
}

}  // extern "C"
