// Runtime part of the C ABI: device memory, copies, streams, events, errors,
// device query and the tuning table.  Stands in for the CUDA runtime calls of
// the reference's common/tensor.cu:8-42 and benchmark drivers.
#include "ko_internal.h"

#include <cstring>
#include <mutex>

namespace ko {

static thread_local char g_last_error[512] = "";

int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return status;
}

int hip_fail(hipError_t err, const char *expr, const char *file, int line) {
    int status = KO_ERR_RUNTIME;
    if (err == hipErrorOutOfMemory) status = KO_ERR_OUT_OF_MEMORY;
    if (err == hipErrorNoDevice || err == hipErrorInvalidDevice) status = KO_ERR_NO_DEVICE;
    // Same information as the reference's checkCudaErrors line (common/common.h:19-21).
    return fail(status, "HIP error at %s:%d code=%d(%s) \"%s\"", file, line, static_cast<int>(err),
                hipGetErrorName(err), expr);
}

std::atomic<int> g_knobs[knob_count];  // zero-initialised: every knob starts at its default

static const char *const kKnobNames[knob_count] = {
#define KO_KNOB_NAME(id, name) name,
    KO_TUNING_KNOBS(KO_KNOB_NAME)
#undef KO_KNOB_NAME
};

// Index of the knob called `name`, or -1.  Only the harness hooks look names up.
static int find_knob(const char *name) {
    for (int i = 0; i < knob_count; ++i)
        if (std::strcmp(kKnobNames[i], name) == 0) return i;
    return -1;
}

int compute_units() {
    constexpr int kCached = 64;
    static std::atomic<int> cus[kCached];  // zero-initialised; 0 = not asked yet
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (dev >= 0 && dev < kCached) {
        const int known = cus[dev].load(std::memory_order_relaxed);
        if (known > 0) return known;
    }
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    if (dev >= 0 && dev < kCached) cus[dev].store(n, std::memory_order_relaxed);
    return n;
}

int allow_dynamic_lds(const void *kernel, size_t bytes, std::atomic<uint64_t> &done) {
    int dev = 0;
    KO_HIP(hipGetDevice(&dev));
    const uint64_t bit = (dev >= 0 && dev < 64) ? (uint64_t{1} << dev) : 0;
    if (bit && (done.load(std::memory_order_acquire) & bit)) return KO_OK;
    KO_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
    if (bit) done.fetch_or(bit, std::memory_order_release);
    return KO_OK;
}

namespace {
// what a (device, stream) pair holds: the GEMMs' workspace, the row operators' small one, or both
struct WorkspaceEntry { int device; hipStream_t stream; void *memory; void *small; };
constexpr int kMaxWorkspaces = 64;
WorkspaceEntry g_workspaces[kMaxWorkspaces];
int g_workspaces_used = 0;
std::mutex g_workspaces_lock;
}  // namespace

namespace {
// The pair's workspace of the asked kind, allocated if it has none yet and nothing forbids it.
int workspace_of(hipStream_t stream, bool small, void **workspace) {
    *workspace = nullptr;
    // one handle value stands for a different stream in every host thread: no workspace can belong to it
    if (stream == hipStreamPerThread) return KO_OK;
    int dev = 0;
    KO_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> guard(g_workspaces_lock);
    int at = -1;
    for (int i = 0; i < g_workspaces_used; ++i)
        if (g_workspaces[i].device == dev && g_workspaces[i].stream == stream) at = i;
    if (at >= 0 && (small ? g_workspaces[at].small : g_workspaces[at].memory) != nullptr) {
        *workspace = small ? g_workspaces[at].small : g_workspaces[at].memory;
        return KO_OK;
    }
    if (at < 0 && g_workspaces_used == kMaxWorkspaces) return KO_OK;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capture) != hipSuccess) {
        (void)hipGetLastError();
        return KO_OK;
    }
    if (capture != hipStreamCaptureStatusNone) return KO_OK;
    void *memory = nullptr;
    // no memory, or an allocation is not allowed right now (another stream of the process is being captured):
    // the caller goes without a workspace this time
    if (hipMalloc(&memory, small ? kStreamSmallWorkspaceBytes : kStreamWorkspaceBytes) != hipSuccess || memory == nullptr) {
        (void)hipGetLastError();
        return KO_OK;
    }
    if (at < 0) {
        at = g_workspaces_used++;
        g_workspaces[at] = WorkspaceEntry{dev, stream, nullptr, nullptr};
    }
    (small ? g_workspaces[at].small : g_workspaces[at].memory) = memory;
    *workspace = memory;
    return KO_OK;
}
}  // namespace

int stream_workspace(hipStream_t stream, void **workspace) { return workspace_of(stream, false, workspace); }
int stream_small_workspace(hipStream_t stream, void **workspace) { return workspace_of(stream, true, workspace); }

int release_stream_workspace(hipStream_t stream) {
    int dev = 0;
    KO_HIP(hipGetDevice(&dev));
    void *memory = nullptr, *small = nullptr;
    {
        std::lock_guard<std::mutex> guard(g_workspaces_lock);
        for (int i = 0; i < g_workspaces_used; ++i)
            if (g_workspaces[i].device == dev && g_workspaces[i].stream == stream) {
                memory = g_workspaces[i].memory;
                small = g_workspaces[i].small;
                g_workspaces[i] = g_workspaces[--g_workspaces_used];
                break;
            }
    }
    if (memory != nullptr) KO_HIP(hipFree(memory));
    if (small != nullptr) KO_HIP(hipFree(small));
    return KO_OK;
}

int stream_workspace_count() {
    std::lock_guard<std::mutex> guard(g_workspaces_lock);
    return g_workspaces_used;
}

}  // namespace ko

KO_EXPORT const char *ko_last_error_string(void) { return ko::g_last_error; }

KO_EXPORT const char *ko_status_name(int status) {
    switch (status) {
        case KO_OK: return "KO_OK";
        case KO_ERR_INVALID_ARGUMENT: return "KO_ERR_INVALID_ARGUMENT";
        case KO_ERR_UNSUPPORTED_SHAPE: return "KO_ERR_UNSUPPORTED_SHAPE";
        case KO_ERR_RUNTIME: return "KO_ERR_RUNTIME";
        case KO_ERR_OUT_OF_MEMORY: return "KO_ERR_OUT_OF_MEMORY";
        case KO_ERR_NO_DEVICE: return "KO_ERR_NO_DEVICE";
        default: return "KO_ERR_UNKNOWN";
    }
}

// ---- the door for libko_harness.so (ko_harness.h): tuning table, planners, workspace table, last error
namespace ko {
namespace {
int hook_set_tuning(const char *name, int value) {
    if (!name) return fail(KO_ERR_INVALID_ARGUMENT, "ko_set_tuning: null name");
    const int k = find_knob(name);
    if (k < 0) return fail(KO_ERR_INVALID_ARGUMENT, "ko_set_tuning: unknown knob \"%s\"", name);
    g_knobs[k].store(value, std::memory_order_relaxed);
    return KO_OK;
}

int hook_get_tuning(const char *name, int *value) {
    if (!name || !value) return fail(KO_ERR_INVALID_ARGUMENT, "ko_get_tuning: null argument");
    const int k = find_knob(name);
    if (k < 0) return fail(KO_ERR_INVALID_ARGUMENT, "ko_get_tuning: unknown knob \"%s\"", name);
    *value = g_knobs[k].load(std::memory_order_relaxed);
    return KO_OK;
}

int hook_set_last_error(int status, const char *message) { return fail(status, "%s", message ? message : ""); }

const ko_harness_hooks_t kHooks = {hook_set_tuning, hook_get_tuning, debug_sgemm_plan, debug_gemm16_plan,
                                   stream_workspace_count, hook_set_last_error};
}  // namespace
}  // namespace ko

KO_EXPORT const ko_harness_hooks_t *ko_harness_hooks(void) { return &ko::kHooks; }

KO_EXPORT int ko_device_info(ko_device_info_t *info) {
    if (!info) return ko::fail(KO_ERR_INVALID_ARGUMENT, "ko_device_info: null info");
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0) {
        (void)hipGetLastError();
        return ko::fail(KO_ERR_NO_DEVICE, "ko_device_info: no HIP device visible");
    }
    int dev = 0;
    KO_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    KO_HIP(hipGetDeviceProperties(&prop, dev));
    std::memset(info, 0, sizeof(*info));
    std::strncpy(info->name, prop.name, sizeof(info->name) - 1);
    std::strncpy(info->arch, prop.gcnArchName, sizeof(info->arch) - 1);
    info->compute_units = prop.multiProcessorCount;
    info->wavefront_size = prop.warpSize;
    info->clock_khz = prop.clockRate;
    info->memory_clock_khz = prop.memoryClockRate;
    info->memory_bus_bits = prop.memoryBusWidth;
    info->l2_bytes = prop.l2CacheSize;
    info->lds_bytes_per_workgroup = static_cast<int>(prop.sharedMemPerBlock);
    info->hbm_bytes = prop.totalGlobalMem;
    return KO_OK;
}

KO_EXPORT int ko_malloc(void **device_ptr, size_t bytes) {
    if (!device_ptr) return ko::fail(KO_ERR_INVALID_ARGUMENT, "ko_malloc: null result pointer");
    *device_ptr = nullptr;
    if (bytes == 0) return KO_OK;
    KO_HIP(hipMalloc(device_ptr, bytes));
    return KO_OK;
}

KO_EXPORT int ko_free(void *device_ptr) {
    if (!device_ptr) return KO_OK;
    KO_HIP(hipFree(device_ptr));
    return KO_OK;
}

KO_EXPORT int ko_memset_async(void *device_ptr, int value, size_t bytes, ko_stream_t stream) {
    if (bytes == 0) return KO_OK;
    if (!device_ptr) return ko::fail(KO_ERR_INVALID_ARGUMENT, "ko_memset_async: null pointer");
    KO_HIP(hipMemsetAsync(device_ptr, value, bytes, ko::as_stream(stream)));
    return KO_OK;
}

static int check_copy(const void *dst, const void *src, size_t bytes, const char *who) {
    if (bytes && (!dst || !src)) return ko::fail(KO_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    return KO_OK;
}

KO_EXPORT int ko_memcpy_h2d(void *device_dst, const void *host_src, size_t bytes) {
    if (int rc = check_copy(device_dst, host_src, bytes, "ko_memcpy_h2d")) return rc;
    if (bytes == 0) return KO_OK;
    KO_HIP(hipMemcpy(device_dst, host_src, bytes, hipMemcpyHostToDevice));
    return KO_OK;
}

KO_EXPORT int ko_memcpy_h2d_async(void *device_dst, const void *host_src, size_t bytes,
                                  ko_stream_t stream) {
    if (int rc = check_copy(device_dst, host_src, bytes, "ko_memcpy_h2d_async")) return rc;
    if (bytes == 0) return KO_OK;
    KO_HIP(hipMemcpyAsync(device_dst, host_src, bytes, hipMemcpyHostToDevice, ko::as_stream(stream)));
    return KO_OK;
}

KO_EXPORT int ko_memcpy_d2h(void *host_dst, const void *device_src, size_t bytes) {
    if (int rc = check_copy(host_dst, device_src, bytes, "ko_memcpy_d2h")) return rc;
    if (bytes == 0) return KO_OK;
    KO_HIP(hipMemcpy(host_dst, device_src, bytes, hipMemcpyDeviceToHost));
    return KO_OK;
}

KO_EXPORT int ko_memcpy_d2h_async(void *host_dst, const void *device_src, size_t bytes,
                                  ko_stream_t stream) {
    if (int rc = check_copy(host_dst, device_src, bytes, "ko_memcpy_d2h_async")) return rc;
    if (bytes == 0) return KO_OK;
    KO_HIP(hipMemcpyAsync(host_dst, device_src, bytes, hipMemcpyDeviceToHost, ko::as_stream(stream)));
    return KO_OK;
}

KO_EXPORT int ko_memcpy_d2d_async(void *device_dst, const void *device_src, size_t bytes,
                                  ko_stream_t stream) {
    if (int rc = check_copy(device_dst, device_src, bytes, "ko_memcpy_d2d_async")) return rc;
    if (bytes == 0) return KO_OK;
    KO_HIP(hipMemcpyAsync(device_dst, device_src, bytes, hipMemcpyDeviceToDevice,
                          ko::as_stream(stream)));
    return KO_OK;
}

KO_EXPORT int ko_stream_create(ko_stream_t *stream) {
    if (!stream) return ko::fail(KO_ERR_INVALID_ARGUMENT, "ko_stream_create: null result pointer");
    hipStream_t s = nullptr;
    // Non-blocking with respect to the default stream, default priority.
    KO_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = reinterpret_cast<ko_stream_t>(s);
    return KO_OK;
}

KO_EXPORT int ko_stream_destroy(ko_stream_t stream) {
    if (!stream) return KO_OK;
    // The stream's workspace goes with it (the reference's Tensor frees what it allocated, common/tensor.cu:23-26):
    // first wait for the launches that may still read or write it.
    KO_HIP(hipStreamSynchronize(ko::as_stream(stream)));
    if (const int st = ko::release_stream_workspace(ko::as_stream(stream)); st != KO_OK) return st;
    KO_HIP(hipStreamDestroy(ko::as_stream(stream)));
    return KO_OK;
}

KO_EXPORT int ko_stream_synchronize(ko_stream_t stream) {
    KO_HIP(hipStreamSynchronize(ko::as_stream(stream)));
    return KO_OK;
}

KO_EXPORT int ko_device_synchronize(void) {
    KO_HIP(hipDeviceSynchronize());
    return KO_OK;
}

KO_EXPORT int ko_event_create(ko_event_t *event) {
    if (!event) return ko::fail(KO_ERR_INVALID_ARGUMENT, "ko_event_create: null result pointer");
    hipEvent_t e = nullptr;
    KO_HIP(hipEventCreate(&e));
    *event = reinterpret_cast<ko_event_t>(e);
    return KO_OK;
}

KO_EXPORT int ko_event_record(ko_event_t event, ko_stream_t stream) {
    if (!event) return ko::fail(KO_ERR_INVALID_ARGUMENT, "ko_event_record: null event");
    KO_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), ko::as_stream(stream)));
    return KO_OK;
}

KO_EXPORT int ko_event_synchronize(ko_event_t event) {
    if (!event) return ko::fail(KO_ERR_INVALID_ARGUMENT, "ko_event_synchronize: null event");
    KO_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
    return KO_OK;
}

KO_EXPORT int ko_event_elapsed_ms(float *ms, ko_event_t start, ko_event_t stop) {
    if (!ms || !start || !stop)
        return ko::fail(KO_ERR_INVALID_ARGUMENT, "ko_event_elapsed_ms: null argument");
    KO_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start),
                               reinterpret_cast<hipEvent_t>(stop)));
    return KO_OK;
}

KO_EXPORT int ko_event_destroy(ko_event_t event) {
    if (!event) return KO_OK;
    KO_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
    return KO_OK;
}
