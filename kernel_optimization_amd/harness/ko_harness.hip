// libko_harness.so: the parts of the test and benchmark harness that are device code or reach into libko.so.
// This file holds the library's own copies of the few helpers of ko_internal.h its kernels use (errors are
// recorded in libko.so's last-error slot through the hooks, so ko_last_error_string() reports them), the
// wrappers over the hooks, and the cross-lane primitive check.
#include "ko_internal.h"
#include "wave64.h"

#include <algorithm>
#include <cstring>

namespace ko {

static const ko_harness_hooks_t *hooks() {
    static const ko_harness_hooks_t *h = ko_harness_hooks();
    return h;
}

int fail(int status, const char *fmt, ...) {
    char message[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(message, sizeof(message), fmt, ap);
    va_end(ap);
    return hooks()->set_last_error(status, message);
}

int hip_fail(hipError_t err, const char *expr, const char *file, int line) {
    int status = KO_ERR_RUNTIME;
    if (err == hipErrorOutOfMemory) status = KO_ERR_OUT_OF_MEMORY;
    if (err == hipErrorNoDevice || err == hipErrorInvalidDevice) status = KO_ERR_NO_DEVICE;
    return fail(status, "HIP error at %s:%d code=%d(%s) \"%s\"", file, line, static_cast<int>(err),
                hipGetErrorName(err), expr);
}

// This library's copy of the knob table: ko_set_tuning keeps it in step with libko.so's, so the copy kernel
// here reads its knobs ("copy.*") the way the operators read theirs.
std::atomic<int> g_knobs[knob_count];

static const char *const kKnobNames[knob_count] = {
#define KO_KNOB_NAME(id, name) name,
    KO_TUNING_KNOBS(KO_KNOB_NAME)
#undef KO_KNOB_NAME
};

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

}  // namespace ko

KO_EXPORT int ko_set_tuning(const char *name, int value) {
    const int st = ko::hooks()->set_tuning(name, value);
    if (st == KO_OK)
        for (int i = 0; i < ko::knob_count; ++i)
            if (std::strcmp(ko::kKnobNames[i], name) == 0) ko::g_knobs[i].store(value, std::memory_order_relaxed);
    return st;
}

KO_EXPORT int ko_get_tuning(const char *name, int *value) { return ko::hooks()->get_tuning(name, value); }

KO_EXPORT int ko_debug_sgemm_plan(int64_t m, int64_t n, int64_t k, int *slices, int *k_slice, int *variant) {
    return ko::hooks()->sgemm_plan(m, n, k, slices, k_slice, variant);
}

KO_EXPORT int ko_debug_gemm16_plan(int64_t m, int64_t n, int64_t k, int b_layout, int *slices, int *k_slice, int *tile) {
    return ko::hooks()->gemm16_plan(m, n, k, b_layout, slices, k_slice, tile);
}

KO_EXPORT int ko_time_gemm16_sets(int64_t m, int64_t n, int64_t k, const void *const *A, const void *const *B,
                                  void *const *D, int nsets, int b_layout, int dtype, int warmup, int reps, int batches,
                                  float *median_us) {
    if (!A || !B || !D || !median_us || nsets <= 0 || warmup < 0 || reps <= 0 || batches <= 0 || batches > 64)
        return ko::fail(KO_ERR_INVALID_ARGUMENT, "ko_time_gemm16_sets: bad argument");
    auto call = [&](int i) {
        const int s = i % nsets;
        return ko_gemm_f16f32acc(m, n, k, 1.0f, A[s], B[s], b_layout, 0.0f, nullptr, D[s], dtype, nullptr);
    };
    for (int i = 0; i < warmup; ++i)
        if (const int st = call(i); st != KO_OK) return st;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    KO_HIP(hipEventCreate(&e0));
    if (const hipError_t e = hipEventCreate(&e1); e != hipSuccess) {
        (void)hipEventDestroy(e0);
        return ko::hip_fail(e, "hipEventCreate", __FILE__, __LINE__);
    }
    float us[64];
    int st = KO_OK;
    for (int b = 0; b < batches && st == KO_OK; ++b) {
        (void)hipEventRecord(e0, nullptr);
        for (int r = 0; r < reps && st == KO_OK; ++r) st = call(warmup + b * reps + r);
        (void)hipEventRecord(e1, nullptr);
        if (const hipError_t e = hipEventSynchronize(e1); e != hipSuccess && st == KO_OK)
            st = ko::hip_fail(e, "hipEventSynchronize", __FILE__, __LINE__);
        float ms = 0.0f;
        (void)hipEventElapsedTime(&ms, e0, e1);
        us[b] = ms * 1e3f / reps;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (st != KO_OK) return st;
    std::sort(us, us + batches);
    *median_us = us[batches / 2];
    return KO_OK;
}

KO_EXPORT int ko_debug_stream_workspace_count(int *count) {
    if (!count) return ko::fail(KO_ERR_INVALID_ARGUMENT, "ko_debug_stream_workspace_count: null argument");
    *count = ko::hooks()->stream_workspace_count();
    return KO_OK;
}

// ---- cross-lane primitive check (see ko_harness.h)
namespace ko {
namespace {
template <int G>
__global__ void wave_allreduce_kernel(const float *in, float *out, int op) {
    float v = in[threadIdx.x];
    out[threadIdx.x] = op == 0 ? wave::allreduce<G, wave::Max>(v) : wave::allreduce<G, wave::Sum>(v);
}
}  // namespace
}  // namespace ko

KO_EXPORT int ko_debug_wave_allreduce(const float *in, float *out, int group, int op,
                                      ko_stream_t stream) {
    if (!in || !out) return ko::fail(KO_ERR_INVALID_ARGUMENT, "wave_allreduce: null pointer");
    if (op != 0 && op != 1) return ko::fail(KO_ERR_INVALID_ARGUMENT, "wave_allreduce: op=%d", op);
    hipStream_t s = ko::as_stream(stream);
    switch (group) {
        case 2: ko::wave_allreduce_kernel<2><<<1, 64, 0, s>>>(in, out, op); break;
        case 4: ko::wave_allreduce_kernel<4><<<1, 64, 0, s>>>(in, out, op); break;
        case 8: ko::wave_allreduce_kernel<8><<<1, 64, 0, s>>>(in, out, op); break;
        case 16: ko::wave_allreduce_kernel<16><<<1, 64, 0, s>>>(in, out, op); break;
        case 32: ko::wave_allreduce_kernel<32><<<1, 64, 0, s>>>(in, out, op); break;
        case 64: ko::wave_allreduce_kernel<64><<<1, 64, 0, s>>>(in, out, op); break;
        default: return ko::fail(KO_ERR_INVALID_ARGUMENT, "wave_allreduce: group=%d", group);
    }
    KO_CHECK_LAUNCH();
    return KO_OK;
}
