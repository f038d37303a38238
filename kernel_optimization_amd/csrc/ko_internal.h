// Shared by the translation units of libko.so: status/last-error plumbing,
// launch checking and the tuning table.  Internal; not installed.
#pragma once

#include <hip/hip_runtime.h>
#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/ko.h"

#define KO_EXPORT extern "C" __attribute__((visibility("default")))

namespace ko {

// Records a formatted message as the calling thread's last error and returns `status`.
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Maps a hipError_t to a ko_status, recording file:line and the HIP error name.
int hip_fail(hipError_t err, const char *expr, const char *file, int line);

// Integer tuning knobs (0 = use the built-in default).
int tuning(const char *name);

inline hipStream_t as_stream(ko_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Number of compute units of the current device (cached per device).
int compute_units();

// Raises the dynamic-LDS limit of `kernel` to `bytes` on the current device. The attribute belongs to the
// device's copy of the kernel, so it is set once per device; `done` is the caller's per-kernel record of the
// devices already served (bit d = device d; devices from 64 on are set every time).
int allow_dynamic_lds(const void *kernel, size_t bytes, std::atomic<uint64_t> &done);

}  // namespace ko

#define KO_HIP(expr)                                                          \
    do {                                                                      \
        hipError_t ko_err_ = (expr);                                          \
        if (ko_err_ != hipSuccess) return ko::hip_fail(ko_err_, #expr, __FILE__, __LINE__); \
    } while (0)

// After a <<<>>> launch: surfaces launch-configuration errors (the reference never checks launches).
#define KO_CHECK_LAUNCH() KO_HIP(hipGetLastError())
