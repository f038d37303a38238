// Shared by the translation units of libko.so: status/last-error plumbing,
// launch checking and the tuning table.  Internal; not installed.
#pragma once

#include <hip/hip_runtime.h>
#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/ko.h"
#include "../../include/ko_harness.h"

#define KO_EXPORT extern "C" __attribute__((visibility("default")))

namespace ko {

// Records a formatted message as the calling thread's last error and returns `status`.
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Maps a hipError_t to a ko_status, recording file:line and the HIP error name.
int hip_fail(hipError_t err, const char *expr, const char *file, int line);

// Integer tuning knobs (0 = use the built-in default).  One relaxed atomic per knob, indexed by an enum: a
// launch path reads several of them per call and takes no lock and builds no string to do so.  The names are
// what ko_set_tuning / ko_get_tuning accept.
#define KO_TUNING_KNOBS(X)                                                                                  \
    X(softmax_lanes_per_row, "softmax.lanes_per_row") X(softmax_blocks_per_cu, "softmax.blocks_per_cu")     \
    X(softmax_nontemporal, "softmax.nontemporal") X(softmax_block_threads, "softmax.block_threads")         \
    X(softmax_wave_threads, "softmax.wave_threads") X(layernorm_lanes_per_row, "layernorm.lanes_per_row")   \
    X(layernorm_blocks_per_cu, "layernorm.blocks_per_cu") X(layernorm_block_threads, "layernorm.block_threads") \
    X(layernorm_wave_threads, "layernorm.wave_threads") X(softmax_wave_lds, "softmax.wave_lds") X(rows_block_grid, "rows.block_grid") X(layernorm_wave_lds, "layernorm.wave_lds") X(layernorm_affine_lds, "layernorm.affine_lds")           \
    X(sgemm_variant, "sgemm.variant") X(sgemm_mapping, "sgemm.mapping") X(sgemm_split_rows, "sgemm.split_rows") \
    X(sgemm_k_slices, "sgemm.k_slices") X(gemm16_k_slices, "gemm16.k_slices") X(layernorm_block_rows, "layernorm.block_rows") X(sgemm_slice_variant, "sgemm.slice_variant") X(sgemm_unaligned, "sgemm.unaligned")                                                                     \
    X(gemm16_variant, "gemm16.variant") X(gemm16_mapping, "gemm16.mapping")                                 \
    X(gemm16_split_rows, "gemm16.split_rows") X(gemm16_wave_k, "gemm16.wave_k") X(copy_blocks_per_cu, "copy.blocks_per_cu")                   \
    X(copy_nontemporal, "copy.nontemporal")
enum Knob {
#define KO_KNOB_ENUM(id, name) knob_##id,
    KO_TUNING_KNOBS(KO_KNOB_ENUM)
#undef KO_KNOB_ENUM
    knob_count
};
extern std::atomic<int> g_knobs[knob_count];
inline int tuning(Knob k) { return g_knobs[k].load(std::memory_order_relaxed); }

// Residency cap for the streaming row kernels.  A one-pass kernel over HBM runs fastest on MI355X with about
// 32-40 KB of loads in flight per compute unit; with more resident wavefronts than that needs, the requests
// of a CU spread over a wider address window and the achieved rate drops (a 1 GiB copy with 2 KB per
// wavefront: 6.32 TB/s at 32 resident wavefronts per CU, 6.84 TB/s at 16).  A single-wavefront workgroup
// therefore asks for dynamic LDS it never touches, sized so that `bytes_in_flight / bytes_per_wave`
// workgroups fit into the 160 KB of a CU.  Returns 0 (no cap) when the hardware limit of 32 is no more.
inline int lds_pad_for_residency(int64_t bytes_per_wave, int64_t bytes_in_flight) {
    if (bytes_per_wave <= 0) return 0;
    int64_t waves = (bytes_in_flight + bytes_per_wave - 1) / bytes_per_wave;
    if (waves >= 32) return 0;
    if (waves < 8) waves = 8;  // fewer leave the memory latency uncovered (8 KB rows: 5 resident 75.7 us, 8 64.0 us)
    return static_cast<int>((160 * 1024 / waves) & ~int64_t{511});
}

inline hipStream_t as_stream(ko_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Number of compute units of the current device (cached per device).
int compute_units();

// Raises the dynamic-LDS limit of `kernel` to `bytes` on the current device. The attribute belongs to the
// device's copy of the kernel, so it is set once per device; `done` is the caller's per-kernel record of the
// devices already served (bit d = device d; devices from 64 on are set every time).
int allow_dynamic_lds(const void *kernel, size_t bytes, std::atomic<uint64_t> &done);

// Device memory for the partial results of calls on `stream` of the current device: kStreamWorkspaceBytes,
// allocated at the first request for that (device, stream) pair and kept until ko_stream_destroy releases it
// (the default stream's until the process ends), so calls on different streams never share it and calls on one
// stream use it in stream order.  `*workspace` stays null, with KO_OK, where nothing may be allocated (the
// stream is being captured into a graph and has no workspace yet, 64 live pairs already hold one, the stream is
// hipStreamPerThread, or the allocation fails): the caller then takes its path without a workspace.
constexpr size_t kStreamWorkspaceBytes = size_t{64} << 20;
// What the SGEMM's K slices use of it at most: the size of the static array that stands in for the workspace in the
// entry point that allocates nothing, so that both entry points plan, and sum, the same slices.
constexpr size_t kSgemmPartialBytes = size_t{32} << 20;
int stream_workspace(hipStream_t stream, void **workspace);
// The same for the row operators, which pass a few kilobytes of per-piece statistics: a small allocation of the pair's
// own (kStreamSmallWorkspaceBytes), made, kept and released like the large one and independent of it.
constexpr size_t kStreamSmallWorkspaceBytes = size_t{1} << 20;
int stream_small_workspace(hipStream_t stream, void **workspace);
// Frees the workspace of (current device, stream), if it has one.  The caller has synchronised the stream.
int release_stream_workspace(hipStream_t stream);
// How many (device, stream) pairs hold a workspace right now.
int stream_workspace_count();

// The 16-bit GEMM's problem as its kernels take it (csrc/ko_gemm16.hip, compiled in four parts).
struct Gemm16Params {
    const uint16_t *A;
    const uint16_t *B;
    const uint16_t *C;
    uint16_t *D;
    int M, N, K;
    float alpha, beta;
    int tiles_n;
    int nblocks;
    int band_rows;              // persistent kernels: > 0 selects the blocked tile order (see tile_of)
    int block_cols;
    const uint16_t *bias;       // [N] or null: added to every row before the activation
    int act;                    // KO_ACT_*
    int ldd;                    // elements between rows of C and D (N, or more when they are a column range of a wider matrix)
    int ldb;                    // row-major B: elements between its rows (N, or more likewise)
    // K slices (gemm16_kernel only): workgroups with blockIdx.y = s multiply k in [s * k_slice, (s + 1) * k_slice) and
    // write their M x N partial product as fp32 (no alpha, C, bias or activation; rows partial_ld(N) floats apart)
    // behind partial + s * M * partial_ld(N)
    int k_slice;                // 0: no slices
    float *partial;
    int ldk;                    // gemm16_kernel: elements between rows of A and of a column-major B (K of the whole problem)
    int tiles;                  // gemm16_pinned_kernel with K slices: output tiles (nblocks = tiles * slices)
    int xcd_cols_log2;          // blocked tile order: the 8 XCDs' regions lie 2^this side by side (0: one below the other)
    int region_cols;            //                     columns of tiles in a region (unused when they lie one below the other)
};
// One call of the 16-bit GEMM on operands of one type and one layout of B: defined by the part of ko_gemm16.hip that
// is compiled for that combination.
template <bool BF16, bool B_ROW_MAJOR>
int gemm16_run(const Gemm16Params &p, hipStream_t stream);
template <> int gemm16_run<false, false>(const Gemm16Params &p, hipStream_t stream);
template <> int gemm16_run<false, true>(const Gemm16Params &p, hipStream_t stream);
template <> int gemm16_run<true, false>(const Gemm16Params &p, hipStream_t stream);
template <> int gemm16_run<true, true>(const Gemm16Params &p, hipStream_t stream);

// What the GEMM planners decide for a shape, for the harness (ko_harness_hooks_t::sgemm_plan, gemm16_plan).
int debug_sgemm_plan(int64_t m, int64_t n, int64_t k, int *slices, int *k_slice, int *variant);
int debug_gemm16_plan(int64_t m, int64_t n, int64_t k, int b_layout, int *slices, int *k_slice, int *tile);

}  // namespace ko

#define KO_HIP(expr)                                                          \
    do {                                                                      \
        hipError_t ko_err_ = (expr);                                          \
        if (ko_err_ != hipSuccess) return ko::hip_fail(ko_err_, #expr, __FILE__, __LINE__); \
    } while (0)

// After a <<<>>> launch: surfaces launch-configuration errors (the reference never checks launches).
#define KO_CHECK_LAUNCH() KO_HIP(hipGetLastError())
