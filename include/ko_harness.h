/*
 * ko_harness.h - C ABI of libko_harness.so: what the tests and the benchmark need beside the operators and is
 * no part of the operator library's seam.  Seeded device fills, the plain copy kernel and the streaming probe
 * the bandwidth figures are judged against, the tuning knobs, and debug views of the cross-lane primitives
 * and of the GEMM planners.  Nothing here has a counterpart in the reference
 * (donglinz/kernel_optimization) beyond the host RNG loops of its drivers, which the fills replace.
 *
 * libko_harness.so links against libko.so.  Errors are reported as in ko.h: a ko_status return value and the
 * calling thread's ko_last_error_string().
 */
#ifndef KO_HARNESS_H
#define KO_HARNESS_H

#include "ko.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- the door: the ONE symbol libko.so exports beside those of ko.h.  libko_harness.so reaches the tuning
 *      table, the GEMM planners, the workspace table and the last-error slot of libko.so through it; nothing
 *      else should call it. */
typedef struct ko_harness_hooks_t {
    int (*set_tuning)(const char *name, int value);
    int (*get_tuning)(const char *name, int *value);
    int (*sgemm_plan)(int64_t m, int64_t n, int64_t k, int *slices, int *k_slice, int *variant);
    int (*gemm16_plan)(int64_t m, int64_t n, int64_t k, int b_layout, int *slices, int *k_slice, int *tile);
    int (*stream_workspace_count)(void);
    int (*set_last_error)(int status, const char *message); /* returns status */
} ko_harness_hooks_t;
const ko_harness_hooks_t *ko_harness_hooks(void); /* in libko.so */

/* ---- everything below is in libko_harness.so ---- */

/* ---- seeded device fills: replace the host RNG loops of the benchmark drivers
 *      (softmax/main.cu:31-36, layernorm/main.cu:30-35, gemm/main.cu:46-66) with a
 *      counter-based generator that gives the same tensor on host and device:
 *      splitmix64(seed, counter) -> u in [0,1); uniform = lo + (hi-lo)*u;
 *      normal = mean + std * sqrt(-2 ln(1-u(2i))) * cos(2 pi u(2i+1)); evaluated in
 *      double, rounded once to the storage type.  `first` is the index of out[0]. */
int ko_fill_normal_f32(float *out, int64_t n, uint64_t seed, double mean, double std,
                       int64_t first, ko_stream_t stream);
int ko_fill_uniform_f32(float *out, int64_t n, uint64_t seed, double lo, double hi, int64_t first,
                        ko_stream_t stream);
int ko_fill_uniform_16(void *out, int64_t n, uint64_t seed, double lo, double hi, int64_t first,
                       int dtype, ko_stream_t stream);
/* int32 lengths lo + floor((hi - lo + 1) * u), uniform on [lo, hi] */
int ko_fill_lengths_i32(int32_t *out, int64_t n, uint64_t seed, int32_t lo, int32_t hi,
                        ko_stream_t stream);

/* ---- measurement helpers (no reference counterpart; used by the benchmark harness) */
/* out[i] = in[i] for n floats, 128-bit accesses: the plain copy whose rate is the
 * practical HBM ceiling the bandwidth kernels are compared with. */
int ko_copy_f32(const float *in, float *out, int64_t n, ko_stream_t stream);
/* Streaming-rate probe: one launch that streams `nbytes` (a multiple of threads * vectors_per_thread * 16)
 * from `in` and/or to `out`: mode 0 write-only, 1 read-only, 2 copy, 3 copy that reads only the vectors whose
 * index modulo 128 is below `read_of_128` (a 512-column fp32 row with a padded tail) and writes all.
 * threads: workgroup size (multiple of 64); vectors_per_thread: 1, 2 or 4 16-byte vectors;
 * blocks_per_cu: 0 = one chunk per workgroup, else a grid of that many workgroups per compute unit walking
 * the chunks; load_policy: 0 plain, 1 non-temporal; store_policy: 0 plain, 1 nt, 2 sc1, 3 sc1 nt,
 * 4 sc0 sc1 nt (the cache-policy bits of the store instruction); lds_pad_bytes: dynamic LDS per workgroup,
 * never touched, which caps how many workgroups are resident per compute unit. */
int ko_stream_probe(const void *in, void *out, int64_t nbytes, int mode, int vectors_per_thread,
                    int threads, int blocks_per_cu, int load_policy, int store_policy, int read_of_128,
                    int lds_pad_bytes, ko_stream_t stream);
/* Times ko_gemm_f16f32acc (alpha 1, no C) from a host loop in C, as the vendor library's kernels are timed by the
 * comparison harness: `warmup` launches, then `batches` batches of `reps` launches between two events on the
 * default stream, launch i on operand set i % nsets (A, B, D: arrays of nsets device pointers); *median_us is the
 * median batch's time per launch.  For kernels of a few microseconds a Python loop cannot launch fast enough. */
int ko_time_gemm16_sets(int64_t m, int64_t n, int64_t k, const void *const *A, const void *const *B, void *const *D,
                        int nsets, int b_layout, int dtype, int warmup, int reps, int batches, float *median_us);
/* Integer tuning knobs by name ("softmax.lanes_per_row", ...); value 0 restores the default.
 * Unknown names return KO_ERR_INVALID_ARGUMENT. */
int ko_set_tuning(const char *name, int value);
int ko_get_tuning(const char *name, int *value);
/* Cross-lane primitives check: each of the 64 lanes of one wavefront contributes
 * in[lane]; out[lane] receives the all-reduce over its group of `group` lanes
 * (group in {2,4,8,16,32,64}; op 0 = max, 1 = sum). */
int ko_debug_wave_allreduce(const float *in, float *out, int group, int op, ko_stream_t stream);
/* How many (device, stream) pairs hold a workspace of the K-sliced paths right now (see ko_sgemm_f32 in ko.h). */
int ko_debug_stream_workspace_count(int *count);
/* What the GEMMs' host-side planners decide for a shape (16-byte aligned operands, 256 compute units when no
 * device is visible): the number of K slices (1 = the problem goes out whole), the depth of every slice but the
 * last, and the tiling of the sliced launch (SGEMM: the kernel variant number, 0 = chosen as for the whole
 * problem; 16-bit GEMM: 128 or 64, the tile edge, or 32 for 32 x 256 tiles).  The 16-bit GEMM with B in layout
 * b_layout (KO_ROW_MAJOR / KO_COL_MAJOR) has one more answer for a problem of few tiles: slices = 1 and tile =
 * 1000 * rows + columns - one launch whose workgroups own one output tile of that size and either split K over
 * their waves (32032, 32064, 64064) or walk K together through a deep ring of LDS stages (64128, 128064, 128128;
 * 1032064: 32 x 64 tiles of that kernel for a problem of at most 32 rows); slices > 1 with tile = 256: the pinned
 * kernel's 256 x 256 tiles in K slices;
 * tile = 0: none of this.  Touches no device memory and launches nothing. */
int ko_debug_sgemm_plan(int64_t m, int64_t n, int64_t k, int *slices, int *k_slice, int *variant);
int ko_debug_gemm16_plan(int64_t m, int64_t n, int64_t k, int b_layout, int *slices, int *k_slice, int *tile);

#ifdef __cplusplus
}
#endif
#endif /* KO_HARNESS_H */
