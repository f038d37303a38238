// LayerNorm over the last dimension for gfx950: one pass over HBM, fp32
// arithmetic, fp32 / binary16 / bfloat16 storage (x, y, gamma, beta; mean and
// rstd are always fp32), Welford statistics, outputs y and (optionally) per-row
// mean and rstd.
//
// Per row (nn_operators/layernorm/layernorm.h): each lane folds its elements
// into a Welford triplet (count, mean, M2) with the streaming update of
// :13-23; lanes are combined with Chan's merge (:36-47) as symmetric DPP /
// permlane-swap exchanges; var = M2 / N (or N-1); rstd = 1/sqrt(var + eps)
// (:184); y = (x - mean) * rstd [* gamma] [+ beta] (:185-195, with the
// intended x - mean; the reference's Subtract functor adds,
// common/functors.h:168, and its merge divides M2 by count-1 at every step,
// layernorm.h:48 - neither is reproduced).
//
// The statistics are taken of x - x0, x0 being the row's first element: fp32
// Welford/Chan arithmetic rounds every partial mean to an ulp of the data's
// magnitude, which costs a few 1e-5 of the variance when |mean| is 1e4 times the
// standard deviation.  After the shift the partial means are of the size of the
// spread, not of the offset, and x - x0 itself is exact or nearly so.
// mean = x0 + mean(x - x0); its error is relative to the spread of the row.
//
// A row that holds a NaN or an infinity has no statistics: M2 becomes NaN (the
// update multiplies inf by inf - inf), and with it rstd and every y of the row;
// mean is reported as NaN as well, whatever the running mean happened to be (the
// reference's own update turns mu into NaN as soon as an element follows an
// infinity: d = x - mu = -inf, mu += d/n, layernorm.h:16-18).
//
// Mappings as in the reference: WARP (LayerNormWarpImpl :145-201) = row in the
// registers of LPR lanes of a wavefront; BLOCK (LayerNormBlockImpl :204-252) =
// row in the registers of a workgroup, per-wave triplets through LDS;
// BLOCK_NOCACHE (LayerNormBlockNoCacheImpl :254-300) = two reads of the row.
#include "ko_internal.h"
#include <type_traits>

#include "wave64.h"

namespace ko {
namespace {

// 1/n for the streaming update: the n-th element a lane folds always has count n,
// so the division of layernorm.h:18 becomes a multiplication by a constant.
template <int N>
struct Reciprocals {
    float v[N + 1];
    constexpr Reciprocals() : v{} {
        v[0] = 0.0f;
        for (int i = 1; i <= N; ++i) v[i] = 1.0f / static_cast<float>(i);
    }
};

// 1 / sqrt(x) from the hardware instruction (1 ulp; the gate on rstd is 1e-5 relative).  A correctly rounded
// square root followed by a correctly rounded division is some 25 instructions that every lane of a row runs.
// Special values as with the division: +inf -> 0, 0 -> +inf, NaN and negative -> NaN.
__device__ __forceinline__ float rsqrt_1ulp(float x) { return __builtin_amdgcn_rsqf(x); }

__device__ __forceinline__ void welford_update(wave::Welford &w, float x, float inv_count) {
    w.count += 1.0f;
    const float d = x - w.mean;
    w.mean = __builtin_fmaf(d, inv_count, w.mean);
    w.m2 = __builtin_fmaf(d, x - w.mean, w.m2);
}

// The same update where the count is not a compile-time constant: 1/count comes from the hardware reciprocal
// (1 ulp).  M2 is accumulated against the mean actually formed, so the triplet stays consistent and the
// deviation is far inside the 1e-5 gate.
__device__ __forceinline__ void welford_update_counted(wave::Welford &w, float x) {
    w.count += 1.0f;
    const float d = x - w.mean;
    w.mean = __builtin_fmaf(d, __builtin_amdgcn_rcpf(w.count), w.mean);
    w.m2 = __builtin_fmaf(d, x - w.mean, w.m2);
}

template <int IO>
struct Args {
    const typename Io<IO>::elem *in;
    typename Io<IO>::elem *out;
    float *mean;
    float *rstd;
    const typename Io<IO>::elem *gamma;
    const typename Io<IO>::elem *beta;
    int64_t rows;
    int cols;
    float eps;
    float inv_denominator;  // 1/N or 1/(N-1)
    hipStream_t stream;
};

// ---------------------------------------------------------------- WARP policy
// A wavefront takes one row group (64 / LPR rows, one per lane group) per trip.
// FULL: cols == LPR * VPL vectors, every lane folds the same number of elements (no per-vector bounds
// checks, and the lanes merge with the equal-count form).
// AFFINE: gamma or beta (or both) given.  Their loads are then unconditional - a missing one is pointed at the
// other and its values ignored - because loads inside `if (gamma)` branches leave the compiler unable to count
// the loads in flight: it then makes the statistics wait for all but the last two of them, gamma and beta
// included, instead of for the row alone.
// AFFINE_LDS (with AFFINE, FULL rows, one row per wavefront, four wavefronts per workgroup, rows a multiple of four):
// gamma and beta come into LDS once per workgroup, straight from global memory, and every wavefront reads its
// lanes' vectors from there.  Fetched per wavefront they are 6 KB of L1 traffic next to a 3 KB row.
template <int IO, int LPR, int VPL, bool FULL, bool AFFINE, bool AFFINE_LDS = false>
__global__ __launch_bounds__(256) void layernorm_wave_kernel(const typename Io<IO>::elem *in,
                                                             typename Io<IO>::elem *out,
                                                             float *__restrict__ mean_out,
                                                             float *__restrict__ rstd_out,
                                                             const typename Io<IO>::elem *__restrict__ gamma,
                                                             const typename Io<IO>::elem *__restrict__ beta,
                                                             int64_t rows, int cols, float eps,
                                                             float inv_denominator) {
    constexpr int E = Io<IO>::E;
    constexpr int RPW = 64 / LPR;
    constexpr bool NT = true;  // streaming accesses: every byte is touched once
    constexpr Reciprocals<VPL * E> rcp;
    const int lane = threadIdx.x & 63;
    const int sub = lane / LPR;
    const int l = lane % LPR;
    const int nvec = cols / E;
    const int64_t waves_per_block = blockDim.x >> 6;
    const int64_t wave = blockIdx.x * waves_per_block + (threadIdx.x >> 6);
    const int64_t stride = static_cast<int64_t>(gridDim.x) * waves_per_block * RPW;

    // gamma/beta of this lane's columns stay in registers across rows.  They are fetched behind the first
    // row's loads: memory returns in order, so loads issued ahead of the row would stand between the row
    // and the statistics, which do not need them.
    // They are kept as loaded (16-bit storage: half the registers of converted values, which decides between
    // four and six resident waves per SIMD at 768 columns) and converted where they are used.
    typename Io<IO>::raw g_raw[VPL], b_raw[VPL];
    const typename Io<IO>::elem *g_from = gamma ? gamma : beta, *b_from = beta ? beta : gamma;
    extern __shared__ __attribute__((aligned(16))) char affine_lds[];  // AFFINE_LDS: raw gamma[nvec], then raw beta[nvec]
    auto load_affine = [&]() {
        if constexpr (AFFINE_LDS) {
            // thread t brings vector t of gamma and of beta in: a wavefront's 64 vectors land, 16 bytes per lane, behind
            // a wave-uniform LDS address
            typedef const __attribute__((address_space(1))) void *gptr_t;
            typedef __attribute__((address_space(3))) void *lptr_t;
            for (int j0 = static_cast<int>(threadIdx.x & ~63u); j0 < nvec; j0 += blockDim.x) {
                if (j0 + lane < nvec) {
                    __builtin_amdgcn_global_load_lds((gptr_t)(g_from + E * (j0 + lane)), (lptr_t)(affine_lds + 16 * j0), 16, 0, 0);
                    __builtin_amdgcn_global_load_lds((gptr_t)(b_from + E * (j0 + lane)), (lptr_t)(affine_lds + 16 * (nvec + j0)), 16, 0, 0);
                }
            }
            return;
        }
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = l + k * LPR;
            g_raw[k] = typename Io<IO>::raw{};
            b_raw[k] = typename Io<IO>::raw{};
            if constexpr (AFFINE) {
                if (FULL || j < nvec) {
                    g_raw[k] = Io<IO>::template load_raw<false>(g_from + E * j);
                    b_raw[k] = Io<IO>::template load_raw<false>(b_from + E * j);
                }
            }
        }
    };

    // All loads of a row go out before any is converted: a conversion inside the branch that holds its load
    // makes the compiler wait for that load before the next one is issued.
    auto load_rows = [&](float (&v)[VPL][E], int64_t row) {
        const bool row_ok = row < rows;
        const typename Io<IO>::elem *src = in + row * cols;
        typename Io<IO>::raw loaded[VPL];
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = l + k * LPR;
            loaded[k] = typename Io<IO>::raw{};  // all-zero bits are 0.0 in every storage type
            if (row_ok && (FULL || j < nvec)) loaded[k] = Io<IO>::template load_raw<NT>(src + E * j);
        }
#pragma unroll
        for (int k = 0; k < VPL; ++k) Io<IO>::unpack(loaded[k], v[k]);
    };

    auto finish_rows = [&](float (&v)[VPL][E], int64_t row, auto between) {
        const bool row_ok = row < rows;
        const float x0 = wave::broadcast_group_first<LPR>(v[0][0]);
        wave::Welford w{0.0f, 0.0f, 0.0f};
        if constexpr (FULL) {
            // Every lane holds VPL * E values in registers: its triplet (count, mean, M2) is formed in two passes
            // over them - sums of independent pairs instead of VPL * E dependent Welford updates.
            float s[E], q[E];
#pragma unroll
            for (int e = 0; e < E; ++e) {
                v[0][e] -= x0;
                s[e] = v[0][e];
            }
#pragma unroll
            for (int k = 1; k < VPL; ++k)
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    v[k][e] -= x0;
                    s[e] += v[k][e];
                }
            float sum = s[0];
#pragma unroll
            for (int e = 1; e < E; ++e) sum += s[e];
            const float lane_mean = sum * (1.0f / (VPL * E));
#pragma unroll
            for (int e = 0; e < E; ++e) q[e] = 0.0f;
#pragma unroll
            for (int k = 0; k < VPL; ++k)
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    const float d = v[k][e] - lane_mean;
                    q[e] = __builtin_fmaf(d, d, q[e]);
                }
            float m2 = q[0];
#pragma unroll
            for (int e = 1; e < E; ++e) m2 += q[e];
            w = wave::Welford{static_cast<float>(VPL * E), lane_mean, m2};
        } else {
#pragma unroll
            for (int k = 0; k < VPL; ++k) {
                const int j = l + k * LPR;
#pragma unroll
                for (int e = 0; e < E; ++e) v[k][e] -= x0;
                if (FULL || j < nvec) {
#pragma unroll
                    for (int e = 0; e < E; ++e) welford_update(w, v[k][e], rcp.v[E * k + e + 1]);
                }
            }
        }
        if constexpr (FULL) w = wave::welford_allreduce_equal<LPR>(w);
        else w = wave::welford_allreduce<LPR>(w);

        const float mean = w.mean;  // of the shifted row
        const float rstd = rsqrt_1ulp(w.m2 * inv_denominator + eps);
        between();

        // streaming stores: wave-uniform base (the wavefront's first row) + per-lane byte offset
        // (written through at once only when rows are whole 64-byte lines: see store_row_vec)
        typename Io<IO>::elem *dst0 = out + (row - sub) * cols;
        const uint32_t sub_off = static_cast<uint32_t>(sub) * static_cast<uint32_t>(cols) * sizeof(typename Io<IO>::elem);
        const bool whole_lines = rows_are_whole_lines<IO>(cols);
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = l + k * LPR;
            if (row_ok && (FULL || j < nvec)) {
                float y[E], g[E], b[E];
                if constexpr (E == 8) {
                    // the conversions stay here, per row: hoisted out of the row loop they would occupy the
                    // registers that keeping the vectors unconverted is meant to save
                    asm volatile("" : "+v"(g_raw[k]), "+v"(b_raw[k]));
                }
                if (AFFINE && gamma) {
                    Io<IO>::unpack(g_raw[k], g);
                } else {
#pragma unroll
                    for (int e = 0; e < E; ++e) g[e] = 1.0f;
                }
                if (AFFINE && beta) {
                    Io<IO>::unpack(b_raw[k], b);
                } else {
#pragma unroll
                    for (int e = 0; e < E; ++e) b[e] = 0.0f;
                }
#pragma unroll
                for (int e = 0; e < E; ++e) y[e] = __builtin_fmaf((v[k][e] - mean) * rstd, g[e], b[e]);
                store_row_vec<IO>(whole_lines, dst0, sub_off + Io<IO>::kBytes * j, y);
            }
        }
        if (row_ok && l == 0) {
            if (mean_out) mean_out[row] = rstd != rstd ? rstd : x0 + mean;  // no statistics for a row with NaN or inf
            if (rstd_out) rstd_out[row] = rstd;
        }
    };

    // The first row group stands outside the loop: its loads and those of gamma and beta are then one
    // straight-line sequence, and the compiler can count which of them the statistics have to wait for.
    int64_t row0 = wave * RPW;
    if (row0 >= rows) return;
    float v[VPL][E];
    load_rows(v, row0 + sub);
    load_affine();
    finish_rows(v, row0 + sub, [&]() {
        if constexpr (AFFINE_LDS) {
            // every wavefront of the workgroup has a row (rows are a multiple of the wavefronts per workgroup), so
            // all of them arrive here; the statistics above have covered the latency of the fetch
            __syncthreads();
            const typename Io<IO>::raw *g_lds = reinterpret_cast<const typename Io<IO>::raw *>(affine_lds);
#pragma unroll
            for (int k = 0; k < VPL; ++k) {
                g_raw[k] = g_lds[l + k * LPR];
                b_raw[k] = g_lds[nvec + l + k * LPR];
            }
        }
    });
    for (row0 += stride; row0 < rows; row0 += stride) {
        load_rows(v, row0 + sub);
        finish_rows(v, row0 + sub, []() {});
    }
}

// --------------------------------------------------------------- BLOCK policy
// Workgroup-wide Welford all-reduce: per-wave triplets through LDS, then merged as a tree by
// every wave in the same way.
template <int THREADS>
__device__ __forceinline__ wave::Welford block_welford_allreduce(wave::Welford w, float *lds) {
    constexpr int WAVES = THREADS / 64;
    w = wave::welford_allreduce<64>(w);
    if constexpr (WAVES == 1) return w;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) {
        const int wv = threadIdx.x >> 6;
        lds[wv] = w.count;
        lds[16 + wv] = w.mean;
        lds[32 + wv] = w.m2;
    }
    __syncthreads();
    // every lane picks up one wave's triplet and the WAVES of them are merged as a tree by the same
    // symmetric exchanges (log2(WAVES) merges instead of WAVES - 1 in a row); all lanes of all waves
    // end with the same bits
    const int i = threadIdx.x & (WAVES - 1);
    return wave::welford_allreduce<WAVES>(wave::Welford{lds[i], lds[16 + i], lds[32 + i]});
}

// base + bytes, for addresses formed from a uniform pointer and a 32-bit per-lane offset
template <class T>
__device__ __forceinline__ T *at_bytes(T *base, uint32_t bytes) {
    typedef typename std::conditional<std::is_const<T>::value, const char, char>::type Byte;
    return reinterpret_cast<T *>(reinterpret_cast<Byte *>(base) + bytes);
}

// y = (x - mean) * rstd [* gamma] [+ beta] for one vector; gamma/beta are read here (long rows:
// they do not fit the registers next to the row).
template <int IO>
__device__ __forceinline__ void normalize_vec(const float (&x)[Io<IO>::E], float mean, float rstd,
                                              const typename Io<IO>::elem *gamma,
                                              const typename Io<IO>::elem *beta, int col, float (&y)[Io<IO>::E]) {
    constexpr int E = Io<IO>::E;
    float g[E], b[E];
    if (gamma) Io<IO>::template load<false>(gamma + col, g);
    if (beta) Io<IO>::template load<false>(beta + col, b);
#pragma unroll
    for (int e = 0; e < E; ++e) {
        float t = (x[e] - mean) * rstd;
        if (gamma) t *= g[e];
        if (beta) t += b[e];
        y[e] = t;
    }
}

// One workgroup per row, the row held on chip between its single read and its single write; both are
// nontemporal (every byte is touched once; measured faster than cached accesses on rows of 16 KB and more).
// VPL vectors per thread live in registers, LV more in LDS (vector k of thread t at tail[k][t], filled by
// direct-to-LDS loads, which cost no registers on the way).  REST: what lies beyond those (VPL + LV) * THREADS
// vectors is streamed - folded into the statistics as it arrives, and read a second time for the output - so a
// row a little longer than the chip holds costs a little more traffic, not half as much again.
template <int IO, int THREADS, int VPL, int LV = 0, bool REST = false>
__global__ __launch_bounds__(THREADS) void layernorm_block_kernel(const typename Io<IO>::elem *in,
                                                                  typename Io<IO>::elem *out,
                                                                  float *__restrict__ mean_out,
                                                                  float *__restrict__ rstd_out,
                                                                  const typename Io<IO>::elem *__restrict__ gamma,
                                                                  const typename Io<IO>::elem *__restrict__ beta,
                                                                  int64_t rows, int cols, float eps,
                                                                  float inv_denominator) {
    constexpr int E = Io<IO>::E;
    typedef typename Io<IO>::raw Raw;
    __shared__ float lds[48];
    extern __shared__ __attribute__((aligned(16))) char tail_bytes[];  // Raw tail[LV][THREADS]
    Raw *tail = reinterpret_cast<Raw *>(tail_bytes);
    constexpr Reciprocals<VPL * E> rcp;
    constexpr int UNROLL = 2;                       // vectors per thread and trip of the streamed part
    constexpr int kCached = (VPL + LV) * THREADS;   // vectors of a row held on chip
    const int nvec = cols / E;
    // gamma/beta of this thread's columns stay in registers across the rows the workgroup walks, when
    // row, gamma and beta fit the register budget of the workgroup size (128 per lane at 1024 threads)
    constexpr bool HOIST = VPL * E * 3 + 48 <= (THREADS == 1024 ? 128 : 256);
    float g[HOIST ? VPL : 1][E], b[HOIST ? VPL : 1][E];
#pragma unroll
    for (int k = 0; k < (HOIST ? VPL : 0); ++k) {
        const int j = threadIdx.x + k * THREADS;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            g[k][e] = 1.0f;
            b[k][e] = 0.0f;
        }
        if (j < nvec) {
            if (gamma) Io<IO>::template load<false>(gamma + E * j, g[k]);
            if (beta) Io<IO>::template load<false>(beta + E * j, b[k]);
        }
    }
    // Byte offset of this thread's first vector in a row (vector k lies k * THREADS * 16 bytes further).  The
    // row loop passes it through an empty asm: addresses are then formed per use from a uniform base and this
    // one register, instead of 2 * VPL pointers to gamma and beta being kept across rows (which spilled).
    uint32_t first = threadIdx.x * Io<IO>::kBytes;
    constexpr uint32_t kStep = THREADS * Io<IO>::kBytes;
    static_assert(LV == 0 || Io<IO>::kBytes == 16, "the LDS tail is filled 16 bytes per lane");
    const bool whole_lines = rows_are_whole_lines<IO>(cols);
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        asm volatile("" : "+v"(first));
        const typename Io<IO>::elem *src = in + row * cols;
        float v[VPL][E];
        {
            typename Io<IO>::raw loaded[VPL];  // all loads first, conversions afterwards
#pragma unroll
            for (int k = 0; k < VPL; ++k) {
                const int j = threadIdx.x + k * THREADS;
                loaded[k] = typename Io<IO>::raw{};
                if (j < nvec) loaded[k] = Io<IO>::template load_raw<true>(at_bytes(src, first + k * kStep));
            }
            if constexpr (LV > 0) {
                // each lane's 16 bytes land at the wave's base plus 16 x lane, i.e. at tail[k][thread]; lanes
                // past the end of the row write nothing
#pragma unroll
                for (int k = 0; k < LV; ++k) {
                    const int j = threadIdx.x + (VPL + k) * THREADS;
                    if (j < nvec)
                        __builtin_amdgcn_global_load_lds(
                            (const __attribute__((address_space(1))) void *)at_bytes(src, first + (VPL + k) * kStep),
                            (__attribute__((address_space(3))) void *)(tail + k * THREADS + (threadIdx.x & ~63u)), 16, 0, 0);
                }
            }
#pragma unroll
            for (int k = 0; k < VPL; ++k) Io<IO>::unpack(loaded[k], v[k]);
        }
        const float x0 = Io<IO>::scalar(src);
        wave::Welford w{0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = threadIdx.x + k * THREADS;
#pragma unroll
            for (int e = 0; e < E; ++e) v[k][e] -= x0;
            if (j < nvec) {
#pragma unroll
                for (int e = 0; e < E; ++e) welford_update(w, v[k][e], rcp.v[E * k + e + 1]);
            }
        }
        // (the loops over the tail are kept rolled: unrolled, the compiler fetches all of it from LDS at once and spills)
#pragma unroll 1
        for (int k = 0; k < LV; ++k) {
            if (static_cast<int>(threadIdx.x) + (VPL + k) * THREADS < nvec) {
                float x[E];
                Io<IO>::unpack(tail[k * THREADS + threadIdx.x], x);
#pragma unroll
                for (int e = 0; e < E; ++e) welford_update_counted(w, x[e] - x0);
            }
        }
        if constexpr (REST) {
            // cached loads here: the second read of these vectors may still find them in L2
            for (int j0 = kCached + threadIdx.x; j0 < nvec; j0 += THREADS * UNROLL) {
                float x[UNROLL][E];
                Raw loaded[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    loaded[u] = Raw{};
                    if (j0 + u * THREADS < nvec) loaded[u] = Io<IO>::template load_raw<false>(src + E * (j0 + u * THREADS));
                }
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) Io<IO>::unpack(loaded[u], x[u]);
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    if (j0 + u * THREADS >= nvec) break;
#pragma unroll
                    for (int e = 0; e < E; ++e) welford_update_counted(w, x[u][e] - x0);
                }
            }
        }
        w = block_welford_allreduce<THREADS>(w, lds);
        const float mean = w.mean;  // of the shifted row
        const float rstd = rsqrt_1ulp(w.m2 * inv_denominator + eps);
        typename Io<IO>::elem *dst = out + row * cols;
        if constexpr (REST) {
            // the streamed part first and from the row's end backwards: what was read last is the likeliest to be
            // in a cache still
            const int rest = nvec - kCached;
            const int trips = rest > 0 ? (rest + THREADS * UNROLL - 1) / (THREADS * UNROLL) : 0;
            for (int t = trips - 1; t >= 0; --t) {
                const int j0 = kCached + threadIdx.x + t * (THREADS * UNROLL);
                float x[UNROLL][E];
                Raw loaded[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    loaded[u] = Raw{};
                    if (j0 + u * THREADS < nvec) loaded[u] = Io<IO>::template load_raw<true>(src + E * (j0 + u * THREADS));
                }
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) Io<IO>::unpack(loaded[u], x[u]);
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const int j = j0 + u * THREADS;
                    if (j >= nvec) break;
                    float y[E];
#pragma unroll
                    for (int e = 0; e < E; ++e) x[u][e] -= x0;
                    normalize_vec<IO>(x[u], mean, rstd, gamma, beta, E * j, y);
                    store_row_vec<IO>(whole_lines, dst, Io<IO>::kBytes * j, y);
                }
            }
        }
#pragma unroll 1
        for (int k = 0; k < LV; ++k) {
            const int j = threadIdx.x + (VPL + k) * THREADS;
            if (j < nvec) {
                float x[E], y[E];
                Io<IO>::unpack(tail[k * THREADS + threadIdx.x], x);
#pragma unroll
                for (int e = 0; e < E; ++e) x[e] -= x0;
                normalize_vec<IO>(x, mean, rstd, gamma, beta, E * j, y);
                store_row_vec<IO>(whole_lines, dst, first + (VPL + k) * kStep, y);
            }
        }
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = threadIdx.x + k * THREADS;
            if (j < nvec) {
                float y[E];
                if constexpr (HOIST) {
#pragma unroll
                    for (int e = 0; e < E; ++e) y[e] = __builtin_fmaf((v[k][e] - mean) * rstd, g[k][e], b[k][e]);
                } else {
                    float gk[E], bk[E];
                    if (gamma) Io<IO>::template load<false>(at_bytes(gamma, first + k * kStep), gk);
                    if (beta) Io<IO>::template load<false>(at_bytes(beta, first + k * kStep), bk);
#pragma unroll
                    for (int e = 0; e < E; ++e) {
                        float t = (v[k][e] - mean) * rstd;
                        if (gamma) t *= gk[e];
                        if (beta) t += bk[e];
                        y[e] = t;
                    }
                }
                store_row_vec<IO>(whole_lines, dst, first + k * kStep, y);
            }
        }
        if (threadIdx.x == 0) {
            if (mean_out) mean_out[row] = rstd != rstd ? rstd : x0 + mean;  // no statistics for a row with NaN or inf
            if (rstd_out) rstd_out[row] = rstd;
        }
    }
}

// ------------------------------------------------------- BLOCK_NOCACHE policy
template <int IO, int THREADS>
__global__ __launch_bounds__(THREADS) void layernorm_nocache_kernel(const typename Io<IO>::elem *in,
                                                                    typename Io<IO>::elem *out,
                                                                    float *__restrict__ mean_out,
                                                                    float *__restrict__ rstd_out,
                                                                    const typename Io<IO>::elem *__restrict__ gamma,
                                                                    const typename Io<IO>::elem *__restrict__ beta,
                                                                    int64_t rows, int cols, float eps,
                                                                    float inv_denominator) {
    constexpr int E = Io<IO>::E;
    __shared__ float lds[48];
    const int nvec = cols / E;
    const bool whole_lines = rows_are_whole_lines<IO>(cols);
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const typename Io<IO>::elem *src = in + row * cols;
        const float x0 = Io<IO>::scalar(src);
        wave::Welford w{0.0f, 0.0f, 0.0f};
        // UNROLL vectors per thread and trip: their loads are issued together, so that a workgroup keeps
        // enough bytes in flight to cover the memory latency (one vector per trip leaves the pipe half empty)
        constexpr int UNROLL = 4;
        for (int j0 = threadIdx.x; j0 < nvec; j0 += THREADS * UNROLL) {
            float x[UNROLL][E];
            typename Io<IO>::raw loaded[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                loaded[u] = typename Io<IO>::raw{};
                if (j0 + u * THREADS < nvec) loaded[u] = Io<IO>::template load_raw<false>(src + E * (j0 + u * THREADS));
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) Io<IO>::unpack(loaded[u], x[u]);
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                if (j0 + u * THREADS >= nvec) break;
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    // streaming update; the count is not a compile-time constant here, and 1/count comes from
                    // the hardware reciprocal (1 ulp): M2 is accumulated against the mean actually formed, so
                    // the triplet stays consistent and the deviation is far inside the 1e-5 gate
                    const float xe = x[u][e] - x0;
                    w.count += 1.0f;
                    const float d = xe - w.mean;
                    w.mean = __builtin_fmaf(d, __builtin_amdgcn_rcpf(w.count), w.mean);
                    w.m2 = __builtin_fmaf(d, xe - w.mean, w.m2);
                }
            }
        }
        w = block_welford_allreduce<THREADS>(w, lds);
        const float mean = w.mean;  // of the shifted row
        const float rstd = rsqrt_1ulp(w.m2 * inv_denominator + eps);
        typename Io<IO>::elem *dst = out + row * cols;
        // Second pass from the row's end backwards (what the first pass read last is the likeliest to be in a
        // cache still), with nontemporal accesses: nothing is touched again.
        const int trips = (nvec + THREADS * UNROLL - 1) / (THREADS * UNROLL);
        for (int t = trips - 1; t >= 0; --t) {
            const int j0 = threadIdx.x + t * (THREADS * UNROLL);
            float x[UNROLL][E];
            typename Io<IO>::raw loaded[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                loaded[u] = typename Io<IO>::raw{};
                if (j0 + u * THREADS < nvec) loaded[u] = Io<IO>::template load_raw<true>(src + E * (j0 + u * THREADS));
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) Io<IO>::unpack(loaded[u], x[u]);
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int j = j0 + u * THREADS;
                if (j >= nvec) break;
                float y[E];
#pragma unroll
                for (int e = 0; e < E; ++e) x[u][e] -= x0;
                normalize_vec<IO>(x[u], mean, rstd, gamma, beta, E * j, y);
                store_row_vec<IO>(whole_lines, dst, Io<IO>::kBytes * j, y);
            }
        }
        if (threadIdx.x == 0) {
            if (mean_out) mean_out[row] = rstd != rstd ? rstd : x0 + mean;  // no statistics for a row with NaN or inf
            if (rstd_out) rstd_out[row] = rstd;
        }
    }
}

// ------------------------------------------- few rows: a row split over workgroups
// With fewer rows than compute units one workgroup per row leaves most of the chip idle.  Such rows are cut into
// `parts` pieces of `piece` vectors each, one workgroup per piece, in two launches with nothing but the kernel
// boundary between them: the first leaves every piece's Welford triplet (of x - x0, x0 the row's first element)
// in a workspace, the second merges a row's triplets - in piece order, every workgroup the same way, so the result
// is the same bits from call to call - and writes its piece of the output, reading the piece a second time.
// blockIdx.x = piece, blockIdx.y = row.
template <int IO, int THREADS>
__global__ __launch_bounds__(THREADS) void layernorm_pieces_stats_kernel(const typename Io<IO>::elem *in, int cols,
                                                                         int piece, wave::Welford *__restrict__ triplets) {
    constexpr int E = Io<IO>::E;
    constexpr int UNROLL = 4;
    __shared__ float lds[48];
    const int nvec = cols / E;
    const int64_t row = blockIdx.y;
    const int lo = static_cast<int>(blockIdx.x) * piece;
    const int hi = lo + piece < nvec ? lo + piece : nvec;
    const typename Io<IO>::elem *src = in + row * cols;
    const float x0 = Io<IO>::scalar(src);
    wave::Welford w{0.0f, 0.0f, 0.0f};
    for (int j0 = lo + threadIdx.x; j0 < hi; j0 += THREADS * UNROLL) {
        float x[UNROLL][E];
        typename Io<IO>::raw loaded[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            loaded[u] = typename Io<IO>::raw{};
            if (j0 + u * THREADS < hi) loaded[u] = Io<IO>::template load_raw<false>(src + E * (j0 + u * THREADS));
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) Io<IO>::unpack(loaded[u], x[u]);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (j0 + u * THREADS >= hi) break;
#pragma unroll
            for (int e = 0; e < E; ++e) welford_update_counted(w, x[u][e] - x0);
        }
    }
    w = block_welford_allreduce<THREADS>(w, lds);
    if (threadIdx.x == 0) {
        triplets[row * gridDim.x + blockIdx.x] = w;
        // x0 goes along (behind all the triplets): in place, the second launch finds the row's first element
        // overwritten by whichever workgroup got to piece 0 first
        if (blockIdx.x == 0) reinterpret_cast<float *>(triplets + static_cast<int64_t>(gridDim.y) * gridDim.x)[row] = x0;
    }
}

template <int IO, int THREADS>
__global__ __launch_bounds__(THREADS) void layernorm_pieces_apply_kernel(const typename Io<IO>::elem *in,
                                                                         typename Io<IO>::elem *out,
                                                                         float *__restrict__ mean_out,
                                                                         float *__restrict__ rstd_out,
                                                                         const typename Io<IO>::elem *__restrict__ gamma,
                                                                         const typename Io<IO>::elem *__restrict__ beta,
                                                                         int cols, float eps, float inv_denominator, int piece,
                                                                         const wave::Welford *__restrict__ triplets) {
    constexpr int E = Io<IO>::E;
    constexpr int UNROLL = 4;
    const int nvec = cols / E;
    const int64_t row = blockIdx.y;
    const int parts = static_cast<int>(gridDim.x);
    const int lo = static_cast<int>(blockIdx.x) * piece;
    const int hi = lo + piece < nvec ? lo + piece : nvec;
    const typename Io<IO>::elem *src = in + row * cols;
    const float x0 = reinterpret_cast<const float *>(triplets + static_cast<int64_t>(gridDim.y) * parts)[row];
    // the row's triplet from its pieces', merged in piece order (wave-uniform loads)
    const wave::Welford *mine = triplets + row * parts;
    wave::Welford w = mine[0];
    for (int i = 1; i < parts; ++i) w = wave::welford_merge(w, mine[i]);
    const float mean = w.mean;  // of the shifted row
    const float rstd = rsqrt_1ulp(w.m2 * inv_denominator + eps);
    typename Io<IO>::elem *dst = out + row * cols;
    const bool whole_lines = rows_are_whole_lines<IO>(cols);
    for (int j0 = lo + threadIdx.x; j0 < hi; j0 += THREADS * UNROLL) {
        float x[UNROLL][E];
        typename Io<IO>::raw loaded[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            loaded[u] = typename Io<IO>::raw{};
            if (j0 + u * THREADS < hi) loaded[u] = Io<IO>::template load_raw<true>(src + E * (j0 + u * THREADS));
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) Io<IO>::unpack(loaded[u], x[u]);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int j = j0 + u * THREADS;
            if (j >= hi) break;
            float y[E];
#pragma unroll
            for (int e = 0; e < E; ++e) x[u][e] -= x0;
            normalize_vec<IO>(x[u], mean, rstd, gamma, beta, E * j, y);
            store_row_vec<IO>(whole_lines, dst, Io<IO>::kBytes * j, y);
        }
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        if (mean_out) mean_out[row] = rstd != rstd ? rstd : x0 + mean;  // no statistics for a row with NaN or inf
        if (rstd_out) rstd_out[row] = rstd;
    }
}

// Rows of a few vectors per thread (up to 2048 vectors: 8192 fp32 columns): one workgroup per group of R rows,
// dispatched in row order and gone when its rows are written (a one-shot launch keeps the memory system busier
// than a grid that walks the rows in step: [32768, 4096] without gamma and beta 181 -> 165 us, the time of the
// softmax on the same rows).  gamma and beta have to be fetched by every workgroup, from L2: with R rows held in
// registers at once they are fetched once per R rows, and the R triplets share the barrier of the
// workgroup-wide all-reduce ([52428, 2560]: walking grid 194 us, one row per workgroup 189 us, two 174 us).
template <int IO, int THREADS, int VPL, int R>
__global__ __launch_bounds__(THREADS) void layernorm_block_batch_kernel(const typename Io<IO>::elem *in,
                                                                        typename Io<IO>::elem *out,
                                                                        float *__restrict__ mean_out,
                                                                        float *__restrict__ rstd_out,
                                                                        const typename Io<IO>::elem *__restrict__ gamma,
                                                                        const typename Io<IO>::elem *__restrict__ beta,
                                                                        int64_t rows, int cols, float eps,
                                                                        float inv_denominator) {
    constexpr int E = Io<IO>::E;
    constexpr int WAVES = THREADS / 64;
    typedef typename Io<IO>::raw Raw;
    __shared__ float lds[R * 3 * 16];
    constexpr Reciprocals<VPL * E> rcp;
    const int nvec = cols / E;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * R;
    const uint32_t first = threadIdx.x * 16u;
    constexpr uint32_t kStep = THREADS * 16u;
    const bool whole_lines = rows_are_whole_lines<IO>(cols);

    Raw loaded[R][VPL];  // all loads first, conversions afterwards
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const typename Io<IO>::elem *src = in + (row0 + r) * cols;
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = threadIdx.x + k * THREADS;
            loaded[r][k] = Raw{};
            if (row0 + r < rows && j < nvec) loaded[r][k] = Io<IO>::template load_raw<true>(at_bytes(src, first + k * kStep));
        }
    }
    float x0[R];
#pragma unroll
    for (int r = 0; r < R; ++r) x0[r] = row0 + r < rows ? Io<IO>::scalar(in + (row0 + r) * cols) : 0.0f;
    // gamma and beta behind the rows: memory returns in order, and the statistics do not need them
    float g[VPL][E], b[VPL][E];
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
        const int j = threadIdx.x + k * THREADS;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            g[k][e] = 1.0f;
            b[k][e] = 0.0f;
        }
        if (j < nvec) {
            if (gamma) Io<IO>::template load<false>(gamma + E * j, g[k]);
            if (beta) Io<IO>::template load<false>(beta + E * j, b[k]);
        }
    }

    float v[R][VPL][E];
    wave::Welford w[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        w[r] = wave::Welford{0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = threadIdx.x + k * THREADS;
            Io<IO>::unpack(loaded[r][k], v[r][k]);
#pragma unroll
            for (int e = 0; e < E; ++e) v[r][k][e] -= x0[r];
            if (j < nvec) {  // a thread's valid vectors are its first ones, so the n-th element it folds has count n
#pragma unroll
                for (int e = 0; e < E; ++e) welford_update(w[r], v[r][k][e], rcp.v[E * k + e + 1]);
            }
        }
        w[r] = wave::welford_allreduce<64>(w[r]);
    }
    if constexpr (WAVES > 1) {
        if ((threadIdx.x & 63) == 0) {
            const int wv = threadIdx.x >> 6;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                lds[(3 * r + 0) * 16 + wv] = w[r].count;
                lds[(3 * r + 1) * 16 + wv] = w[r].mean;
                lds[(3 * r + 2) * 16 + wv] = w[r].m2;
            }
        }
        __syncthreads();
        const int i = threadIdx.x & (WAVES - 1);
#pragma unroll
        for (int r = 0; r < R; ++r)
            w[r] = wave::welford_allreduce<WAVES>(
                wave::Welford{lds[(3 * r + 0) * 16 + i], lds[(3 * r + 1) * 16 + i], lds[(3 * r + 2) * 16 + i]});
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t row = row0 + r;
        if (row >= rows) break;
        const float mean = w[r].mean;  // of the shifted row
        const float rstd = rsqrt_1ulp(w[r].m2 * inv_denominator + eps);
        typename Io<IO>::elem *dst = out + row * cols;
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = threadIdx.x + k * THREADS;
            if (j < nvec) {
                float y[E];
#pragma unroll
                for (int e = 0; e < E; ++e) y[e] = __builtin_fmaf((v[r][k][e] - mean) * rstd, g[k][e], b[k][e]);
                store_row_vec<IO>(whole_lines, dst, first + k * kStep, y);
            }
        }
        if (threadIdx.x == 0) {
            if (mean_out) mean_out[row] = rstd != rstd ? rstd : x0[r] + mean;  // no statistics for a row with NaN or inf
            if (rstd_out) rstd_out[row] = rstd;
        }
    }
}

// ------------------------------------------------------------------ dispatch
template <int IO, int LPR, int VPL, bool FULL>
int launch_wave_full(const Args<IO> &a) {
    constexpr int RPW = 64 / LPR;
    // Single-wavefront workgroups by default (measured slightly faster than 256 threads).
    int threads = tuning(knob_layernorm_wave_threads);
    if (threads != 128 && threads != 256) threads = 64;
    const int64_t rows_per_block = static_cast<int64_t>(RPW) * (threads / 64);
    const int64_t needed = (a.rows + rows_per_block - 1) / rows_per_block;
    // One row group per wavefront by default; a positive knob caps the grid (grid-stride loop) instead.
    int64_t grid = needed;
    const int per_cu = tuning(knob_layernorm_blocks_per_cu);
    if (per_cu > 0 && grid > static_cast<int64_t>(compute_units()) * per_cu)
        grid = static_cast<int64_t>(compute_units()) * per_cu;
    if (grid > 0x7fffffff) grid = 0x7fffffff;
    // Residency cap (see lds_pad_for_residency).  The statistics keep a wavefront busy for a while after its
    // loads have landed, so more bytes' worth of wavefronts are kept resident than for softmax: 72 KB
    // ([16384, 768]: 24 wavefronts per CU 18.7 us, 32 19.2 us, 16 19.0 us, 12 20.0 us).  Knob: bytes, or -1.
    int lds = tuning(knob_layernorm_wave_lds);
    if (lds == 0 && threads == 64)
        lds = lds_pad_for_residency(static_cast<int64_t>(RPW) * a.cols * sizeof(typename Io<IO>::elem), 72 * 1024);
    if (lds < 0) lds = 0;
    if constexpr (FULL && LPR == 64 && sizeof(typename Io<IO>::raw) == 16 && VPL >= 2) {
        // gamma and beta through LDS, four rows per workgroup: from two vectors per lane on, where fetching them per
        // wavefront is a third or more of its L1 traffic.  Knob layernorm.affine_lds: 1 never, 2 whenever the shape allows.
        const int knob = tuning(knob_layernorm_affine_lds);
        if ((a.gamma || a.beta) && knob != 1 && a.rows % 4 == 0 && per_cu <= 0 &&
            (knob == 2 || tuning(knob_layernorm_wave_threads) == 0)) {
            const int64_t wgrid = a.rows / 4;
            if (wgrid <= 0x7fffffff) {
                const int need = 2 * (a.cols / Io<IO>::E) * 16;
                // Residency cap (see lds_pad_for_residency): workgroups of four rows, about 56 KB of rows in flight per
                // compute unit but never fewer than three workgroups.  Interleaved runs, workgroups per CU 8 / 6 / 5 / 4 / 3,
                // us: [16384, 768] 18.7 / 18.5 / 18.3 / 18.2 / 19.2 (gamma and beta per wavefront: 18.7), [262144, 768]
                // 258 / 257 / 254 / 254 / 257 (265), [196608, 1024] 259 / 259 / 253 / 253 / 253 (260), [65536, 1536]
                // 130 / 130 / 130 / 130 / 127 (138), [32768, 512] 23.4 / 23.1 / 23.8 / 23.8 / 25.8 (23.5).
                // Knob layernorm.wave_lds: bytes per workgroup, or -1 for no cap.
                const int64_t wg_bytes = 4 * static_cast<int64_t>(a.cols) * sizeof(typename Io<IO>::elem);
                int64_t wgs = (56 * 1024 + wg_bytes / 2) / wg_bytes;
                wgs = wgs < 3 ? 3 : (wgs > 8 ? 8 : wgs);
                // (a KB short of an even share of the 160 KB, so that the count fits whatever the allocation rounds to)
                int pad = wgs >= 8 ? 0 : static_cast<int>((160 * 1024 / wgs - 1024) & ~int64_t{511});
                if (tuning(knob_layernorm_wave_lds) != 0) pad = tuning(knob_layernorm_wave_lds) > 0 ? tuning(knob_layernorm_wave_lds) : 0;
                layernorm_wave_kernel<IO, LPR, VPL, FULL, true, true>
                    <<<dim3(static_cast<unsigned>(wgrid)), dim3(256), static_cast<size_t>(pad > need ? pad : need), a.stream>>>(
                        a.in, a.out, a.mean, a.rstd, a.gamma, a.beta, a.rows, a.cols, a.eps, a.inv_denominator);
                KO_CHECK_LAUNCH();
                return KO_OK;
            }
        }
    }
    if (a.gamma || a.beta)
        layernorm_wave_kernel<IO, LPR, VPL, FULL, true><<<dim3(static_cast<unsigned>(grid)), dim3(threads), lds, a.stream>>>(
            a.in, a.out, a.mean, a.rstd, a.gamma, a.beta, a.rows, a.cols, a.eps, a.inv_denominator);
    else
        layernorm_wave_kernel<IO, LPR, VPL, FULL, false><<<dim3(static_cast<unsigned>(grid)), dim3(threads), lds, a.stream>>>(
            a.in, a.out, a.mean, a.rstd, a.gamma, a.beta, a.rows, a.cols, a.eps, a.inv_denominator);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <int IO, int LPR, int VPL>
int launch_wave(const Args<IO> &a) {
    // One row group per wavefront: batches of 2 and 4 row groups per wave (gamma and beta fetched once per
    // batch, the next group's loads issued before the current one is reduced) measured 5-8 % slower on
    // MI355X at [16384, 768] - the hardware keeps more independent waves in flight than a batch keeps loads.
    if (a.cols == LPR * VPL * Io<IO>::E) return launch_wave_full<IO, LPR, VPL, true>(a);
    return launch_wave_full<IO, LPR, VPL, false>(a);
}

template <int IO, int LPR>
int launch_wave_vpl(const Args<IO> &a, int vpl) {
    switch (vpl) {
        case 1: return launch_wave<IO, LPR, 1>(a);
        case 2: return launch_wave<IO, LPR, 2>(a);
        case 3: return launch_wave<IO, LPR, 3>(a);
        case 4: return launch_wave<IO, LPR, 4>(a);
        case 5:
        case 6: return launch_wave<IO, LPR, 6>(a);
        default: return launch_wave<IO, LPR, 8>(a);
    }
}

template <int IO>
int launch_wave_lpr(const Args<IO> &a, int lpr) {
    const int nvec = a.cols / Io<IO>::E;
    const int vpl = (nvec + lpr - 1) / lpr;
    // rows of one to four vectors: 1, 2 or 4 lanes per row with one vector each, 16 to 64 rows per wavefront, one
    // load of which still covers a contiguous stretch of memory
    if (vpl == 1 && lpr == 1) return launch_wave<IO, 1, 1>(a);
    if (vpl == 1 && lpr == 2) return launch_wave<IO, 2, 1>(a);
    if (vpl == 1 && lpr == 4) return launch_wave<IO, 4, 1>(a);
    switch (lpr) {
        case 8: return launch_wave_vpl<IO, 8>(a, vpl);
        case 16: return launch_wave_vpl<IO, 16>(a, vpl);
        case 32: return launch_wave_vpl<IO, 32>(a, vpl);
        default: return launch_wave_vpl<IO, 64>(a, vpl);
    }
}

// Longest row per policy, in 16-byte vectors: 512 per wavefront (2048 fp32 or 4096 16-bit columns); per
// workgroup 80 values per thread of 1024 threads (81920 columns).
constexpr int kWaveMaxVpl = 8;
constexpr int kWaveMaxVecs = 64 * kWaveMaxVpl;
constexpr int kTailMaxVecs = 9;  // 16-byte vectors per thread of a 1024-thread workgroup kept in LDS (9 x 16 KB)
template <int IO>
constexpr int kBlockMaxVecs = 1024 * (80 / Io<IO>::E);  // in registers; BLOCK takes longer rows too (LDS, then streaming)

// Lanes per row for the WARP policy.  A group of LPR lanes holds a row in VPL vectors per lane, VPL from
// {1, 2, 3, 4, 6, 8}; the choice wastes the fewest vector slots (idle lanes still cost issue cycles
// and a wavefront's worth of latency), and among equals takes the widest group: one load instruction
// of the group then covers the longest contiguous piece of the row.
int default_lanes_per_row(int nvec) {
    int best = 64, best_waste = 1 << 30;
    for (int lpr = 1; lpr <= 64; lpr <<= 1) {  // (groups of 1, 2 and 4 lanes: one vector per lane)
        int vpl = (nvec + lpr - 1) / lpr;
        if (vpl > (lpr < 8 ? 1 : 8)) continue;
        if (vpl == 5) vpl = 6;
        if (vpl == 7) vpl = 8;
        const int waste = lpr * vpl - nvec;
        if (waste <= best_waste) {
            best_waste = waste;
            best = lpr;
        }
    }
    return best;
}

template <int IO>
int launch_wave_any(const Args<IO> &a) {
    const int nvec = a.cols / Io<IO>::E;
    int lpr = tuning(knob_layernorm_lanes_per_row);
    if (lpr != 8 && lpr != 16 && lpr != 32 && lpr != 64) lpr = default_lanes_per_row(nvec);
    while (lpr < 64 && (nvec + lpr - 1) / lpr > (lpr < 8 ? 1 : kWaveMaxVpl)) lpr <<= 1;
    return launch_wave_lpr<IO>(a, lpr);
}

template <int IO, int THREADS>
int launch_block_threads(const Args<IO> &a) {
    const int nvec = a.cols / Io<IO>::E;
    const int vpl = (nvec + THREADS - 1) / THREADS;
    int64_t grid = static_cast<int64_t>(compute_units()) * (2048 / THREADS) * 2;
    if (tuning(knob_rows_block_grid) == 1) grid = a.rows;  // one workgroup per row
    if (grid > a.rows) grid = a.rows;
    if (grid > 0x7fffffff) grid = 0x7fffffff;
    dim3 g(static_cast<unsigned>(grid)), b(THREADS);
#define KO_LN_BLOCK(V)                                                                                 \
    layernorm_block_kernel<IO, THREADS, V><<<g, b, 0, a.stream>>>(a.in, a.out, a.mean, a.rstd, a.gamma, \
                                                                  a.beta, a.rows, a.cols, a.eps,        \
                                                                  a.inv_denominator)
    if (vpl <= 1) KO_LN_BLOCK(1);
    else if (vpl <= 2) KO_LN_BLOCK(2);
    else if (vpl <= 4) KO_LN_BLOCK(4);
    else if (vpl <= 8) KO_LN_BLOCK(8);
    else if constexpr (THREADS == 1024) {
        // a single resident workgroup of 1024 threads has 128 registers per thread: up to 80 hold the row
        constexpr int kRegs = 80 / Io<IO>::E;  // vectors per thread held in registers
        if constexpr (Io<IO>::E == 4) {
            if (vpl <= 12) KO_LN_BLOCK(12);
            else if (vpl <= 16) KO_LN_BLOCK(16);
            else if (vpl <= 20) KO_LN_BLOCK(20);
        } else if (vpl <= 10) {
            KO_LN_BLOCK(10);
        }
        if (vpl > kRegs) {
            // longer rows: nine more vectors per thread in LDS (9 x 16 KB), the rest of the row streamed twice
            constexpr int kRegsTail = Io<IO>::E == 4 ? 20 : 8;  // 16-bit storage: 64 values, the conversions need registers too
            auto kernel = layernorm_block_kernel<IO, THREADS, kRegsTail, kTailMaxVecs, true>;
            static std::atomic<uint64_t> done{0};
            if (const int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), 160 * 1024 - 256, done); rc != KO_OK)
                return rc;
            kernel<<<g, b, static_cast<size_t>(kTailMaxVecs) * THREADS * 16, a.stream>>>(
                a.in, a.out, a.mean, a.rstd, a.gamma, a.beta, a.rows, a.cols, a.eps, a.inv_denominator);
        }
    }
#undef KO_LN_BLOCK
    KO_CHECK_LAUNCH();
    return KO_OK;
}

// Rows of 513 to 2048 vectors: layernorm_block_batch_kernel with 512 threads, one row per workgroup without
// gamma and beta, two rows with them.
template <int IO>
int launch_block_batch(const Args<IO> &a) {
    const int nvec = a.cols / Io<IO>::E;
    const int vpl = (nvec + 511) / 512;
    int r = tuning(knob_layernorm_block_rows);
    if (r != 1 && r != 2) r = a.gamma != nullptr || a.beta != nullptr ? 2 : 1;
    const int64_t grid = (a.rows + r - 1) / r;
    if (grid > 0x7fffffff) return fail(KO_ERR_UNSUPPORTED_SHAPE, "layernorm: too many rows");
    const dim3 g(static_cast<unsigned>(grid)), b(512);
#define KO_LN_BATCH(V)                                                                                          \
    do {                                                                                                        \
        if (r == 1)                                                                                             \
            layernorm_block_batch_kernel<IO, 512, V, 1><<<g, b, 0, a.stream>>>(a.in, a.out, a.mean, a.rstd, a.gamma, \
                                                                              a.beta, a.rows, a.cols, a.eps,   \
                                                                              a.inv_denominator);              \
        else                                                                                                    \
            layernorm_block_batch_kernel<IO, 512, V, 2><<<g, b, 0, a.stream>>>(a.in, a.out, a.mean, a.rstd, a.gamma, \
                                                                              a.beta, a.rows, a.cols, a.eps,   \
                                                                              a.inv_denominator);              \
    } while (0)
    if (vpl <= 2) KO_LN_BATCH(2);
    else if (vpl <= 3) KO_LN_BATCH(3);
    else KO_LN_BATCH(4);
#undef KO_LN_BATCH
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <int IO>
int launch_block(const Args<IO> &a) {
    const int nvec = a.cols / Io<IO>::E;
    int threads = tuning(knob_layernorm_block_threads);
    // Rows of 513 to 2048 vectors (2052 to 8192 fp32 columns) as a one-shot launch: without gamma and beta one row
    // per workgroup; with them two rows per workgroup, which share their fetch - unless rows lie a multiple of
    // 8 KB apart: two rows, gamma and beta then fall on the same memory channels at the same moment, and the
    // walking grid below, which keeps gamma and beta in registers, is the faster one ([32768, 4096]: 181 us
    // walking, 188 us two rows per workgroup; [43690, 3072]: 192 and 175 us; without gamma and beta 181 -> 165 us
    // and 191 -> 162 us).  Knob layernorm.block_rows: -1 walking grid always, 1 or 2 rows per workgroup.
    // 16-bit storage (eight values per vector: twice the arithmetic and twice the registers per byte) keeps the
    // walking grid, whose workgroups hold gamma and beta across rows ([32768, 5120] binary16: one-shot launch with
    // one or two rows per workgroup 186 and 169 us, walking grid of 256 threads 125 us), and grows the workgroup
    // to 512 threads from four vectors per thread on ([8192, 16384]: 256 threads 116 us, 512 threads 98 us).
    constexpr bool WIDE = Io<IO>::E > 4;
    if (nvec > 512 && nvec <= 2048 && threads == 0 && tuning(knob_rows_block_grid) == 0) {
        const int forced = tuning(knob_layernorm_block_rows);
        const bool affine = a.gamma != nullptr || a.beta != nullptr;
        const bool rows_on_one_channel = (static_cast<int64_t>(a.cols) * sizeof(typename Io<IO>::elem)) % 8192 == 0;
        if (forced == 1 || forced == 2 || (forced == 0 && !WIDE && (!affine || !rows_on_one_channel)))
            return launch_block_batch<IO>(a);
    }
    if (threads != 256 && threads != 512 && threads != 1024) {
        // up to eight vectors per thread before the workgroup grows: gamma and beta then still fit the registers
        // next to the row at 256 and 512 threads ([8192, 16384]: 512 threads 181 us, 1024 threads 186 us)
        threads = 256;
        if (WIDE && (nvec + threads - 1) / threads > 4) threads = 512;  // ([4096, 32768] binary16: 512 threads 117 us, 1024 threads 136 us)
        while (threads < 1024 && (nvec + threads - 1) / threads > 8) threads <<= 1;
    }
    while (threads < 1024 && (nvec + threads - 1) / threads > 8) threads <<= 1;
    if (threads == 256) return launch_block_threads<IO, 256>(a);
    if (threads == 512) return launch_block_threads<IO, 512>(a);
    return launch_block_threads<IO, 1024>(a);
}

template <int IO, int THREADS>
int launch_nocache_threads(const Args<IO> &a) {
    int64_t grid = static_cast<int64_t>(compute_units()) * (2048 / THREADS) * 2;
    if (tuning(knob_rows_block_grid) == 1) grid = a.rows;  // one workgroup per row
    if (grid > a.rows) grid = a.rows;
    if (grid > 0x7fffffff) grid = 0x7fffffff;
    layernorm_nocache_kernel<IO, THREADS><<<dim3(static_cast<unsigned>(grid)), dim3(THREADS), 0, a.stream>>>(
        a.in, a.out, a.mean, a.rstd, a.gamma, a.beta, a.rows, a.cols, a.eps, a.inv_denominator);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

// Workgroup size by row length: a thread should have several trips of four vectors to make.
template <int IO>
int launch_nocache(const Args<IO> &a) {
    const int nvec = a.cols / Io<IO>::E;
    if (nvec <= 2048) return launch_nocache_threads<IO, 256>(a);
    if (nvec <= 8192) return launch_nocache_threads<IO, 512>(a);
    return launch_nocache_threads<IO, 1024>(a);
}

// A row in the registers of one 1024-thread workgroup, element by element: 1024 * VPL columns, and with REST what
// lies beyond them streamed (read twice).
template <int IO, int VPL, bool REST>
int launch_block_by_element(const Args<IO> &a) {
    int64_t grid = static_cast<int64_t>(compute_units()) * 4;  // two workgroups per resident slot walk the rows
    if (grid > a.rows) grid = a.rows;
    layernorm_block_kernel<IO, 1024, VPL, 0, REST><<<dim3(static_cast<unsigned>(grid)), dim3(1024), 0, a.stream>>>(
        a.in, a.out, a.mean, a.rstd, a.gamma, a.beta, a.rows, a.cols, a.eps, a.inv_denominator);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

// Rows walked element by element (IO is one of the *_1 kinds): up to 2048 columns a row sits in the registers of
// 16 or 64 lanes (column j in lane j % lanes, slot j / lanes), up to 65536 in those of a workgroup, and is read
// once; of longer rows the far end is read twice.
// An explicit policy is honoured: WARP takes the wavefront kernels (up to 2048 columns here), BLOCK the workgroup
// kernel, BLOCK_NOCACHE the one that reads every row twice; AUTO the first that holds the row.
template <int IO>
int launch_by_element(const Args<IO> &a, int policy) {
    static_assert(Io<IO>::E == 1, "");
    const int cols = a.cols;
    if (policy == KO_POLICY_BLOCK_NOCACHE) return launch_nocache<IO>(a);
    if (policy == KO_POLICY_WARP && cols > 2048)
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "layernorm: WARP policy holds at most 2048 columns of a row walked "
                                              "element by element, got %d", cols);
    if (policy == KO_POLICY_BLOCK) {
        if (cols <= 4096) return launch_block_by_element<IO, 4, false>(a);
        if (cols <= 8192) return launch_block_by_element<IO, 8, false>(a);
        if (cols <= 16384) return launch_block_by_element<IO, 16, false>(a);
        if (cols <= 32768) return launch_block_by_element<IO, 32, false>(a);
        return launch_block_by_element<IO, 64, true>(a);
    }
    if (cols <= 1) return launch_wave_full<IO, 1, 1, false>(a);  // rows of a few columns: as many lanes as columns
    if (cols <= 2) return launch_wave_full<IO, 2, 1, false>(a);
    if (cols <= 4) return launch_wave_full<IO, 4, 1, false>(a);
    if (cols <= 8) return launch_wave_full<IO, 8, 1, false>(a);
    if (cols <= 16) return launch_wave_full<IO, 16, 1, false>(a);
    if (cols <= 32) return launch_wave_full<IO, 16, 2, false>(a);
    if (cols <= 64) return launch_wave_full<IO, 16, 4, false>(a);
    if (cols <= 128) return launch_wave_full<IO, 64, 2, false>(a);
    if (cols <= 256) return launch_wave_full<IO, 64, 4, false>(a);
    if (cols <= 512) return launch_wave_full<IO, 64, 8, false>(a);
    if (cols <= 1024) return launch_wave_full<IO, 64, 16, false>(a);
    if (cols <= 2048) return launch_wave_full<IO, 64, 32, false>(a);
    if (cols <= 4096) return launch_block_by_element<IO, 4, false>(a);
    if (cols <= 8192) return launch_block_by_element<IO, 8, false>(a);
    if (cols <= 16384) return launch_block_by_element<IO, 16, false>(a);
    if (cols <= 32768) return launch_block_by_element<IO, 32, false>(a);
    return launch_block_by_element<IO, 64, true>(a);  // (without REST this one spills; with it, it does not)
}

// Few long rows (see layernorm_pieces_stats_kernel).  Pieces of at least 1024 vectors (16 KB), two workgroups per
// compute unit in all.  Returns -1 when the
// shape is left to the one-workgroup-per-row kernels, or when the stream has no workspace to be had (inside a
// graph capture on a stream that never ran a call that needs one).
template <int IO>
int launch_pieces(const Args<IO> &a) {
    constexpr int THREADS = 256;
    const int nvec = a.cols / Io<IO>::E;
    const int cu = compute_units();
    // two launches have a fixed cost of some 10 us: it pays from rows of 256 KB on for up to a quarter of the
    // compute units' worth of rows ([64, 128256]: 29 -> 22 us, [32, 128256] 28 -> 14 us, [1, 16777216] 3.8 ms ->
    // 96 us; [64, 32768] 9 against 10 us), from rows of 1 MB on for up to half ([128, 524288]: 168 -> 149 us;
    // [128, 128256] 35 against 42 us)
    if (!((a.rows * 4 <= cu && nvec >= 16384) || (a.rows * 2 <= cu && nvec >= 65536))) return -1;
    int parts = static_cast<int>(2 * cu / a.rows);
    if (parts > nvec / 1024) parts = nvec / 1024;
    if (parts < 2) return -1;
    int piece = (nvec + parts - 1) / parts;
    piece = (piece + THREADS - 1) / THREADS * THREADS;  // whole trips of the workgroup; the last piece is the short one
    parts = (nvec + piece - 1) / piece;
    void *workspace = nullptr;
    if (const int st = stream_small_workspace(a.stream, &workspace); st != KO_OK) return st;
    if (workspace == nullptr || static_cast<size_t>(a.rows) * (parts * sizeof(wave::Welford) + sizeof(float)) > kStreamSmallWorkspaceBytes)
        return -1;
    wave::Welford *triplets = static_cast<wave::Welford *>(workspace);
    const dim3 grid(static_cast<unsigned>(parts), static_cast<unsigned>(a.rows));
    layernorm_pieces_stats_kernel<IO, THREADS><<<grid, dim3(THREADS), 0, a.stream>>>(a.in, a.cols, piece, triplets);
    KO_CHECK_LAUNCH();
    layernorm_pieces_apply_kernel<IO, THREADS><<<grid, dim3(THREADS), 0, a.stream>>>(
        a.in, a.out, a.mean, a.rstd, a.gamma, a.beta, a.cols, a.eps, a.inv_denominator, piece, triplets);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <int IO>
int entry(const void *in, void *out, float *mean, float *rstd, const void *gamma, const void *beta, int64_t rows,
          int64_t cols, float eps, int unbiased, int policy, ko_stream_t stream) {
    constexpr int E = Io<IO>::E;
    typedef typename Io<IO>::elem elem;
    if (rows < 0 || cols <= 0)
        return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: rows=%lld cols=%lld", (long long)rows, (long long)cols);
    if (cols > (1 << 30)) return fail(KO_ERR_UNSUPPORTED_SHAPE, "layernorm: cols=%lld too large", (long long)cols);
    if (rows == 0) return KO_OK;
    if (!in || !out) return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: null in/out pointer");
    const uintptr_t addresses = reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out) |
                                reinterpret_cast<uintptr_t>(gamma) | reinterpret_cast<uintptr_t>(beta);
    if (addresses & (sizeof(elem) - 1))
        return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: in/out/gamma/beta must be aligned to their element type");
    if ((reinterpret_cast<uintptr_t>(mean) | reinterpret_cast<uintptr_t>(rstd)) & 3)
        return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: mean/rstd must be 4-byte aligned");
    if (!(eps >= 0.0f)) return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: eps must be >= 0");
    const double denom = unbiased ? static_cast<double>(cols - 1) : static_cast<double>(cols);
    if (cols % E != 0 || (addresses & 15) != 0) {
        // Rows that do not start on 16-byte boundaries (the reference's descriptors with vec_len = 1 or 2, or
        // tensors that start off one): every policy walks such a row element by element (launch_by_element); the
        // WARP policy's row limit stays.
        constexpr int BY_ELEMENT = io_by_element(IO);
        if (policy != KO_POLICY_AUTO && policy != KO_POLICY_WARP && policy != KO_POLICY_BLOCK && policy != KO_POLICY_BLOCK_NOCACHE)
            return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: unknown policy %d", policy);
        if (policy == KO_POLICY_WARP && (cols + E - 1) / E > kWaveMaxVecs)
            return fail(KO_ERR_UNSUPPORTED_SHAPE, "layernorm: WARP policy holds at most %d columns per row, got %lld",
                        kWaveMaxVecs * E, (long long)cols);
        Args<BY_ELEMENT> a1{static_cast<const elem *>(in), static_cast<elem *>(out), mean, rstd,
                            static_cast<const elem *>(gamma), static_cast<const elem *>(beta), rows,
                            static_cast<int>(cols), eps, static_cast<float>(1.0 / denom), as_stream(stream)};
        return launch_by_element<BY_ELEMENT>(a1, policy);
    }
    Args<IO> a{static_cast<const elem *>(in), static_cast<elem *>(out), mean, rstd, static_cast<const elem *>(gamma),
               static_cast<const elem *>(beta), rows, static_cast<int>(cols), eps, static_cast<float>(1.0 / denom),
               as_stream(stream)};
    const int nvec = a.cols / E;
    if (policy == KO_POLICY_AUTO) {
        if (const int st = launch_pieces<IO>(a); st != -1) return st;
        policy = nvec <= kWaveMaxVecs ? KO_POLICY_WARP
                                      : KO_POLICY_BLOCK;  // rows past what the chip holds stream their far end twice
    }
    switch (policy) {
        case KO_POLICY_WARP:
            if (nvec > kWaveMaxVecs)
                return fail(KO_ERR_UNSUPPORTED_SHAPE,
                            "layernorm: WARP policy holds at most %d columns per row, got %d", kWaveMaxVecs * E, a.cols);
            return launch_wave_any<IO>(a);
        case KO_POLICY_BLOCK:
            return launch_block<IO>(a);
        case KO_POLICY_BLOCK_NOCACHE: return launch_nocache<IO>(a);
        default: return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: unknown policy %d", policy);
    }
}

}  // namespace
}  // namespace ko

KO_EXPORT int ko_layernorm_f32_policy(const float *in, float *out, float *mean, float *rstd,
                                      const float *gamma, const float *beta, int64_t rows,
                                      int64_t cols, float eps, int unbiased, int policy,
                                      ko_stream_t stream) {
    return ko::entry<ko::IO_F32>(in, out, mean, rstd, gamma, beta, rows, cols, eps, unbiased, policy, stream);
}

KO_EXPORT int ko_layernorm_f32(const float *in, float *out, float *mean, float *rstd,
                               const float *gamma, const float *beta, int64_t rows, int64_t cols,
                               float eps, int unbiased, ko_stream_t stream) {
    return ko_layernorm_f32_policy(in, out, mean, rstd, gamma, beta, rows, cols, eps, unbiased,
                                   KO_POLICY_AUTO, stream);
}

KO_EXPORT int ko_layernorm_16(const void *in, void *out, float *mean, float *rstd, const void *gamma,
                              const void *beta, int64_t rows, int64_t cols, float eps, int unbiased, int dtype,
                              int policy, ko_stream_t stream) {
    if (dtype == KO_F16)
        return ko::entry<ko::IO_F16>(in, out, mean, rstd, gamma, beta, rows, cols, eps, unbiased, policy, stream);
    if (dtype == KO_BF16)
        return ko::entry<ko::IO_BF16>(in, out, mean, rstd, gamma, beta, rows, cols, eps, unbiased, policy, stream);
    return ko::fail(KO_ERR_INVALID_ARGUMENT, "layernorm: dtype=%d is neither KO_F16 nor KO_BF16", dtype);
}
