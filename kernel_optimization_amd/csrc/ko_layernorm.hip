// LayerNorm over the last dimension for gfx950: one pass over HBM, fp32,
// Welford statistics, outputs y and (optionally) per-row mean and rstd.
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
// Mappings as in the reference: WARP (LayerNormWarpImpl :145-201) = row in the
// registers of LPR lanes of a wavefront; BLOCK (LayerNormBlockImpl :204-252) =
// row in the registers of a workgroup, per-wave triplets through LDS;
// BLOCK_NOCACHE (LayerNormBlockNoCacheImpl :254-300) = two reads of the row.
#include "ko_internal.h"
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

__device__ __forceinline__ void welford_update(wave::Welford &w, float x, float inv_count) {
    w.count += 1.0f;
    const float d = x - w.mean;
    w.mean = __builtin_fmaf(d, inv_count, w.mean);
    w.m2 = __builtin_fmaf(d, x - w.mean, w.m2);
}

struct Args {
    const float *in;
    float *out;
    float *mean;
    float *rstd;
    const float *gamma;
    const float *beta;
    int64_t rows;
    int cols;
    float eps;
    float inv_denominator;  // 1/N or 1/(N-1)
    hipStream_t stream;
};

// ---------------------------------------------------------------- WARP policy
// A wavefront takes BATCH consecutive row groups (a row group = 64 / LPR rows, one per lane
// group); the loads of group b + 1 are issued before group b is reduced and stored, so reads
// and writes of a wave overlap and gamma/beta are fetched once per BATCH groups.
template <int LPR, int VPL, bool NT, int BATCH>
__global__ __launch_bounds__(256) void layernorm_wave_kernel(const float *in,
                                                             float *out,
                                                             float *__restrict__ mean_out,
                                                             float *__restrict__ rstd_out,
                                                             const float *__restrict__ gamma,
                                                             const float *__restrict__ beta, int64_t rows,
                                                             int cols, float eps, float inv_denominator) {
    constexpr int RPW = 64 / LPR;
    constexpr Reciprocals<VPL * 4> rcp;
    const int lane = threadIdx.x & 63;
    const int sub = lane / LPR;
    const int l = lane % LPR;
    const int nvec = cols >> 2;
    const int64_t waves_per_block = blockDim.x >> 6;
    const int64_t wave = blockIdx.x * waves_per_block + (threadIdx.x >> 6);
    const int64_t stride = static_cast<int64_t>(gridDim.x) * waves_per_block * (RPW * BATCH);

    // gamma/beta of this lane's columns stay in registers across rows.
    float4v g[VPL], b[VPL];
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
        const int j = l + k * LPR;
        g[k] = float4v{1.0f, 1.0f, 1.0f, 1.0f};
        b[k] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
        if (j < nvec) {
            if (gamma) g[k] = load4<false>(gamma + 4 * j);
            if (beta) b[k] = load4<false>(beta + 4 * j);
        }
    }

    auto load_rows = [&](float4v (&v)[VPL], int64_t row) {
        const bool row_ok = row < rows;
        const float *src = in + row * cols;
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = l + k * LPR;
            if (row_ok && j < nvec) v[k] = load4<NT>(src + 4 * j);
            else v[k] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
        }
    };

    auto finish_rows = [&](float4v (&v)[VPL], int64_t row) {
        const bool row_ok = row < rows;
        const float x0 = wave::broadcast_group_first<LPR>(v[0][0]);
        wave::Welford w{0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = l + k * LPR;
            v[k] = v[k] - x0;
            if (j < nvec) {
#pragma unroll
                for (int e = 0; e < 4; ++e) welford_update(w, v[k][e], rcp.v[4 * k + e + 1]);
            }
        }
        w = wave::welford_allreduce<LPR>(w);

        const float mean = w.mean;  // of the shifted row
        const float rstd = 1.0f / sqrtf(w.m2 * inv_denominator + eps);

        float *dst = out + row * cols;
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = l + k * LPR;
            if (row_ok && j < nvec) {
                float4v y;
#pragma unroll
                for (int e = 0; e < 4; ++e) y[e] = __builtin_fmaf((v[k][e] - mean) * rstd, g[k][e], b[k][e]);
                store4<NT>(dst + 4 * j, y);
            }
        }
        if (row_ok && l == 0) {
            if (mean_out) mean_out[row] = x0 + mean;
            if (rstd_out) rstd_out[row] = rstd;
        }
    };

    for (int64_t row0 = wave * (RPW * BATCH); row0 < rows; row0 += stride) {
        float4v v[2][VPL];
        load_rows(v[0], row0 + sub);
#pragma unroll
        for (int bt = 0; bt < BATCH; ++bt) {
            if (bt + 1 < BATCH) load_rows(v[(bt + 1) & 1], row0 + (bt + 1) * RPW + sub);
            finish_rows(v[bt & 1], row0 + bt * RPW + sub);
        }
    }
}

// --------------------------------------------------------------- BLOCK policy
// Workgroup-wide Welford all-reduce: per-wave triplets through LDS, folded by
// every thread in the same order.
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
    wave::Welford r{lds[0], lds[16], lds[32]};
#pragma unroll
    for (int i = 1; i < WAVES; ++i) r = wave::welford_merge(r, wave::Welford{lds[i], lds[16 + i], lds[32 + i]});
    return r;
}

template <int THREADS, int VPL>
__global__ __launch_bounds__(THREADS) void layernorm_block_kernel(const float *in,
                                                                  float *out,
                                                                  float *__restrict__ mean_out,
                                                                  float *__restrict__ rstd_out,
                                                                  const float *__restrict__ gamma,
                                                                  const float *__restrict__ beta,
                                                                  int64_t rows, int cols, float eps,
                                                                  float inv_denominator) {
    __shared__ float lds[48];
    constexpr Reciprocals<VPL * 4> rcp;
    const int nvec = cols >> 2;
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const float *src = in + row * cols;
        float4v v[VPL];
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = threadIdx.x + k * THREADS;
            if (j < nvec) v[k] = load4<false>(src + 4 * j);
            else v[k] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
        }
        const float x0 = src[0];
        wave::Welford w{0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = threadIdx.x + k * THREADS;
            v[k] = v[k] - x0;
            if (j < nvec) {
#pragma unroll
                for (int e = 0; e < 4; ++e) welford_update(w, v[k][e], rcp.v[4 * k + e + 1]);
            }
        }
        w = block_welford_allreduce<THREADS>(w, lds);
        const float mean = w.mean;  // of the shifted row
        const float rstd = 1.0f / sqrtf(w.m2 * inv_denominator + eps);
        float *dst = out + row * cols;
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = threadIdx.x + k * THREADS;
            if (j < nvec) {
                float4v y;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float t = (v[k][e] - mean) * rstd;
                    if (gamma) t *= gamma[4 * j + e];
                    if (beta) t += beta[4 * j + e];
                    y[e] = t;
                }
                store4<false>(dst + 4 * j, y);
            }
        }
        if (threadIdx.x == 0) {
            if (mean_out) mean_out[row] = x0 + mean;
            if (rstd_out) rstd_out[row] = rstd;
        }
    }
}

// ------------------------------------------------------- BLOCK_NOCACHE policy
template <int THREADS>
__global__ __launch_bounds__(THREADS) void layernorm_nocache_kernel(const float *in,
                                                                    float *out,
                                                                    float *__restrict__ mean_out,
                                                                    float *__restrict__ rstd_out,
                                                                    const float *__restrict__ gamma,
                                                                    const float *__restrict__ beta,
                                                                    int64_t rows, int cols, float eps,
                                                                    float inv_denominator) {
    __shared__ float lds[48];
    const int nvec = cols >> 2;
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const float *src = in + row * cols;
        const float x0 = src[0];
        wave::Welford w{0.0f, 0.0f, 0.0f};
        for (int j = threadIdx.x; j < nvec; j += THREADS) {
            float4v x = load4<false>(src + 4 * j) - x0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // streaming update with a true division: the count is not a compile-time constant here
                w.count += 1.0f;
                const float d = x[e] - w.mean;
                w.mean += d / w.count;
                w.m2 = __builtin_fmaf(d, x[e] - w.mean, w.m2);
            }
        }
        w = block_welford_allreduce<THREADS>(w, lds);
        const float mean = w.mean;  // of the shifted row
        const float rstd = 1.0f / sqrtf(w.m2 * inv_denominator + eps);
        float *dst = out + row * cols;
        for (int j = threadIdx.x; j < nvec; j += THREADS) {
            float4v x = load4<false>(src + 4 * j) - x0;
            float4v y;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float t = (x[e] - mean) * rstd;
                if (gamma) t *= gamma[4 * j + e];
                if (beta) t += beta[4 * j + e];
                y[e] = t;
            }
            store4<false>(dst + 4 * j, y);
        }
        if (threadIdx.x == 0) {
            if (mean_out) mean_out[row] = x0 + mean;
            if (rstd_out) rstd_out[row] = rstd;
        }
    }
}

// ------------------------------------------------------------------ dispatch
template <int LPR, int VPL, bool NT, int BATCH>
int launch_wave_batch(const Args &a) {
    constexpr int RPW = 64 / LPR;
    // Single-wavefront workgroups by default (measured slightly faster than 256 threads).
    int threads = tuning("layernorm.wave_threads");
    if (threads != 128 && threads != 256) threads = 64;
    const int64_t rows_per_block = static_cast<int64_t>(RPW) * BATCH * (threads / 64);
    const int64_t needed = (a.rows + rows_per_block - 1) / rows_per_block;
    // One batch per wavefront by default; a positive knob caps the grid (grid-stride loop) instead.
    int64_t grid = needed;
    const int per_cu = tuning("layernorm.blocks_per_cu");
    if (per_cu > 0 && grid > static_cast<int64_t>(compute_units()) * per_cu)
        grid = static_cast<int64_t>(compute_units()) * per_cu;
    if (grid > 0x7fffffff) grid = 0x7fffffff;
    layernorm_wave_kernel<LPR, VPL, NT, BATCH><<<dim3(static_cast<unsigned>(grid)), dim3(threads), 0, a.stream>>>(
        a.in, a.out, a.mean, a.rstd, a.gamma, a.beta, a.rows, a.cols, a.eps, a.inv_denominator);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <int LPR, int VPL, bool NT>
int launch_wave(const Args &a) {
    // One row group per wavefront by default: on MI355X batching measured slower at every size tried
    // (the hardware keeps more independent waves in flight than a batch keeps loads).
    int batch = tuning("layernorm.batch");
    if (batch != 2 && batch != 4) batch = 1;
    if (batch == 4) return launch_wave_batch<LPR, VPL, NT, 4>(a);
    if (batch == 2) return launch_wave_batch<LPR, VPL, NT, 2>(a);
    return launch_wave_batch<LPR, VPL, NT, 1>(a);
}

template <int LPR, bool NT>
int launch_wave_vpl(const Args &a, int vpl) {
    switch (vpl) {
        case 1: return launch_wave<LPR, 1, NT>(a);
        case 2: return launch_wave<LPR, 2, NT>(a);
        case 3: return launch_wave<LPR, 3, NT>(a);
        case 4: return launch_wave<LPR, 4, NT>(a);
        case 5:
        case 6: return launch_wave<LPR, 6, NT>(a);
        default: return launch_wave<LPR, 8, NT>(a);
    }
}

template <bool NT>
int launch_wave_lpr(const Args &a, int lpr) {
    const int nvec = a.cols / 4;
    const int vpl = (nvec + lpr - 1) / lpr;
    switch (lpr) {
        case 8: return launch_wave_vpl<8, NT>(a, vpl);
        case 16: return launch_wave_vpl<16, NT>(a, vpl);
        case 32: return launch_wave_vpl<32, NT>(a, vpl);
        default: return launch_wave_vpl<64, NT>(a, vpl);
    }
}

constexpr int kWaveMaxVpl = 8;
constexpr int kWaveMaxCols = 64 * kWaveMaxVpl * 4;  // 2048
constexpr int kBlockMaxCols = 1024 * 8 * 4;         // 32768

// Lanes per row for the WARP policy: the narrowest group that gives every lane at most
// one vector, so that one load instruction of the group covers the row contiguously;
// rows longer than 64 vectors take the whole wavefront and several vectors per lane.
int default_lanes_per_row(int cols) {
    const int nvec = cols / 4;
    int lpr = 8;
    while (lpr < 64 && lpr < nvec) lpr <<= 1;
    return lpr;
}

int launch_wave_any(const Args &a) {
    int lpr = tuning("layernorm.lanes_per_row");
    if (lpr != 8 && lpr != 16 && lpr != 32 && lpr != 64) lpr = default_lanes_per_row(a.cols);
    while (lpr < 64 && (a.cols / 4 + lpr - 1) / lpr > kWaveMaxVpl) lpr <<= 1;
    // Streaming (non-temporal) accesses by default: every byte is touched once.  Knob: 2 = off.
    if (tuning("layernorm.nontemporal") == 2) return launch_wave_lpr<false>(a, lpr);
    return launch_wave_lpr<true>(a, lpr);
}

template <int THREADS>
int launch_block_threads(const Args &a) {
    const int nvec = a.cols / 4;
    const int vpl = (nvec + THREADS - 1) / THREADS;
    int64_t grid = static_cast<int64_t>(compute_units()) * (2048 / THREADS) * 2;
    if (grid > a.rows) grid = a.rows;
    dim3 g(static_cast<unsigned>(grid)), b(THREADS);
#define KO_LN_BLOCK(V)                                                                             \
    layernorm_block_kernel<THREADS, V><<<g, b, 0, a.stream>>>(a.in, a.out, a.mean, a.rstd, a.gamma, \
                                                              a.beta, a.rows, a.cols, a.eps,        \
                                                              a.inv_denominator)
    if (vpl <= 1) KO_LN_BLOCK(1);
    else if (vpl <= 2) KO_LN_BLOCK(2);
    else if (vpl <= 4) KO_LN_BLOCK(4);
    else KO_LN_BLOCK(8);
#undef KO_LN_BLOCK
    KO_CHECK_LAUNCH();
    return KO_OK;
}

int launch_block(const Args &a) {
    const int nvec = a.cols / 4;
    int threads = tuning("layernorm.block_threads");
    if (threads != 256 && threads != 512 && threads != 1024) {
        threads = 256;
        while (threads < 1024 && (nvec + threads - 1) / threads > 4) threads <<= 1;
    }
    while (threads < 1024 && (nvec + threads - 1) / threads > 8) threads <<= 1;
    if (threads == 256) return launch_block_threads<256>(a);
    if (threads == 512) return launch_block_threads<512>(a);
    return launch_block_threads<1024>(a);
}

int launch_nocache(const Args &a) {
    constexpr int kThreads = 1024;
    int64_t grid = static_cast<int64_t>(compute_units()) * 4;
    if (grid > a.rows) grid = a.rows;
    layernorm_nocache_kernel<kThreads><<<dim3(static_cast<unsigned>(grid)), dim3(kThreads), 0, a.stream>>>(
        a.in, a.out, a.mean, a.rstd, a.gamma, a.beta, a.rows, a.cols, a.eps, a.inv_denominator);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

}  // namespace
}  // namespace ko

KO_EXPORT int ko_layernorm_f32_policy(const float *in, float *out, float *mean, float *rstd,
                                      const float *gamma, const float *beta, int64_t rows,
                                      int64_t cols, float eps, int unbiased, int policy,
                                      ko_stream_t stream) {
    using namespace ko;
    if (rows < 0 || cols <= 0)
        return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: rows=%lld cols=%lld", (long long)rows, (long long)cols);
    if (cols % 4 != 0)
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "layernorm: cols=%lld is not a multiple of the vector width 4",
                    (long long)cols);
    if (cols > (1 << 30)) return fail(KO_ERR_UNSUPPORTED_SHAPE, "layernorm: cols=%lld too large", (long long)cols);
    if (rows == 0) return KO_OK;
    if (!in || !out) return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: null in/out pointer");
    uintptr_t align = reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out) |
                      reinterpret_cast<uintptr_t>(gamma) | reinterpret_cast<uintptr_t>(beta);
    if (align & 15) return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: in/out/gamma/beta must be 16-byte aligned");
    if (!(eps >= 0.0f)) return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: eps must be >= 0");
    const double denom = unbiased ? static_cast<double>(cols - 1) : static_cast<double>(cols);
    Args a{in, out, mean, rstd, gamma, beta, rows, static_cast<int>(cols), eps,
           static_cast<float>(1.0 / denom), as_stream(stream)};
    if (policy == KO_POLICY_AUTO) {
        policy = a.cols <= kWaveMaxCols ? KO_POLICY_WARP
                 : a.cols <= kBlockMaxCols ? KO_POLICY_BLOCK
                                           : KO_POLICY_BLOCK_NOCACHE;
    }
    switch (policy) {
        case KO_POLICY_WARP:
            if (a.cols > kWaveMaxCols)
                return fail(KO_ERR_UNSUPPORTED_SHAPE,
                            "layernorm: WARP policy holds at most %d columns per row, got %d", kWaveMaxCols, a.cols);
            return launch_wave_any(a);
        case KO_POLICY_BLOCK:
            if (a.cols > kBlockMaxCols)
                return fail(KO_ERR_UNSUPPORTED_SHAPE,
                            "layernorm: BLOCK policy holds at most %d columns per row, got %d", kBlockMaxCols, a.cols);
            return launch_block(a);
        case KO_POLICY_BLOCK_NOCACHE: return launch_nocache(a);
        default: return fail(KO_ERR_INVALID_ARGUMENT, "layernorm: unknown policy %d", policy);
    }
}

KO_EXPORT int ko_layernorm_f32(const float *in, float *out, float *mean, float *rstd,
                               const float *gamma, const float *beta, int64_t rows, int64_t cols,
                               float eps, int unbiased, ko_stream_t stream) {
    return ko_layernorm_f32_policy(in, out, mean, rstd, gamma, beta, rows, cols, eps, unbiased,
                                   KO_POLICY_AUTO, stream);
}
