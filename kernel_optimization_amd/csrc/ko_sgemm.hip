// SIMT-path SGEMM for gfx950: fp32 operands, fp32 matrix-core accumulation
// (v_mfma_f32_32x32x2_f32; true fp32 products and sums), row-major A[M,K],
// B[K,N], C/D[M,N].  D = alpha * A * B + beta * C.
//
// Stands in for GemmKernelSimt (nn_operators/gemm/simt_gemm.h:46-376): a 64x64x8
// block tile computed by 4 warps with scalar FMAs (:202-222), shared-memory double
// buffer and register prefetch (:224-297), epilogue D = acc (+ C) (:325-373).  The
// same pipeline skeleton is kept (global -> registers -> LDS double buffer ->
// fragments -> multiply, one barrier per K tile); the multiply is the fp32 MFMA
// and the tile shapes are sized for 64-lane wavefronts:
//
//   workgroup tile  BM x BN x 32, WAVES_M x WAVES_N wavefronts
//   LDS             A stage [BM][32] floats, 16-byte chunks XOR-swizzled by row (a
//                   lane reads 4 consecutive k of one row with one ds_read_b128);
//                   B stage [32][BN] floats as in memory (a lane reads one float per
//                   k; 32 consecutive lanes read 32 consecutive columns)
//   K order         within an 8-wide K group, MFMA t (t = 0..3) multiplies
//                   k = 4*(lane/32) + t; the sum over the group covers every k once
//   no prefetch past the end of K (the reference reads one tile out of bounds,
//   simt_gemm.h:287-292)
#include "ko_internal.h"

namespace ko {
namespace {

typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kBK = 32;
constexpr int kAChunks = kBK / 4;  // 16-byte chunks per A row

struct Params {
    const float *A;
    const float *B;
    const float *C;
    float *D;
    int M, N, K;
    float alpha, beta;
    int tiles_n;
};

// VEC: K % 4 == 0, N % 4 == 0 and 16-byte aligned A and B (128-bit global loads);
// otherwise every element is loaded on its own with bounds checks.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool VEC>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void sgemm_kernel(const Params p) {
    constexpr int THREADS = 64 * WAVES_M * WAVES_N;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int A_CHUNKS = BM * kAChunks;      // float4 chunks of the A stage
    constexpr int B_CHUNKS = kBK * BN / 4;       // float4 chunks of the B stage
    constexpr int A_ITERS = A_CHUNKS / THREADS, B_ITERS = B_CHUNKS / THREADS;
    constexpr int BNC = BN / 4;                  // chunks per B row
    static_assert(A_CHUNKS % THREADS == 0 && B_CHUNKS % THREADS == 0, "");

    __shared__ float4v lds_a[2][A_CHUNKS];
    __shared__ float4v lds_b[2][B_CHUNKS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int m0 = (blockIdx.x / p.tiles_n) * BM;
    const int n0 = (blockIdx.x % p.tiles_n) * BN;
    const int M = p.M, N = p.N, K = p.K;

    float4v ra[A_ITERS], rb[B_ITERS];

    auto load_global = [&](int kt) {
        const int k0 = kt * kBK;
#pragma unroll
        for (int i = 0; i < A_ITERS; ++i) {
            const int idx = tid + i * THREADS;
            const int row = idx / kAChunks, c = idx % kAChunks;
            int gr = m0 + row;
            gr = gr < M ? gr : M - 1;
            const int kc = k0 + c * 4;
            const float *src = p.A + static_cast<int64_t>(gr) * K + kc;
            float4v v = {0.0f, 0.0f, 0.0f, 0.0f};
            if constexpr (VEC) {
                if (kc < K) v = *reinterpret_cast<const float4v *>(src);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (kc + e < K) v[e] = src[e];
            }
            ra[i] = v;
        }
#pragma unroll
        for (int i = 0; i < B_ITERS; ++i) {
            const int idx = tid + i * THREADS;
            const int kr = idx / BNC, c = idx % BNC;
            const int gk = k0 + kr;
            const int gn = n0 + c * 4;
            float4v v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (gk < K) {
                const float *src = p.B + static_cast<int64_t>(gk) * N + gn;
                if constexpr (VEC) {
                    if (gn < N) v = *reinterpret_cast<const float4v *>(src);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (gn + e < N) v[e] = src[e];
                }
            }
            rb[i] = v;
        }
    };

    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_ITERS; ++i) {
            const int idx = tid + i * THREADS;
            const int row = idx / kAChunks, c = idx % kAChunks;
            lds_a[buf][row * kAChunks + (c ^ (row & 7))] = ra[i];
        }
#pragma unroll
        for (int i = 0; i < B_ITERS; ++i) lds_b[buf][tid + i * THREADS] = rb[i];
    };

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int KT = (K + kBK - 1) / kBK;
    load_global(0);
    store_lds(0);
    __syncthreads();

    const int frow = lane & 31;
    const int fhalf = lane >> 5;

    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) load_global(kt + 1);
        const float4v *sa = lds_a[cur];
        const float *sb = reinterpret_cast<const float *>(lds_b[cur]);
#pragma unroll
        for (int kg = 0; kg < kBK / 8; ++kg) {  // groups of 8 k
            float4v af[TM];
            float bf[TN][4];
            const int chunk = 2 * kg + fhalf;   // this lane's 4 consecutive k
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int row = wm * WTM + i * 32 + frow;
                af[i] = sa[row * kAChunks + (chunk ^ (row & 7))];
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int col = wn * WTN + j * 32 + frow;
#pragma unroll
                for (int t = 0; t < 4; ++t) bf[j][t] = sb[(4 * chunk + t) * BN + col];
            }
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][t], bf[j][t], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < KT) store_lds(cur ^ 1);
        __syncthreads();
    }

    // acc[i][j][r] is D[m][n] with m = 8*(r/4) + 4*(lane/32) + r%4, n = lane%32 inside
    // the 32x32 tile: for a fixed r the 32 lanes of a half-wave write 128 contiguous bytes.
    const float alpha = p.alpha, beta = p.beta;
    const bool use_c = p.C != nullptr && beta != 0.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * WTN + j * 32 + frow;
            if (n >= N) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * WTM + i * 32 + 8 * (r / 4) + 4 * fhalf + (r % 4);
                if (m >= M) continue;
                const int64_t off = static_cast<int64_t>(m) * N + n;
                float v = alpha * acc[i][j][r];
                if (use_c) v += beta * p.C[off];
                p.D[off] = v;
            }
        }
    }
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
int launch(Params p, hipStream_t stream) {
    constexpr int THREADS = 64 * WAVES_M * WAVES_N;
    const int tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int64_t nblocks = static_cast<int64_t>(tiles_m) * p.tiles_n;
    if (nblocks > 0x7fffffff) return fail(KO_ERR_UNSUPPORTED_SHAPE, "sgemm: too many tiles");
    const bool vec = (p.K % 4 == 0) && (p.N % 4 == 0) &&
                     ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15) == 0;
    dim3 grid(static_cast<unsigned>(nblocks)), block(THREADS);
    if (vec) sgemm_kernel<BM, BN, WAVES_M, WAVES_N, true><<<grid, block, 0, stream>>>(p);
    else sgemm_kernel<BM, BN, WAVES_M, WAVES_N, false><<<grid, block, 0, stream>>>(p);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

}  // namespace
}  // namespace ko

KO_EXPORT int ko_sgemm_f32(int64_t m, int64_t n, int64_t k, float alpha, const float *A,
                           const float *B, float beta, const float *C, float *D,
                           ko_stream_t stream) {
    using namespace ko;
    if (m < 0 || n < 0 || k < 0)
        return fail(KO_ERR_INVALID_ARGUMENT, "sgemm: m=%lld n=%lld k=%lld", (long long)m, (long long)n, (long long)k);
    if (m == 0 || n == 0) return KO_OK;
    if (k == 0) return fail(KO_ERR_UNSUPPORTED_SHAPE, "sgemm: k must be positive");
    if (m > (1 << 30) || n > (1 << 30) || k > (1 << 30)) return fail(KO_ERR_UNSUPPORTED_SHAPE, "sgemm: dimension too large");
    if (!A || !B || !D) return fail(KO_ERR_INVALID_ARGUMENT, "sgemm: null A/B/D pointer");
    Params p{A, B, C, D, static_cast<int>(m), static_cast<int>(n), static_cast<int>(k), alpha, beta, 0};
    hipStream_t s = as_stream(stream);
    int variant = tuning("sgemm.variant");
    if (variant <= 0) {
        const int64_t t128 = ((m + 127) / 128) * ((n + 127) / 128);
        variant = t128 >= 2 * compute_units() ? 3 : 1;
    }
    switch (variant) {
        case 1: return launch<64, 64, 2, 2>(p, s);
        case 2: return launch<128, 64, 2, 2>(p, s);
        case 3: return launch<128, 128, 2, 2>(p, s);
        case 4: return launch<64, 64, 1, 1>(p, s);
        case 5: return launch<64, 128, 2, 2>(p, s);
        default: return fail(KO_ERR_INVALID_ARGUMENT, "sgemm: unknown variant %d", variant);
    }
}
