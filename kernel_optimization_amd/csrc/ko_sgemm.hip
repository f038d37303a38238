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
//   workgroup tile  BM x BN x BK, WAVES_M x WAVES_N x KSPLIT wavefronts: the KSPLIT waves
//                   that share an output sub-tile take every KSPLIT-th group of 8 k
//                   of each K tile and their accumulators are summed through LDS at
//                   the end.  A 1024^3 problem has only 256 tiles of 64 x 64 (one per
//                   compute unit); splitting K inside the workgroup is what puts
//                   several waves on every SIMD so that LDS and barrier latencies of
//                   one wave are covered by the MFMAs of another
//   LDS             A stage [BM][BK] floats, 16-byte chunks XOR-swizzled by row (a
//                   lane reads 4 consecutive k of one row with one ds_read_b128);
//                   B stage [BK][BN] floats as in memory, with the two 32-column
//                   halves of every 64 columns exchanged in rows whose (k / 4) is odd
//                   (a lane reads one float per k; the two half-waves read rows k and
//                   k + 4 and so hit different banks)
//   K order         within an 8-wide K group, MFMA t (t = 0..3) multiplies
//                   k = 4*(lane/32) + t; the sum over the group covers every k once
//   no prefetch past the end of K (the reference reads one tile out of bounds,
//   simt_gemm.h:287-292)
#include "ko_internal.h"

namespace ko {
namespace {

typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));

// Workgroup barrier that waits for this wave's LDS traffic only; global loads stay in flight across it.
// The wait is the compiler's own s_waitcnt instruction (lgkmcnt(0); vmcnt and expcnt left at their
// maxima), not inline assembly, so that its wait-count bookkeeping knows the LDS reads issued before
// the barrier have landed and does not wait for them again behind younger reads.  The barrier builtin
// does not order memory accesses for the compiler; the empty asm statements do (no LDS access may move
// across them in either direction).
__device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

struct Params {
    const float *A;
    const float *B;
    const float *C;
    float *D;
    int M, N, K;
    float alpha, beta;
    int tiles_n;
    int blocked;  // 1: the tile grid is cut into 4 x 8 blocks, one per XCD and round (see tile_of)
};

// Workgroup -> output tile.  Workgroups go to the 8 XCDs round-robin by index, each XCD has its own
// L2 and runs 32 workgroups at a time (one per compute unit).  In the blocked order workgroups
// 8j + x, j = 32r .. 32r + 31, which are resident on XCD x together, form one 4 x 8 block of tiles:
// 256 rows of A and 512 columns of B instead of whole matrices.  Needs tiles_m % 4 == 0,
// tiles_n % 8 == 0 and a block count that is a multiple of 8; otherwise tiles are taken row-major.
__device__ __forceinline__ void tile_of(const Params &p, int b, int &tile_m, int &tile_n) {
    if (p.blocked) {
        const int x = b & 7, j = b >> 3;
        const int block = (j >> 5) * 8 + x;  // blocks are numbered row-major over the (tiles_m / 4) x (tiles_n / 8) grid
        const int blocks_n = p.tiles_n >> 3;
        tile_m = (block / blocks_n) * 4 + ((j & 31) >> 3);
        tile_n = (block % blocks_n) * 8 + (j & 7);
    } else {
        tile_m = b / p.tiles_n;
        tile_n = b % p.tiles_n;
    }
}

// VEC: K % 4 == 0, N % 4 == 0 and 16-byte aligned A and B (128-bit global loads);
// otherwise every element is loaded on its own with bounds checks.
// FULL (implies VEC): M % BM == 0, N % BN == 0, K % BK == 0 - no bounds checks at all.
// PIPE: global loads run two K tiles ahead (two sets of staging registers) and a wave holds all of its
// fragments of a K tile in registers, so the fragments of the next tile are read right after the
// barrier that publishes it, under the MFMAs of the current tile.  Needs FULL and an even number of K tiles.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int KSPLIT, bool PIPE, bool VEC, bool FULL>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N * KSPLIT) void sgemm_kernel(const Params p) {
    constexpr int THREADS = 64 * WAVES_M * WAVES_N * KSPLIT;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int A_ROW_CHUNKS = BK / 4;         // 16-byte chunks per A row
    constexpr int A_CHUNKS = BM * A_ROW_CHUNKS;  // float4 chunks of the A stage
    constexpr int B_CHUNKS = BK * BN / 4;        // float4 chunks of the B stage
    constexpr int BNC = BN / 4;                  // chunks per B row
    constexpr int CHUNKS = A_CHUNKS + B_CHUNKS;
    constexpr int ITERS = CHUNKS / THREADS;      // chunks a thread moves per K tile
    constexpr int KGROUPS = BK / 8;
    constexpr int STAGE_BYTES = CHUNKS * 16;
    constexpr int REDUCE_BYTES = (KSPLIT - 1) * BM * BN * 4;
    constexpr int LDS_BYTES = 2 * STAGE_BYTES > REDUCE_BYTES ? 2 * STAGE_BYTES : REDUCE_BYTES;
    static_assert(CHUNKS % THREADS == 0 && A_CHUNKS % 64 == 0, "");
    static_assert(KGROUPS % KSPLIT == 0 && (BK == 32 || BK == 64) && BN % 64 == 0, "");
    static_assert((!FULL || VEC) && (!PIPE || FULL), "");

    __shared__ float4v lds[LDS_BYTES / 16];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: address math on the scalar unit
    const int split = wave / (WAVES_M * WAVES_N);
    const int wm = (wave / WAVES_N) % WAVES_M, wn = wave % WAVES_N;
    int tile_m, tile_n;
    tile_of(p, static_cast<int>(blockIdx.x), tile_m, tile_n);
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;
    const int M = p.M, N = p.N, K = p.K;

    // A rows of 128 bytes: two rows share one line of the 64 banks, so the row pair number goes
    // into the swizzle; rows of 256 bytes fill a bank line on their own.
    auto swz_a = [](int row) { return BK == 32 ? (row >> 1) & 7 : row & 15; };
    // B: exchange the 32-column halves (8 chunks) when (k / 4) is odd.
    auto swz_b = [](int k) { return ((k >> 2) & 1) << 3; };

    auto load_global = [&](int kt, float4v (&staged)[ITERS]) {
        const int k0 = kt * BK;
#pragma unroll
        for (int i = 0; i < ITERS; ++i) {
            const int idx = tid + i * THREADS;
            float4v v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (idx < A_CHUNKS) {  // wave-uniform
                const int row = idx / A_ROW_CHUNKS, c = idx % A_ROW_CHUNKS;
                int gr = m0 + row;
                if constexpr (!FULL) gr = gr < M ? gr : M - 1;
                const int kc = k0 + c * 4;
                const float *src = p.A + static_cast<int64_t>(gr) * K + kc;
                if constexpr (FULL) {
                    v = *reinterpret_cast<const float4v *>(src);
                } else if constexpr (VEC) {
                    if (kc < K) v = *reinterpret_cast<const float4v *>(src);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (kc + e < K) v[e] = src[e];
                }
            } else {
                const int b = idx - A_CHUNKS;
                const int kr = b / BNC, c = b % BNC;
                const int gk = k0 + kr;
                const int gn = n0 + c * 4;
                const float *src = p.B + static_cast<int64_t>(gk) * N + gn;
                if constexpr (FULL) {
                    v = *reinterpret_cast<const float4v *>(src);
                } else if (gk < K) {
                    if constexpr (VEC) {
                        if (gn < N) v = *reinterpret_cast<const float4v *>(src);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (gn + e < N) v[e] = src[e];
                    }
                }
            }
            staged[i] = v;
        }
    };

    auto store_lds = [&](int buf, const float4v (&staged)[ITERS]) {
        float4v *sa = lds + buf * CHUNKS;
        float4v *sb = sa + A_CHUNKS;
#pragma unroll
        for (int i = 0; i < ITERS; ++i) {
            const int idx = tid + i * THREADS;
            if (idx < A_CHUNKS) {
                const int row = idx / A_ROW_CHUNKS, c = idx % A_ROW_CHUNKS;
                sa[row * A_ROW_CHUNKS + (c ^ swz_a(row))] = staged[i];
            } else {
                const int b = idx - A_CHUNKS;
                const int kr = b / BNC, c = b % BNC;
                sb[kr * BNC + (c ^ swz_b(kr))] = staged[i];
            }
        }
    };

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int KT = (K + BK - 1) / BK;
    const int frow = lane & 31;
    const int fhalf = lane >> 5;
    constexpr int GROUPS = KGROUPS / KSPLIT;  // groups of 8 k per wave and K tile

    // fragments of this wave's group g of the K tile held in stage `buf`
    auto read_frags = [&](int buf, int g, float4v (&af)[TM], float (&bf)[TN][4]) {
        const float4v *sa = lds + buf * CHUNKS;
        const float *sb = reinterpret_cast<const float *>(sa + A_CHUNKS);
        const int kg = split + g * KSPLIT;
        const int chunk = 2 * kg + fhalf;   // this lane's 4 consecutive k
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int row = wm * WTM + i * 32 + frow;
            af[i] = sa[row * A_ROW_CHUNKS + (chunk ^ swz_a(row))];
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            // (k / 4) % 2 == fhalf for all four k of this lane: the upper half-wave reads the exchanged halves
            const int col = (wn * WTN + j * 32 + frow) ^ (fhalf << 5);
#pragma unroll
            for (int t = 0; t < 4; ++t) bf[j][t] = sb[(4 * chunk + t) * BN + col];
        }
    };
    auto multiply = [&](const float4v (&af)[TM], const float (&bf)[TN][4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][t], bf[j][t], acc[i][j], 0, 0, 0);
    };

    if constexpr (PIPE) {
        float4v staged0[ITERS], staged1[ITERS];       // tiles with even / odd index on their way to LDS
        float4v af0[GROUPS][TM], af1[GROUPS][TM];     // fragments of the even / odd tile
        float bf0[GROUPS][TN][4], bf1[GROUPS][TN][4];
        // Loads and stores past the last K tile are not branched around but redirected to the last tile
        // (its data is stored once more into the stage nobody reads any more): with the same memory
        // operations on every path the compiler's wait counts stay exact, and it waits for the oldest
        // staging set only instead of for everything in flight.
        const int last = KT - 1;
        load_global(0, staged0);
        load_global(1, staged1);
        store_lds(0, staged0);
        load_global(2 < KT ? 2 : last, staged0);
        lds_barrier();
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) read_frags(0, g, af0[g], bf0[g]);
        // One K tile: publish the next tile's stage, start reading its fragments, multiply this tile.
        // The stage written here was last read before the previous barrier (every wave had its reads
        // of it completed by then), and global loads stay in flight across the barrier.
        auto step = [&](int kt, float4v (&st_next)[ITERS], float4v (&af_cur)[GROUPS][TM], float (&bf_cur)[GROUPS][TN][4],
                        float4v (&af_next)[GROUPS][TM], float (&bf_next)[GROUPS][TN][4]) {
            const int next = (kt + 1) & 1;
            store_lds(next, st_next);
            load_global(kt + 3 < KT ? kt + 3 : last, st_next);
            lds_barrier();
            // after the last K tile this reads stale (in-bounds) LDS contents that nothing uses; keeping
            // the reads unconditional keeps the count of outstanding LDS operations the same on every path
#pragma unroll
            for (int g = 0; g < GROUPS; ++g) read_frags(next, g, af_next[g], bf_next[g]);
            __builtin_amdgcn_sched_barrier(0);  // the reads are issued before the MFMAs that cover their latency
#pragma unroll
            for (int g = 0; g < GROUPS; ++g) multiply(af_cur[g], bf_cur[g]);
            __builtin_amdgcn_sched_barrier(0);
        };
        // KT is even here (the launcher sees to it): with no branch between the two steps the
        // fragment reads stay where they are written, right behind the barrier
        for (int kt = 0; kt < KT; kt += 2) {
            step(kt, staged1, af0, bf0, af1, bf1);
            step(kt + 1, staged0, af1, bf1, af0, bf0);
        }
        lds_barrier();  // the stages are reused by the split-K reduction
    } else {
        float4v staged[ITERS];
        load_global(0, staged);
        store_lds(0, staged);
        __syncthreads();
        for (int kt = 0; kt < KT; ++kt) {
            const int cur = kt & 1;
            if (kt + 1 < KT) load_global(kt + 1, staged);
#pragma unroll
            for (int g = 0; g < GROUPS; ++g) {
                float4v af[TM];
                float bf[TN][4];
                read_frags(cur, g, af, bf);
                multiply(af, bf);
            }
            if (kt + 1 < KT) store_lds(cur ^ 1, staged);
            __syncthreads();
        }
    }

    if constexpr (KSPLIT > 1) {
        // Sum the partial accumulators of the K splits into split 0 (fixed order: 1, 2, ...).
        // Every wave is past the last barrier of the main loop, so the stages are free.
        constexpr int PER_WAVE = TM * TN * 4 * 64;  // float4 slots of one wave's accumulators
        const int sub = wave % (WAVES_M * WAVES_N);
        if (split > 0) {
            float4v *dst = lds + ((split - 1) * WAVES_M * WAVES_N + sub) * PER_WAVE;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float4v v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                        dst[((i * TN + j) * 4 + q) * 64 + lane] = v;
                    }
        }
        __syncthreads();
        if (split > 0) return;
#pragma unroll
        for (int s = 1; s < KSPLIT; ++s) {
            const float4v *src = lds + ((s - 1) * WAVES_M * WAVES_N + sub) * PER_WAVE;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float4v v = src[((i * TN + j) * 4 + q) * 64 + lane];
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] += v[e];
                    }
        }
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
            if (!FULL && n >= N) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * WTM + i * 32 + 8 * (r / 4) + 4 * fhalf + (r % 4);
                if (!FULL && m >= M) continue;
                const int64_t off = static_cast<int64_t>(m) * N + n;
                float v = alpha * acc[i][j][r];
                if (use_c) v += beta * p.C[off];
                __builtin_nontemporal_store(v, &p.D[off]);
            }
        }
    }
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int KSPLIT, bool PIPE = false>
int launch(Params p, hipStream_t stream) {
    constexpr int THREADS = 64 * WAVES_M * WAVES_N * KSPLIT;
    const int tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int64_t nblocks = static_cast<int64_t>(tiles_m) * p.tiles_n;
    if (nblocks > 0x7fffffff) return fail(KO_ERR_UNSUPPORTED_SHAPE, "sgemm: too many tiles");
    p.blocked = tuning("sgemm.mapping") != 1 && tiles_m % 4 == 0 && p.tiles_n % 8 == 0 &&
                ((tiles_m / 4) * (p.tiles_n / 8)) % 8 == 0;
    const bool vec = (p.K % 4 == 0) && (p.N % 4 == 0) &&
                     ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15) == 0;
    const bool full = vec && p.M % BM == 0 && p.N % BN == 0 && p.K % BK == 0;
    dim3 grid(static_cast<unsigned>(nblocks)), block(THREADS);
    if (PIPE && full && (p.K / BK) % 2 == 0)
        sgemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, KSPLIT, PIPE, true, true><<<grid, block, 0, stream>>>(p);
    else if (full) sgemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, KSPLIT, false, true, true><<<grid, block, 0, stream>>>(p);
    else if (vec) sgemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, KSPLIT, false, true, false><<<grid, block, 0, stream>>>(p);
    else sgemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, KSPLIT, false, false, false><<<grid, block, 0, stream>>>(p);
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
    Params p{A, B, C, D, static_cast<int>(m), static_cast<int>(n), static_cast<int>(k), alpha, beta, 0, 0};
    hipStream_t s = as_stream(stream);
    int variant = tuning("sgemm.variant");
    if (variant <= 0) {
        // Few tiles (fewer 128 x 128 tiles than compute units): 64 x 64 tiles with K split four ways inside
        // the workgroup; otherwise 128 x 128 tiles with K split two ways (2048^3, one tile per compute unit:
        // 136 us against 148 us).
        // Very few (64 x 64 tiles for at most half of the compute units): 32 x 64 tiles (512^3: 8.8 us against
        // 12.2 us).
        const int64_t t128 = ((m + 127) / 128) * ((n + 127) / 128);
        const int64_t t64 = ((m + 63) / 64) * ((n + 63) / 64);
        variant = t128 >= compute_units() ? 16 : (2 * t64 <= compute_units() ? 21 : 13);
    }
    switch (variant) {
        case 1: return launch<64, 64, 32, 2, 2, 1>(p, s);
        case 2: return launch<128, 64, 32, 2, 2, 1>(p, s);
        case 3: return launch<128, 128, 32, 2, 2, 1>(p, s);
        case 4: return launch<64, 64, 32, 1, 1, 1>(p, s);
        case 5: return launch<64, 128, 32, 2, 2, 1>(p, s);
        case 6: return launch<64, 64, 32, 2, 2, 2>(p, s);
        case 7: return launch<64, 64, 32, 2, 2, 4>(p, s);
        case 8: return launch<64, 64, 64, 2, 2, 2>(p, s);
        case 9: return launch<64, 64, 64, 2, 2, 4>(p, s);
        case 10: return launch<128, 128, 32, 2, 2, 2>(p, s);
        case 11: return launch<128, 64, 32, 2, 2, 2>(p, s);
        case 12: return launch<64, 64, 64, 2, 2, 2, true>(p, s);
        case 13: return launch<64, 64, 64, 2, 2, 4, true>(p, s);
        case 14: return launch<64, 64, 32, 2, 2, 4, true>(p, s);
        case 15: return launch<64, 64, 32, 2, 2, 2, true>(p, s);
        case 16: return launch<128, 128, 32, 2, 2, 2, true>(p, s);
        case 17: return launch<128, 128, 32, 2, 2, 1, true>(p, s);
        case 18: return launch<128, 64, 32, 2, 2, 2, true>(p, s);
        case 19: return launch<128, 64, 64, 2, 2, 2, true>(p, s);
        case 21: return launch<32, 64, 64, 1, 2, 4, true>(p, s);
        default: return fail(KO_ERR_INVALID_ARGUMENT, "sgemm: unknown variant %d", variant);
    }
}
