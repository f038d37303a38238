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

#include <type_traits>
#include <utility>

// Partial products of the entry point that allocates nothing (ko_sgemm_f32_static_scratch): as large as the
// part of a stream's workspace that the allocating entry point uses.  Every device the library runs on holds its own copy
// until the process ends.  In host code the name is a stand-in, not a device address: host code uses the
// address that ko::static_scratch() asks the runtime for, once per device.
static __device__ __align__(256) unsigned char scratch[ko::kSgemmPartialBytes];

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
    int lda;      // floats between rows of A (K, or more when A is a column range of a wider matrix)
    int k_slice;  // 0, or: workgroups with blockIdx.y = s multiply columns [s * k_slice, (s + 1) * k_slice) of A by
                  // the same rows of B and write their M x N partial product (alpha 1, no C) behind D + s * M * N
};

// The problem a workgroup of a K-sliced launch works on: its slice of A and B and its own partial product.
__device__ __forceinline__ Params slice_of(Params p) {
    if (p.k_slice > 0) {
        const int s = static_cast<int>(blockIdx.y);
        const int k0 = s * p.k_slice;
        p.A += k0;
        p.B += static_cast<int64_t>(k0) * p.N;
        p.D += static_cast<int64_t>(s) * p.M * p.N;
        p.K = p.K - k0 < p.k_slice ? p.K - k0 : p.k_slice;
    }
    return p;
}

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

// Sums the partial accumulators of the K splits through LDS (every wave must be past its last use of
// the stages) and writes D = alpha * acc + beta * C.
template <int BM, int BN, int WAVES_M, int WAVES_N, int KSPLIT, int TM, int TN, bool FULL>
__device__ __forceinline__ void reduce_and_store(const Params &p, float16v (&acc)[TM][TN], float4v *lds, int wave,
                                                 int lane, int m0, int n0) {
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    const int split = wave / (WAVES_M * WAVES_N);
    const int wm = (wave / WAVES_N) % WAVES_M, wn = wave % WAVES_N;
    const int frow = lane & 31;
    const int fhalf = lane >> 5;
    const int M = p.M, N = p.N;
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
                        // one 32 x 32 accumulator at a time: with all reads issued first, a 128 x 128 tile
                        // needs 64 more registers here than anywhere in the K loop
                        if (q == 3) __builtin_amdgcn_sched_barrier(0);
                    }
        }
    }

    // acc[i][j][r] is D[m][n] with m = 8*(r/4) + 4*(lane/32) + r%4, n = lane%32 inside
    // the 32x32 tile: for a fixed r the 32 lanes of a half-wave write 128 contiguous bytes.
    const float alpha = p.alpha, beta = p.beta;
    // streaming stores while rows of D start on 64-byte boundaries (a half-wave's 128 bytes are two whole sectors then);
    // off them the ends of a row segment share their sectors with a neighbour's, and go through the L2 to meet there
    // (4096 x 4072 x 128: 60.5 us streamed, against 54.4 at N = 4064)
    const bool whole_sectors = (N & 15) == 0;
    // The choice between "with C" and "without" is made once, not per element, and the 32 x 32 sub-tiles
    // are written one after the other (the addresses of all of them at once would not fit the registers).
    auto store_all = [&](auto with_c, auto streaming) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int n = n0 + wn * WTN + j * 32 + frow;
                if (FULL || n < N) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int m = m0 + wm * WTM + i * 32 + 8 * (r / 4) + 4 * fhalf + (r % 4);
                        if (!FULL && m >= M) continue;
                        const int64_t off = static_cast<int64_t>(m) * N + n;
                        float v = alpha * acc[i][j][r];
                        if constexpr (decltype(with_c)::value) v += beta * p.C[off];
                        if constexpr (decltype(streaming)::value) __builtin_nontemporal_store(v, &p.D[off]);
                        else p.D[off] = v;
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    if (p.C != nullptr && beta != 0.0f) {
        if (whole_sectors) store_all(std::true_type{}, std::true_type{});
        else store_all(std::true_type{}, std::false_type{});
    } else {
        if (whole_sectors) store_all(std::false_type{}, std::true_type{});
        else store_all(std::false_type{}, std::false_type{});
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
                const float *src = p.A + static_cast<int64_t>(gr) * p.lda + kc;
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

    reduce_and_store<BM, BN, WAVES_M, WAVES_N, KSPLIT, TM, TN, FULL>(p, acc, lds, wave, lane, m0, n0);
}

template <int IMM>
__device__ __forceinline__ void lds_read_b128(float4v &dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(IMM));
}
template <int IMM>
__device__ __forceinline__ void lds_read_b32(float &dst, uint32_t addr) {
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(IMM));
}
template <int N>
__device__ __forceinline__ void wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}) in order
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// What lanes fetch in place of operand elements past the end of K.
__device__ __attribute__((aligned(16))) const float zero_chunk[4] = {0.0f, 0.0f, 0.0f, 0.0f};

// One direct-to-LDS load: LB (16 or 4) bytes per lane from `from` (per lane) to `to` + LB * lane (`to` wave-uniform).
template <int LB>
__device__ __forceinline__ void load_to_lds(const char *from, char *to) {
    typedef const __attribute__((address_space(1))) void *gptr_t;
    typedef __attribute__((address_space(3))) void *lptr_t;
    if constexpr (LB == 16) __builtin_amdgcn_global_load_lds((gptr_t)from, (lptr_t)to, 16, 0, 0);
    else __builtin_amdgcn_global_load_lds((gptr_t)from, (lptr_t)to, 4, 0, 0);
}

// Direct-to-LDS kernel (EDGE false: full tiles and an even number of K tiles): the same tiles, LDS layout, fragment
// order and epilogue as the PIPE form of sgemm_kernel, but global_load_lds_dwordx4 moves 16 bytes per
// lane from global memory straight into LDS (lane l of a wave-level load fills the l-th 16-byte slot
// after the wave-uniform LDS base), so the staging registers, the LDS writes and their address
// arithmetic leave the K loop.  The swizzles are applied on the global side: the lane that fills slot
// (row, c) fetches chunk c ^ swz(row) of that row.  NSTAGE stages of LDS: while tile kt is multiplied
// out of registers, the fragments of tile kt + 1 are read from its stage and tiles up to kt + NSTAGE are
// in flight (the newest one into the stage tile kt has just left).
//
// The compiler counts a direct-to-LDS load as an LDS write that any LDS read may alias and would wait
// for all of them (vmcnt(0)) before every fragment read it knows of; so the fragment reads and their
// waits are inline assembly.  Registers filled by such a read pass through an empty assembly statement
// behind the wait before the MFMAs use them, which keeps every use (and every copy) behind the wait.
//
// LB = 4 (with EDGE): operand rows that do not start on 16-byte boundaries (N, K or the row stride of A not a
// multiple of 4, or unaligned base pointers).  The same LDS layout is filled four bytes per lane instead of
// sixteen (global_load_lds_dword: lane l fills the l-th dword behind the wave-uniform base), four times as
// many loads; each lane fetches the element that belongs in its dword, a zero where k is past the end.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int KSPLIT, int NSTAGE, bool EDGE, int LB = 16>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N * KSPLIT) void sgemm_direct_kernel(const Params whole) {
    const Params p = slice_of(whole);
    constexpr int THREADS = 64 * WAVES_M * WAVES_N * KSPLIT;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int A_ROW_CHUNKS = BK / 4;
    constexpr int A_CHUNKS = BM * A_ROW_CHUNKS;
    constexpr int B_CHUNKS = BK * BN / 4;
    constexpr int BNC = BN / 4;
    constexpr int CHUNKS = A_CHUNKS + B_CHUNKS;
    constexpr int PER_CHUNK = 16 / LB;                       // loads that fill one 16-byte chunk
    constexpr int LOADS = CHUNKS * PER_CHUNK / THREADS;      // wave-level loads per wave and K tile
    constexpr int A_LOADS = A_CHUNKS * PER_CHUNK / THREADS;  // the first A_LOADS of them fetch A
    constexpr int KGROUPS = BK / 8;
    constexpr int GROUPS = KGROUPS / KSPLIT;
    constexpr int STAGE_BYTES = CHUNKS * 16;
    static_assert(LB == 16 || (LB == 4 && EDGE), "the dword form is an edge form");
    static_assert(A_CHUNKS % THREADS == 0 && B_CHUNKS % THREADS == 0, "a wave-level load stays inside A or B");
    static_assert(KGROUPS % KSPLIT == 0 && (BK == 32 || BK == 64 || BK == 128) && BN % 64 == 0 && NSTAGE >= 2, "");
    static_assert((NSTAGE - 1) * LOADS < 64 && BK * BN * 4 < 65536 && TM * 32 * A_ROW_CHUNKS * 16 < 65536, "");
    typedef const __attribute__((address_space(1))) void *gptr_t;
    typedef __attribute__((address_space(3))) void *lptr_t;

    extern __shared__ float4v lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int split = wave / (WAVES_M * WAVES_N);
    const int wm = (wave / WAVES_N) % WAVES_M, wn = wave % WAVES_N;
    int tile_m, tile_n;
    tile_of(p, static_cast<int>(blockIdx.x), tile_m, tile_n);
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;
    const int N = p.N, K = p.K;
    // EDGE: K (a multiple of 4 unless LB = 4) is padded with zeros up to the next pair of K tiles.
    const int KT = EDGE ? 2 * ((K + 2 * BK - 1) / (2 * BK)) : K / BK;

    // A rows of 256 bytes or more fill lines of the 64 banks; of 128 bytes two rows share one, and the
    // number of the row pair goes into the swizzle.
    auto swz_a = [](int row) { return BK == 32 ? (row >> 1) & 7 : row & 15; };
    auto swz_b = [](int k) { return ((k >> 2) & 1) << 3; };

    // What this thread fetches with each of its loads: LDS slot (of LB bytes) tid + i * THREADS of the stage, K tile 0.
    const char *src[LOADS];
    int koff[EDGE ? LOADS : 1];  // EDGE: the k, within a K tile, of the chunk or element (A) or row (B) this lane fetches
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int slot = tid + i * THREADS;
        const int idx = slot / PER_CHUNK, d = slot % PER_CHUNK;  // 16-byte chunk of the stage, element within it (LB = 4)
        if (i < A_LOADS) {
            const int row = idx / A_ROW_CHUNKS, c = idx % A_ROW_CHUNKS;
            const int k = 4 * (c ^ swz_a(row)) + d;
            if constexpr (EDGE) koff[i] = k;
            int gr = m0 + row;
            if constexpr (EDGE) gr = gr < p.M ? gr : p.M - 1;  // rows past M fetch the last row again; never stored
            src[i] = reinterpret_cast<const char *>(p.A + static_cast<int64_t>(gr) * p.lda + k);
        } else {
            const int b = idx - A_CHUNKS;
            const int kr = b / BNC, c = b % BNC;
            if constexpr (EDGE) koff[i] = kr;
            int gn = n0 + 4 * (c ^ swz_b(kr)) + d;
            // columns past N fetch the last chunk (N a multiple of 4) or element again: they only feed columns never stored
            if constexpr (EDGE) gn = gn < N ? gn : N - (LB == 16 ? 4 : 1);
            src[i] = reinterpret_cast<const char *>(p.B + static_cast<int64_t>(kr) * N + gn);
        }
    }
    const int64_t step_a = BK * 4, step_b = static_cast<int64_t>(BK) * N * 4;
    int ld_kt = 0;  // the K tile the sources point at
    int k_left = K;  // EDGE: K - ld_kt * BK; chunks and rows at or past it are fetched from zeros instead
    const char *zeros = reinterpret_cast<const char *>(&zero_chunk);
    auto source = [&](int i) {
        if constexpr (EDGE) return koff[i] < k_left ? src[i] : zeros;
        else return src[i];
    };
    // Loads past the last K tile are not branched around: they fetch the last tile once more, into a
    // stage nobody reads any more, so that the count of loads in flight is the same on every path.
    auto advance = [&]() {
        const bool more = ld_kt + 1 < KT;
        ld_kt += more ? 1 : 0;
        const int64_t da = more ? step_a : 0, db = more ? step_b : 0;
#pragma unroll
        for (int i = 0; i < LOADS; ++i) src[i] += i < A_LOADS ? da : db;
        if constexpr (EDGE) k_left = K - ld_kt * BK;
    };
    auto issue = [&](int stage) {
        char *dst = reinterpret_cast<char *>(lds) + stage * STAGE_BYTES + wave * (64 * LB);
#pragma unroll
        for (int i = 0; i < LOADS; ++i)
            load_to_lds<LB>(source(i), dst + i * THREADS * LB);
        advance();
    };

    // LDS byte addresses of this lane's fragments in stage 0 (see read_frags of sgemm_kernel): per group
    // of 8 k for A (the swizzle depends on the chunk), per 32 columns for B; the rest are immediates.
    const int frow = lane & 31;
    const int fhalf = lane >> 5;
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));  // LDS aperture offset
    uint32_t addr_a[GROUPS], addr_b[TN];
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
        const int chunk = 2 * (split + g * KSPLIT) + fhalf;
        const int row = wm * WTM + frow;  // rows 32 apart share the swizzle
        addr_a[g] = lds_base + (row * A_ROW_CHUNKS + (chunk ^ swz_a(row))) * 16;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int col = (wn * WTN + j * 32 + frow) ^ (fhalf << 5);
        addr_b[j] = lds_base + A_CHUNKS * 16 + ((8 * split + 4 * fhalf) * BN + col) * 4;
    }
    auto read_frags = [&](int stage, float4v (&af)[GROUPS][TM], float (&bf)[GROUPS][TN][4]) {
        const uint32_t off = static_cast<uint32_t>(stage) * STAGE_BYTES;
        static_for<GROUPS>([&](auto g_c) {
            constexpr int g = decltype(g_c)::value;
            const uint32_t a = addr_a[g] + off;
            static_for<TM>([&](auto i_c) {
                constexpr int i = decltype(i_c)::value;
                lds_read_b128<i * 32 * A_ROW_CHUNKS * 16>(af[g][i], a);
            });
        });
        static_for<TN>([&](auto j_c) {
            constexpr int j = decltype(j_c)::value;
            const uint32_t b = addr_b[j] + off;
            static_for<GROUPS * 4>([&](auto gt_c) {
                constexpr int g = decltype(gt_c)::value / 4, t = decltype(gt_c)::value % 4;
                lds_read_b32<(8 * g * KSPLIT + t) * BN * 4>(bf[g][j][t], b);
            });
        });
    };
    // All LDS reads of this wave have landed; the fragments become usable.
    auto frags_ready = [&](float4v (&af)[GROUPS][TM], float (&bf)[GROUPS][TN][4]) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
#pragma unroll
            for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(af[g][i]));
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t) asm volatile("" : "+v"(bf[g][j][t]));
        }
    };

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    float4v af0[GROUPS][TM], af1[GROUPS][TM];  // fragments of the even / odd K tile
    float bf0[GROUPS][TN][4], bf1[GROUPS][TN][4];
#pragma unroll
    for (int s = 0; s < NSTAGE; ++s) issue(s);  // K tiles 0 .. NSTAGE - 1
    wait_vm<(NSTAGE - 1) * LOADS>();
    asm volatile("s_barrier" ::: "memory");
    read_frags(0, af0, bf0);
    int wr = 0, rd = 1;  // stages of K tiles kt and kt + 1
    // One K tile.  Before the barrier: this wave's share of tile kt + 1 has landed and its reads of tile
    // kt's stage are complete.  Behind it: that stage takes tile kt + NSTAGE, the fragments of tile
    // kt + 1 are read under the MFMAs of tile kt.  After the last tile the reads fetch stale (in-bounds)
    // LDS contents that nothing uses.
    auto step = [&](float4v (&af_cur)[GROUPS][TM], float (&bf_cur)[GROUPS][TN][4], float4v (&af_next)[GROUPS][TM],
                    float (&bf_next)[GROUPS][TN][4]) {
        wait_vm<(NSTAGE - 2) * LOADS>();
        frags_ready(af_cur, bf_cur);
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        // The loads of tile kt + NSTAGE and the fragment reads of tile kt + 1 are spread over the MFMAs
        // of tile kt, PER of them behind each MFMA until they run out, loads first: the wave never
        // stands between two MFMAs for longer than that, so the matrix core's queue does not run dry
        // while all waves of the workgroup are in the same part of the step.
        constexpr int NMFMA = GROUPS * 4 * TM * TN;
        constexpr int A_READS = GROUPS * TM, B_READS = TN * GROUPS * 4;
        constexpr int PIECES = LOADS + A_READS + B_READS;
        constexpr int PER = (PIECES + NMFMA - 1) / NMFMA;
        char *dst = reinterpret_cast<char *>(lds) + wr * STAGE_BYTES + wave * (64 * LB);
        const uint32_t off = static_cast<uint32_t>(rd) * STAGE_BYTES;
        static_for<NMFMA>([&](auto q_c) {
            constexpr int q = decltype(q_c)::value;
            constexpr int g = q / (4 * TM * TN), t = (q / (TM * TN)) % 4, i = (q / TN) % TM, j = q % TN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af_cur[g][i][t], bf_cur[g][j][t], acc[i][j], 0, 0, 0);
            static_for<PER>([&](auto r_c) {
                constexpr int pc = q * PER + decltype(r_c)::value;
                if constexpr (pc < LOADS) {
                    load_to_lds<LB>(source(pc), dst + pc * THREADS * LB);
                    if constexpr (pc == LOADS - 1) advance();
                } else if constexpr (pc < LOADS + A_READS) {
                    constexpr int u = pc - LOADS, g2 = u / TM, i2 = u % TM;
                    lds_read_b128<i2 * 32 * A_ROW_CHUNKS * 16>(af_next[g2][i2], addr_a[g2] + off);
                } else if constexpr (pc < PIECES) {
                    constexpr int u = pc - LOADS - A_READS, j2 = u / (GROUPS * 4), g2 = (u / 4) % GROUPS, t2 = u % 4;
                    lds_read_b32<(8 * g2 * KSPLIT + t2) * BN * 4>(bf_next[g2][j2][t2], addr_b[j2] + off);
                }
            });
            __builtin_amdgcn_sched_barrier(0);
        });
        wr = rd;
        rd = rd + 1 == NSTAGE ? 0 : rd + 1;
    };
    for (int kt = 0; kt < KT; kt += 2) {
        step(af0, bf0, af1, bf1);
        step(af1, bf1, af0, bf0);
    }
    // The redirected loads still in flight write LDS, and the last fragment reads are pending: both end
    // before the reduction reuses the stages.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    reduce_and_store<BM, BN, WAVES_M, WAVES_N, KSPLIT, TM, TN, !EDGE>(p, acc, lds, wave, lane, m0, n0);
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int KSPLIT, bool PIPE = false>
int launch(Params p, hipStream_t stream) {
    constexpr int THREADS = 64 * WAVES_M * WAVES_N * KSPLIT;
    if (p.k_slice > 0) return fail(KO_ERR_INVALID_ARGUMENT, "sgemm: this tiling takes no K slices");
    const int tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int64_t nblocks = static_cast<int64_t>(tiles_m) * p.tiles_n;
    if (nblocks > 0x7fffffff) return fail(KO_ERR_UNSUPPORTED_SHAPE, "sgemm: too many tiles");
    p.blocked = tuning(knob_sgemm_mapping) != 1 && tiles_m % 4 == 0 && p.tiles_n % 8 == 0 &&
                ((tiles_m / 4) * (p.tiles_n / 8)) % 8 == 0;
    const bool vec = (p.K % 4 == 0) && (p.lda % 4 == 0) && (p.N % 4 == 0) &&
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

// The direct-to-LDS kernel where it applies (operand rows on 16-byte boundaries, at least one pair of K
// tiles), else the register pipeline with the same tiling.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int KSPLIT, int NSTAGE, int FALLBACK_BK = BK>
int launch_direct(Params p, hipStream_t stream) {
    constexpr int THREADS = 64 * WAVES_M * WAVES_N * KSPLIT;
    constexpr size_t stage_bytes = static_cast<size_t>(NSTAGE) * (BM * BK + BK * BN) * 4;
    constexpr size_t reduce_bytes = static_cast<size_t>(KSPLIT - 1) * BM * BN * 4;  // the split-K reduction reuses the stages
    constexpr size_t lds_bytes = stage_bytes > reduce_bytes ? stage_bytes : reduce_bytes;
    // Ragged shapes are handled in the kernel's EDGE form (rows past M and columns past N fetch valid data
    // that is never stored, K is padded with zeros up to a pair of K tiles, stores are bounds-checked).
    // Operand rows have to start on 16-byte boundaries and K must not end inside a 16-byte chunk.
    const bool aligned = ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15) == 0 &&
                         p.lda % 4 == 0 && p.N % 4 == 0 && p.K % 4 == 0;
    if (!aligned && p.k_slice == 0 && tuning(knob_sgemm_unaligned) == 1) return launch<BM, BN, FALLBACK_BK, WAVES_M, WAVES_N, KSPLIT, true>(p, stream);
    // K-sliced launches: every slice but the last is k_slice deep (a multiple of 4, so aligned operand rows stay
    // aligned in every slice), the last takes the rest.
    const int slices = p.k_slice > 0 ? (p.K + p.k_slice - 1) / p.k_slice : 1;
    const int k_last = p.K - (slices - 1) * (p.k_slice > 0 ? p.k_slice : 0);
    const int k_each = slices > 1 ? p.k_slice : p.K;
    const bool edge = p.M % BM != 0 || p.N % BN != 0 || k_each % (2 * BK) != 0 || k_last % (2 * BK) != 0;
    const int tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int64_t nblocks = static_cast<int64_t>(tiles_m) * p.tiles_n;
    if (nblocks > 0x7fffffff) return fail(KO_ERR_UNSUPPORTED_SHAPE, "sgemm: too many tiles");
    p.blocked = tuning(knob_sgemm_mapping) != 1 && tiles_m % 4 == 0 && p.tiles_n % 8 == 0 &&
                ((tiles_m / 4) * (p.tiles_n / 8)) % 8 == 0;
    // Operand rows off 16-byte boundaries: the edge form that fills LDS four bytes per lane.
    auto kernel = !aligned ? sgemm_direct_kernel<BM, BN, BK, WAVES_M, WAVES_N, KSPLIT, NSTAGE, true, 4>
                  : edge   ? sgemm_direct_kernel<BM, BN, BK, WAVES_M, WAVES_N, KSPLIT, NSTAGE, true>
                           : sgemm_direct_kernel<BM, BN, BK, WAVES_M, WAVES_N, KSPLIT, NSTAGE, false>;
    static std::atomic<uint64_t> configured[3] = {{0}, {0}, {0}};  // per instantiation: the devices whose LDS limit is raised
    if (const int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds_bytes, configured[!aligned ? 2 : edge]); st != KO_OK)
        return st;
    kernel<<<dim3(static_cast<unsigned>(nblocks), static_cast<unsigned>(slices)), dim3(THREADS), lds_bytes, stream>>>(p);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

// D = alpha * (P_0 + P_1 + ... + P_{slices-1}) + beta * C over the M x N partial products a K-sliced launch
// left behind `partials`, summed in slice order whatever order the slices finished in.  slices == 0 is the
// empty product (k == 0): nothing is read through `partials` and D = beta * C, or zero without a C - what the
// reference's kernel leaves when its main loop runs no K tile (simt_gemm.h:325-354).
// One 64-lane workgroup per 256 outputs: the problems that are sliced have few outputs, and small
// workgroups spread them over more compute units.  The partial products of eight slices are fetched together
// (they come from memory behind the L2s: another XCD wrote them) and added one after the other.
__global__ __launch_bounds__(64) void sgemm_slices_sum_kernel(const float *__restrict__ partials, int slices,
                                                              int64_t count, float alpha, float beta,
                                                              const float *C, float *D) {  // C may be D
    // four floats that start on any 4-byte boundary (an odd M x N puts every other partial product off the
    // 16-byte grid): still one access each
    typedef float vec_t __attribute__((ext_vector_type(4)));
    typedef vec_t vec_any_t __attribute__((aligned(4)));
    const int64_t i = (static_cast<int64_t>(blockIdx.x) * 64 + threadIdx.x) * 4;
    if (i >= count) return;
    const float *src = partials + i;
    if (i + 4 <= count) {
        vec_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
        if (slices > 0) acc = *reinterpret_cast<const vec_any_t *>(src);
        int s = 1;
        for (; s + 8 <= slices; s += 8) {
            vec_t v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const vec_any_t *>(src + (s + j) * count);
#pragma unroll
            for (int j = 0; j < 8; ++j) acc += v[j];
        }
        for (; s < slices; ++s) acc += *reinterpret_cast<const vec_any_t *>(src + s * count);
        acc *= alpha;
        if (C != nullptr && beta != 0.0f) acc += beta * *reinterpret_cast<const vec_any_t *>(C + i);
        __builtin_nontemporal_store(acc, reinterpret_cast<vec_any_t *>(D + i));
    } else {
        for (int64_t e = i; e < count; ++e) {  // the last one to three outputs
            float acc = slices > 0 ? partials[e] : 0.0f;
            for (int s = 1; s < slices; ++s) acc += partials[e + s * count];
            acc *= alpha;
            if (C != nullptr && beta != 0.0f) acc += beta * C[e];
            D[e] = acc;
        }
    }
}

int sum_slices(const float *partials, int slices, const Params &p, hipStream_t stream) {
    const int64_t count = static_cast<int64_t>(p.M) * p.N;
    const dim3 grid(static_cast<unsigned>(((count + 3) / 4 + 63) / 64));
    sgemm_slices_sum_kernel<<<grid, 64, 0, stream>>>(partials, slices, count, p.alpha, p.beta, p.C, p.D);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

// One launch: the tiling by shape (variant <= 0) or the one asked for.
int run(Params p, hipStream_t s, int variant) {
    const int64_t m = p.M, n = p.N, k = p.k_slice > 0 ? p.k_slice : p.K;
    if (variant <= 0) {
        // Few tiles (fewer 128 x 128 tiles than compute units): 64 x 64 tiles with K split four ways inside
        // the workgroup; otherwise 128 x 128 tiles with K split two ways (2048^3, one tile per compute unit:
        // 130 us against 149 us).
        // Very few (64 x 64 tiles for at most half of the compute units): 32 x 64 tiles (512^3: 8.0 us against
        // 12.1 us).
        // All three as direct-to-LDS kernels; shapes those do not take fall back to the register pipeline
        // with the same tiling.  The 64 x 64 tiles take 128 k per step (two LDS stages of 64 KB) where K
        // allows: half as many barriers of the 16 waves (1024 x 1024 x 4096: 67 us against 73 us).
        // The 128 x 128 tiles take 64 k per step from K = 2048 on (2048^3: 126 us against 143 us; the same
        // at 4096^3; shallower K loses more to the larger first tile than it gains).
        const int64_t t128 = ((m + 127) / 128) * ((n + 127) / 128);
        const int64_t t64 = ((m + 63) / 64) * ((n + 63) / 64);
        // K is padded up to a pair of K tiles: the deeper step is taken where its padding costs less than it gains.
        const int64_t k_pad128 = (k + 127) / 128 * 128, k_pad256 = (k + 255) / 256 * 256;
        // A round of 64 x 64 tiles takes 0.29-0.31 of the time of a round of 128 x 128 tiles (2048 x 3072 x 1024:
        // 19 us against 62 us; K = 2048: 35 against 121): the big tiles do the same work in 0.8 of the time
        // when their rounds are full, but one and a half rounds of them cost two (384 tiles on 256 compute
        // units: 125 us, as 1536 small tiles in six rounds 114 us).
        const int64_t cu = compute_units();
        const bool big = t128 >= cu && 97 * ((t128 + cu - 1) / cu) <= 31 * ((t64 + cu - 1) / cu);
        variant = big ? (k >= 2048 ? 40 : 36)
                      : (2 * t64 <= cu ? 41 : (15 * k_pad256 <= 16 * k_pad128 ? 35 : 33));
        // a K of one 32-deep K tile or less (a low-rank update: the time is the output's): the register pipeline
        // takes it as one K tile, the direct-to-LDS kernels pad it to a pair of them (8192 x 3072 x 8: 31 us
        // against 47 us)
        if (big && k <= 32) variant = 16;
        // A shallow K on many small tiles: the time is the output's, and the direct-to-LDS 64 x 64 kernels - three
        // stages, K padded to a pair of 64-deep tiles - spend it on their prologue (9523 x 344 x 32: 22 us; the
        // 128 x 128 register pipeline 10.5; x 256: 38 against 28 on direct 128 x 128 tiles).  128 x 128 tiles
        // where their rounds come out nearly full, else the 64 x 64 register pipeline (597 x 7992 x 128, 315 big
        // tiles on 256 compute units: 23 us against 30 and 32).
        if (!big && k <= 256 && t64 >= 2 * cu) {
            const int64_t rounds128 = (t128 + cu - 1) / cu;
            variant = k <= 32 ? 16 : (5 * t128 >= 4 * rounds128 * cu ? 36 : 13);
        }
        // Operand rows off 16-byte boundaries are loaded four bytes per lane, four times as many loads with an
        // address each: the 128 x 128 x 64 form would spill registers there.
        const bool aligned = ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15) == 0 &&
                             p.lda % 4 == 0 && p.N % 4 == 0 && p.K % 4 == 0;
        if (!aligned && variant == 40) variant = 36;
        // a slice of K (a forced slice count can bring one here with any depth): only the direct-to-LDS kernels
        // take slices, so the register pipeline's shapes go to the direct-to-LDS kernel of the same tile
        if (p.k_slice > 0) {
            if (variant == 13) variant = 33;
            if (variant == 16) variant = 36;
        }
    }
    switch (variant) {
        case 13: return launch<64, 64, 64, 2, 2, 4, true>(p, s);
        case 16: return launch<128, 128, 32, 2, 2, 2, true>(p, s);
        case 21: return launch<32, 64, 64, 1, 2, 4, true>(p, s);
        case 33: return launch_direct<64, 64, 64, 2, 2, 4, 3>(p, s);
        case 35: return launch_direct<64, 64, 128, 2, 2, 4, 2, 64>(p, s);
        case 36: return launch_direct<128, 128, 32, 2, 2, 2, 2>(p, s);
        case 37: return launch_direct<128, 128, 32, 2, 2, 2, 3>(p, s);
        case 40: return launch_direct<128, 128, 64, 2, 2, 2, 2, 32>(p, s);
        case 41: return launch_direct<32, 64, 64, 1, 2, 4, 3>(p, s);
        default: return fail(KO_ERR_INVALID_ARGUMENT, "sgemm: unknown variant %d", variant);
    }
}

// K slices.  The slices are workgroups of one launch (blockIdx.y); their partial products go to a workspace and
// a second kernel sums them in slice order, so the result does not depend on which slice finished first.
// Two cases:
//   - few output tiles (tiles for at most half of the compute units, 256 x 256 x 2048: 32 tiles of 32 x 64 on 256
//     CUs) and K >= 768: as many slices as bring the launch up to one workgroup per compute unit, each at
//     least 256 deep and a multiple of 128 (whole pairs of K tiles); the tiling as for the unsliced problem;
//   - more tiles, but rounds that do not fill the chip, and K >= 2048 (768 x 768 x 16384: 144 tiles of 64 x 64 on
//     256 CUs, a round of K = 16384 at 56 % of the chip): the tiling and slice count that a cost model of the
//     three tilings puts lowest - rounds x (fixed + per-64-k x depth / 64) + the summing kernel, the constants
//     from K sweeps on this device - when that is at least a tenth below the best unsliced estimate (36 tiles
//     of 128 x 128 in 7 slices: 252 workgroups, 253 -> 153 us; hipBLASLt 159 us).
struct SlicePlan {
    int slices = 1;   // 1: do not slice
    int k_slice = 0;  // depth of every slice but the last
    int variant = 0;  // tiling of the sliced launch (0: as run() picks it)
};

SlicePlan plan_k_slices(const Params &p, size_t workspace_bytes) {
    SlicePlan plan;
    const int forced = tuning(knob_sgemm_k_slices);
    if (forced == 1) return plan;
    // operand rows off 16-byte boundaries: the same plans (the four-byte loads make every tiling slower by about
    // the same factor), without the 128 x 128 x 64 form
    const bool aligned = ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15) == 0 &&
                         p.lda % 4 == 0 && p.N % 4 == 0 && p.K % 4 == 0;
    const int64_t cu = compute_units();
    const int64_t t64 = ((p.M + 63) / 64) * ((p.N + 63) / 64);
    auto set = [&](int64_t slices, int variant) {
        if (slices < 2) return;
        const int64_t depth = ((p.K + slices - 1) / slices + 127) / 128 * 128;
        slices = (p.K + depth - 1) / depth;
        if (slices < 2 || slices > 65535) return;
        plan.slices = static_cast<int>(slices);
        plan.k_slice = static_cast<int>(depth);
        plan.variant = variant;
    };
    if (forced >= 2) {
        set(forced, tuning(knob_sgemm_slice_variant));
        return plan;
    }
    if (2 * t64 <= cu) {
        // The second launch costs 2-3 us: below K = 768 the slices do not win them back (256 x 256 x 512: 7.0 us
        // whole, 7.5 us in two slices; K = 768: 9.2 against 8.3; K = 2048: 19.8 against 11.1).
        if (p.K < 768) return plan;
        const int64_t tiles = ((p.M + 31) / 32) * ((p.N + 63) / 64);  // run() takes 32 x 64 tiles here
        int64_t slices = cu / tiles;
        if (slices > p.K / 256) slices = p.K / 256;
        set(slices, 0);
        return plan;
    }
    if (p.K < 2048) return plan;
    // us of one round of workgroups that are `depth` deep: {fixed, per 64 k}; rounds of one workgroup per
    // compute unit (32 x 64 tiles: of two, which then take 1.2 us per 64 k instead of 0.5)
    struct Tiling { int bm, bn, variant; double fixed, per64; int per_cu; };
    const Tiling tilings[3] = {{128, 128, 0, 6.0, 3.67, 1}, {64, 64, 0, 5.2, 0.95, 1}, {32, 64, 41, 4.2, 1.2, 2}};
    const double out_bytes = 4.0 * p.M * p.N;
    double best_whole = 1e30, best_sliced = 1e30;
    int64_t best_slices = 1;
    int best_variant = 0;
    for (const Tiling &t : tilings) {
        const int64_t tiles = static_cast<int64_t>((p.M + t.bm - 1) / t.bm) * ((p.N + t.bn - 1) / t.bn);
        const int64_t slots = cu * t.per_cu;
        for (int64_t slices = 1; slices <= 64 && p.K / slices >= 512; ++slices) {
            if (slices > 1 && slices * out_bytes > static_cast<double>(workspace_bytes)) break;
            const int64_t depth = slices == 1 ? p.K : ((p.K + slices - 1) / slices + 127) / 128 * 128;
            const int64_t groups = tiles * ((p.K + depth - 1) / depth);
            const int64_t rounds = (groups + slots - 1) / slots;
            const double per64 = t.per_cu == 2 && groups <= cu ? 0.5 : t.per64;
            double us = rounds * (t.fixed + per64 * depth / 64.0);
            if (slices == 1) {
                if (us < best_whole) best_whole = us;
                continue;
            }
            us += 2.5 + (slices + 1) * out_bytes / 5e6;  // the summing kernel: its launch, partial products in, D out
            if (us < best_sliced) {
                best_sliced = us;
                best_slices = slices;
                best_variant = t.variant != 0 ? t.variant
                               : t.bm == 128  ? (depth >= 2048 && aligned ? 40 : 36)
                                              : (depth % 256 == 0 ? 35 : 33);
            }
        }
    }
    if (best_sliced < 0.9 * best_whole) set(best_slices, best_variant);
    return plan;
}

// The K-sliced form of one problem: partial products into `workspace`, then their sum and the epilogue.
int run_sliced(const Params &p, const SlicePlan &plan, float *workspace, hipStream_t s) {
    Params part = p;
    part.C = nullptr;
    part.D = workspace;
    part.alpha = 1.0f;
    part.beta = 0.0f;
    part.k_slice = plan.k_slice;
    if (const int st = run(part, s, plan.variant); st != KO_OK) return st;
    return sum_slices(workspace, plan.slices, p, s);
}

// The address of `scratch` on the current device (looked up once per device).
int static_scratch(void **address) {
    constexpr int kCached = 64;
    static std::atomic<void *> known[kCached];  // zero-initialised
    int dev = 0;
    KO_HIP(hipGetDevice(&dev));
    if (dev >= 0 && dev < kCached) {
        if (void *a = known[dev].load(std::memory_order_acquire)) {
            *address = a;
            return KO_OK;
        }
    }
    void *a = nullptr;
    KO_HIP(hipGetSymbolAddress(&a, HIP_SYMBOL(scratch)));
    if (a == nullptr) return fail(KO_ERR_RUNTIME, "sgemm: the static scratch array has no address on device %d", dev);
    if (dev >= 0 && dev < kCached) known[dev].store(a, std::memory_order_release);
    *address = a;
    return KO_OK;
}

// Both SGEMM entry points.  `own_scratch`: partial products of a K-sliced problem go to the static array of the
// device instead of the stream's allocated workspace, and a slice plan that does not fit is an error.
int sgemm(int64_t m, int64_t n, int64_t k, float alpha, const float *A, const float *B, float beta, const float *C,
          float *D, ko_stream_t stream, bool own_scratch) {
    if (m < 0 || n < 0 || k < 0)
        return fail(KO_ERR_INVALID_ARGUMENT, "sgemm: m=%lld n=%lld k=%lld", (long long)m, (long long)n, (long long)k);
    if (m == 0 || n == 0) return KO_OK;
    if (m > (1 << 30) || n > (1 << 30) || k > (1 << 30)) return fail(KO_ERR_UNSUPPORTED_SHAPE, "sgemm: dimension too large");
    if (!D || (k > 0 && (!A || !B))) return fail(KO_ERR_INVALID_ARGUMENT, "sgemm: null A/B/D pointer");
    if (k == 0) {  // the empty product: D = beta * C (one scale-and-copy launch; A and B are not touched)
        const Params empty{A, B, C, D, static_cast<int>(m), static_cast<int>(n), 0, alpha, beta, 0, 0, 0, 0};
        return sum_slices(nullptr, 0, empty, as_stream(stream));
    }
    Params p{A, B, C, D, static_cast<int>(m), static_cast<int>(n), static_cast<int>(k), alpha, beta, 0, 0, static_cast<int>(k), 0};
    hipStream_t s = as_stream(stream);
    const int variant = tuning(knob_sgemm_variant);
    if (variant <= 0) {
        if (const SlicePlan plan = plan_k_slices(p, sizeof(scratch)); plan.slices > 1) {
            const int slices = plan.slices;
            const uint64_t need = static_cast<uint64_t>(slices) * m * n * sizeof(float);
            void *workspace = nullptr;
            if (own_scratch) {
                if (need > sizeof(scratch))
                    return fail(KO_ERR_UNSUPPORTED_SHAPE,
                                "sgemm: the partial products of %d slices of K (%llu bytes) do not fit the static scratch array (%zu bytes)",
                                slices, (unsigned long long)need, sizeof(scratch));
                if (const int st = static_scratch(&workspace); st != KO_OK) return st;
            } else if (need <= kSgemmPartialBytes) {
                if (const int st = stream_workspace(s, &workspace); st != KO_OK) return st;
            }
            if (workspace != nullptr) return run_sliced(p, plan, static_cast<float *>(workspace), s);
        }
    }
    if (variant <= 0 && tuning(knob_sgemm_split_rows) != 1 && k >= 512) {
        // A last round of 128 x 128 tiles that fills at most half of the compute units costs a whole round:
        // the tile rows that fill whole rounds go out as one launch, the rows below them as a second one
        // with the smaller tiles its own size asks for (4096 x 4224 x 4096, 1056 tiles on 256 compute
        // units: 1023 tiles in four rounds plus 132 tiles of 64 x 64 instead of five rounds).
        const int64_t cu = compute_units();
        const int64_t tm = (m + 127) / 128, tn = (n + 127) / 128;
        const int64_t rounds = tm * tn / cu;
        const int64_t rows1 = rounds * cu / tn;          // whole tile rows within the full rounds
        const int64_t below = (tm - rows1) * tn;         // 128 x 128 tiles left for the second launch
        if (rounds >= 1 && rows1 >= 1 && rows1 < tm && (tm * tn) % cu != 0 && 2 * below <= cu) {
            const int64_t m1 = rows1 * 128;
            Params top = p, bottom = p;
            top.M = static_cast<int>(m1);
            bottom.M = static_cast<int>(m - m1);
            bottom.A = A + m1 * k;
            bottom.C = C ? C + m1 * n : nullptr;
            bottom.D = D + m1 * n;
            if (const int st = run(top, s, 0); st != KO_OK) return st;
            return run(bottom, s, 0);
        }
    }
    return run(p, s, variant);
}

}  // namespace
}  // namespace ko

KO_EXPORT int ko_sgemm_f32(int64_t m, int64_t n, int64_t k, float alpha, const float *A, const float *B, float beta,
                           const float *C, float *D, ko_stream_t stream) {
    return ko::sgemm(m, n, k, alpha, A, B, beta, C, D, stream, false);
}

KO_EXPORT int ko_sgemm_f32_static_scratch(int64_t m, int64_t n, int64_t k, float alpha, const float *A, const float *B,
                                          float beta, const float *C, float *D, ko_stream_t stream) {
    return ko::sgemm(m, n, k, alpha, A, B, beta, C, D, stream, true);
}

int ko::debug_sgemm_plan(int64_t m, int64_t n, int64_t k, int *slices, int *k_slice, int *variant) {
    using namespace ko;
    if (!slices || !k_slice || !variant || m <= 0 || n <= 0 || k <= 0 || m > (1 << 30) || n > (1 << 30) || k > (1 << 30))
        return fail(KO_ERR_INVALID_ARGUMENT, "sgemm_plan: bad argument");
    // operands that the planner takes for 16-byte aligned; nothing is read through them
    const float *aligned = reinterpret_cast<const float *>(uintptr_t{256});
    const Params p{aligned, aligned, nullptr, nullptr, static_cast<int>(m), static_cast<int>(n), static_cast<int>(k),
                   1.0f, 0.0f, 0, 0, static_cast<int>(k), 0};
    const SlicePlan plan = plan_k_slices(p, kSgemmPartialBytes);
    *slices = plan.slices;
    *k_slice = plan.k_slice;
    *variant = plan.variant;
    return KO_OK;
}
