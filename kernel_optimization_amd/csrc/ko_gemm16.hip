// Tensor-core-path GEMM for gfx950: binary16 / bfloat16 operands, fp32
// accumulation on the matrix cores (v_mfma_f32_32x32x16_{f16,bf16}), 16-bit
// output.  D[m,n] = alpha * sum_k A[m,k] B[k,n] + beta * C[m,n].
//
// Stands in for GemmKernelTensorCore (nn_operators/gemm/tensor_core_gemm.h:101-399),
// which stages 128x128x32 tiles in shared memory, feeds mma.sync.m16n8k8 with
// f16 accumulation (:33-48) and has an unfinished epilogue (:366-397).  The
// skeleton is the same - global -> registers -> LDS double buffer -> fragments
// -> matrix instruction, one barrier per K tile (:237-339) - the tiling is not:
//
//   workgroup tile  BM x BN x 64, WAVES_M x WAVES_N wavefronts of 64 lanes
//   wave tile       (BM/WAVES_M) x (BN/WAVES_N), made of 32x32 MFMA tiles
//   LDS             2 stages x (BM + BN) rows x 128 B; both operands are stored
//                   K-contiguous ([row][k]); 16-byte chunks are XOR-swizzled with
//                   the row index so that fragment reads (one 16-byte chunk per
//                   lane, 32 consecutive rows) and staging writes (8 chunks of one
//                   row) are both bank-conflict free
//   fragments       lane l reads row l%32, k-chunk l/32 of a 16-wide K step: the
//                   operand layout of the 32x32x16 MFMA; 8 halfs = one ds_read_b128
//   operands swapped: the B fragment is passed as the first MFMA operand, so the
//                   accumulator holds the tile transposed and every lane owns 4
//                   consecutive columns of one output row
//   pipeline        tile kt+2 is in flight from global memory into registers while
//                   tile kt is multiplied out of one LDS stage and tile kt+1 moves
//                   from registers into the other; the barrier waits for LDS only
//   epilogue        full tiles: each wave transposes its tile through LDS and writes
//                   16 bytes per lane, whole rows of the wave tile contiguously
//
// Column-major B (memory [n][k]) is the fast layout: both operands are then
// K-contiguous in global memory.  Row-major B (the reference's layout,
// tensor_core_gemm.h:178) is transposed while it is staged into LDS.
#include "ko_internal.h"

#include <type_traits>

namespace ko {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kBK = 64;          // K extent of a stage
constexpr int kChunks = kBK / 8; // 16-byte chunks per LDS row

template <bool BF16>
__device__ __forceinline__ float16v mfma16(u32x4 a, u32x4 b, float16v c) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a),
                                                      __builtin_bit_cast(half8, b), c, 0, 0, 0);
}

template <bool BF16>
__device__ __forceinline__ float to_float(uint16_t bits) {
    if constexpr (BF16) return __builtin_bit_cast(float, static_cast<uint32_t>(bits) << 16);
    else return static_cast<float>(__builtin_bit_cast(_Float16, bits));
}

template <bool BF16>
__device__ __forceinline__ uint16_t from_float(float v) {
    if constexpr (BF16) {
        uint32_t u = __builtin_bit_cast(uint32_t, v);
        if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);  // quiet NaN
        return static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
    } else {
        return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
    }
}

// Workgroup -> output tile.  Workgroups are handed to the 8 XCDs round-robin by
// their index, and each XCD has its own L2; the remap gives every XCD one
// contiguous band of tiles (tile_n fastest), so the tiles resident on an XCD at any
// moment share A rows and B columns in that XCD's L2.
__device__ __forceinline__ int xcd_remap(int block, int nblocks) {
    constexpr int kXcds = 8;
    const int per = nblocks / kXcds;
    const int main_blocks = per * kXcds;
    if (block >= main_blocks) return block;  // remainder keeps its index
    return (block % kXcds) * per + block / kXcds;
}

// Workgroup barrier that waits for this wave's LDS traffic only.  __syncthreads() also
// drains the global loads in flight, which here are meant to stay in flight across it.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Orders this wave's earlier LDS writes before its later LDS reads.
__device__ __forceinline__ void wave_lds_fence() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

struct Params {
    const uint16_t *A;
    const uint16_t *B;
    const uint16_t *C;
    uint16_t *D;
    int M, N, K;
    float alpha, beta;
    int tiles_n;
    int nblocks;
};

// EDGE = false: M % BM == 0, N % BN == 0 and K % 64 == 0, so no load or store needs a bounds check.
// REG_STAGES = 2: global loads run two K tiles ahead (two sets of staging registers);
// REG_STAGES = 1: one tile ahead.  FRAG_DB: fragments of the next K step are read into a
// second register set while the MFMAs of the current step run.
template <int BM, int BN, int WAVES_M, int WAVES_N, int REG_STAGES, bool FRAG_DB, bool BF16, bool B_ROW_MAJOR,
          bool EDGE>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm16_kernel(const Params p) {
    constexpr int THREADS = 64 * WAVES_M * WAVES_N;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int A_CHUNKS = BM * kChunks, B_CHUNKS = BN * kChunks;
    constexpr int A_ITERS = A_CHUNKS / THREADS, B_ITERS = B_CHUNKS / THREADS;
    constexpr int STAGE = A_CHUNKS + B_CHUNKS;  // chunks per stage
    static_assert(A_CHUNKS % THREADS == 0 && B_CHUNKS % THREADS == 0, "");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "");

    extern __shared__ u32x4 lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    const int tile = xcd_remap(blockIdx.x, p.nblocks);
    const int m0 = (tile / p.tiles_n) * BM;
    const int n0 = (tile % p.tiles_n) * BN;
    const int M = p.M, N = p.N, K = p.K;

    const int KT = (K + kBK - 1) / kBK;

    // Two register stages: the tile two steps ahead is in flight from global memory
    // while the tile one step ahead waits to be written to LDS.
    u32x4 ra[REG_STAGES][A_ITERS], rb[REG_STAGES][B_ITERS];

    auto load_global = [&](int kt, auto slot) {
        constexpr int S = decltype(slot)::value;
        const int k0 = kt * kBK;
#pragma unroll
        for (int i = 0; i < A_ITERS; ++i) {
            const int idx = tid + i * THREADS;
            const int row = idx / kChunks, c = idx % kChunks;
            int gr = m0 + row;
            const int kc = k0 + c * 8;
            if constexpr (EDGE) {
                gr = gr < M ? gr : M - 1;  // rows past the edge re-read the last row; their results are never stored
                u32x4 v = {0u, 0u, 0u, 0u};
                if (kc < K) v = *reinterpret_cast<const u32x4 *>(p.A + static_cast<int64_t>(gr) * K + kc);
                ra[S][i] = v;
            } else {
                ra[S][i] = *reinterpret_cast<const u32x4 *>(p.A + static_cast<int64_t>(gr) * K + kc);
            }
        }
        if constexpr (!B_ROW_MAJOR) {
#pragma unroll
            for (int i = 0; i < B_ITERS; ++i) {
                const int idx = tid + i * THREADS;
                const int row = idx / kChunks, c = idx % kChunks;
                int gr = n0 + row;
                const int kc = k0 + c * 8;
                if constexpr (EDGE) {
                    gr = gr < N ? gr : N - 1;
                    u32x4 v = {0u, 0u, 0u, 0u};
                    if (kc < K) v = *reinterpret_cast<const u32x4 *>(p.B + static_cast<int64_t>(gr) * K + kc);
                    rb[S][i] = v;
                } else {
                    rb[S][i] = *reinterpret_cast<const u32x4 *>(p.B + static_cast<int64_t>(gr) * K + kc);
                }
            }
        } else {
            // B[k][n] row-major: a chunk is 8 consecutive n of one k.
#pragma unroll
            for (int i = 0; i < B_ITERS; ++i) {
                const int idx = tid + i * THREADS;
                constexpr int NCH = BN / 8;
                const int kr = idx / NCH, c = idx % NCH;
                const int gk = k0 + kr;
                const int gn = n0 + c * 8;
                u32x4 v = {0u, 0u, 0u, 0u};
                if (!EDGE || gk < K) {
                    const uint16_t *src = p.B + static_cast<int64_t>(gk) * N + gn;
                    if (!EDGE || (gn + 8 <= N && (N & 7) == 0)) {
                        v = *reinterpret_cast<const u32x4 *>(src);
                    } else {
                        uint16_t t[8];
#pragma unroll
                        for (int e = 0; e < 8; ++e) t[e] = gn + e < N ? src[e] : static_cast<uint16_t>(0);
                        v = u32x4{t[0] | (uint32_t(t[1]) << 16), t[2] | (uint32_t(t[3]) << 16),
                                  t[4] | (uint32_t(t[5]) << 16), t[6] | (uint32_t(t[7]) << 16)};
                    }
                }
                rb[S][i] = v;
            }
        }
    };

    auto store_lds = [&](int buf, auto slot) {
        constexpr int S = decltype(slot)::value;
        u32x4 *sa = lds + buf * STAGE;
        u32x4 *sb = sa + A_CHUNKS;
#pragma unroll
        for (int i = 0; i < A_ITERS; ++i) {
            const int idx = tid + i * THREADS;
            const int row = idx / kChunks, c = idx % kChunks;
            sa[row * kChunks + (c ^ (row & 7))] = ra[S][i];
        }
        if constexpr (!B_ROW_MAJOR) {
#pragma unroll
            for (int i = 0; i < B_ITERS; ++i) {
                const int idx = tid + i * THREADS;
                const int row = idx / kChunks, c = idx % kChunks;
                sb[row * kChunks + (c ^ (row & 7))] = rb[S][i];
            }
        } else {
            uint16_t *sb16 = reinterpret_cast<uint16_t *>(sb);
#pragma unroll
            for (int i = 0; i < B_ITERS; ++i) {
                const int idx = tid + i * THREADS;
                constexpr int NCH = BN / 8;
                const int kr = idx / NCH, c = idx % NCH;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int n = c * 8 + e;
                    const uint16_t h = static_cast<uint16_t>(rb[S][i][e >> 1] >> ((e & 1) * 16));
                    const int chunk = (kr >> 3) ^ (n & 7);
                    sb16[(n * kChunks + chunk) * 8 + (kr & 7)] = h;
                }
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

    const int frow = lane & 31;  // row of the 32-row fragment this lane reads
    const int fhalf = lane >> 5; // which 8-wide K chunk of the 16-wide step

    auto compute_tile = [&](int cur) {
        const u32x4 *sa = lds + cur * STAGE;
        const u32x4 *sb = sa + A_CHUNKS;
        constexpr int SLOTS = FRAG_DB ? 2 : 1;
        u32x4 af[SLOTS][TM], bf[SLOTS][TN];
        auto read_frags = [&](int ks, int slot) {
            const int chunk = 2 * ks + fhalf;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int row = wm * WTM + i * 32 + frow;
                af[slot][i] = sa[row * kChunks + (chunk ^ (row & 7))];
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int row = wn * WTN + j * 32 + frow;
                bf[slot][j] = sb[row * kChunks + (chunk ^ (row & 7))];
            }
        };
        if constexpr (FRAG_DB) read_frags(0, 0);
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) {
            if constexpr (FRAG_DB) {
                if (ks + 1 < kBK / 16) read_frags(ks + 1, (ks + 1) & 1);
            } else {
                read_frags(ks, 0);
            }
            const int slot = FRAG_DB ? (ks & 1) : 0;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = mfma16<BF16>(bf[slot][j], af[slot][i], acc[i][j]);
        }
    };

    // One K tile.  REG_STAGES = 2: start the loads of tile kt+2, multiply tile kt out of LDS,
    // then move tile kt+1 (loaded one step earlier) from registers to the other LDS stage.
    // REG_STAGES = 1: the same with the loads of tile kt+1 started at the top of the step.
    auto step = [&](int kt, auto parity) {
        constexpr int P = decltype(parity)::value;  // kt & 1
        constexpr int LOAD_SLOT = REG_STAGES == 2 ? P : 0;
        constexpr int STORE_SLOT = REG_STAGES == 2 ? (P ^ 1) : 0;
        if (kt + REG_STAGES < KT) load_global(kt + REG_STAGES, std::integral_constant<int, LOAD_SLOT>{});
        compute_tile(P);
        if (kt + 1 < KT) store_lds(P ^ 1, std::integral_constant<int, STORE_SLOT>{});
        lds_barrier();
    };

    load_global(0, std::integral_constant<int, 0>{});
    store_lds(0, std::integral_constant<int, 0>{});
    if constexpr (REG_STAGES == 2) {
        if (KT > 1) load_global(1, std::integral_constant<int, 1>{});
    }
    lds_barrier();
    for (int kt = 0; kt < KT; kt += 2) {
        step(kt, std::integral_constant<int, 0>{});
        if (kt + 1 < KT) step(kt + 1, std::integral_constant<int, 1>{});
    }

    // Epilogue.  acc[i][j][4q + e] is D[m][n] with m = tile row (lane % 32) and
    // n = 8q + 4*(lane / 32) + e: four consecutive columns per (i, j, q).
    const float alpha = p.alpha, beta = p.beta;
    const bool use_c = p.C != nullptr && beta != 0.0f;

    if (!EDGE && !use_c) {
        // Full tiles, no C: each wave transposes its own tile through LDS (free now: the last
        // barrier of the K loop is behind every wave) and writes whole 16-byte chunks, a
        // contiguous WTN*2-byte run per row.  8-byte units of a row are XOR-swizzled with the
        // row index: the accumulator writes (32 consecutive rows, one unit) and the row reads
        // (all chunks of a row) are then both free of bank conflicts; a chunk read from an odd
        // row has its two units swapped.
        constexpr int ROW_CHUNKS = WTN / 8;         // 16-byte chunks per row of the wave tile
        constexpr int ROWS_PER_ITER = 64 / ROW_CHUNKS;
        constexpr int SWZ = (2 * ROW_CHUNKS < 16 ? 2 * ROW_CHUNKS : 16) - 1;  // swizzle stays inside the row
        static_assert(BM * BN * 2 <= 2 * STAGE * 16, "epilogue tile must fit the pipeline LDS");
        u32x2 *region8 = reinterpret_cast<u32x2 *>(lds) + wave * (WTM * WTN / 4);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int row = i * 32 + frow;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int unit = j * 8 + 2 * q + fhalf;
                    u32x2 o;
                    o[0] = from_float<BF16>(alpha * acc[i][j][4 * q]) |
                           (static_cast<uint32_t>(from_float<BF16>(alpha * acc[i][j][4 * q + 1])) << 16);
                    o[1] = from_float<BF16>(alpha * acc[i][j][4 * q + 2]) |
                           (static_cast<uint32_t>(from_float<BF16>(alpha * acc[i][j][4 * q + 3])) << 16);
                    region8[row * (2 * ROW_CHUNKS) + (unit ^ (row & SWZ))] = o;
                }
            }
        }
        wave_lds_fence();
        const u32x4 *region16 = reinterpret_cast<const u32x4 *>(region8);
        const int c = lane % ROW_CHUNKS;
#pragma unroll
        for (int it = 0; it < WTM / ROWS_PER_ITER; ++it) {
            const int row = it * ROWS_PER_ITER + lane / ROW_CHUNKS;
            u32x4 v = region16[row * ROW_CHUNKS + (c ^ ((row & SWZ) >> 1))];
            if (row & 1) v = u32x4{v[2], v[3], v[0], v[1]};
            const int gm = m0 + wm * WTM + row;
            const int gn = n0 + wn * WTN + c * 8;
            *reinterpret_cast<u32x4 *>(p.D + static_cast<int64_t>(gm) * N + gn) = v;
        }
        return;
    }

    const bool vec_ok = (N & 3) == 0;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm * WTM + i * 32 + frow;
        if (EDGE && m >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = n0 + wn * WTN + j * 32 + 8 * q + 4 * fhalf;
                if (EDGE && n >= N) continue;
                const int64_t off = static_cast<int64_t>(m) * N + n;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = alpha * acc[i][j][4 * q + e];
                if (!EDGE || vec_ok) {  // n is a multiple of 4 and n + 3 < N
                    if (use_c) {
                        const u32x2 c2 = *reinterpret_cast<const u32x2 *>(p.C + off);
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            v[e] += beta * to_float<BF16>(static_cast<uint16_t>(c2[e >> 1] >> ((e & 1) * 16)));
                    }
                    u32x2 o;
                    o[0] = from_float<BF16>(v[0]) | (static_cast<uint32_t>(from_float<BF16>(v[1])) << 16);
                    o[1] = from_float<BF16>(v[2]) | (static_cast<uint32_t>(from_float<BF16>(v[3])) << 16);
                    *reinterpret_cast<u32x2 *>(p.D + off) = o;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (n + e < N) {
                            float t = v[e];
                            if (use_c) t += beta * to_float<BF16>(p.C[off + e]);
                            p.D[off + e] = from_float<BF16>(t);
                        }
                    }
                }
            }
        }
    }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int REG_STAGES, bool FRAG_DB, bool BF16, bool B_ROW_MAJOR,
          bool EDGE>
int launch_edge(const Params &p, hipStream_t stream) {
    constexpr int THREADS = 64 * WAVES_M * WAVES_N;
    constexpr size_t lds_bytes = 2u * (BM + BN) * kBK * sizeof(uint16_t);
    auto kernel = gemm16_kernel<BM, BN, WAVES_M, WAVES_N, REG_STAGES, FRAG_DB, BF16, B_ROW_MAJOR, EDGE>;
    static bool configured = false;  // per instantiation
    if (!configured) {
        KO_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
        configured = true;
    }
    kernel<<<dim3(static_cast<unsigned>(p.nblocks)), dim3(THREADS), lds_bytes, stream>>>(p);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int REG_STAGES, bool FRAG_DB, bool BF16, bool B_ROW_MAJOR>
int launch(Params p, hipStream_t stream) {
    const int tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    p.nblocks = tiles_m * p.tiles_n;
    const bool edge = (p.M % BM) != 0 || (p.N % BN) != 0 || (p.K % kBK) != 0;
    if (edge) return launch_edge<BM, BN, WAVES_M, WAVES_N, REG_STAGES, FRAG_DB, BF16, B_ROW_MAJOR, true>(p, stream);
    return launch_edge<BM, BN, WAVES_M, WAVES_N, REG_STAGES, FRAG_DB, BF16, B_ROW_MAJOR, false>(p, stream);
}

template <bool BF16, bool B_ROW_MAJOR>
int launch_variant(const Params &p, hipStream_t stream) {
    int variant = tuning("gemm16.variant");
    if (variant <= 0) {
        // Large problems: 256x256 tiles; small ones: 128x128 so that the grid still fills the chip.
        const int64_t big_tiles = static_cast<int64_t>((p.M + 255) / 256) * ((p.N + 255) / 256);
        variant = big_tiles >= compute_units() ? 6 : 3;
    }
    switch (variant) {
        case 1: return launch<256, 256, 2, 2, 1, true, BF16, B_ROW_MAJOR>(p, stream);
        case 2: return launch<256, 256, 2, 4, 2, false, BF16, B_ROW_MAJOR>(p, stream);
        case 3: return launch<128, 128, 2, 2, 2, true, BF16, B_ROW_MAJOR>(p, stream);
        case 4: return launch<256, 128, 2, 2, 2, true, BF16, B_ROW_MAJOR>(p, stream);
        case 5: return launch<128, 256, 2, 2, 2, true, BF16, B_ROW_MAJOR>(p, stream);
        case 6: return launch<256, 256, 2, 4, 1, true, BF16, B_ROW_MAJOR>(p, stream);
        case 7: return launch<256, 256, 4, 2, 2, false, BF16, B_ROW_MAJOR>(p, stream);
        case 8: return launch<256, 128, 2, 4, 2, true, BF16, B_ROW_MAJOR>(p, stream);
        default: return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: unknown variant %d", variant);
    }
}

}  // namespace
}  // namespace ko

KO_EXPORT int ko_gemm_f16f32acc(int64_t m, int64_t n, int64_t k, float alpha, const void *A,
                                const void *B, int b_layout, float beta, const void *C, void *D,
                                int in_dtype, ko_stream_t stream) {
    using namespace ko;
    if (m < 0 || n < 0 || k < 0)
        return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: m=%lld n=%lld k=%lld", (long long)m, (long long)n, (long long)k);
    if (in_dtype != KO_F16 && in_dtype != KO_BF16) return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: in_dtype=%d", in_dtype);
    if (b_layout != KO_ROW_MAJOR && b_layout != KO_COL_MAJOR)
        return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: b_layout=%d", b_layout);
    if (m == 0 || n == 0) return KO_OK;
    if (k == 0 || k % 8 != 0)
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: k=%lld must be a positive multiple of 8", (long long)k);
    if (m > (1 << 30) || n > (1 << 30) || k > (1 << 30))
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: dimension too large");
    if (!A || !B || !D) return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: null A/B/D pointer");
    uintptr_t align = reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B);
    if (align & 15) return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: A and B must be 16-byte aligned");
    if ((reinterpret_cast<uintptr_t>(D) | reinterpret_cast<uintptr_t>(C)) & 7)
        return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: C and D must be 8-byte aligned");
    Params p{static_cast<const uint16_t *>(A), static_cast<const uint16_t *>(B),
             static_cast<const uint16_t *>(C), static_cast<uint16_t *>(D),
             static_cast<int>(m), static_cast<int>(n), static_cast<int>(k), alpha, beta, 0, 0};
    hipStream_t s = as_stream(stream);
    if (in_dtype == KO_F16)
        return b_layout == KO_COL_MAJOR ? launch_variant<false, false>(p, s) : launch_variant<false, true>(p, s);
    return b_layout == KO_COL_MAJOR ? launch_variant<true, false>(p, s) : launch_variant<true, true>(p, s);
}
