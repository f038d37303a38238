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
#include <utility>

// This file is compiled four times, once per combination of operand type and layout of B - the kernels of one
// combination take over a minute to compile: by itself for binary16 operands and a column-major B, together with the
// entry points, and through ko_gemm16_f16_row.hip, ko_gemm16_bf16_col.hip and ko_gemm16_bf16_row.hip, which set the
// three macros and include it.  Each part defines its gemm16_run<BF16, B_ROW_MAJOR>.
#ifndef KO_GEMM16_BF16
#define KO_GEMM16_BF16 0
#define KO_GEMM16_B_ROW 0
#define KO_GEMM16_ENTRY 1
#endif

namespace ko {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
// The same vectors where only the element's own alignment is known: rows of C and D start on 2-byte boundaries when
// the row stride is not a multiple of 8.  Global memory takes 8- and 16-byte accesses at any element boundary (the
// compiler emits the same one instruction for them), so such rows keep the coalesced epilogue.
typedef u32x4 u32x4_rows __attribute__((aligned(2)));
typedef u32x2 u32x2_rows __attribute__((aligned(2)));

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

// Two floats -> two 16-bit values in one register (low half first), each rounded to nearest even by the
// hardware conversions (v_cvt_pk_bf16_f32 / v_cvt_f16_f32).
template <bool BF16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef float float2v __attribute__((ext_vector_type(2)));
    if constexpr (BF16) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2v{lo, hi}, bf16x2));
    } else {
        typedef _Float16 half2v __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2v{lo, hi}, half2v));
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

using Params = Gemm16Params;  // (ko_internal.h: the four parts this file is compiled into share it)

// x/2 (1 + tanh u) = x / (1 + exp(-2u)) with u = sqrt(2/pi) (x + 0.044715 x^3), written as
// x * rcp(1 + 2^(x (c1 + c2 x^2))), c1 = -2 sqrt(2/pi) log2(e), c2 = 0.044715 c1: two multiplies, one FMA,
// one add and the hardware 2^x and reciprocal (about 1 ulp each; the result is rounded to 16 bits next).
// Large negative x: 2^(+big) = inf, rcp = 0, result -0; large positive x: 2^(-big) = 0, result x.
__device__ __forceinline__ float gelu_tanh(float x) {
    constexpr float c1 = -2.0f * 0.79788456080286535588f * 1.44269504088896340736f;
    constexpr float c2 = 0.044715f * c1;
    const float t = x * __builtin_fmaf(c2 * x, x, c1);
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t));
}

// Epilogue of one group of four consecutive columns n .. n+3 of row m (all inside the matrix):
// v = act(alpha * acc + beta * C + bias).  c2 and b2 hold the group's four C and bias values (8 bytes
// each, loaded by the caller - several groups at a time, so that the loads overlap).
template <bool BF16>
__device__ __forceinline__ void finish4(const Params &p, float (&v)[4], u32x2 c2, u32x2 b2, bool use_c) {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] *= p.alpha;
    if (use_c) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += p.beta * to_float<BF16>(static_cast<uint16_t>(c2[e >> 1] >> ((e & 1) * 16)));
    }
    if (p.bias) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += to_float<BF16>(static_cast<uint16_t>(b2[e >> 1] >> ((e & 1) * 16)));
    }
    if (p.act == KO_ACT_GELU_ERF) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = 0.5f * v[e] * (1.0f + erff(v[e] * 0.70710678118654752440f));
    } else if (p.act == KO_ACT_GELU_TANH) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = gelu_tanh(v[e]);
    }
}

// Persistent kernels: tile number t (0, 1, ...) of workgroup b when the grid has `grid` workgroups.
// Workgroup b runs on XCD b % 8 and is the (b / 8)-th of the workgroups there.  With band_rows > 0
// the tile grid is cut into 8 regions, 8 >> xcd_cols_log2 of them below each other and 1 << xcd_cols_log2
// side by side, one per XCD, each band_rows rows of tiles high and region_cols columns wide (the whole width
// when they all lie below each other); an XCD walks its region in blocks of block_cols columns: the
// workgroups that are resident on it at a time cover a band_rows x block_cols block of tiles, a compact
// footprint (few distinct A and B panels) in their shared L2, and the A panels of the band are reused
// from block to block.  Otherwise tiles are dealt in row-major order from one contiguous range per XCD.
__device__ __forceinline__ void tile_of(const Params &p, int b, int grid, int t, int &tile_m, int &tile_n) {
    if (p.band_rows > 0) {
        const int x = b & 7, j = b >> 3;
        const int xr = x >> p.xcd_cols_log2, xc = x & ((1 << p.xcd_cols_log2) - 1);  // the XCD's place among the regions
        tile_m = xr * p.band_rows + j % p.band_rows;
        tile_n = xc * p.region_cols + t * p.block_cols + j / p.band_rows;
    } else {
        const int tile = xcd_remap(b + grid * t, p.nblocks);
        tile_m = tile / p.tiles_n;
        tile_n = tile % p.tiles_n;
    }
}

// EDGE = false: M % BM == 0, N % BN == 0 and K % 64 == 0, so no load or store needs a bounds check.
// Writes one wave's WTM x WTN accumulator tile to D (rows row0.., columns col0..).
// acc[i][j][4q + e] is D[m][n] with m = 32i + lane % 32 and n = 32j + 8q + 4*(lane / 32) + e:
// four consecutive columns per (i, j, q).  `region` is this wave's own piece of LDS, free for reuse.
// The LDS transpose runs in PARTS passes over WTM / PARTS rows each, so that a wave needs
// only WTM * WTN * 2 / PARTS bytes of LDS.
// WAIT_VM: wait for this wave's outstanding vector memory operations right before the first global store
// (the caller has loads in flight that it wants confirmed while they are still the only ones outstanding).
// GUARD_M (full-tile form): the tile may reach past row M - rows at or past M hold the products of rows fetched from
// elsewhere in A: they take no C and are not stored.
// STREAM (full-tile form): the stores are streaming (non-temporal) ones - see store_tile below, which chooses.
template <int WTM, int WTN, int SWIZZLE, bool BF16, bool EDGE, int PARTS, bool WAIT_VM, bool GUARD_M, bool STREAM>
__device__ __forceinline__ void store_tile_as(const Params &p, float16v (&acc)[WTM / 32][WTN / 32], u32x4 *region,
                                              int lane, int row0, int col0) {
    constexpr int TM = WTM / 32, TN = WTN / 32;
    const int M = p.M, N = p.N;
    const int64_t ldd = p.ldd;
    const int frow = lane & 31, fhalf = lane >> 5;
    const float alpha = p.alpha;
    const bool use_c = p.C != nullptr && p.beta != 0.0f;
    const bool plain = !use_c && p.bias == nullptr && p.act == KO_ACT_NONE;  // D = alpha * acc

    if (!EDGE) {
        // Full tiles: each wave transposes its own tile through LDS (free now: the last
        // barrier of the K loop is behind every wave) and writes whole 16-byte chunks, a
        // contiguous WTN*2-byte run per row.  8-byte units of a row are XOR-swizzled with the
        // row index: the accumulator writes (32 consecutive rows, one unit) and the row reads
        // (all chunks of a row) are then both free of bank conflicts; a chunk read from an odd
        // row has its two units swapped.
        constexpr int ROW_CHUNKS = WTN / 8;         // 16-byte chunks per row of the wave tile
        constexpr int ROWS_PER_ITER = 64 / ROW_CHUNKS;
        constexpr int SWZ = (2 * ROW_CHUNKS < 16 ? 2 * ROW_CHUNKS : 16) - 1;  // swizzle stays inside the row
        // rows of WTN*2 = 128 bytes pair up into one 64-bank line: then the row pair index drives the swizzle
        auto erow = [](int row) { return (SWIZZLE == 1 && WTN * 2 <= 128) ? (row >> 1) : row; };
        constexpr int PTM = TM / PARTS;             // 32-row blocks per pass
        constexpr int PROWS = WTM / PARTS;          // rows per pass
        static_assert(TM % PARTS == 0, "");
        u32x2 *region8 = reinterpret_cast<u32x2 *>(region);
        const u32x4 *region16 = reinterpret_cast<const u32x4 *>(region8);
        const int c = lane % ROW_CHUNKS;
        // the bias of this lane's column groups, once per tile
        u32x2 bias_q[TN][4];
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                bias_q[j][q] = u32x2{0, 0};
                if (p.bias) bias_q[j][q] = *reinterpret_cast<const u32x2 *>(p.bias + col0 + j * 32 + 8 * q + 4 * fhalf);
            }
#pragma unroll
        for (int part = 0; part < PARTS; ++part) {
            if (part > 0) wave_lds_fence();  // the previous pass has read its rows
#pragma unroll
            for (int ii = 0; ii < PTM; ++ii) {
                const int i = part * PTM + ii;
                const int row = ii * 32 + frow;
                // C of this 32-row block: all loads first, so that their latencies overlap
                u32x2 c_q[TN][4];
                if (use_c) {
                    // (a row at or past M reads the matrix's last row instead: a valid address, a value never stored)
                    const int crow_index = GUARD_M && row0 + i * 32 + frow >= M ? M - 1 : row0 + i * 32 + frow;
                    const uint16_t *crow = p.C + crow_index * ldd + col0 + 4 * fhalf;
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q) c_q[j][q] = *reinterpret_cast<const u32x2_rows *>(crow + j * 32 + 8 * q);
                }
#pragma unroll
                for (int j = 0; j < TN; ++j) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int unit = j * 8 + 2 * q + fhalf;
                        float v[4] = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                        if (plain) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] *= alpha;
                        } else {  // C, bias and the activation enter before the one rounding to 16 bits
                            finish4<BF16>(p, v, use_c ? c_q[j][q] : u32x2{0, 0}, bias_q[j][q], use_c);
                        }
                        u32x2 o;
                        o[0] = pack2<BF16>(v[0], v[1]);
                        o[1] = pack2<BF16>(v[2], v[3]);
                        region8[row * (2 * ROW_CHUNKS) + (unit ^ (erow(row) & SWZ))] = o;
                    }
                }
            }
            wave_lds_fence();
            if constexpr (WAIT_VM) {
                if (part == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
#pragma unroll
            for (int it = 0; it < PROWS / ROWS_PER_ITER; ++it) {
                const int row = it * ROWS_PER_ITER + lane / ROW_CHUNKS;
                u32x4 v = region16[row * ROW_CHUNKS + (c ^ ((erow(row) & SWZ) >> 1))];
                if (erow(row) & 1) v = u32x4{v[2], v[3], v[0], v[1]};
                const int gm = row0 + part * PROWS + row;
                const int gn = col0 + c * 8;
                if (!GUARD_M || gm < M) {
                    if constexpr (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<u32x4_rows *>(p.D + gm * ldd + gn));
                    else *reinterpret_cast<u32x4_rows *>(p.D + gm * ldd + gn) = v;
                }
            }
        }
        return;
    }

#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = row0 + i * 32 + frow;
        if (EDGE && m >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = col0 + j * 32 + 8 * q + 4 * fhalf;
                if (EDGE && n >= N) continue;
                const int64_t off = m * ldd + n;
                float v[4] = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                if (!EDGE || n + 3 < N) {  // the group's four columns are inside the matrix (n is a multiple of 4)
                    u32x2 c2 = {0, 0}, b2 = {0, 0};
                    if (use_c) c2 = *reinterpret_cast<const u32x2_rows *>(p.C + off);
                    if (p.bias) b2 = *reinterpret_cast<const u32x2 *>(p.bias + n);
                    finish4<BF16>(p, v, c2, b2, use_c);
                    u32x2 o;
                    o[0] = pack2<BF16>(v[0], v[1]);
                    o[1] = pack2<BF16>(v[2], v[3]);
                    *reinterpret_cast<u32x2_rows *>(p.D + off) = o;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (n + e < N) {
                            float t = alpha * v[e];
                            if (use_c) t += p.beta * to_float<BF16>(p.C[off + e]);
                            if (p.bias) t += to_float<BF16>(p.bias[n + e]);
                            if (p.act == KO_ACT_GELU_ERF) t = 0.5f * t * (1.0f + erff(t * 0.70710678118654752440f));
                            else if (p.act == KO_ACT_GELU_TANH) t = gelu_tanh(t);
                            p.D[off + e] = from_float<BF16>(t);
                        }
                    }
                }
            }
        }
    }
}

// The epilogue with the kind of store that the rows of D ask for, chosen once per tile (the two forms are two copies of
// the code: a choice per store inside the loop cost the 16384 x 3072 x 768 problem 6 us - and the persistent kernels,
// whose tiles are whole 256-column ones of rows that as a rule start on such boundaries, keep the one streaming copy).  D is written once and not read
// again, and while its rows start on 64-byte boundaries a wave's 128-byte row segments are whole sectors and streaming
// (non-temporal) stores are the faster ones (that problem, on operand sets that rotate through more than the caches
// hold: 77 us against 85 with plain stores).  Off such boundaries the segments end inside sectors that a neighbouring
// wave or tile completes; streamed out, each part goes to memory on its own, and the kernel takes a third longer
// (4096 x 11928 x 64: 44.1 us, with plain stores - which meet in the L2 - 35.0; 9329 x 4948 x 32 44.3 / 34.6).
template <int WTM, int WTN, int SWIZZLE, bool BF16, bool EDGE, int PARTS = 1, bool WAIT_VM = false, bool GUARD_M = false>
__device__ __forceinline__ void store_tile(const Params &p, float16v (&acc)[WTM / 32][WTN / 32], u32x4 *region,
                                           int lane, int row0, int col0) {
    if (EDGE || (p.ldd & 31) == 0)
        store_tile_as<WTM, WTN, SWIZZLE, BF16, EDGE, PARTS, WAIT_VM, GUARD_M, true>(p, acc, region, lane, row0, col0);
    else
        store_tile_as<WTM, WTN, SWIZZLE, BF16, EDGE, PARTS, WAIT_VM, GUARD_M, false>(p, acc, region, lane, row0, col0);
}

// Tiling of one kernel instantiation.
// REG_STAGES = 2: global loads run two K tiles ahead (two sets of staging registers);
// REG_STAGES = 1: one tile ahead.  FRAG_DB: fragments of the next K step are read into a
// second register set while the MFMAs of the current step run.  SWIZZLE selects the row
// function XOR-ed into the chunk index of the LDS stages: 0 = row % 8 (conflict free for 8
// consecutive rows when two rows share a bank line of 32 banks), 1 = (row / 2) % 8 (conflict
// free for 16 consecutive rows on 64 banks, where two 128-byte rows make one bank line).
template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int REG_STAGES_, bool FRAG_DB_, int SWIZZLE_,
          bool SPARE_EPILOGUE_ = false, bool SPREAD_LOADS_ = false>
struct Tiling {
    static constexpr bool SPARE_EPILOGUE = SPARE_EPILOGUE_;  // pinned kernel: see SPARE there
    static constexpr bool SPREAD_LOADS = SPREAD_LOADS_;      // pinned kernel with SPARE: loads one by one in K step 3
    static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, REG_STAGES = REG_STAGES_;
    static constexpr bool FRAG_DB = FRAG_DB_;
    static constexpr int SWIZZLE = SWIZZLE_;
    static constexpr int THREADS = 64 * WAVES_M * WAVES_N;
};

template <int SWIZZLE>
__device__ __forceinline__ int swz(int row) {
    if constexpr (SWIZZLE == 1) return (row >> 1) & 7;
    else return row & 7;
}

// B fragment of a 32x32x16 MFMA out of a row-major [k][BN] LDS tile (16-byte chunks swizzled with k & 3, see the
// store): columns n0 .. n0+31, rows k0 .. k0+7 for this lane's half of the K step.  ds_read_b64_tr_b16 works on
// groups of 16 lanes: lane i of a group supplies the address of four consecutive 16-bit values (here: row
// k + i / 4, columns 4 * (i % 4) .. + 3 of the group's 16 columns) and receives, of the 16 x 4 values the group
// read, column i of rows 0..3 - i.e. the four k values of its own column n0 + i.  Two reads give the eight
// consecutive k that the MFMA wants per lane.
template <int BN>
__device__ __forceinline__ u32x4 read_b_transposed(const u32x4 *sb, int k0, int n0, int lane) {
    typedef short short4v __attribute__((ext_vector_type(4)));
    typedef short short8v __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) short4v *lds_ptr;
    constexpr int NCH = BN / 8;
    const int i = lane & 15, g = (lane >> 4) & 1;
    const int kq = i >> 2;  // row within the four rows of one read (k0 is a multiple of 4: (k0 + kq) & 3 == kq)
    const int chunk = ((n0 + g * 16 + 4 * (i & 3)) >> 3) ^ ((kq << 2) & (NCH - 1));
    const char *base = reinterpret_cast<const char *>(sb) + ((k0 + kq) * NCH + chunk) * 16 + (i & 1) * 8;
    const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(base));
    const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(base + 4 * NCH * 16));
    return __builtin_bit_cast(u32x4, static_cast<short8v>(__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7)));
}

// Floats between rows of a partial product: N rounded up to whole groups of four columns, so that every group a
// lane holds is stored and fetched as one aligned 16-byte access whatever N is.
__host__ __device__ __forceinline__ int64_t partial_ld(int n) { return (static_cast<int64_t>(n) + 3) & ~int64_t{3}; }

// The problem a workgroup of a K-sliced launch works on: its K range of A and B, its own partial product.
template <bool B_ROW_MAJOR>
__device__ __forceinline__ Params slice_of(Params p) {
    if (p.k_slice > 0) {
        const int s = static_cast<int>(blockIdx.y);
        const int k0 = s * p.k_slice;
        p.A += k0;
        p.B += B_ROW_MAJOR ? static_cast<int64_t>(k0) * p.ldb : static_cast<int64_t>(k0);
        p.partial += static_cast<int64_t>(s) * p.M * partial_ld(p.N);
        p.K = p.K - k0 < p.k_slice ? p.K - k0 : p.k_slice;
    }
    return p;
}

// One wave's accumulator tile as fp32 into a partial product.  A lane's four consecutive columns start at a
// multiple of 4: a group that starts inside the matrix ends inside the padded row.
template <int WTM, int WTN>
__device__ __forceinline__ void store_partial(const Params &p, float16v (&acc)[WTM / 32][WTN / 32], int lane, int row0,
                                              int col0) {
    typedef float float4v __attribute__((ext_vector_type(4)));
    const int frow = lane & 31, fhalf = lane >> 5;
#pragma unroll
    for (int i = 0; i < WTM / 32; ++i) {
        const int m = row0 + i * 32 + frow;
        if (m >= p.M) continue;
#pragma unroll
        for (int j = 0; j < WTN / 32; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = col0 + j * 32 + 8 * q + 4 * fhalf;
                if (n >= p.N) continue;
                const float4v v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                *reinterpret_cast<float4v *>(p.partial + m * partial_ld(p.N) + n) = v;
            }
    }
}

// Sixteen bytes of zeros in device memory: what a load fetches in place of a chunk that lies past the end of K.
__device__ __attribute__((aligned(16))) const uint32_t zero_chunk16[4] = {0u, 0u, 0u, 0u};

template <class T, bool BF16, bool B_ROW_MAJOR, bool EDGE>
__global__ __launch_bounds__(T::THREADS) void gemm16_kernel(const Params whole) {
    const Params p = slice_of<B_ROW_MAJOR>(whole);
    constexpr int BM = T::BM, BN = T::BN, WAVES_M = T::WAVES_M, WAVES_N = T::WAVES_N, REG_STAGES = T::REG_STAGES;
    constexpr bool FRAG_DB = T::FRAG_DB;
    constexpr int SWIZZLE = T::SWIZZLE;
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
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: lets address math run on the scalar unit
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    const int tile = xcd_remap(blockIdx.x, p.nblocks);
    const int m0 = (tile / p.tiles_n) * BM;
    const int n0 = (tile % p.tiles_n) * BN;
    const int M = p.M, N = p.N, K = p.K;
    const int ldk = p.ldk;

    const int KT = (K + kBK - 1) / kBK;

    // Two register stages: the tile two steps ahead is in flight from global memory
    // while the tile one step ahead waits to be written to LDS.
    u32x4 ra[REG_STAGES][A_ITERS], rb[REG_STAGES][B_ITERS];

    // Full tiles: the address of a 16-byte chunk is a wave-uniform base (tile origin, step i
    // and K tile: scalar registers) plus a per-lane byte offset that never changes, so the
    // loads need one offset register instead of a 64-bit pointer each.
    constexpr int ROWS_PER_ITER = THREADS / kChunks;  // rows covered by one load instruction of the workgroup
    const uint32_t lane_off_a = static_cast<uint32_t>((tid / kChunks) * ldk + (tid % kChunks) * 8) * 2u;

    // EDGE: no load sits under a per-lane branch - the compiler could not count the loads in flight behind one
    // and would wait for all of them, the tile fetched ahead included, before it touches the older set.  Each
    // lane keeps the addresses of its chunks of K tile 0, rows past M or N clamped to the last one (they feed
    // outputs that are never stored); in the last K tile the chunks at or past K are fetched from a chunk of
    // zeros instead (a select of the address, not a branch).
    // Row-major B: a chunk of eight columns that begins past N starts at column 0 instead, and one that ends past
    // N is fetched whole where the next row of B lies behind it - columns past N of B only reach columns past N
    // of D.  That needs a row of at least eight columns and is not done in the last K tile, whose elements are
    // fetched one by one, again from zeros where they lie past N or K; shorter rows go that way in every K tile.
    // (the chunk of zeros and the operands are both global memory: said in the pointer type, or the loads become
    // flat ones, which also count as LDS operations)
    typedef const __attribute__((address_space(1))) u32x4 *global_chunk_t;
    typedef const __attribute__((address_space(1))) uint16_t *global_elem_t;
    typedef const __attribute__((address_space(1))) u32x4_rows *global_rows_t;
    const uint16_t *edge_a[EDGE ? A_ITERS : 1], *edge_b[EDGE ? B_ITERS : 1];
    const uint16_t *const zeros = reinterpret_cast<const uint16_t *>(&zero_chunk16);
    const bool past_k_last = (tid % kChunks) * 8 >= K - (KT - 1) * kBK;  // this lane's chunk of the last K tile (A, column-major B)
    if constexpr (EDGE) {
#pragma unroll
        for (int i = 0; i < A_ITERS; ++i) {
            const int idx = tid + i * THREADS;
            const int gr = m0 + idx / kChunks;
            edge_a[i] = p.A + static_cast<int64_t>(gr < M ? gr : M - 1) * ldk + (idx % kChunks) * 8;
        }
#pragma unroll
        for (int i = 0; i < B_ITERS; ++i) {
            const int idx = tid + i * THREADS;
            if constexpr (B_ROW_MAJOR) {
                constexpr int NCH = BN / 8;
                const int gn = n0 + (idx % NCH) * 8;
                edge_b[i] = p.B + static_cast<int64_t>(idx / NCH) * p.ldb + (gn < N ? gn : 0);
            } else {
                const int gr = n0 + idx / kChunks;
                edge_b[i] = p.B + static_cast<int64_t>(gr < N ? gr : N - 1) * ldk + (idx % kChunks) * 8;
            }
        }
    }
    // The addresses run along with the K tile they point at, in their own registers: an address formed in a
    // temporary per load would take the registers of a load still in flight and wait for it.
    int edge_kt = 0;                                  // the K tile edge_a and edge_b point at
    const bool whole_chunks = !B_ROW_MAJOR || N >= 8; // K tiles before the last one need no per-lane care

    auto load_global = [&](int kt, auto slot) {
        constexpr int S = decltype(slot)::value;
        const int k0 = kt * kBK;
        if constexpr (EDGE) {
            const int64_t ahead = static_cast<int64_t>(kt - edge_kt) * kBK;  // wave-uniform; K tiles are asked for in rising order
            edge_kt = kt;
            const bool last = kt == KT - 1;  // wave-uniform
            // in the last K tile (which may be asked for again, never left) the chunks at or past K turn to the zeros
            const bool to_zeros = last && past_k_last;
#pragma unroll
            for (int i = 0; i < A_ITERS; ++i) edge_a[i] = to_zeros ? zeros : edge_a[i] + ahead;
#pragma unroll
            for (int i = 0; i < B_ITERS; ++i) {
                if constexpr (B_ROW_MAJOR) edge_b[i] += ahead * p.ldb;
                else edge_b[i] = to_zeros ? zeros : edge_b[i] + ahead;
            }
            if constexpr (B_ROW_MAJOR) {
                // both sides of this branch issue their loads unmasked, so the loads in flight can still be counted
                if (!last && whole_chunks) {
#pragma unroll
                    for (int i = 0; i < A_ITERS; ++i) ra[S][i] = *(global_chunk_t)edge_a[i];
#pragma unroll
                    for (int i = 0; i < B_ITERS; ++i) rb[S][i] = *(global_rows_t)edge_b[i];
                    return;
                }
            }
#pragma unroll
            for (int i = 0; i < A_ITERS; ++i) ra[S][i] = *(global_chunk_t)edge_a[i];
#pragma unroll
            for (int i = 0; i < B_ITERS; ++i) {
                if constexpr (!B_ROW_MAJOR) {
                    rb[S][i] = *(global_chunk_t)edge_b[i];
                } else {
                    const int idx = tid + i * THREADS;
                    constexpr int NCH = BN / 8;
                    const int gk = k0 + idx / NCH;
                    const int gn = n0 + (idx % NCH) * 8;
                    const uint16_t *src = p.B + static_cast<int64_t>(gk) * p.ldb + gn;
                    uint32_t t[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) t[e] = *(global_elem_t)(gk < K && gn + e < N ? src + e : zeros);
                    rb[S][i] = u32x4{t[0] | (t[1] << 16), t[2] | (t[3] << 16), t[4] | (t[5] << 16), t[6] | (t[7] << 16)};
                }
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < A_ITERS; ++i) {
            const char *base = reinterpret_cast<const char *>(p.A + static_cast<int64_t>(m0 + i * ROWS_PER_ITER) * ldk + k0);
            ra[S][i] = *reinterpret_cast<const u32x4 *>(base + lane_off_a);
        }
#pragma unroll
        for (int i = 0; i < B_ITERS; ++i) {
            if constexpr (!B_ROW_MAJOR) {
                const char *base = reinterpret_cast<const char *>(p.B + static_cast<int64_t>(n0 + i * ROWS_PER_ITER) * ldk + k0);
                rb[S][i] = *reinterpret_cast<const u32x4 *>(base + lane_off_a);
            } else {
                // B[k][n] row-major: a chunk is 8 consecutive n of one k; rows of B may start at any element (ldb
                // not a multiple of 8)
                const int idx = tid + i * THREADS;
                constexpr int NCH = BN / 8;
                rb[S][i] = *reinterpret_cast<const u32x4_rows *>(p.B + static_cast<int64_t>(k0 + idx / NCH) * p.ldb + n0 + (idx % NCH) * 8);
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
            sa[row * kChunks + (c ^ swz<SWIZZLE>(row))] = ra[S][i];
        }
        if constexpr (!B_ROW_MAJOR) {
#pragma unroll
            for (int i = 0; i < B_ITERS; ++i) {
                const int idx = tid + i * THREADS;
                const int row = idx / kChunks, c = idx % kChunks;
                sb[row * kChunks + (c ^ swz<SWIZZLE>(row))] = rb[S][i];
            }
        } else {
            // Row-major B stays row-major in LDS ([k][n], 16-byte chunks of 8 consecutive n); the chunk index is
            // swizzled with k & 3 so that the four k rows one transposing read touches lie in different banks.
#pragma unroll
            for (int i = 0; i < B_ITERS; ++i) {
                const int idx = tid + i * THREADS;
                constexpr int NCH = BN / 8;
                const int kr = idx / NCH, c = idx % NCH;
                sb[kr * NCH + (c ^ (((kr & 3) << 2) & (NCH - 1)))] = rb[S][i];  // the swizzle stays inside the row
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
                af[slot][i] = sa[row * kChunks + (chunk ^ swz<SWIZZLE>(row))];
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (!B_ROW_MAJOR) {
                    const int row = wn * WTN + j * 32 + frow;
                    bf[slot][j] = sb[row * kChunks + (chunk ^ swz<SWIZZLE>(row))];
                } else {
                    bf[slot][j] = read_b_transposed<BN>(sb, ks * 16 + fhalf * 8, wn * WTN + j * 32, lane);
                }
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
        // Past the last K tile the loads and the LDS stores are not branched around but redirected to the last
        // tile (fetched and stored once more, into the stage nobody reads any more): with loads under a branch
        // the compiler cannot count the loads in flight and waits for all of them - the set issued one step
        // ago included - before it reuses the registers of the older set.
        load_global(kt + REG_STAGES < KT ? kt + REG_STAGES : KT - 1, std::integral_constant<int, LOAD_SLOT>{});
        compute_tile(P);
        store_lds(P ^ 1, std::integral_constant<int, STORE_SLOT>{});
        lds_barrier();
    };

    load_global(0, std::integral_constant<int, 0>{});
    store_lds(0, std::integral_constant<int, 0>{});
    if constexpr (REG_STAGES == 2) load_global(KT > 1 ? 1 : 0, std::integral_constant<int, 1>{});
    lds_barrier();
    for (int kt = 0; kt < KT; kt += 2) {
        step(kt, std::integral_constant<int, 0>{});
        if (kt + 1 < KT) step(kt + 1, std::integral_constant<int, 1>{});
    }

    if (p.partial != nullptr) {
        store_partial<WTM, WTN>(p, acc, lane, m0 + wm * WTM, n0 + wn * WTN);
    } else if (!EDGE || (m0 + BM <= M && n0 + BN <= N)) {
        // a tile that lies inside the matrix takes the coalesced epilogue in the edge form of the kernel too (a
        // ragged K, or the inner tiles of a ragged M or N: 16384 x 3072 x 8 is 100 MB of output and nothing else)
        store_tile<WTM, WTN, SWIZZLE, BF16, false>(p, acc, lds + wave * (WTM * WTN / 8), lane, m0 + wm * WTM, n0 + wn * WTN);
    } else {
        store_tile<WTM, WTN, SWIZZLE, BF16, true>(p, acc, lds + wave * (WTM * WTN / 8), lane, m0 + wm * WTM, n0 + wn * WTN);
    }
}

// Direct-to-LDS kernels for full tiles with K-contiguous operands (column-major B):
// global_load_lds_dwordx4 moves 16 bytes per lane from global memory straight into LDS
// (lane l of a wave-level load fills the l-th 16-byte slot after the wave-uniform LDS
// base), so the staging registers and the ds_write instructions of the register pipeline
// disappear.  The XOR swizzle is applied on the global side: the lane that fills slot
// (row, p) fetches chunk p ^ swz(row) of that row, still one 128-byte segment per 8 lanes.
// Each wave-level load covers 8 tile rows; wave w issues loads w, w + WAVES, ...
// One K tile ahead is in flight while the current one is multiplied; a wave waits for its
// own loads (vmcnt) before the barrier that publishes the stage.
//
// Persistent form: one workgroup per compute unit walks over
// its tiles, and the K tiles of all of them form one stream through the two LDS stages.
// While the last K tile of an output tile is multiplied, the first K tile of the next
// output tile is already in flight into the other stage; the epilogue then transposes
// through the stage that was just consumed (in two passes, half of LDS), and its global
// stores drain while the next tile's main loop runs.
template <class T, bool BF16>
__global__ __launch_bounds__(T::THREADS) void gemm16_persistent_kernel(const Params p) {
    constexpr int BM = T::BM, BN = T::BN, WAVES_M = T::WAVES_M, WAVES_N = T::WAVES_N;
    constexpr bool FRAG_DB = T::FRAG_DB;
    constexpr int SWIZZLE = T::SWIZZLE;
    constexpr int WAVES = WAVES_M * WAVES_N;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int A_CHUNKS = BM * kChunks, B_CHUNKS = BN * kChunks;
    constexpr int STAGE = A_CHUNKS + B_CHUNKS;
    constexpr int A_LOADS = A_CHUNKS / 64 / WAVES, B_LOADS = B_CHUNKS / 64 / WAVES;
    constexpr int EPI_PARTS = (BM * BN * 2) / (STAGE * 16);  // passes so that the transpose fits one stage
    static_assert(WAVES % 2 == 0 && A_CHUNKS % (64 * WAVES) == 0 && B_CHUNKS % (64 * WAVES) == 0, "");
    static_assert(EPI_PARTS >= 1 && TM % EPI_PARTS == 0, "");

    extern __shared__ u32x4 lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: lets address math run on the scalar unit
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int K = p.K;
    const int KT = K / kBK;
    const int grid = gridDim.x;
    const int my_tiles = (p.nblocks - static_cast<int>(blockIdx.x) + grid - 1) / grid;
    const int total = my_tiles * KT;

    const int row_in = lane >> 3;
    const uint32_t lane_off =
        static_cast<uint32_t>(row_in * K + (((lane & 7) ^ swz<SWIZZLE>(8 * wave + row_in)) << 3)) * 2u;

    typedef const __attribute__((address_space(1))) void *gptr_t;
    typedef __attribute__((address_space(3))) void *lptr_t;

    auto tile_origin = [&](int t, int &m0, int &n0) {
        const int tile = xcd_remap(static_cast<int>(blockIdx.x) + grid * t, p.nblocks);
        m0 = (tile / p.tiles_n) * BM;
        n0 = (tile % p.tiles_n) * BN;
    };

    auto issue = [&](int step, int stage) {
        const int t = step / KT, kt = step - t * KT;
        int m0, n0;
        tile_origin(t, m0, n0);
        const int k0 = kt * kBK;
        u32x4 *dst = lds + stage * STAGE;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const int g = wave + WAVES * i;
            const char *base = reinterpret_cast<const char *>(p.A + static_cast<int64_t>(m0 + 8 * g) * K + k0);
            __builtin_amdgcn_global_load_lds((gptr_t)(base + lane_off), (lptr_t)(dst + 64 * g), 16, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            const int g = wave + WAVES * i;
            const char *base = reinterpret_cast<const char *>(p.B + static_cast<int64_t>(n0 + 8 * g) * K + k0);
            __builtin_amdgcn_global_load_lds((gptr_t)(base + lane_off), (lptr_t)(dst + A_CHUNKS + 64 * g), 16, 0, 0);
        }
    };

    float16v acc[TM][TN];
    auto clear_acc = [&]() {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
        // The zeroes are written by vector-ALU moves, and the matrix instructions that read them as their addend
        // are inline assembly: the compiler does not know them for what they are and keeps no distance between
        // such a move and the instruction that reads its register (it is free to sink the moves down to right in
        // front of the first of them).  Pin the moves here and put the wait states behind them.
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(acc[i][j]));
        asm volatile("s_nop 7");
    };
    clear_acc();

    const int frow = lane & 31;
    const int fhalf = lane >> 5;

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
                af[slot][i] = sa[row * kChunks + (chunk ^ swz<SWIZZLE>(row))];
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int row = wn * WTN + j * 32 + frow;
                bf[slot][j] = sb[row * kChunks + (chunk ^ swz<SWIZZLE>(row))];
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

    if (total == 0) return;
    issue(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
    int kt = 0, t = 0;
    for (int step = 0; step < total; ++step) {
        const int cur = step & 1;
        if (step + 1 < total) issue(step + 1, cur ^ 1);
        compute_tile(cur);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        lds_barrier();
        if (++kt == KT) {
            int m0, n0;
            tile_origin(t, m0, n0);
            // stage `cur` is free (every wave is past the barrier); stage cur^1 holds the next tile's first K tile
            store_tile_as<WTM, WTN, SWIZZLE, BF16, false, EPI_PARTS, false, false, true>(
                p, acc, lds + cur * STAGE + wave * (WTM * WTN / 8 / EPI_PARTS), lane, m0 + wm * WTM, n0 + wn * WTN);
            clear_acc();
            lds_barrier();  // the next step loads into stage `cur`
            kt = 0;
            ++t;
        }
    }
}

// Persistent direct-to-LDS kernel with a pinned inner loop.  LDS holds
// [A stage 0][A stage 1][B stage 0][B stage 1]; the byte offset of a lane's fragment for K step ks
// is precomputed once (4 registers for A, 4 for B: the swizzle term depends on the lane only), and
// the stage, the 32-row block and the operand enter as immediate offsets of ds_read_b128.  The K
// loop is unrolled by two so that the stage is a compile-time constant (hence K % 128 == 0), and
// the loads walk the K tiles with a cursor instead of dividing the step number.
// The inner loop is a fixed sequence of inline-assembly instructions so that its order is exactly
// the one below (left to itself the compiler folds the two fragment register sets into one and
// waits for every LDS read right after issuing it).  Per K tile held in stage S:
//
//   K step 0..2 : MFMA, 2 reads, MFMA, 2 reads, MFMA, 2 reads, 5 MFMA    (reads = next step's fragments)
//   wait for the LDS reads and for this wave's direct-to-LDS loads, barrier
//                                 -> stage S^1 (next K tile) is published, stage S is free
//   start the direct-to-LDS loads of the K tile after next into stage S
//   K step 3    : the same pattern, the reads being step 0 of the next K tile out of stage S^1
//
// so neither the barrier nor the first fragment reads of a K tile stand between two MFMAs.
// At the last K tile of an output tile the loads into stage S start only after the epilogue
// has used that stage for its transpose.
template <int IMM>
__device__ __forceinline__ void lds_read16(u32x4 &dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(IMM));
}

template <int IMM>
__device__ __forceinline__ void lds_read_tr(u32x2 &dst, uint32_t addr) {
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(IMM));
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

template <bool BF16>
__device__ __forceinline__ void mfma_asm(float16v &acc, const u32x4 &a, const u32x4 &b) {
    if constexpr (BF16) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}


// EDGE_K: K is any multiple of 8 and is padded with zeros up to the next multiple of 128 - a lane whose
// 16-byte chunk (or, for a row-major B, whose row) lies at or past K fetches 16 zero bytes instead, chosen per
// load with a compare and two selects, so nothing is read past the end of a row or of the matrix.
// EDGE_M: any M; the last row of tiles may reach past it.  A lane whose row of A lies at or past M fetches row
// M - 1 instead - its byte offset from the cursor, one 32-bit register per load, is recomputed once per output tile -
// a valid address, whose products land in rows of the tile that the epilogue does not store.
// SLICED: K slices.  The workgroups walk p.nblocks = p.tiles * slices pairs (slice, output tile) - tile_of's grid of
// tiles with the slices' tile grids below each other; pair
// (s, tile) multiplies k in [s * p.k_slice, (s + 1) * p.k_slice) - p.k_slice a multiple of 128, the last slice
// padded with zeros when K ends inside it (EDGE_K) - and stores its accumulators as fp32 into partial product s
// (see Params::partial) instead of the epilogue; p.K stays the whole K, the distance between rows.
template <class T, bool BF16, bool B_ROW, bool EDGE_K = false, bool EDGE_M = false, bool SLICED = false>
__global__ __launch_bounds__(T::THREADS) void gemm16_pinned_kernel(const Params p) {
    constexpr int BM = T::BM, BN = T::BN, WAVES_M = T::WAVES_M, WAVES_N = T::WAVES_N;
    constexpr int WAVES = WAVES_M * WAVES_N;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int KS = kBK / 16;
    constexpr int A_BYTES = BM * kBK * 2, B_BYTES = BN * kBK * 2;  // per stage
    constexpr int A_LOADS = A_BYTES / 1024 / WAVES, B_LOADS = B_BYTES / 1024 / WAVES;
    // passes of the epilogue's transpose: half of the waves put their part of a pass into the A stage just
    // consumed, the other half into the B stage, and both halves must fit
    constexpr int EPI_PARTS = (WTM * WTN * 2 * (WAVES / 2) + (A_BYTES < B_BYTES ? A_BYTES : B_BYTES) - 1) /
                              (A_BYTES < B_BYTES ? A_BYTES : B_BYTES);
    constexpr int READS = TM + TN;
    static_assert(T::SWIZZLE == 1 && KS == 4, "");
    static_assert(WAVES % 2 == 0 && A_BYTES % (1024 * WAVES) == 0 && B_BYTES % (1024 * WAVES) == 0, "");
    static_assert(A_BYTES + (TM - 1) * 4096 < 65536 && B_BYTES + (TN - 1) * 4096 < 65536, "");
    static_assert(EPI_PARTS >= 1 && TM % EPI_PARTS == 0 && READS % 2 == 0 && TM * TN > READS / 2, "");

    extern __shared__ u32x4 lds[];
    char *const lds_bytes = reinterpret_cast<char *>(lds);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: lets address math run on the scalar unit
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int K = p.K;
    const int KT = SLICED ? p.k_slice / kBK : EDGE_K ? 2 * ((K + 2 * kBK - 1) / (2 * kBK)) : K / kBK;
    const int grid = gridDim.x;
    const int my_tiles = (p.nblocks - static_cast<int>(blockIdx.x) + grid - 1) / grid;
    const int total = my_tiles * KT;
    if (total == 0) return;

    const int row_in = lane >> 3;
    const int lane_k = ((lane & 7) ^ swz<1>(8 * wave + row_in)) << 3;  // first k, within a K tile, of this lane's chunk
    const uint32_t lane_off = static_cast<uint32_t>(row_in * K + lane_k) * 2u;
    const char *const zeros = reinterpret_cast<const char *>(&zero_chunk16);

    // Row-major B ([K][N]): the K tile of B is 64 rows of BN values and stays row-major in LDS.  A load
    // instruction of a wave covers two rows (k = 2 * (wave + WAVES * J) + r, r = lane / 32); the 16-byte chunk a
    // lane fetches is permuted with k & 3 (= 2 * (wave & 1) + r) so that the four rows of a transposing fragment
    // read lie in different banks (see read_b_transposed).
    static_assert(!B_ROW || (BN == 256 && WTN == 64), "");
    uint32_t lane_off_b = lane_off;
    if constexpr (B_ROW) {
        const int r = lane >> 5;
        lane_off_b = static_cast<uint32_t>(r * p.ldb + 8 * ((lane & 31) ^ ((2 * (wave & 1) + r) << 2))) * 2u;
    }

    typedef const __attribute__((address_space(1))) void *gptr_t;
    typedef __attribute__((address_space(3))) void *lptr_t;

    auto tile_origin = [&](int t, int &m0, int &n0, int &slice) {
        int tile_m, tile_n;
        tile_of(p, static_cast<int>(blockIdx.x), grid, t, tile_m, tile_n);
        if constexpr (SLICED) {
            // the pairs are laid out as a grid of tiles with the slices below each other: row = slice * tiles_m + tile_m
            const int tiles_m = p.tiles / p.tiles_n;
            slice = tile_m / tiles_m;
            tile_m -= slice * tiles_m;
        } else {
            slice = 0;
        }
        m0 = tile_m * BM;
        n0 = tile_n * BN;
    };

    // The loads walk the K tiles of this workgroup's output tiles in order.  The cursor is a pair of
    // wave-uniform pointers (row 8 * wave of the A and of the B panel, at the K tile to fetch next), moved
    // on by 128 bytes per K tile and recomputed when an output tile is finished, so that a load costs a
    // scalar 64-bit add, the lane offset and the LDS address in M0 - no multiplication per load.
    int ld_kt = 0, ld_t = 0;
    const char *cur_a, *cur_b;
    const int64_t group_stride = static_cast<int64_t>(8 * WAVES) * K * 2;  // bytes between a wave's consecutive loads
    // EDGE_M: load i of A, this lane: bytes from the cursor (row m0 + 8 * wave, the K tile's first k) to its chunk;
    // fits 32 bits (at most 256 rows either way, K below 2^22: the launcher checks)
    int32_t a_lane_off[EDGE_M ? A_LOADS : 1];
    int k_end = K;  // EDGE_K: the K tiles of the cursor's output tile count from k = K - k_end
    auto set_cursor = [&]() {
        int m0, n0, slice;
        tile_origin(ld_t, m0, n0, slice);
        const int k0 = SLICED ? slice * p.k_slice : 0;
        if constexpr (SLICED) k_end = K - k0;
        if constexpr (EDGE_M) {
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) {
                const int row = m0 + 8 * (wave + WAVES * i) + row_in;
                a_lane_off[i] = (((row < p.M ? row : p.M - 1) - (m0 + 8 * wave)) * K + lane_k) * 2;
            }
        }
        cur_a = reinterpret_cast<const char *>(p.A + static_cast<int64_t>(m0 + 8 * wave) * K + k0);
        if constexpr (B_ROW) cur_b = reinterpret_cast<const char *>(p.B + static_cast<int64_t>(k0 + 2 * wave) * p.ldb + n0);
        else cur_b = reinterpret_cast<const char *>(p.B + static_cast<int64_t>(n0 + 8 * wave) * K + k0);
    };
    set_cursor();
    const int64_t group_stride_b = B_ROW ? static_cast<int64_t>(2 * WAVES) * p.ldb * 2 : group_stride;
    const int64_t ktile_step_b = B_ROW ? static_cast<int64_t>(kBK) * p.ldb * 2 : kBK * 2;  // bytes from a K tile to the next
    auto advance_cursor = [&]() {
        if (ld_kt + 1 < KT) {
            ++ld_kt;
            cur_a += kBK * 2;
            cur_b += ktile_step_b;
        } else if (ld_t + 1 < my_tiles) {
            ld_kt = 0;
            ++ld_t;
            set_cursor();
        }
    };
    // load number I of the cursor's K tile (the A loads first, then the B loads); the last one moves the cursor
    // EDGE_K: where load I of the cursor's K tile reads from - its place in A or B, or the zero chunk when the
    // lane's k lies at or past K (for a row-major B the k is the row the load fetches)
    auto source_a = [&](int i) {
        const char *at = EDGE_M ? cur_a + a_lane_off[EDGE_M ? i : 0] : cur_a + i * group_stride + lane_off;
        if constexpr (EDGE_K) at = ld_kt * kBK + lane_k < k_end ? at : zeros;
        return at;
    };
    auto source_b = [&](int j) {
        const char *at = cur_b + j * group_stride_b + lane_off_b;
        if constexpr (EDGE_K) {
            const int k = B_ROW ? 2 * (wave + WAVES * j) + (lane >> 5) : lane_k;
            at = ld_kt * kBK + k < k_end ? at : zeros;
        }
        return at;
    };
    auto issue_one = [&](int stage, auto i_c) {
        constexpr int I = decltype(i_c)::value;
        if constexpr (I < A_LOADS) {
            __builtin_amdgcn_global_load_lds((gptr_t)source_a(I),
                                             (lptr_t)(lds_bytes + stage * A_BYTES + 1024 * (wave + WAVES * I)), 16, 0, 0);
        } else {
            constexpr int J = I - A_LOADS;
            __builtin_amdgcn_global_load_lds(
                (gptr_t)source_b(J),
                (lptr_t)(lds_bytes + 2 * A_BYTES + stage * B_BYTES + 1024 * (wave + WAVES * J)), 16, 0, 0);
            if constexpr (J == B_LOADS - 1) advance_cursor();
        }
    };
    auto issue_next = [&](int stage) {
        char *dst_a = lds_bytes + stage * A_BYTES;
        char *dst_b = lds_bytes + 2 * A_BYTES + stage * B_BYTES;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)source_a(i), (lptr_t)(dst_a + 1024 * (wave + WAVES * i)), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)source_b(i), (lptr_t)(dst_b + 1024 * (wave + WAVES * i)), 16, 0, 0);
        if (ld_kt + 1 < KT) {
            ++ld_kt;
            cur_a += kBK * 2;
            cur_b += ktile_step_b;
        } else if (ld_t + 1 < my_tiles) {
            ld_kt = 0;
            ++ld_t;
            set_cursor();
        }
    };

    // LDS byte addresses of this lane's fragments (stage 0, block 0) for the four K steps.
    const int frow = lane & 31;
    const int fhalf = lane >> 5;
    const int sw = (frow >> 1) & 7;
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_bytes));  // LDS aperture offset
    uint32_t off_a[KS], off_b[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const uint32_t o = static_cast<uint32_t>(frow * 128 + (((2 * ks + fhalf) ^ sw) << 4));
        off_a[ks] = lds_base + o + wm * WTM * 128;
        off_b[ks] = lds_base + o + 2 * A_BYTES + wn * WTN * 128;
    }

    float16v acc[TM][TN];
    auto clear_acc = [&]() {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
        // The zeroes are written by vector-ALU moves, and the matrix instructions that read them as their addend
        // are inline assembly: the compiler does not know them for what they are and keeps no distance between
        // such a move and the instruction that reads its register (it is free to sink the moves down to right in
        // front of the first of them).  Pin the moves here and put the wait states behind them.
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(acc[i][j]));
        asm volatile("s_nop 7");
    };
    clear_acc();

    u32x4 af[2][TM], bf[2][TN];
    // row-major B: the halves of a B fragment as the two reads deliver them; bf is put together from them behind
    // the wait (the compiler may need copies for that, and before the wait the registers hold nothing yet)
    u32x2 b_lo[2][B_ROW ? TN : 1], b_hi[2][B_ROW ? TN : 1];
    uint32_t off_br[B_ROW ? TN : 1];
    if constexpr (B_ROW) {
        const int i = lane & 15, g = (lane >> 4) & 1, kq = i >> 2;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int chunk = ((wn * WTN + j * 32 + g * 16 + 4 * (i & 3)) >> 3) ^ (kq << 2);
            off_br[j] = lds_base + 2 * A_BYTES + (fhalf * 8 + kq) * (BN * 2) + chunk * 16 + (i & 1) * 8;
        }
    }

    // read number R (0 .. READS-1) of K step KSTEP out of stage S into fragment set SLOT
    auto read_one = [&](auto r_c, auto ks_c, auto slot_c, auto stage_c) {
        constexpr int R = decltype(r_c)::value, KSTEP = decltype(ks_c)::value, SLOT = decltype(slot_c)::value,
                      S = decltype(stage_c)::value;
        if constexpr (R < TM) {
            lds_read16<S * A_BYTES + R * 4096>(af[SLOT][R], off_a[KSTEP]);
        } else if constexpr (!B_ROW) {
            lds_read16<S * B_BYTES + (R - TM) * 4096>(bf[SLOT][R - TM], off_b[KSTEP]);
        } else {
            // two transposing reads: k .. k+3 and k+4 .. k+7 of this lane's column (rows of BN * 2 bytes)
            constexpr int IMM = S * B_BYTES + KSTEP * 16 * BN * 2;
            lds_read_tr<IMM>(b_lo[SLOT][R - TM], off_br[R - TM]);
            lds_read_tr<IMM + 4 * BN * 2>(b_hi[SLOT][R - TM], off_br[R - TM]);
        }
    };

    // MFMAs of one K step out of fragment set SLOT, with the reads reader(R) spread over the first ones
    // and after(IDX) called behind every MFMA
    auto mfma_step = [&](auto slot_c, auto reader, auto after) {
        constexpr int SLOT = decltype(slot_c)::value;
        static_for<TM * TN>([&](auto idx_c) {
            constexpr int IDX = decltype(idx_c)::value;
            constexpr int I = IDX / TN, J = IDX % TN;
            mfma_asm<BF16>(acc[I][J], bf[SLOT][J], af[SLOT][I]);
            if constexpr (IDX < READS / 2) {
                reader(std::integral_constant<int, 2 * IDX>{});
                reader(std::integral_constant<int, 2 * IDX + 1>{});
            }
            after(idx_c);
        });
    };
    auto nothing = [](auto) {};

    // all reads issued so far have landed; the fake operands keep later MFMAs behind this point
    auto wait_frags = [&](int slot) {
        if constexpr (B_ROW) {
            static_assert(!B_ROW || ((TM == 4 || TM == 2) && TN == 2), "");
            if constexpr (TM == 4)
                asm volatile("s_waitcnt lgkmcnt(0)"
                             : "+v"(af[slot][0]), "+v"(af[slot][1]), "+v"(af[slot][2]), "+v"(af[slot][3]),
                               "+v"(b_lo[slot][0]), "+v"(b_hi[slot][0]), "+v"(b_lo[slot][TN - 1]), "+v"(b_hi[slot][TN - 1]));
            else
                asm volatile("s_waitcnt lgkmcnt(0)"
                             : "+v"(af[slot][0]), "+v"(af[slot][TM - 1]), "+v"(b_lo[slot][0]), "+v"(b_hi[slot][0]),
                               "+v"(b_lo[slot][TN - 1]), "+v"(b_hi[slot][TN - 1]));
#pragma unroll
            for (int j = 0; j < TN; ++j)
                bf[slot][j] = u32x4{b_lo[slot][j][0], b_lo[slot][j][1], b_hi[slot][j][0], b_hi[slot][j][1]};
            // where the halves did not land in adjacent registers the line above is vector-ALU moves, and the matrix
            // instructions that read bf are inline assembly the compiler keeps no distance to (see clear_acc)
#pragma unroll
            for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(bf[slot][j]));
            asm volatile("s_nop 3");
        } else if constexpr (TM == 4 && TN == 2) {
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(af[slot][0]), "+v"(af[slot][1]), "+v"(af[slot][2]), "+v"(af[slot][3]),
                           "+v"(bf[slot][0]), "+v"(bf[slot][1]));
        } else if constexpr (TM == 2 && TN == 2) {
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[slot][0]), "+v"(af[slot][1]), "+v"(bf[slot][0]), "+v"(bf[slot][1]));
        } else if constexpr (TM == 2 && TN == 4) {
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(af[slot][0]), "+v"(af[slot][1]), "+v"(bf[slot][0]), "+v"(bf[slot][1]),
                           "+v"(bf[slot][2]), "+v"(bf[slot][3]));
        } else {
            static_assert(TM == 4 && TN == 4, "");
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(af[slot][0]), "+v"(af[slot][1]), "+v"(af[slot][2]), "+v"(af[slot][3]),
                           "+v"(bf[slot][0]), "+v"(bf[slot][1]), "+v"(bf[slot][2]), "+v"(bf[slot][3]));
        }
    };

    // SPARE: the epilogue transposes through the 32 KB of LDS that the two stages leave free (four passes of
    // 32 rows per wave) instead of through the stage just consumed.  The loads of the K tile after next then
    // go out at their usual place, ahead of the epilogue; each wave confirms them (vmcnt(0)) before its first
    // store, while they are still its only outstanding memory operations, and the next K tile's barrier skips
    // the vmcnt wait.  Stores count in vmcnt too on this architecture: waiting there would mean waiting for
    // the whole chip's 32 MB burst of output to drain before the next K tile could be published.
    constexpr int SPARE_BYTES = 160 * 1024 - 2 * (A_BYTES + B_BYTES);
    constexpr bool SPARE = T::SPARE_EPILOGUE && TM % 4 == 0 && WTM * WTN * 2 / 4 * WAVES <= SPARE_BYTES;
    bool stores_in_flight = false;  // SPARE: set by the epilogue, cleared at the next barrier

    int t = 0;
    auto step_fn = [&](int step, auto last_c, auto stage_c) {
        constexpr int S = decltype(stage_c)::value;
        constexpr bool last_of_tile = decltype(last_c)::value;  // last K tile of an output tile
        using Other = std::integral_constant<int, S ^ 1>;
        using C0 = std::integral_constant<int, 0>;
        using C1 = std::integral_constant<int, 1>;
        using C2 = std::integral_constant<int, 2>;
        using C3 = std::integral_constant<int, 3>;
        // K steps 0..2: their MFMAs, with the next step's fragments read early in each
        mfma_step(C0{}, [&](auto r) { read_one(r, C1{}, C1{}, stage_c); }, nothing);
        wait_frags(1);
        mfma_step(C1{}, [&](auto r) { read_one(r, C2{}, C0{}, stage_c); }, nothing);
        wait_frags(0);
        mfma_step(C0{}, [&](auto r) { read_one(r, C3{}, C1{}, stage_c); }, nothing);
        wait_frags(1);
        if constexpr (SPARE) {
            // right after an epilogue the loads this barrier publishes were confirmed before the stores went out
            if (!stores_in_flight) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            stores_in_flight = false;
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        lds_barrier();
        // K step 3, with step 0 of the next K tile read out of the other stage (after the very last
        // K tile these reads fetch stale but in-bounds LDS contents that nothing uses)
        if constexpr (SPARE && T::SPREAD_LOADS) {
            // one load of the K tile after next behind each MFMA, unconditionally: past the end of the work
            // the cursor stands still and the loads fetch the last K tile again into a stage nobody reads
            // (the epilogue waits for them before its first store, so none is in flight at the end)
            static_assert(TM * TN >= A_LOADS + B_LOADS, "");
            mfma_step(C1{}, [&](auto r) { read_one(r, C0{}, C0{}, Other{}); }, [&](auto i_c) {
                if constexpr (decltype(i_c)::value < A_LOADS + B_LOADS) issue_one(S, i_c);
            });
        } else {
            if ((SPARE || !last_of_tile) && step + 2 < total) issue_next(S);
            mfma_step(C1{}, [&](auto r) { read_one(r, C0{}, C0{}, Other{}); }, nothing);
        }
        wait_frags(0);
        if constexpr (last_of_tile) {
            int m0, n0, slice;
            tile_origin(t, m0, n0, slice);
            // MFMA results are read by vector ALU instructions next: cover the issue-to-write latency
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
            if constexpr (SLICED) {
                static_assert(!SLICED || SPARE, "");
                // the loads in flight (the next pair's first K tiles) are confirmed before the first store, as in
                // the epilogue below
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                Params mine = p;
                mine.partial = p.partial + static_cast<int64_t>(slice) * p.M * partial_ld(p.N);
                store_partial<WTM, WTN>(mine, acc, lane, m0 + wm * WTM, n0 + wn * WTN);
                clear_acc();
                stores_in_flight = true;
            } else if constexpr (SPARE) {
                constexpr int REGION = WTM * WTN * 2 / 4;  // bytes per wave and pass
                char *region = lds_bytes + 2 * (A_BYTES + B_BYTES) + wave * REGION;
                store_tile_as<WTM, WTN, 1, BF16, false, 4, true, EDGE_M, true>(p, acc, reinterpret_cast<u32x4 *>(region), lane,
                                                                      m0 + wm * WTM, n0 + wn * WTN);
                clear_acc();
                stores_in_flight = true;
            } else {
                constexpr int REGION = WTM * WTN * 2 / EPI_PARTS;  // bytes per wave
                static_assert(REGION * (WAVES / 2) <= A_BYTES && REGION * (WAVES / 2) <= B_BYTES, "");
                char *region = wave < WAVES / 2 ? lds_bytes + S * A_BYTES + wave * REGION
                                                : lds_bytes + 2 * A_BYTES + S * B_BYTES + (wave - WAVES / 2) * REGION;
                store_tile_as<WTM, WTN, 1, BF16, false, EPI_PARTS, false, EDGE_M, true>(p, acc, reinterpret_cast<u32x4 *>(region), lane,
                                                                               m0 + wm * WTM, n0 + wn * WTN);
                clear_acc();
                lds_barrier();  // every wave is done with its transpose region in stage S
                if (step + 2 < total) issue_next(S);
            }
            ++t;
        }
    };

    // Prologue: K tile 0 into stage 0, published; K tile 1 on its way into stage 1; fragments of step 0.
    issue_next(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
    if (total > 1) issue_next(1);
    static_for<READS>([&](auto r) {
        read_one(r, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
    });
    wait_frags(0);

    int step = 0;
    for (int tile_i = 0; tile_i < my_tiles; ++tile_i) {
        for (int kt = 0; kt + 2 < KT; kt += 2, step += 2) {
            step_fn(step, std::false_type{}, std::integral_constant<int, 0>{});
            step_fn(step + 1, std::false_type{}, std::integral_constant<int, 1>{});
        }
        step_fn(step, std::false_type{}, std::integral_constant<int, 0>{});
        step_fn(step + 1, std::true_type{}, std::integral_constant<int, 1>{});  // ends with the epilogue
        step += 2;
    }
}

// EDGE_M: any M (the last row of tiles then reaches past M, see the kernel); K below 2^22.
// SLICED: p.k_slice (a multiple of 128) and p.partial are set: the fp32 partial products of the K slices, no epilogue.
template <class T, bool BF16, bool B_ROW = false, bool EDGE_M = false, bool SLICED = false>
int launch_pinned(Params p, hipStream_t stream) {
    constexpr size_t lds_bytes = T::SPARE_EPILOGUE ? 160u * 1024u : 2u * (T::BM + T::BN) * kBK * sizeof(uint16_t);
    if ((!EDGE_M && p.M % T::BM != 0) || p.M < 1 || (EDGE_M && p.K >= (1 << 22)) || (p.N % T::BN) != 0 || (p.K % 8) != 0)
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: this persistent variant needs full tiles and K %% 8 == 0");
    if (SLICED && (p.k_slice < 2 * kBK || p.k_slice % (2 * kBK) != 0 || p.partial == nullptr))
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: K slices of this variant are multiples of 128 deep");
    const int slices = SLICED ? (p.K + p.k_slice - 1) / p.k_slice : 1;
    // padded with zeros inside the kernel: up to a pair of K tiles, or to the end of the last slice
    const bool edge_k = SLICED ? p.K % p.k_slice != 0 : p.K % (2 * kBK) != 0;
    auto kernel = edge_k ? gemm16_pinned_kernel<T, BF16, B_ROW, true, EDGE_M, SLICED>
                         : gemm16_pinned_kernel<T, BF16, B_ROW, false, EDGE_M, SLICED>;
    static std::atomic<uint64_t> configured[2] = {{0}, {0}};  // per instantiation: the devices whose LDS limit is raised
    if (const int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds_bytes, configured[edge_k]); st != KO_OK)
        return st;
    p.tiles_n = p.N / T::BN;
    const int tiles_m = (p.M + T::BM - 1) / T::BM;
    p.tiles = tiles_m * p.tiles_n;
    p.nblocks = p.tiles * slices;
    int grid = compute_units() / 8 * 8;
    if (grid > p.nblocks) grid = p.nblocks;
    // Blocked tile order when the tile grid divides evenly over 8 XCDs x (grid / 8) workgroups: of the ways to lay
    // the 8 regions out (8 x 1, 4 x 2, 2 x 4, 1 x 8) the one whose resident block of tiles needs the fewest bytes
    // of A and B panels - for a short, wide output regions side by side (1024 x 8192 x 4096 on 128 x 256 tiles took
    // 102 us as eight bands of one tile row, its transpose 88).
    p.band_rows = 0;
    p.block_cols = 0;
    p.xcd_cols_log2 = 0;
    p.region_cols = 0;
    const int per_xcd = grid / 8;
    // (K slices: the grid of tiles is the slices' grids below each other; a band lies inside a slice or is whole
    // slices, and the resident block then holds a panel of B per slice and column)
    const int rows = tiles_m * slices;
    if (tuning(knob_gemm16_mapping) != 1 && grid % 8 == 0) {
        int64_t best = 0;
        for (int lg = 0; lg <= 3; ++lg) {
            const int across = 1 << lg, down = 8 >> lg;
            if (rows % down != 0 || p.tiles_n % across != 0) continue;
            const int band = rows / down, region = p.tiles_n / across;
            if (band > per_xcd || per_xcd % band != 0 || region % (per_xcd / band) != 0) continue;
            if (tiles_m % band != 0 && band % tiles_m != 0) continue;
            const int band_slices = (band + tiles_m - 1) / tiles_m;
            const int64_t bytes = static_cast<int64_t>(band) * T::BM + static_cast<int64_t>(per_xcd / band) * band_slices * T::BN;
            if (p.band_rows == 0 || bytes < best) {
                best = bytes;
                p.band_rows = band;
                p.block_cols = per_xcd / band;
                p.xcd_cols_log2 = lg;
                p.region_cols = region;
            }
        }
    }
    kernel<<<dim3(static_cast<unsigned>(grid)), dim3(T::THREADS), lds_bytes, stream>>>(p);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

// K split over the waves of a workgroup, for a problem of few output tiles (a few hundred rows against a weight
// matrix): every kernel above walks K in steps that all waves of a workgroup take together - a barrier per K tile,
// one or two K tiles in flight per workgroup - and with a workgroup or less per compute unit such a step costs its
// latencies (0.4 us per 64 k on 64 x 64 tiles, whatever the arithmetic).  Here a workgroup owns one (32 TM) x (32 TN)
// output tile (32 x 32 to 128 x 64) and wave w multiplies the w-th of WAVES ranges of K tiles of it: the whole tile over its own share of K, out of two
// LDS stages of its own that it fills with direct-to-LDS loads (eight rows of 128 bytes per wave-level load, as
// in the kernels above) - no barrier in the loop, WAVES times fewer steps in a row, and two K tiles per wave in
// flight.  At the end the waves leave their fp32 tiles in LDS and the workgroup adds them in wave order (the same
// bits from call to call) and applies alpha, beta * C, the bias and the activation once.
// Any M, N and any K that is a multiple of 8: a row at or past M (N) is fetched from the last row instead and its
// results are not stored; a 16-byte chunk at or past the end of the wave's range of K - in the last K tile, or in a K
// tile past the range that a wave's second stage asks for - is fetched from sixteen zero bytes, chosen per load with a
// compare and two selects.
// B_ROW: B as [K][N] (rows ldb apart, N and ldb multiples of 8).  A wave's K tile of B is 64 rows of 32 TN values and
// stays row-major in LDS; a wave-level load covers 1 KB of it (16, 8 or 4 rows), the 16-byte chunk a lane fetches
// is permuted with the row number modulo 4 - as far as the row has chunks for it - and the fragments come out of
// transposing LDS reads as in the pinned kernel (read_b_transposed has the lane arithmetic); a chunk at or past N
// or a row at or past K is fetched from the zeros.
template <int TM, int TN, int WAVES, bool BF16, bool B_ROW = false>
__global__ __launch_bounds__(64 * WAVES) void gemm16_wave_k_kernel(const Params p) {
    constexpr int WTM = 32 * TM, WTN = 32 * TN;
    constexpr int KS = kBK / 16;
    constexpr int STAGES = 2;
    constexpr int A_LOADS = WTM / 8, B_LOADS = WTN / 8, LOADS = A_LOADS + B_LOADS;
    constexpr int A_BYTES = WTM * kBK * 2, STAGE_BYTES = (WTM + WTN) * kBK * 2, WAVE_BYTES = STAGES * STAGE_BYTES;
    constexpr int LDP = WTN + 4;  // floats between the rows of a wave's fp32 tile in LDS
    static_assert(KS == 4 && (STAGES - 1) * LOADS <= 63 && STAGES >= 2, "the loads in flight must fit the 6-bit counter");
    static_assert(WTM * LDP * 4 <= WAVE_BYTES && WAVES * WAVE_BYTES <= 160 * 1024, "");
    static_assert(TM * TN <= 8 && TM + TN <= 6, "");

    extern __shared__ u32x4 lds[];
    char *const lds_bytes = reinterpret_cast<char *>(lds);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Tiles in row-major order, workgroup b on XCD b % 8: the tiles of one row of tiles - which share their rows of
    // A - are spread over the XCDs.  (One contiguous range of the tile list per XCD, along the smaller operand, so
    // that the larger one is shared out between the L2s, was slower: 256 x 4096 x 4096 18.1 -> 20.2 us, 1000 x 1024 x
    // 4096 18.6 -> 20.5, 100 x 4096 x 4096 11.7 -> 13.0 - the workgroups of an XCD then ask for the same few blocks
    // at the same moment.)
    const int tile = static_cast<int>(blockIdx.x);
    const int m0 = (tile / p.tiles_n) * WTM, n0 = (tile % p.tiles_n) * WTN;
    const int M = p.M, N = p.N, K = p.K;
    const int64_t ldk = p.ldk;
    // wave w takes the K tiles [w * per, (w + 1) * per), a range of its own.  (Dealt round-robin - w, w + WAVES, ... - the
    // waves of a workgroup walk through adjacent 128-byte pieces of every row together, and weights that come from memory
    // stream more slowly: 8 x 8192 x 8192 31.3 us against 28.6, 8 x 4096 x 4096 11.2 against 10.1; problems that live in
    // the L2s are level, within 3 %.  A read-only loop with this kernel's loads - eight rows of 128 bytes per wave-level
    // load - over the same 134 MB: 4.6 TB/s round-robin, 5.9 in ranges.  Three or four stages per wave on a K tile
    // of A cut down to 8 rows gained nothing over two.)  p.band_rows == 0 deals round-robin, for comparison.
    const int KT = (K + kBK - 1) / kBK;
    const bool ranges = p.band_rows != 0;
    const int per = (KT + WAVES - 1) / WAVES;
    const int k_first = ranges ? wave * per * kBK : wave * kBK;             // first k of this wave's K tiles
    const int k_step = ranges ? kBK : WAVES * kBK;                          // from one of them to the next
    // ranges: where this wave's range ends - chunks at or past it are fetched as zeros
    const int k_end = ranges && k_first + per * kBK < K ? k_first + per * kBK : K;
    const int my_tiles = k_first < k_end ? (k_end - k_first + k_step - 1) / k_step : 0;

    typedef const __attribute__((address_space(1))) void *gptr_t;
    typedef __attribute__((address_space(3))) void *lptr_t;
    const char *const zeros = reinterpret_cast<const char *>(&zero_chunk16);

    // Lane l of a wave-level load fills the l-th 16-byte slot of eight LDS rows: row l / 8, slot l % 8, which holds
    // chunk (l % 8) ^ swz(row) of the row.  The row within the tile is 8 i + l / 8 for load i, so the swizzle term
    // takes two values, by the parity of i.
    const int row_in = lane >> 3;
    int lane_k[2];  // first k, within a K tile, of the chunk this lane fetches in an even / odd load
#pragma unroll
    for (int par = 0; par < 2; ++par) lane_k[par] = ((lane & 7) ^ ((4 * par + (row_in >> 1)) & 7)) << 3;
    const char *src_a[A_LOADS], *src_b[B_LOADS];  // this lane's chunk of load i in the K tile to fetch next
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const int r = m0 + 8 * i + row_in;
        src_a[i] = reinterpret_cast<const char *>(p.A + static_cast<int64_t>(r < M ? r : M - 1) * ldk + k_first + lane_k[i & 1]);
    }
    // row-major B: NCH chunks per LDS row, RPL rows per wave-level load; lane l fills position l % NCH of row
    // l / NCH of its load's rows, with chunk (l % NCH) ^ b_swz(row) of that row of the tile
    constexpr int NCH = WTN / 8, RPL = 64 / NCH, B_ROW_BYTES = WTN * 2;
    auto b_swz = [](int k) { return ((k & 3) << 2) & (NCH - 1); };
    const int b_krow = lane / NCH;  // + RPL * j: the row, within the K tile, that this lane fetches in load j
    bool b_inside = true;           // row-major B: this lane's chunk lies inside N (the same chunk in every load: RPL % 4 == 0)
#pragma unroll
    for (int j = 0; j < B_LOADS; ++j) {
        if constexpr (B_ROW) {
            static_assert(RPL % 4 == 0, "");
            const int c = n0 + 8 * ((lane % NCH) ^ b_swz(b_krow));
            b_inside = c < N;
            src_b[j] = reinterpret_cast<const char *>(p.B + static_cast<int64_t>(k_first + RPL * j + b_krow) * p.ldb + (b_inside ? c : 0));
        } else {
            const int r = n0 + 8 * j + row_in;
            src_b[j] = reinterpret_cast<const char *>(p.B + static_cast<int64_t>(r < N ? r : N - 1) * ldk + k_first + lane_k[j & 1]);
        }
    }
    int ld_k0 = k_first;  // first k of the K tile to fetch next
    char *const wave_lds = lds_bytes + wave * WAVE_BYTES;
    const int64_t b_tile_step = B_ROW ? static_cast<int64_t>(k_step) * p.ldb * 2 : k_step * 2;  // bytes to this wave's next K tile
    auto issue = [&](int stage) {
        const bool in0 = ld_k0 + lane_k[0] < k_end, in1 = ld_k0 + lane_k[1] < k_end;
        char *dst = wave_lds + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            __builtin_amdgcn_global_load_lds((gptr_t)((i & 1 ? in1 : in0) ? src_a[i] : zeros), (lptr_t)(dst + 1024 * i), 16, 0, 0);
            src_a[i] += k_step * 2;
        }
#pragma unroll
        for (int j = 0; j < B_LOADS; ++j) {
            bool in = j & 1 ? in1 : in0;
            if constexpr (B_ROW) in = b_inside && ld_k0 + RPL * j + b_krow < k_end;
            __builtin_amdgcn_global_load_lds((gptr_t)(in ? src_b[j] : zeros), (lptr_t)(dst + A_BYTES + 1024 * j), 16, 0, 0);
            src_b[j] += b_tile_step;
        }
        ld_k0 += k_step;
    };

    // LDS byte addresses of this lane's fragments (stage 0, block 0) for the four K steps
    const int frow = lane & 31, fhalf = lane >> 5;
    const int sw = (frow >> 1) & 7;
    const uint32_t frag_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(wave_lds));
    uint32_t off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) off[ks] = frag_base + static_cast<uint32_t>(frow * 128 + (((2 * ks + fhalf) ^ sw) << 4));

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    u32x4 af[2][TM], bf[2][TN];
    // row-major B: the two halves of a B fragment as the transposing reads deliver them (k .. k+3 and k+4 .. k+7 of
    // this lane's column), and where the lane reads them (K step 0 of stage 0): lane i of a group of 16 points at row
    // i / 4 of the K step's rows, columns 4 (i % 4) .. + 3 of the group's 16
    u32x2 b_lo[2][B_ROW ? TN : 1], b_hi[2][B_ROW ? TN : 1];
    uint32_t off_br[B_ROW ? TN : 1];
    if constexpr (B_ROW) {
        const int i = lane & 15, g = (lane >> 4) & 1, kq = i >> 2;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int chunk = ((j * 32 + g * 16 + 4 * (i & 3)) >> 3) ^ b_swz(kq);
            off_br[j] = frag_base + A_BYTES + (fhalf * 8 + kq) * B_ROW_BYTES + chunk * 16 + (i & 1) * 8;
        }
    }
    auto read_frags = [&](auto ks_c, auto slot_c, auto stage_c) {
        constexpr int KSTEP = decltype(ks_c)::value, SLOT = decltype(slot_c)::value, S = decltype(stage_c)::value;
        static_for<TM>([&](auto i_c) {
            constexpr int I = decltype(i_c)::value;
            lds_read16<S * STAGE_BYTES + I * 4096>(af[SLOT][I], off[KSTEP]);
        });
        static_for<TN>([&](auto j_c) {
            constexpr int J = decltype(j_c)::value;
            if constexpr (B_ROW) {
                constexpr int IMM = S * STAGE_BYTES + KSTEP * 16 * B_ROW_BYTES;
                lds_read_tr<IMM>(b_lo[SLOT][J], off_br[J]);
                lds_read_tr<IMM + 4 * B_ROW_BYTES>(b_hi[SLOT][J], off_br[J]);
            } else {
                lds_read16<S * STAGE_BYTES + A_BYTES + J * 4096>(bf[SLOT][J], off[KSTEP]);
            }
        });
    };
    // every read issued so far has landed; each register the reads wrote passes through an empty statement behind the
    // wait, which keeps the matrix instructions that use it behind this point
    auto wait_frags = [&](int slot) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(af[slot][i]));
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            if constexpr (B_ROW) {
                asm volatile("" : "+v"(b_lo[slot][j]), "+v"(b_hi[slot][j]));
                bf[slot][j] = u32x4{b_lo[slot][j][0], b_lo[slot][j][1], b_hi[slot][j][0], b_hi[slot][j][1]};
            } else {
                asm volatile("" : "+v"(bf[slot][j]));
            }
        }
    };
    auto multiply = [&](int slot) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = mfma16<BF16>(bf[slot][j], af[slot][i], acc[i][j]);
    };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using C2 = std::integral_constant<int, 2>;
    using C3 = std::integral_constant<int, 3>;
    // One K tile out of stage S; the loads of the K tile STAGES further on go out as soon as the stage's last fragments
    // are in registers.  Loads complete in order: with STAGES K tiles' worth in flight, all but the last
    // (STAGES - 1) LOADS done means that this stage has landed.
    auto k_tile = [&](auto stage_c) {
        constexpr int S = decltype(stage_c)::value;
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 1) * LOADS) : "memory");
        read_frags(C0{}, C0{}, stage_c);
        read_frags(C1{}, C1{}, stage_c);
        wait_frags(0);
        wait_frags(1);
        multiply(0);
        read_frags(C2{}, C0{}, stage_c);
        multiply(1);
        read_frags(C3{}, C1{}, stage_c);
        wait_frags(0);
        wait_frags(1);
        issue(S);
        multiply(0);
        multiply(1);
    };
    static_for<STAGES>([&](auto s_c) { issue(decltype(s_c)::value); });
    for (int t = 0; t < my_tiles; t += STAGES) static_for<STAGES>(k_tile);  // past this wave's last K tile: stages of zeros
    // the loads still in flight (K tiles past the end: zeros) must land before the stages are written over
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // this wave's tile as fp32 into its own LDS; a lane holds, of row frow of each 32 x 32 block, columns 8 q + 4 fhalf .. + 3
    typedef float float4v __attribute__((ext_vector_type(4)));
    float *const mine = reinterpret_cast<float *>(wave_lds);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4v v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                *reinterpret_cast<float4v *>(mine + (i * 32 + frow) * LDP + j * 32 + 8 * q + 4 * fhalf) = v;
            }
    __syncthreads();
    // one thread per four consecutive columns of a row; the waves' tiles are added in wave order
    constexpr int GROUPS = WTN / 4, ROWS_PER_PASS = 64 * WAVES / GROUPS;
    static_assert(64 * WAVES % GROUPS == 0, "");
    const bool use_c = p.C != nullptr && p.beta != 0.0f;
    const int g = tid % GROUPS;
    const int n = n0 + 4 * g;
    for (int r = tid / GROUPS; r < WTM; r += ROWS_PER_PASS) {
        const int m = m0 + r;
        if (m >= M || n >= N) continue;
        float4v sum = *reinterpret_cast<const float4v *>(reinterpret_cast<const float *>(lds_bytes) + r * LDP + 4 * g);
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
            sum += *reinterpret_cast<const float4v *>(reinterpret_cast<const float *>(lds_bytes + w * WAVE_BYTES) + r * LDP + 4 * g);
        float v[4] = {sum[0], sum[1], sum[2], sum[3]};
        const int64_t at = static_cast<int64_t>(m) * p.ldd + n;
        u32x2 c2 = {0, 0}, b2 = {0, 0};
        if (n + 3 < N) {
            if (use_c) c2 = *reinterpret_cast<const u32x2_rows *>(p.C + at);
            if (p.bias) b2 = *reinterpret_cast<const u32x2_rows *>(p.bias + n);
            finish4<BF16>(p, v, c2, b2, use_c);
            u32x2 o;
            o[0] = pack2<BF16>(v[0], v[1]);
            o[1] = pack2<BF16>(v[2], v[3]);
            *reinterpret_cast<u32x2_rows *>(p.D + at) = o;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (n + e >= N) continue;
                if (use_c) c2[e >> 1] |= static_cast<uint32_t>(p.C[at + e]) << ((e & 1) * 16);
                if (p.bias) b2[e >> 1] |= static_cast<uint32_t>(p.bias[n + e]) << ((e & 1) * 16);
            }
            finish4<BF16>(p, v, c2, b2, use_c);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n + e < N) p.D[at + e] = from_float<BF16>(v[e]);
        }
    }
}

template <int TM, int TN, int WAVES, bool BF16, bool B_ROW = false>
int launch_wave_k(Params p, hipStream_t stream) {
    constexpr size_t lds_bytes = static_cast<size_t>(WAVES) * 2 * (32 * TM + 32 * TN) * kBK * 2;
    if (p.K % 8 != 0 || p.k_slice != 0) return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: the wave-K variant takes a whole K that is a multiple of 8");
    if (B_ROW && (p.N % 8 != 0 || p.ldb % 8 != 0))
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: the wave-K variant takes a row-major B whose N and row stride are multiples of 8");
    auto kernel = gemm16_wave_k_kernel<TM, TN, WAVES, BF16, B_ROW>;
    static std::atomic<uint64_t> configured{0};  // per instantiation: the devices whose LDS limit is raised
    if (const int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds_bytes, configured); st != KO_OK) return st;
    p.tiles_n = (p.N + 32 * TN - 1) / (32 * TN);
    const int64_t tiles = static_cast<int64_t>((p.M + 32 * TM - 1) / (32 * TM)) * p.tiles_n;
    if (tiles > 0x7fffffff) return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: too many tiles for the wave-K variant");
    p.nblocks = static_cast<int>(tiles);
    p.band_rows = tuning(knob_gemm16_mapping) == 2 ? 0 : 1;  // knob gemm16.mapping = 2: K tiles dealt round-robin
    kernel<<<dim3(static_cast<unsigned>(p.nblocks)), dim3(64 * WAVES), lds_bytes, stream>>>(p);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

// A deep ring of LDS stages for mid-size problems (a few thousand rows against a weight matrix: tens to a few
// hundred tiles of 128 x 128).  What a compute unit takes in through direct-to-LDS loads is the bytes it has in flight
// over a latency of 1 - 1.5 us, and the bytes in flight are LDS stages: two stages of a 256 x 256 tile (or of any
// other) give a K tile that takes one latency whatever its size.  Here the tile is small enough (BM + BN rows of
// 128 bytes per stage) for STAGES - 1 K tiles to be on their way while one is multiplied: the loads of K tile
// t + STAGES - 1 go out right behind the barrier that publishes K tile t, into the stage that K tile t - 1 was read
// from; a wave waits only for its own loads of K tile t (loads complete in order: all but the last (STAGES - 2) K
// tiles' worth done) and one barrier per K tile publishes them.  The waves share the stages as in the kernels
// above (WAVES_M x WAVES_N wave tiles of 32 TM x 32 TN, eight rows of 128 bytes per wave-level load, the same
// swizzle, inline-assembly fragment reads two K steps deep); the stage is a compile-time number (the loop is
// unrolled by STAGES and K is padded with K tiles of zeros up to a multiple of that - at most STAGES - 1 K tiles
// of multiplying zeros).  One workgroup per tile and per compute unit; the epilogue is store_tile's, through the
// stages once the last K tile has been read.  Any M and N (rows past the end are fetched from the last row, edge tiles take the
// element-wise epilogue), K a multiple of 8 (chunks at or past K come from sixteen zero bytes).
// B_ROW: B as [K][N] (rows ldb apart, N and ldb multiples of 8): the K tile of B is 64 rows of BN values and stays
// row-major in LDS, a wave-level load covers four or eight of its rows with the 16-byte chunks permuted by the row
// number modulo 4, and the fragments come out of pairs of transposing reads - as in gemm16_wave_k_kernel.
// K slices: workgroups with blockIdx.y = s take k in [s * k_slice, (s + 1) * k_slice) and leave their fp32 partial
// products in the workspace (see slice_of, store_partial).
template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, bool BF16, bool B_ROW = false>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm16_ring_kernel(const Params whole) {
    const Params p = slice_of<B_ROW>(whole);
    constexpr int WAVES = WAVES_M * WAVES_N;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N, TM = WTM / 32, TN = WTN / 32;
    constexpr int KS = kBK / 16;
    constexpr int A_BYTES = BM * kBK * 2, B_BYTES = BN * kBK * 2, STAGE_BYTES = A_BYTES + B_BYTES;
    constexpr int A_LOADS = BM / 8 / WAVES, B_LOADS = BN / 8 / WAVES, LOADS = A_LOADS + B_LOADS;  // per wave and K tile
    constexpr int EPILOGUE_BYTES = WTM * WTN * 2;                                                 // per wave
    static_assert(KS == 4 && WAVES % 2 == 0 && (BM / 8) % WAVES == 0 && (BN / 8) % WAVES == 0, "");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && STAGES >= 3 && (STAGES - 1) * LOADS <= 63, "");
    static_assert(STAGES * STAGE_BYTES <= 160 * 1024 && WAVES * EPILOGUE_BYTES <= STAGES * STAGE_BYTES, "");
    constexpr int SET_BYTES = 32768;                                       // fragment address registers this far apart (see off_a)
    constexpr int OFFSET_SETS = ((STAGES - 1) * STAGE_BYTES) / SET_BYTES + 1;
    constexpr int NCH = BN / 8, RPL = 64 / NCH, B_ROW_BYTES = BN * 2;      // row-major B: chunks per LDS row, rows per wave-level load
    static_assert(SET_BYTES + (TM > TN ? TM : TN) * 4096 <= 65536 && (!B_ROW || (SET_BYTES + 52 * B_ROW_BYTES < 65536 && RPL % 4 == 0)), "");

    extern __shared__ u32x4 lds[];
    char *const lds_bytes = reinterpret_cast<char *>(lds);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int tile = xcd_remap(static_cast<int>(blockIdx.x), p.nblocks);
    const int m0 = (tile / p.tiles_n) * BM, n0 = (tile % p.tiles_n) * BN;
    const int M = p.M, N = p.N, K = p.K;
    const int64_t ldk = p.ldk;
    const int KT = (K + kBK - 1) / kBK;
    const int KT_padded = (KT + STAGES - 1) / STAGES * STAGES;

    typedef const __attribute__((address_space(1))) void *gptr_t;
    typedef __attribute__((address_space(3))) void *lptr_t;
    const char *const zeros = reinterpret_cast<const char *>(&zero_chunk16);

    // wave w issues the wave-level loads w, w + WAVES, ... of a K tile (eight tile rows each); lane l fills slot
    // l % 8 of row l / 8 with chunk (l % 8) ^ swz(row) - the same for all of a wave's loads, as 8 WAVES rows apart
    // the swizzle repeats
    const int row_in = lane >> 3;
    const int lane_k = ((lane & 7) ^ swz<1>(8 * wave + row_in)) << 3;  // first k, within a K tile, of this lane's chunk
    const char *src_a[A_LOADS], *src_b[B_LOADS];  // this lane's chunk of this wave's load i in the K tile to fetch next
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const int r = m0 + 8 * (wave + WAVES * i) + row_in;
        src_a[i] = reinterpret_cast<const char *>(p.A + static_cast<int64_t>(r < M ? r : M - 1) * ldk + lane_k);
    }
    // row-major B: lane l fills position l % NCH of row l / NCH of its load's RPL rows with chunk (l % NCH) ^ b_swz(row)
    auto b_swz = [](int k) { return ((k & 3) << 2) & (NCH - 1); };
    const int b_krow = lane / NCH;  // + RPL * (wave + WAVES * j): the row, within the K tile, this lane fetches in load j
    bool b_inside = true;           // row-major B: this lane's chunk lies inside N (the same chunk in every load)
#pragma unroll
    for (int j = 0; j < B_LOADS; ++j) {
        if constexpr (B_ROW) {
            const int c = n0 + 8 * ((lane % NCH) ^ b_swz(b_krow));
            b_inside = c < N;
            src_b[j] = reinterpret_cast<const char *>(p.B + static_cast<int64_t>(RPL * (wave + WAVES * j) + b_krow) * p.ldb + (b_inside ? c : 0));
        } else {
            const int r = n0 + 8 * (wave + WAVES * j) + row_in;
            src_b[j] = reinterpret_cast<const char *>(p.B + static_cast<int64_t>(r < N ? r : N - 1) * ldk + lane_k);
        }
    }
    const int64_t b_tile_step = B_ROW ? static_cast<int64_t>(kBK) * p.ldb * 2 : kBK * 2;  // bytes from a K tile to the next
    int ld_k0 = 0;     // first k of the K tile to fetch next
    bool ld_in = lane_k < K;  // this lane's chunk of that K tile lies inside K
    // load number L (the A loads first, then the B loads) of the K tile to fetch next, into stage `stage`; the last
    // one moves on to the next K tile
    auto issue_one = [&](int stage, auto l_c) {
        constexpr int L = decltype(l_c)::value;
        char *dst = lds_bytes + stage * STAGE_BYTES + 1024 * wave;
        if constexpr (L < A_LOADS) {
            __builtin_amdgcn_global_load_lds((gptr_t)(ld_in ? src_a[L] : zeros), (lptr_t)(dst + 1024 * WAVES * L), 16, 0, 0);
            src_a[L] += kBK * 2;
        } else {
            constexpr int J = L - A_LOADS;
            bool in = ld_in;
            if constexpr (B_ROW) in = b_inside && ld_k0 + RPL * (wave + WAVES * J) + b_krow < K;
            __builtin_amdgcn_global_load_lds((gptr_t)(in ? src_b[J] : zeros), (lptr_t)(dst + A_BYTES + 1024 * WAVES * J), 16, 0, 0);
            src_b[J] += b_tile_step;
        }
        if constexpr (L == LOADS - 1) {
            ld_k0 += kBK;
            ld_in = ld_k0 + lane_k < K;
        }
    };

    // LDS byte addresses of this lane's fragments (stage 0, block 0) for the four K steps; further sets 32 KB up
    // each, for the stages that the 16-bit offset field of the read does not reach from the first
    const int frow = lane & 31, fhalf = lane >> 5;
    const int sw = (frow >> 1) & 7;
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_bytes));
    uint32_t off_a[OFFSET_SETS][KS], off_b[OFFSET_SETS][KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const uint32_t o = lds_base + static_cast<uint32_t>(frow * 128 + (((2 * ks + fhalf) ^ sw) << 4));
#pragma unroll
        for (int set = 0; set < OFFSET_SETS; ++set) {
            off_a[set][ks] = o + wm * WTM * 128 + set * SET_BYTES;
            off_b[set][ks] = o + A_BYTES + wn * WTN * 128 + set * SET_BYTES;
        }
    }
    // row-major B: where this lane's transposing reads of K step 0 start (lane i of a group of 16: row i / 4 of the
    // step's rows, columns 4 (i % 4) .. + 3 of the group's 16), and the halves of a fragment as the reads deliver them
    uint32_t off_br[OFFSET_SETS][B_ROW ? TN : 1];
    u32x2 b_lo[2][B_ROW ? TN : 1], b_hi[2][B_ROW ? TN : 1];
    if constexpr (B_ROW) {
        const int i = lane & 15, g = (lane >> 4) & 1, kq = i >> 2;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int chunk = ((wn * WTN + j * 32 + g * 16 + 4 * (i & 3)) >> 3) ^ b_swz(kq);
#pragma unroll
            for (int set = 0; set < OFFSET_SETS; ++set)
                off_br[set][j] = lds_base + A_BYTES + (fhalf * 8 + kq) * B_ROW_BYTES + chunk * 16 + (i & 1) * 8 + set * SET_BYTES;
        }
    }

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    // the matrix instructions are inline assembly: pin the moves that zero their addends and keep the distance the
    // compiler does not know it has to keep (see gemm16_pinned_kernel)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(acc[i][j]));
    asm volatile("s_nop 7");

    constexpr int READS = B_ROW ? TM + 2 * TN : TM + TN, MFMAS = TM * TN;
    u32x4 af[2][TM], bf[2][TN];
    // read number R (the A blocks first, then the B blocks - row-major B: their halves) of K step KSTEP out of stage S
    // into fragment set SLOT
    auto read_one = [&](auto r_c, auto ks_c, auto slot_c, auto stage_c) {
        constexpr int R = decltype(r_c)::value, KSTEP = decltype(ks_c)::value, SLOT = decltype(slot_c)::value,
                      S = decltype(stage_c)::value;
        constexpr int HI = S * STAGE_BYTES / SET_BYTES, BASE = S * STAGE_BYTES - HI * SET_BYTES;
        if constexpr (R < TM) {
            lds_read16<BASE + R * 4096>(af[SLOT][R], off_a[HI][KSTEP]);
        } else if constexpr (!B_ROW) {
            lds_read16<BASE + (R - TM) * 4096>(bf[SLOT][R - TM], off_b[HI][KSTEP]);
        } else {
            constexpr int J = (R - TM) / 2, IMM = BASE + KSTEP * 16 * B_ROW_BYTES;
            if constexpr ((R - TM) % 2 == 0) lds_read_tr<IMM>(b_lo[SLOT][J], off_br[HI][J]);
            else lds_read_tr<IMM + 4 * B_ROW_BYTES>(b_hi[SLOT][J], off_br[HI][J]);
        }
    };
    // every read issued so far has landed; each register the reads wrote passes through an empty statement behind the
    // wait, which keeps the matrix instructions that use it behind this point
    auto wait_frags = [&](int slot) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(af[slot][i]));
        if constexpr (B_ROW) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                asm volatile("" : "+v"(b_lo[slot][j]), "+v"(b_hi[slot][j]));
                bf[slot][j] = u32x4{b_lo[slot][j][0], b_lo[slot][j][1], b_hi[slot][j][0], b_hi[slot][j][1]};
            }
            // where the halves did not land in adjacent registers the line above is vector-ALU moves, and the matrix
            // instructions that read bf are inline assembly the compiler keeps no distance to
#pragma unroll
            for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(bf[slot][j]));
            asm volatile("s_nop 3");
        } else {
#pragma unroll
            for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(bf[slot][j]));
        }
    };
    // The matrix instructions of one K step out of fragment set SLOT; behind the IDX-th of them go its share of the
    // step's fragment reads (reader(R), R = 0 .. READS - 1) and of the step's loads (loader(L), L = FIRST_LOAD ..
    // FIRST_LOAD + STEP_LOADS - 1), so that a wave held at the issue of a read or a load has a matrix instruction running.
    // (the reads go out behind the first matrix instructions of the step, two behind each, so that the rest of the
    // step covers their latency; with one read behind each of four the last one's latency lay open: 0.31 us per K
    // tile without any loads, against 0.21 us of matrix instructions)
    constexpr int RPM = MFMAS >= 2 * READS ? 1 : (READS > 2 * MFMAS ? (READS + MFMAS - 1) / MFMAS : 2);  // reads behind one matrix instruction
    static_assert(RPM * MFMAS >= READS, "");
    constexpr int STEP_LOADS = (LOADS + 1) / 2, LPM = (STEP_LOADS + MFMAS - 1) / MFMAS;
    auto mfma_step = [&](auto slot_c, auto reader, auto first_load_c, auto loader) {
        constexpr int SLOT = decltype(slot_c)::value, FIRST_LOAD = decltype(first_load_c)::value;
        static_for<MFMAS>([&](auto idx_c) {
            constexpr int IDX = decltype(idx_c)::value;
            mfma_asm<BF16>(acc[IDX / TN][IDX % TN], bf[SLOT][IDX % TN], af[SLOT][IDX / TN]);
            static_for<RPM>([&](auto r_c) {
                constexpr int R = IDX * RPM + decltype(r_c)::value;
                if constexpr (R < READS) reader(std::integral_constant<int, R>{});
            });
            static_for<LPM>([&](auto l_c) {
                constexpr int L = IDX * LPM + decltype(l_c)::value;
                if constexpr (FIRST_LOAD >= 0 && L < STEP_LOADS && FIRST_LOAD + L < LOADS) loader(std::integral_constant<int, FIRST_LOAD + L>{});
            });
        });
    };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using C2 = std::integral_constant<int, 2>;
    using C3 = std::integral_constant<int, 3>;
    using NoLoads = std::integral_constant<int, -1>;
    auto nothing = [](auto) {};
    // One K tile, held in stage S, its K step 0 already in fragment set 0.  Per K step the matrix instructions run out
    // of one fragment set while the next step's fragments are read into the other.  Between steps 1 and 2: this wave's
    // loads of the next K tile have landed (loads complete in order; those of the STAGES - 3 K tiles behind it may
    // still be on their way) - and behind the barrier every wave's have, and every wave has left the stage before S,
    // which the loads of the K tile STAGES - 1 ahead, one behind each matrix instruction of steps 2 and 3, fill
    // next.  Step 3 reads step 0 of the next K tile out of the next stage.
    auto k_tile = [&](auto stage_c) {
        constexpr int S = decltype(stage_c)::value;
        using Next = std::integral_constant<int, (S + 1) % STAGES>;
        constexpr int FREE = (S + STAGES - 1) % STAGES;
        mfma_step(C0{}, [&](auto r) { read_one(r, C1{}, C1{}, stage_c); }, NoLoads{}, nothing);
        wait_frags(1);
        mfma_step(C1{}, [&](auto r) { read_one(r, C2{}, C0{}, stage_c); }, NoLoads{}, nothing);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 3) * LOADS) : "memory");
        lds_barrier();
        wait_frags(0);
        mfma_step(C0{}, [&](auto r) { read_one(r, C3{}, C1{}, stage_c); }, C0{}, [&](auto l) { issue_one(FREE, l); });
        wait_frags(1);
        mfma_step(C1{}, [&](auto r) { read_one(r, C0{}, C0{}, Next{}); }, std::integral_constant<int, STEP_LOADS>{},
                  [&](auto l) { issue_one(FREE, l); });
        wait_frags(0);
    };
    // Prologue: K tiles 0 .. STAGES - 2 on their way into stages 0 .. STAGES - 2; K tile 0 landed and published; its
    // K step 0 in fragment set 0.
    static_for<STAGES - 1>([&](auto s_c) {
        static_for<LOADS>([&](auto l_c) { issue_one(decltype(s_c)::value, l_c); });
    });
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * LOADS) : "memory");
    lds_barrier();
    static_for<READS>([&](auto r) { read_one(r, C0{}, C0{}, C0{}); });
    wait_frags(0);
    for (int kt = 0; kt < KT_padded; kt += STAGES) static_for<STAGES>([&](auto s_c) { k_tile(s_c); });
    // matrix-instruction results are read by vector-ALU instructions next: cover the issue-to-write latency
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    // the loads still in flight (K tiles past the end: zeros) land, and every wave is done reading, before the
    // stages are written over by the epilogue's transposes
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();

    if (p.partial != nullptr) {
        store_partial<WTM, WTN>(p, acc, lane, m0 + wm * WTM, n0 + wn * WTN);
        return;
    }
    // whole tiles, and tiles that only reach past M, take the coalesced epilogue (rows at or past M are not stored)
    u32x4 *region = reinterpret_cast<u32x4 *>(lds_bytes + wave * EPILOGUE_BYTES);
    if (n0 + BN > N)
        store_tile<WTM, WTN, 1, BF16, true>(p, acc, region, lane, m0 + wm * WTM, n0 + wn * WTN);
    else if (m0 + BM <= M)
        store_tile<WTM, WTN, 1, BF16, false>(p, acc, region, lane, m0 + wm * WTM, n0 + wn * WTN);
    else
        store_tile<WTM, WTN, 1, BF16, false, 1, false, true>(p, acc, region, lane, m0 + wm * WTM, n0 + wn * WTN);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, bool BF16, bool B_ROW = false>
int launch_ring(Params p, hipStream_t stream) {
    constexpr size_t lds_bytes = static_cast<size_t>(STAGES) * (BM + BN) * kBK * 2;
    if (p.K % 8 != 0 || p.k_slice % 8 != 0) return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: the ring variant takes a K (and K slices) that are multiples of 8");
    if (B_ROW && (p.N % 8 != 0 || p.ldb % 8 != 0))
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: the ring variant takes a row-major B whose N and row stride are multiples of 8");
    const int slices = p.k_slice > 0 ? (p.K + p.k_slice - 1) / p.k_slice : 1;
    auto kernel = gemm16_ring_kernel<BM, BN, WAVES_M, WAVES_N, STAGES, BF16, B_ROW>;
    static std::atomic<uint64_t> configured{0};  // per instantiation: the devices whose LDS limit is raised
    if (const int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds_bytes, configured); st != KO_OK) return st;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int64_t tiles = static_cast<int64_t>((p.M + BM - 1) / BM) * p.tiles_n;
    if (tiles > 0x7fffffff) return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: too many tiles for the ring variant");
    p.nblocks = static_cast<int>(tiles);
    kernel<<<dim3(static_cast<unsigned>(p.nblocks), static_cast<unsigned>(slices)), dim3(64 * WAVES_M * WAVES_N), lds_bytes, stream>>>(p);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <class T, bool BF16>
int launch_persistent(Params p, hipStream_t stream) {
    constexpr size_t lds_bytes = 2u * (T::BM + T::BN) * kBK * sizeof(uint16_t);
    if ((p.M % T::BM) != 0 || (p.N % T::BN) != 0 || (p.K % kBK) != 0)
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: the persistent variant needs full tiles");
    auto kernel = gemm16_persistent_kernel<T, BF16>;
    static std::atomic<uint64_t> configured{0};  // per instantiation: the devices whose LDS limit is raised
    if (const int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds_bytes, configured); st != KO_OK)
        return st;
    p.tiles_n = p.N / T::BN;
    p.nblocks = (p.M / T::BM) * p.tiles_n;
    int grid = compute_units() / 8 * 8;  // a multiple of the XCD count keeps a workgroup's tiles on its XCD's band
    if (grid > p.nblocks) grid = p.nblocks;
    kernel<<<dim3(static_cast<unsigned>(grid)), dim3(T::THREADS), lds_bytes, stream>>>(p);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <class T, bool BF16, bool B_ROW_MAJOR, bool EDGE>
int launch_edge(const Params &p, hipStream_t stream) {
    constexpr int THREADS = T::THREADS;
    constexpr size_t lds_bytes = 2u * (T::BM + T::BN) * kBK * sizeof(uint16_t);
    auto kernel = gemm16_kernel<T, BF16, B_ROW_MAJOR, EDGE>;
    static std::atomic<uint64_t> configured{0};  // per instantiation: the devices whose LDS limit is raised
    if (const int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds_bytes, configured); st != KO_OK)
        return st;
    const int slices = p.k_slice > 0 ? (p.K + p.k_slice - 1) / p.k_slice : 1;
    kernel<<<dim3(static_cast<unsigned>(p.nblocks), static_cast<unsigned>(slices)), dim3(THREADS), lds_bytes, stream>>>(p);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <class T, bool BF16, bool B_ROW_MAJOR>
int launch(Params p, hipStream_t stream) {
    const int tiles_m = (p.M + T::BM - 1) / T::BM;
    p.tiles_n = (p.N + T::BN - 1) / T::BN;
    p.nblocks = tiles_m * p.tiles_n;
    // K slices are a multiple of the K tile deep; only the last one can end inside a K tile
    const bool edge = (p.M % T::BM) != 0 || (p.N % T::BN) != 0 || (p.K % kBK) != 0 || (p.k_slice % kBK) != 0;
    if (edge) return launch_edge<T, BF16, B_ROW_MAJOR, true>(p, stream);
    return launch_edge<T, BF16, B_ROW_MAJOR, false>(p, stream);
}

using TileBig = Tiling<256, 256, 2, 4, 1, true, 1>;     // 8 waves, wave tile 128x64
using TileSmall = Tiling<128, 128, 2, 2, 2, true, 1>;   // 4 waves, wave tile 64x64, two register stages
using TileSmallN = Tiling<128, 64, 2, 2, 2, true, 1>;   // 4 waves, wave tile 64x32
using TileTiny = Tiling<64, 64, 2, 2, 2, true, 1>;      // 4 waves, wave tile 32x32
using TileSkinny = Tiling<32, 256, 1, 4, 2, true, 1>;   // 4 waves side by side, wave tile 32x64: at most 32 rows of A

using TileHalf = Tiling<128, 256, 2, 4, 1, true, 1>;    // pinned kernel only: 8 waves, wave tile 64x64
using TileBigSpare = Tiling<256, 256, 2, 4, 1, true, 1, true>;  // the same, epilogue through the spare 32 KB of LDS
using TileBigSpread = Tiling<256, 256, 2, 4, 1, true, 1, true, true>;  // and the loads issued one by one in K step 3

// The direct-to-LDS kernels need full 256x256x64 tiles; the pinned one takes B in either layout, the
// compiler-scheduled one K-contiguous (column-major) B only.
template <class T, bool BF16, bool B_ROW_MAJOR, bool PINNED>
int launch_direct(const Params &p, hipStream_t stream) {
    if constexpr (PINNED) {
        return launch_pinned<T, BF16, B_ROW_MAJOR>(p, stream);
    } else if constexpr (B_ROW_MAJOR) {
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: this direct-to-LDS variant needs column-major B");
    } else {
        return launch_persistent<T, BF16>(p, stream);
    }
}

// D = act(alpha * (P_0 + ... + P_{slices-1}) + beta * C + bias), rounded once, from the fp32 partial products of a
// K-sliced launch, summed in slice order.  One thread per four consecutive columns; the last group of a row whose
// length is not a multiple of 4 finishes its columns one by one.  slices == 0 is the empty product (k == 0): nothing
// is read through p.partial and D = act(beta * C + bias).
template <bool BF16>
__global__ __launch_bounds__(64) void gemm16_slices_sum_kernel(const Params p, int slices) {
    typedef float float4v __attribute__((ext_vector_type(4)));
    const int64_t ldp = partial_ld(p.N);
    const int groups_per_row = static_cast<int>(ldp / 4);
    const int64_t g = static_cast<int64_t>(blockIdx.x) * 64 + threadIdx.x;
    if (g >= static_cast<int64_t>(p.M) * groups_per_row) return;
    const int m = static_cast<int>(g / groups_per_row), n = static_cast<int>(g % groups_per_row) * 4;
    const int64_t count = p.M * ldp;
    const float *src = p.partial + m * ldp + n;
    float4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
    if (slices > 0) acc = *reinterpret_cast<const float4v *>(src);
    int s = 1;
    for (; s + 8 <= slices; s += 8) {
        float4v t[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) t[j] = *reinterpret_cast<const float4v *>(src + (s + j) * count);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc += t[j];
    }
    for (; s < slices; ++s) acc += *reinterpret_cast<const float4v *>(src + s * count);
    const bool use_c = p.C != nullptr && p.beta != 0.0f;
    const int64_t off = static_cast<int64_t>(m) * p.ldd + n;
    float v[4] = {acc[0], acc[1], acc[2], acc[3]};
    if (n + 3 < p.N) {
        u32x2 c2 = {0, 0}, b2 = {0, 0};
        if (use_c) c2 = *reinterpret_cast<const u32x2_rows *>(p.C + off);
        if (p.bias) b2 = *reinterpret_cast<const u32x2_rows *>(p.bias + n);
        finish4<BF16>(p, v, c2, b2, use_c);
        u32x2 o;
        o[0] = pack2<BF16>(v[0], v[1]);
        o[1] = pack2<BF16>(v[2], v[3]);
        *reinterpret_cast<u32x2_rows *>(p.D + off) = o;
    } else {
        u32x2 c2 = {0, 0}, b2 = {0, 0};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (n + e >= p.N) continue;
            if (use_c) c2[e >> 1] |= static_cast<uint32_t>(p.C[off + e]) << ((e & 1) * 16);
            if (p.bias) b2[e >> 1] |= static_cast<uint32_t>(p.bias[n + e]) << ((e & 1) * 16);
        }
        finish4<BF16>(p, v, c2, b2, use_c);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (n + e < p.N) p.D[off + e] = from_float<BF16>(v[e]);
    }
}

// K slices for a deep K on few output tiles (weight-gradient shapes: 768 x 768 x 16384 is 36 tiles of 128 x 128).
// As in the SGEMM: the slices are workgroups of one launch of the register pipeline (blockIdx.y), their fp32 partial
// products go to the stream's workspace, a second kernel sums them in slice order and applies the whole epilogue
// once.  From K = 2048 on, by tile count (measured against the whole problem, us):
//   - at most a quarter of the compute units' worth of 128 x 128 tiles: slices at least 512 deep up to one
//     workgroup per compute unit, of 128 x 128 or 64 x 64 tiles, whichever comes closer to that (64 x 64 on a tie):
//     768 x 768 x 16384 82 -> 40 (7 slices of 36 tiles), 512 x 512 x 8192 43 -> 18, 256 x 256 x 16384 81 -> 15,
//     1024 x 1024 x 8192 46 -> 34;
//   - up to one such tile per compute unit: slices at least 2048 deep up to two workgroups per compute unit:
//     768 x 2304 x 16384 130 -> 97 (4 slices of 108 tiles), 768 x 3072 x 16384 172 -> 121; shallower slices lose
//     (2048 x 768 x 3072: 25.5 whole, 27 in four slices).
struct SlicePlan16 {
    int slices = 1, k_slice = 0;
    int tile = 64;  // 128: 128 x 128 tiles, 64: 64 x 64, 32: the 32 x 256 tiles of a problem with at most 32 rows
};

SlicePlan16 plan_k_slices16(const Params &p, size_t workspace_bytes) {
    SlicePlan16 plan;
    const int forced = tuning(knob_gemm16_k_slices);
    if (forced == 1) return plan;
    const int64_t cu = compute_units();
    const double out_bytes = 4.0 * p.M * partial_ld(p.N);  // of one partial product
    auto set = [&](int64_t slices, int tile) {
        if (slices < 2) return;
        const int64_t unit = tile == 256 ? 2 * kBK : kBK;  // the pinned kernel takes K tiles in pairs
        const int64_t depth = ((p.K + slices - 1) / slices + unit - 1) / unit * unit;
        slices = (p.K + depth - 1) / depth;
        if (slices < 2 || slices > 65535 || slices * out_bytes > static_cast<double>(workspace_bytes)) return;
        plan.slices = static_cast<int>(slices);
        plan.k_slice = static_cast<int>(depth);
        plan.tile = tile;
    };
    const int64_t t128 = static_cast<int64_t>((p.M + 127) / 128) * ((p.N + 127) / 128);
    const int64_t t64 = static_cast<int64_t>((p.M + 63) / 64) * ((p.N + 63) / 64);
    const bool pinned_ok = p.N % 256 == 0 && p.K % 8 == 0 && p.K < (1 << 22);  // the pinned kernel's 256 x 256 tiles
    if (forced >= 2) {
        if (tuning(knob_gemm16_variant) == 62 && pinned_ok) set(forced, 256);
        else set(forced, p.M <= 32 && p.N >= 256 ? 32 : t128 * forced >= cu / 2 ? 128 : 64);
        return plan;
    }
    const int64_t fit = static_cast<int64_t>(static_cast<double>(workspace_bytes) / out_bytes);  // slices the workspace holds
    auto capped = [&](int64_t slices, int64_t min_depth) {
        if (slices > p.K / min_depth) slices = p.K / min_depth;
        return slices < fit ? slices : fit;
    };
    if (p.M <= 32 && p.N >= 256 && p.K >= 2048) {
        // A batch of a few rows against a weight matrix: the time is B's, read once.  32 x 256 tiles (one matrix
        // instruction's worth of rows), slices at least 256 deep up to two workgroups per compute unit, so that
        // every compute unit streams its share of B.
        const int64_t skinny = (p.N + 255) / 256;
        if (skinny <= cu) set(capped(2 * cu / skinny, 256), 32);
        if (plan.slices > 1) return plan;
    }
    // (few tiles: from K = 1536 on - 128 x 128 x 1536 9.9 us whole, 8.7 in three slices; 100 x 100 x 1536 13.2 and
    // 9.1; at K = 1024 the second launch costs what the slices gain)
    if (p.K < (4 * t128 <= cu ? 1536 : 2048)) return plan;
    // More than a quarter of the compute units' worth of 128 x 128 tiles, at most half of them of 256 x 256, and a K
    // beyond what the ring kernel takes whole: the pinned kernel's 256 x 256 tiles in as many slices, at least 2048
    // deep, as give every compute unit at most one (us, hipBLASLt in brackets: 2048 x 4096 x 16384 314 -> 260 (239),
    // 1536 x 4096 x 16392 384 -> 272 (224), 1024 x 3072 x 16384 168 -> 124 (97), 768 x 3072 x 16384 127 -> 102 (79) - in
    // four slices 116, in two 199; at K = 8192 the ring kernel's 80 us for 1024 x 4096 become 90)
    const int64_t t256 = static_cast<int64_t>((p.M + 255) / 256) * ((p.N + 255) / 256);
    if (pinned_ok && tuning(knob_gemm16_wave_k) != 1 && 4 * t128 > cu && 2 * t256 <= cu && p.K > 8192) {
        set(capped(cu / t256, 2048), 256);
        if (plan.slices > 1) return plan;
    }
    if (4 * t128 <= cu) {
        // (128 x 128 tiles when their slices come to three quarters of the compute units or more - they run the ring
        // kernel, one workgroup per compute unit: 1024 x 512 x 32768 two slices of 64 x 64 tiles 123 us, eight of
        // 128 x 128 57 (hipBLASLt 50); 512 x 512 x 32768 64 -> 39 (32), 512 x 1024 x 16384 52 -> 36 (27), 256 x 1024 x 16384
        // 30 -> 23 (19); 256 x 256 x 16384, four such tiles, stays on 16 slices of 64 x 64: 14.7 us)
        // (the partial products cost what more workgroups gain: 768 x 768 x 16384 7 slices 39.3 us, 5 37.6; 512 x 1024 x 16384
        // 8 33.4, 5 31.6; 256 x 1024 x 16384 16 27.3, 8 22.9; 512 x 768 x 12288 10 27.7, 6 23.4)
        // Measured on the ring kernel's tiles, us by slices: 768 x 768 x 8192 4: 23.3, 5: 28.4, 8: 31.6; 1412 x 440 x 8952
        // 2: 43.5, 4: 31.3, 5: 33.1; 1856 x 320 x 6144 3: 21.7, 4: 22.6, 6: 30.1; 1024 x 512 x 32768 6: 64.8, 8: 56.7.  So:
        // three quarters of the compute units' worth of workgroups - all of them when the slices are still 4096 deep -
        // in slices at least 2048 deep, or a quarter of K while K is at most 8192 (and 1024).
        const int64_t s_fill = cu / t128, s_most = (3 * cu + 2 * t128) / (4 * t128);
        const int64_t quarter = p.K / 4 > 1024 ? p.K / 4 : 1024;
        const int64_t min128 = p.K <= 8192 ? quarter : 2048;
        const int64_t s128 = capped(p.K / s_fill >= 4096 ? s_fill : s_most, min128), s64 = t64 <= cu ? capped(cu / t64, 512) : 1;
        if (s64 >= 2 && s64 * t64 >= s128 * t128 && 2 * s128 * t128 < cu) set(s64, 64);
        else set(s128, 128);
    } else if (t128 <= cu) {
        set(capped(2 * cu / t128, 2048), 128);
    }
    return plan;
}

template <bool BF16, bool B_ROW_MAJOR>
int run_sliced16(const Params &p, const SlicePlan16 &plan, float *workspace, hipStream_t stream) {
    Params part = p;
    part.k_slice = plan.k_slice;
    part.partial = workspace;
    // 128 x 128 tiles: the ring kernel while the slices are at most one workgroup per compute unit (it is one
    // workgroup per compute unit; the register pipeline runs two): 1024 x 768 x 16384 in 5 slices 51.7 -> 45.8 us,
    // 1024 x 1024 x 16384 62.3 -> 55.1, 2048 x 512 x 32768 119 -> 98; with more it loses (1024 x 2304 x 16384, 432 workgroups:
    // 119 us against 144)
    const int64_t t128 = static_cast<int64_t>((p.M + 127) / 128) * ((p.N + 127) / 128);
    const bool ring = plan.tile == 128 && tuning(knob_gemm16_wave_k) != 1 && t128 * plan.slices <= compute_units() &&
                      (!B_ROW_MAJOR || (p.N % 8 == 0 && p.ldb % 8 == 0));
    int st = plan.tile == 256 ? launch_pinned<TileBigSpread, BF16, B_ROW_MAJOR, true, true>(part, stream)
             : ring            ? launch_ring<128, 128, 2, 2, 4, BF16, B_ROW_MAJOR>(part, stream)
             : plan.tile == 128 ? launch<TileSmall, BF16, B_ROW_MAJOR>(part, stream)
             : plan.tile == 32 ? launch<TileSkinny, BF16, B_ROW_MAJOR>(part, stream)
                               : launch<TileTiny, BF16, B_ROW_MAJOR>(part, stream);
    if (st != KO_OK) return st;
    const int64_t groups = p.M * (partial_ld(p.N) / 4);
    gemm16_slices_sum_kernel<BF16><<<dim3(static_cast<unsigned>((groups + 63) / 64)), dim3(64), 0, stream>>>(part, plan.slices);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

// Which problems go to the kernel that splits K over the waves of a workgroup (gemm16_wave_k_kernel; timings with B column-major):
// those whose output is at most one workgroup per compute unit of its tiles - the smallest of 32 x 32 (K over eight
// waves), 32 x 64 and 64 x 64 (over four) that the problem does not exceed that with - and whose K is neither so
// shallow that the other kernels' few steps cost nothing, nor so deep that the bytes a small tile draws from the
// L2s per flop outweigh the steps saved (a compute unit takes in some 85 GB/s this way: 768 x 768 x 16384 on
// 64 x 64 tiles 47 us, in K slices of 128 x 128 tiles 42).  Measured against the dispatch below (hipBLASLt), us:
// 100 x 1024 x 1024 9.0 -> 5.7 (5.5), 256 x 768 x 3072 12.5 -> 8.1 (8.6), 512 x 1024 x 4096 17.7 -> 12.3 (13.6),
// 100 x 4096 x 4096 19.5 -> 11.7 (14.4), 1000 x 1024 x 4096 24.4 -> 18.3 (18.0), 768 x 768 x 4096 19.8 -> 16.0 (16.2),
// 32 x 768 x 3072 11.4 -> 6.5 (7.1); with more tiles than compute units it loses (512 x 3072 x 768: 10.3 against 14.1).
// (64 x 128 and 128 x 64 tiles over three waves gained less - 512 x 4096 x 4096 38.0 -> 31.7, 2048 x 768 x 3072 27.6 ->
// 24.9 - than the ring kernel below does on those problems, and are gone.)
// With B as [K][N] the tiles gain as much (100 x 1024 x 1024 12.2 -> 4.4 us, 1000 x 1024 x 4096 30.4 -> 20.4; hipBLASLt
// 5.7 and 17.3).  Returns 0, or 1000 * rows + columns of the tile: 32032, 32064, 64064.
int wave_k_tile(int64_t m, int64_t n, int64_t k, bool b_row_major) {
    if (tuning(knob_gemm16_wave_k) == 1 || tuning(knob_gemm16_k_slices) != 0 || k > 8192) return 0;
    const int64_t cu = compute_units();
    const int64_t m32 = (m + 31) / 32, m64 = (m + 63) / 64, n32 = (n + 31) / 32, n64 = (n + 63) / 64;
    if (m32 * n32 <= cu) return k >= 128 ? 32032 : 0;
    // (the larger tiles up to a K where K slices of the ring kernel's 128 x 128 tiles take over: 1856 x 320 x 6144 27.1 us
    // here, 21.7 in three slices; 768 x 768 x 8192 28.7 / 23.3; 1536 x 512 x 6144 29.1 / 22.4; 2048 x 256 x 8192 on 32 x 64
    // tiles 24.4 / 21.0; at K = 4096 level - 768 x 768 16.7 / 16.8, 1024 x 1024 18.5 / 22.8)
    if (m32 * n64 <= cu) return k >= 256 && k < 8192 ? 32064 : 0;
    // (with at most three quarters of the compute units' worth of tiles from K = 5120 on: 1868 x 303 x 5720 34.3 / 23.6)
    if (m64 * n64 <= cu) return k >= 1024 && k < (4 * m64 * n64 <= 3 * cu ? 5120 : 6144) ? 64064 : 0;
    return 0;
}

// Which problems go to the kernel with the deep ring of LDS stages (gemm16_ring_kernel; B column-major): those that
// are at most one tile of 128 x 128 per compute unit - of 128 x 64 or 64 x 128 when that still holds with those (the
// short side of the tile along the longer side of the output: fewer distinct panels of A and B per XCD) - and too
// many small tiles for the kernel above.  Measured against the dispatch below (hipBLASLt), us: 4096 x 1024 x 4096
// 59.5 -> 36.8 (36.8), 3000 x 1024 x 4096 51.3 -> 33.0 (30.1), 1000 x 4096 x 4096 62.9 -> 45.3 (37.7), 4096 x 768 x
// 3072 37.1 -> 26.4 (25.0), 3000 x 768 x 3072 35.9 -> 25.3 (21.9), 4096 x 1024 x 1024 16.2 -> 13.2 (13.4); on the half
// tiles 2048 x 768 x 3072 23.7 -> 17.7 (17.3), 2048 x 1024 x 4096 33.2 -> 25.9 (24.4), 512 x 4096 x 4096 31.4 -> 27.4
// (24.5), 512 x 4096 x 1024 13.1 -> 10.4 (9.8); with more tiles than compute units the pinned kernel wins (6000 x 768
// x 3072: 43.4 us against 48.6; 256 x 128 and 128 x 256 tiles of this kernel, three stages of 48 KB, four waves of
// 128 x 64, came out level with the pinned kernel there - 46.4, 8192 x 1024 x 4096 76 - 80 against 80 - and are not kept).
// With B as [K][N] (hipBLASLt on that layout in brackets): 3000 x 768 x 3072 45.2 -> 24.2
// (26.0), 4096 x 1024 x 4096 56.2 -> 40.3 (40.8), 1000 x 4096 x 4096 74.2 -> 43.4 (40.4), 3000 x 1024 x 1024 21.7 -> 11.5
// (12.8), 512 x 4096 x 1024 16.1 -> 11.2 (11.4); the half tile there is 128 x 64 whatever the shape (64 x 128 - rows of
// 256 bytes in the stage of B - is the slower one: 2048 x 768 x 3072 22.7 against 20.6).
// Returns 0, or 1000 * rows + columns of the tile: 64128, 128064, 128128; 1032064 for the 32 x 64 tiles of a problem of
// at most 32 rows (the million tells them from the other kernel's 32 x 64).
int ring_tile(int64_t m, int64_t n, int64_t k, bool b_row_major) {
    // (a K beyond 8192 is left to the K slices below, which run this kernel's 128 x 128 tiles: 512 x 2304 x 16384 whole on
    // 144 tiles of 128 x 64 103 us, in slices 67)
    if (tuning(knob_gemm16_wave_k) == 1 || tuning(knob_gemm16_k_slices) != 0 || k < 512) return 0;
    const int64_t cu = compute_units();
    const int64_t m64 = (m + 63) / 64, m128 = (m + 127) / 128, n64 = (n + 63) / 64, n128 = (n + 127) / 128;
    // At most 32 rows against more columns than the kernel above takes (a decoding step against a vocabulary or a wide
    // feed-forward weight): 32 x 64 tiles, two waves, two workgroups per compute unit, however many rounds - the time is
    // the weights' way out of memory, and rows of A that a taller tile would fetch again and again are not.  Before
    // -> now (hipBLASLt), us: 8 x 28672 x 4096 52.3 -> 42.7 (37.5), 32 x 32000 x 4096 58.5 -> 51.2 (43.6), 8 x 128256 x 4096
    // 237 -> 177 (151), 8 x 50304 x 1024 27.2 -> 23.7 (18.5); 32 x 128 tiles with six stages (one workgroup per compute
    // unit) 47.6 / 56.1 / 181 / 24.0, with three 61 / 70 / 190 / 20.7.
    if (m <= 32 && n64 > cu) return 1032064;
    // (a K beyond 8192 only where neither two slices fit a round nor the pinned kernel's slices apply - more than half
    // a chip's worth of 128 x 128 tiles, N not whole 256 x 256 tiles: 311 x 7983 x 8216 in two slices of the register
    // pipeline 111 us, whole here 97; x 12000 143 / 128)
    if (k > 8192 && !(k <= 16384 && n % 256 != 0 && m128 * n128 <= cu && 2 * m128 * n128 > cu)) return 0;
    // One row of tiles against more columns than compute units (64 or 128 rows against a vocabulary): this kernel in
    // several rounds, where the persistent kernels' 256 x 256 tiles are mostly rows that do not exist
    // (64 x 128256 x 4096 258 -> 187 us (hipBLASLt 174), 128 x 128256 x 4096 274 -> 215 (204), 64 x 50304 x 1024 31.8 -> 27.8
    // (21.7); 128 x 50304 x 1024 stays: 31.9 against 33.6)
    if (m > 32 && m <= 64 && n128 > cu && !b_row_major) return 64128;
    if (m > 32 && m <= 128 && n128 > cu && k >= 2048) return 128128;
    if (m64 * n64 <= cu) return 0;  // few tiles: the kernel above
    if (b_row_major) {
        if (m128 * n64 <= cu) return 128064;
    } else if (n > m ? m128 * n64 <= cu : m64 * n128 <= cu) {
        return n > m ? 128064 : 64128;
    }
    if (m128 * n128 <= cu) return 128128;
    return 0;
}

// One call becomes at most five launches: one column cut (left, right), then at most two row cuts in the left
// part (the rows below the last full round, and of those the rows below the last full tile row) and one in the
// right part.  col_cut / row_cuts are what a (sub-)problem may still spend; the knobs are read once per call.
template <bool BF16, bool B_ROW_MAJOR>
int launch_variant(const Params &p, hipStream_t stream, bool col_cut = true, int row_cuts = 2, int variant = -1,
                   int split_knob = -1) {
    if (variant < 0) {
        variant = tuning(knob_gemm16_variant);
        split_knob = tuning(knob_gemm16_split_rows);
        if (variant < 0) variant = 0;
    }
    if (variant <= 0 && p.k_slice == 0 && (!B_ROW_MAJOR || (p.N % 8 == 0 && p.ldb % 8 == 0))) {
        // the whole problem, or a part cut off it, when it is small
        switch (wave_k_tile(p.M, p.N, p.K, B_ROW_MAJOR)) {
            case 32032: return launch_wave_k<1, 1, 8, BF16, B_ROW_MAJOR>(p, stream);
            case 32064: return launch_wave_k<1, 2, 4, BF16, B_ROW_MAJOR>(p, stream);
            case 64064: return launch_wave_k<2, 2, 4, BF16, B_ROW_MAJOR>(p, stream);
            default: break;
        }
    }
    if (variant <= 0 && p.k_slice == 0 && (!B_ROW_MAJOR || (p.N % 8 == 0 && p.ldb % 8 == 0))) {
        switch (ring_tile(p.M, p.N, p.K, B_ROW_MAJOR)) {
            case 1032064: return launch_ring<32, 64, 1, 2, 6, BF16, B_ROW_MAJOR>(p, stream);
            case 64128: return launch_ring<64, 128, 2, 2, 6, BF16, B_ROW_MAJOR>(p, stream);
            case 128064: return launch_ring<128, 64, 2, 2, 6, BF16, B_ROW_MAJOR>(p, stream);
            case 128128: return launch_ring<128, 128, 2, 2, 4, BF16, B_ROW_MAJOR>(p, stream);
            default: break;
        }
    }
    if ((variant <= 0 || variant == 62) && p.k_slice == 0) {
        // the whole problem, or a part cut off it (the launches of one call follow each other on the stream and may
        // use its workspace one after the other): few tiles and a deep K go out as K slices
        const int64_t big = static_cast<int64_t>((p.M + 255) / 256) * ((p.N + 255) / 256);
        if (2 * big <= compute_units() || p.M <= 32 || variant == 62) {
            if (const SlicePlan16 plan = plan_k_slices16(p, kStreamWorkspaceBytes); plan.slices > 1) {
                void *workspace = nullptr;
                if (const int st = stream_workspace(stream, &workspace); st != KO_OK) return st;
                if (workspace != nullptr) return run_sliced16<BF16, B_ROW_MAJOR>(p, plan, static_cast<float *>(workspace), stream);
            }
        }
    }
    if (variant <= 0) {
        // Enough 256x256 tiles to fill the chip: the big tiling - as a persistent direct-to-LDS kernel
        // when the tiles are full (the pinned one from K = 128 on; a K that is not a multiple of 128 is padded
        // with zeros inside the kernel), else as the register pipeline.
        // Fewer: smaller tiles so that the grid still covers the compute units.
        const int64_t big_tiles = static_cast<int64_t>((p.M + 255) / 256) * ((p.N + 255) / 256);
        // Two reasons to send the last rows out as a launch of their own, with the tiling their size asks for:
        // rows that do not fill the last row of big tiles would take the whole problem off the pinned kernel
        // (16000 x 3072 x 768: 123 us, against 78 us as 15872 + 128 rows), and a last round of a few big
        // tiles costs a whole round - that one pays while the rows cut off hold at most a sixth of a round
        // (4352 x 4096 x 1024, 272 tiles on 256 compute units: 52.7 -> 42.7 us; 8192 x 2304 x 768, 288 tiles:
        // 41.1 -> 37.4 us; with 65 or 72 tiles below the cut the small tilings take as long as the round they
        // replace).
        // Columns that do not fill the last column of big tiles: the full tile columns go out on their own -
        // to the pinned kernel when the rest of the shape allows - and the remaining columns (fewer than 256)
        // as a launch of their own; C, D and a row-major B keep their row strides.
        // A shallow K on a shape that is not whole 256 x 256 tiles: the time is the output's, and what counts is that
        // a compute unit has a second workgroup to load and multiply while the first one stores (128 x 128 tiles,
        // two workgroups per compute unit), not the rate of the main loop - neither the cuts below (whose parts
        // run one after the other, each a launch that ends in a round of stores) nor 256 x 256 tiles pay.  Measured,
        // whole on 128 x 128 tiles against cut (hipBLASLt), us: 4197 x 11928 x 64 48 / 58 (31), x 128 55 / 78 (38),
        // x 256 81 / 71 (58); 4880 x 7768 x 256 52 / 60 (41), x 512 82 / 82; 1351 x 18488 x 256 41 / 45, x 512 65 / 60;
        // 8148 x 1800 x 512 30 / 37 (27); 3000 x 5000 x 256 22 / 29 (22), x 512 34 / 38 (28); 4071 x 2328 x 768
        // (160 big tiles) 32 / 41 (24), 12521 x 989 x 768 40 / 52 (30), 3000 x 5000 x 768 (240) 46 / 48.
        // A row count that is not a multiple of the tile height (any: 4093 x 3072 x 768 40.3 -> 26.6 us, at 4096 rows
        // 25.5), on whole tile columns: the pinned kernel
        // takes it as it is (its last row of tiles fetches rows it has, and stores what lies inside the matrix),
        // so such a shape is neither cut nor taken off that kernel.  3000 x 3072 x 768: 30.0 -> 22.1 us (hipBLASLt
        // 19.5), 12000 x 768 x 3072 84 -> 73, 3000 x 4096 x 4096 112 -> 93, 16000 x 3072 x 768 82 -> 76; on
        // 128 x 256 tiles 6000 x 1024 x 1024 25.5 -> 18.0 (17.8), 6000 x 768 x 3072 55 -> 44.
        const bool m_edge = p.M % 256 != 0 && p.N % 256 == 0 && p.K >= 2 * kBK && p.K < (1 << 22);
        {
            const int64_t cu = compute_units();
            const bool ragged = p.M % 256 != 0 || p.N % 256 != 0;
            if (ragged && split_knob != 1 && 2 * big_tiles >= cu && !(m_edge && p.K > 512) &&
                (p.K <= 128 || (p.K <= 256 && 2 * big_tiles <= 5 * cu) || (p.K <= 512 && 4 * big_tiles <= 5 * cu) ||
                 (p.K <= 768 && 5 * big_tiles <= 4 * cu)))
                return launch<TileSmall, BF16, B_ROW_MAJOR>(p, stream);
        }
        if (col_cut && split_knob != 1 && p.N % 256 != 0 && p.N > 256 && (!B_ROW_MAJOR || (p.ldd % 8 == 0 && p.ldb % 8 == 0)) &&
            p.K >= 2 * kBK && 2 * static_cast<int64_t>(p.M / 256) * (p.N / 256) >= compute_units()) {
            const int n1 = p.N - p.N % 256;
            Params left = p, right = p;
            left.N = n1;
            right.N = p.N - n1;
            right.B = B_ROW_MAJOR ? p.B + n1 : p.B + static_cast<int64_t>(n1) * p.K;
            right.C = p.C ? p.C + n1 : nullptr;
            right.D = p.D + n1;
            right.bias = p.bias ? p.bias + n1 : nullptr;
            if (const int st = launch_variant<BF16, B_ROW_MAJOR>(left, stream, false, 2, variant, split_knob); st != KO_OK)
                return st;
            return launch_variant<BF16, B_ROW_MAJOR>(right, stream, false, 1, variant, split_knob);
        }
        // Between half a chip's and a whole chip's worth of 128 x 256 tiles: the pinned kernel on those (8 waves
        // of 64 x 64).  A K tile takes it as long as one of a 256 x 256 tile (a third LDS stage did not change
        // that), but twice as many compute units work: 1536 x 4096 x 4096 (96 big tiles)
        // 93 -> 79 us, 7168 x 768 x 3072 (84) 62 -> 52, 8192 x 1024 x 1024 (128) 27 -> 21, 2048 x 2304 x 768 (72)
        // 17.4 -> 15.3; with 128 or fewer of them (4096 x 1024 x 1024 18.5 against 16.5) or more than one per
        // compute unit (3072 x 4096 x 4096: 143 against 113) the other tilings win.  Rows below the last whole
        // 128 go out as a launch of their own.
        if (split_knob != 1 && p.N % 256 == 0 && p.K >= 256) {
            const int64_t cu = compute_units();
            const int64_t rows128 = m_edge ? (p.M + 127) / 128 : p.M / 128;
            const int64_t half_tiles = rows128 * (p.N / 256);
            // (the second launch costs about 2 us: 2000 x 3072 x 768 22 us whole on 128 x 128 tiles, 24 cut; from
            // K = 1536 on the first one gains more than that - 7000 x 768 x 3072 66 -> 58, 2000 x 4096 x 4096 117 -> 103)
            if (20 * half_tiles >= 11 * cu && half_tiles <= cu && (p.M % 128 == 0 || m_edge || (row_cuts > 0 && p.K >= 1536))) {
                if (p.M % 128 == 0) return launch_pinned<TileHalf, BF16, B_ROW_MAJOR>(p, stream);
                if (m_edge) return launch_pinned<TileHalf, BF16, B_ROW_MAJOR, true>(p, stream);
                const int64_t m1 = rows128 * 128;
                Params top = p, bottom = p;
                top.M = static_cast<int>(m1);
                bottom.M = p.M - static_cast<int>(m1);
                bottom.A = p.A + m1 * p.K;
                bottom.C = p.C ? p.C + m1 * p.ldd : nullptr;
                bottom.D = p.D + m1 * p.ldd;
                if (const int st = launch_pinned<TileHalf, BF16, B_ROW_MAJOR>(top, stream); st != KO_OK) return st;
                return launch_variant<BF16, B_ROW_MAJOR>(bottom, stream, false, row_cuts - 1, variant, split_knob);
            }
        }
        if (row_cuts > 0 && split_knob != 1 && p.K >= 256) {
            const int64_t cu = compute_units();
            const int64_t tn = (p.N + 255) / 256;
            const bool pinned_ok = p.N % 256 == 0 && p.K >= 2 * kBK;
            int64_t rows_top = p.M % 256 != 0 && pinned_ok && !m_edge ? p.M / 256 : (p.M + 255) / 256;  // in tile rows
            const int64_t tiles = rows_top * tn, rounds = tiles / cu;
            if (rounds >= 1 && tiles % cu != 0) {
                const int64_t rows1 = rounds * cu / tn;  // whole tile rows within the full rounds
                const int64_t rest = (rows_top - rows1) * tn;
                // (up to a quarter of a round when the rows cut off then are one pass of the ring kernel's 128 x 128
                // tiles: 20000 x 1024 x 4096, 316 tiles, 199 -> 171 us; 20000 x 1024 x 1024 53.6 -> 47.0)
                const bool ring_rest = p.K >= 1024 && p.K <= 8192 && 4 * rest <= cu && tuning(knob_gemm16_wave_k) != 1 &&
                                       (!B_ROW_MAJOR || (p.N % 8 == 0 && p.ldb % 8 == 0));
                if (rows1 >= 1 && (6 * rest <= cu || ring_rest)) rows_top = rows1;
            }
            if (rows_top * 256 < p.M && 2 * rows_top * tn >= cu) {
                const int64_t m1 = rows_top * 256;
                Params top = p, bottom = p;
                top.M = static_cast<int>(m1);
                bottom.M = p.M - static_cast<int>(m1);
                bottom.A = p.A + m1 * p.K;
                bottom.C = p.C ? p.C + m1 * p.ldd : nullptr;
                bottom.D = p.D + m1 * p.ldd;
                // the top part holds whole rounds or whole tile rows: it is not cut again
                if (const int st = launch_variant<BF16, B_ROW_MAJOR>(top, stream, false, 0, variant, split_knob); st != KO_OK)
                    return st;
                return launch_variant<BF16, B_ROW_MAJOR>(bottom, stream, false, row_cuts - 1, variant, split_knob);
            }
        }
        // The pinned kernel is so much faster per tile that it wins from half a chip's worth of full tiles on
        // (192 tiles on 256 CUs: 16384 x 768 x 3072 takes 69 us against 103 us with 128 x 128 tiles; at 96 tiles
        // the two are level).
        if (2 * big_tiles >= compute_units() && p.M % 256 == 0 && p.N % 256 == 0 && p.K >= 2 * kBK)
            return launch_pinned<TileBigSpread, BF16, B_ROW_MAJOR>(p, stream);
        if (2 * big_tiles >= compute_units() && m_edge) return launch_pinned<TileBigSpread, BF16, B_ROW_MAJOR, true>(p, stream);
        // at most 32 rows and tiles for every compute unit: one matrix instruction's worth of rows per tile, 256
        // columns wide (64 x 64 tiles load 64 rows of A per tile and multiply most of them for nothing); with
        // fewer tiles the smaller tilings below put more workgroups to work (8 x 3072 x 768: 8 us against 13 us)
        if (p.M <= 32 && (p.N + 255) / 256 >= compute_units()) return launch<TileSkinny, BF16, B_ROW_MAJOR>(p, stream);
        if (big_tiles < compute_units()) {
            // Fewer big tiles than that: the largest of the small tilings that still gives every compute unit one
            // and a half workgroups (two are resident at a time), else the smallest (1024^3: 64 x 64 tiles 8.8 us,
            // 128 x 128 tiles 16.3 us).
            const int64_t want = static_cast<int64_t>(compute_units()) * 3 / 2;
            const int64_t tm128 = (p.M + 127) / 128, tn128 = (p.N + 127) / 128, tn64 = (p.N + 63) / 64;
            // up to one and a half rounds of 128 x 128 tiles: the ring kernel in two rounds still beats the register
            // pipeline (657 x 7834 x 1544, 372 tiles: 49.2 -> 43.1 us; hipBLASLt 28.0)
            if (tm128 * tn128 > compute_units() && 2 * tm128 * tn128 <= 3 * compute_units() && p.K >= 512 && p.K <= 16384 &&
                tuning(knob_gemm16_wave_k) != 1 && (!B_ROW_MAJOR || (p.N % 8 == 0 && p.ldb % 8 == 0)))
                return launch_ring<128, 128, 2, 2, 4, BF16, B_ROW_MAJOR>(p, stream);
            // from one 128 x 128 tile per compute unit on when K is deep: the longer main loop then outweighs the
            // idle second slot (2048^3: 30.1 us against 31.3 with 128 x 64 tiles; 4096 x 1024 x 4096: 50.9 against 53.0)
            if (tm128 * tn128 >= want || (tm128 * tn128 >= compute_units() && p.K >= 2048))
                return launch<TileSmall, BF16, B_ROW_MAJOR>(p, stream);
            if (tm128 * tn64 >= want) return launch<TileSmallN, BF16, B_ROW_MAJOR>(p, stream);
            return launch<TileTiny, BF16, B_ROW_MAJOR>(p, stream);
        }
        if constexpr (!B_ROW_MAJOR) {
            if (p.M % 256 == 0 && p.N % 256 == 0 && p.K % kBK == 0) return launch_persistent<TileBig, BF16>(p, stream);
        }
        return launch<TileBig, BF16, B_ROW_MAJOR>(p, stream);
    }
    switch (variant) {  // explicit choices, for tuning and for the tests
        case 3: return launch<Tiling<128, 128, 2, 2, 2, true, 0>, BF16, B_ROW_MAJOR>(p, stream);
        case 6: return launch<Tiling<256, 256, 2, 4, 1, true, 0>, BF16, B_ROW_MAJOR>(p, stream);
        case 9: return launch<TileBig, BF16, B_ROW_MAJOR>(p, stream);
        case 10: return launch<TileSmall, BF16, B_ROW_MAJOR>(p, stream);
        case 11: return launch<TileTiny, BF16, B_ROW_MAJOR>(p, stream);
        case 12: return launch<TileSmallN, BF16, B_ROW_MAJOR>(p, stream);
        case 13: return launch<TileSkinny, BF16, B_ROW_MAJOR>(p, stream);
        case 30: return launch_direct<TileBig, BF16, B_ROW_MAJOR, false>(p, stream);
        case 50: return launch_direct<TileBig, BF16, B_ROW_MAJOR, true>(p, stream);
        case 52: return launch_direct<TileBigSpare, BF16, B_ROW_MAJOR, true>(p, stream);
        case 53: return launch_direct<TileBigSpread, BF16, B_ROW_MAJOR, true>(p, stream);
        case 54: return launch_direct<TileHalf, BF16, B_ROW_MAJOR, true>(p, stream);
        case 60: return launch_pinned<TileBigSpread, BF16, B_ROW_MAJOR, true>(p, stream);  // any M
        case 61: return launch_pinned<TileHalf, BF16, B_ROW_MAJOR, true>(p, stream);
        case 62:  // the pinned kernel in gemm16.k_slices K slices: reached only when the plan above came out whole
            return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: variant 62 needs gemm16.k_slices >= 2, N %% 256 == 0 and a workspace");
        case 80:
        case 81:
        case 82:
        case 83:
            if (variant == 80) return launch_ring<128, 128, 2, 2, 4, BF16, B_ROW_MAJOR>(p, stream);  // 4 stages of 32 KB
            if (variant == 81) return launch_ring<128, 64, 2, 2, 6, BF16, B_ROW_MAJOR>(p, stream);   // 6 stages of 24 KB
            if (variant == 82) return launch_ring<64, 128, 2, 2, 6, BF16, B_ROW_MAJOR>(p, stream);
            return launch_ring<128, 128, 2, 4, 5, BF16, B_ROW_MAJOR>(p, stream);  // 8 waves of 64 x 32, 5 stages
        case 84: return launch_ring<32, 64, 1, 2, 6, BF16, B_ROW_MAJOR>(p, stream);  // two waves of 32 x 32, 6 stages of 12 KB
        case 70:
        case 71:
        case 72:
        case 73:
            if (variant == 70) return launch_wave_k<2, 2, 4, BF16, B_ROW_MAJOR>(p, stream);  // 64 x 64 tiles, K over 4 waves
            if (variant == 71) return launch_wave_k<1, 2, 4, BF16, B_ROW_MAJOR>(p, stream);  // 32 x 64
            if (variant == 72) return launch_wave_k<1, 1, 8, BF16, B_ROW_MAJOR>(p, stream);  // 32 x 32, K over 8 waves
            return launch_wave_k<1, 2, 6, BF16, B_ROW_MAJOR>(p, stream);                     // 32 x 64, K over 6 waves
        default: return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: unknown variant %d", variant);
    }
}

}  // namespace

template <>
int gemm16_run<KO_GEMM16_BF16 != 0, KO_GEMM16_B_ROW != 0>(const Gemm16Params &p, hipStream_t stream) {
    return launch_variant<KO_GEMM16_BF16 != 0, KO_GEMM16_B_ROW != 0>(p, stream);
}
}  // namespace ko

#if KO_GEMM16_ENTRY
KO_EXPORT int ko_gemm_f16f32acc_bias_act(int64_t m, int64_t n, int64_t k, float alpha, const void *A,
                                         const void *B, int b_layout, float beta, const void *C, const void *bias,
                                         int activation, void *D, int in_dtype, ko_stream_t stream) {
    using namespace ko;
    if (m < 0 || n < 0 || k < 0)
        return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: m=%lld n=%lld k=%lld", (long long)m, (long long)n, (long long)k);
    if (in_dtype != KO_F16 && in_dtype != KO_BF16) return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: in_dtype=%d", in_dtype);
    if (b_layout != KO_ROW_MAJOR && b_layout != KO_COL_MAJOR)
        return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: b_layout=%d", b_layout);
    if (activation != KO_ACT_NONE && activation != KO_ACT_GELU_ERF && activation != KO_ACT_GELU_TANH)
        return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: activation=%d", activation);
    if (m == 0 || n == 0) return KO_OK;
    if (k % 8 != 0)
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: k=%lld must be a multiple of 8", (long long)k);
    if (m > (1 << 30) || n > (1 << 30) || k > (1 << 30))
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "gemm16: dimension too large");
    if (!D || (k > 0 && (!A || !B))) return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: null A/B/D pointer");
    uintptr_t align = reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) |
                      reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(D);
    if (align & 15) return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: A, B, C and D must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(bias) & 7) return fail(KO_ERR_INVALID_ARGUMENT, "gemm16: bias must be 8-byte aligned");
    Params p{static_cast<const uint16_t *>(A), static_cast<const uint16_t *>(B),
             static_cast<const uint16_t *>(C), static_cast<uint16_t *>(D),
             static_cast<int>(m), static_cast<int>(n), static_cast<int>(k), alpha, beta, 0, 0, 0, 0,
             static_cast<const uint16_t *>(bias), activation, static_cast<int>(n), static_cast<int>(n),
             0, nullptr, static_cast<int>(k)};
    hipStream_t s = as_stream(stream);
    if (k == 0) {  // the empty product: D = act(beta * C + bias), one launch of the epilogue kernel; A and B are not touched
        const int64_t groups = m * (partial_ld(p.N) / 4);
        const dim3 grid(static_cast<unsigned>((groups + 63) / 64));
        if (in_dtype == KO_F16) gemm16_slices_sum_kernel<false><<<grid, 64, 0, s>>>(p, 0);
        else gemm16_slices_sum_kernel<true><<<grid, 64, 0, s>>>(p, 0);
        KO_CHECK_LAUNCH();
        return KO_OK;
    }
    if (in_dtype == KO_F16) return b_layout == KO_COL_MAJOR ? gemm16_run<false, false>(p, s) : gemm16_run<false, true>(p, s);
    return b_layout == KO_COL_MAJOR ? gemm16_run<true, false>(p, s) : gemm16_run<true, true>(p, s);
}

KO_EXPORT int ko_gemm_f16f32acc(int64_t m, int64_t n, int64_t k, float alpha, const void *A,
                                const void *B, int b_layout, float beta, const void *C, void *D,
                                int in_dtype, ko_stream_t stream) {
    return ko_gemm_f16f32acc_bias_act(m, n, k, alpha, A, B, b_layout, beta, C, nullptr, KO_ACT_NONE, D, in_dtype,
                                      stream);
}

int ko::debug_gemm16_plan(int64_t m, int64_t n, int64_t k, int b_layout, int *slices, int *k_slice, int *tile) {
    using namespace ko;
    if (!slices || !k_slice || !tile || m <= 0 || n <= 0 || k <= 0 || m > (1 << 30) || n > (1 << 30) || k > (1 << 30) ||
        (b_layout != KO_ROW_MAJOR && b_layout != KO_COL_MAJOR))
        return fail(KO_ERR_INVALID_ARGUMENT, "gemm16_plan: bad argument");
    if ((b_layout == KO_COL_MAJOR || n % 8 == 0) && k % 8 == 0) {  // (a row-major B: rows of whole 16-byte chunks)
        int one_launch = wave_k_tile(m, n, k, b_layout == KO_ROW_MAJOR);
        if (one_launch == 0) one_launch = ring_tile(m, n, k, b_layout == KO_ROW_MAJOR);
        if (one_launch != 0) {
            *slices = 1;
            *k_slice = 0;
            *tile = one_launch;
            return KO_OK;
        }
    }
    Params p{};
    p.M = static_cast<int>(m);
    p.N = static_cast<int>(n);
    p.K = static_cast<int>(k);
    p.ldd = p.ldb = p.N;
    p.ldk = p.K;
    const int64_t big = ((m + 255) / 256) * ((n + 255) / 256);
    SlicePlan16 plan;
    if (2 * big <= compute_units() || m <= 32 || tuning(knob_gemm16_variant) == 62)
        plan = plan_k_slices16(p, kStreamWorkspaceBytes);  // as launch_variant asks
    *slices = plan.slices;
    *k_slice = plan.k_slice;
    *tile = plan.slices > 1 ? plan.tile : 0;
    return KO_OK;
}
#endif  // KO_GEMM16_ENTRY
