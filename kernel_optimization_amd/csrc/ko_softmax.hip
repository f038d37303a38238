// Row softmax for gfx950: one pass over HBM (each element read once, written
// once), fp32 arithmetic, fp32 / binary16 / bfloat16 storage, optional
// per-sequence padding mask.
//
// Three mappings, the counterparts of the reference's three policies
// (nn_operators/softmax/softmax.h):
//   WARP          a row lives in the registers of a group of LPR lanes of one
//                 wavefront (LPR in {8,16,32,64}; 64/LPR rows per wavefront),
//                 VPL 128-bit vectors per lane; max and sum are DPP /
//                 permlane-swap all-reduces; no LDS.      (SoftMaxWarpImpl, :11-60)
//   BLOCK         a row lives in the registers of one workgroup; LDS carries only
//                 the per-wave partials.                  (SoftMaxBlockImpl, :62-113)
//   BLOCK_NOCACHE rows of any length: pass 1 keeps a running (max, sum) per
//                 thread (online rescaling), pass 2 re-reads the row and writes:
//                 two reads + one write instead of the reference's three reads.
//                                                        (SoftMaxBlockNoCacheImpl, :116-166)
//
// Per row: m = max_j x_j (running max starts at -FLT_MAX, softmax.h:33),
// e_j = exp(x_j - m), s = sum_j e_j, y_j = e_j / s  (softmax.h:35-57; the
// intended x - m, not the x + m the reference's Subtract functor computes,
// common/functors.h:168).
//
// Special values follow from that arithmetic as they do in the reference: a NaN
// element, or a +inf element (inf - inf), makes exp(x - m) NaN and with it the
// row's sum and every output of the row; -inf elements get probability 0; a row
// of nothing but -inf keeps m = -FLT_MAX, sums to 0 and comes out as 0/0 = NaN.
// The maximum itself ignores NaN (fmaxf), which changes nothing: the sum is NaN
// either way.  Vector slots past the end of a row hold -inf, so they add
// nothing to any sum.  Masked columns are replaced before any of this.
//
// Mask: columns j >= valid_len[row / rows_per_seq] take the value -10000.  Vectors
// that lie wholly in the padded part are not loaded.
#include "ko_internal.h"
#include <type_traits>

#include "wave64.h"

#include <cfloat>

namespace ko {
namespace {

constexpr float kMaskValue = -10000.0f;

// A row vector is fetched in two steps so that a thread can issue all of its loads before it looks at any of
// them: unpacking or masking inside the branch that holds a load makes the compiler wait for that load before
// the next one goes out.
// fetch: the 16 bytes at `p` (vector j of the row) if the vector holds valid columns, else nothing is loaded.
template <int IO, bool MASKED, bool NT>
__device__ __forceinline__ typename Io<IO>::raw fetch_row_vec(const typename Io<IO>::elem *p, int j, int vlen) {
    typename Io<IO>::raw r{};
    if (!MASKED || Io<IO>::E * j < vlen) r = Io<IO>::template load_raw<NT>(p);
    return r;
}
// finish: converted values of vector j, with the columns from `vlen` on replaced by the mask value.
template <int IO, bool MASKED>
__device__ __forceinline__ void finish_row_vec(typename Io<IO>::raw r, int j, int vlen, float (&v)[Io<IO>::E]) {
    constexpr int E = Io<IO>::E;
    Io<IO>::unpack(r, v);
    if constexpr (MASKED) {
#pragma unroll
        for (int e = 0; e < E; ++e)
            if (E * j + e >= vlen) v[e] = kMaskValue;
    }
}

// base + bytes, for addresses formed from a uniform pointer and a 32-bit per-lane offset
template <class T>
__device__ __forceinline__ T *at_bytes(T *base, uint32_t bytes) {
    typedef typename std::conditional<std::is_const<T>::value, const char, char>::type Byte;
    return reinterpret_cast<T *>(reinterpret_cast<Byte *>(base) + bytes);
}

template <int E>
__device__ __forceinline__ float vec_max(const float (&v)[E], float m) {
#pragma unroll
    for (int e = 0; e < E; ++e) m = fmaxf(m, v[e]);
    return m;
}

__device__ __forceinline__ int clamp_len(int v, int cols) { return v < 0 ? 0 : (v > cols ? cols : v); }

// ---------------------------------------------------------------- WARP policy
template <int IO, int LPR, int VPL, bool MASKED, bool NT>
__global__ __launch_bounds__(256) void softmax_wave_kernel(const typename Io<IO>::elem *in,
                                                           typename Io<IO>::elem *out, int64_t rows,
                                                           int cols, const int32_t *__restrict__ valid_len,
                                                           int64_t rows_per_seq) {
    constexpr int E = Io<IO>::E;
    constexpr int RPW = 64 / LPR;  // rows per wavefront
    const int lane = threadIdx.x & 63;
    const int sub = lane / LPR;
    const int l = lane % LPR;
    const int nvec = cols / E;
    const int64_t waves_per_block = blockDim.x >> 6;
    const int64_t wave = blockIdx.x * waves_per_block + (threadIdx.x >> 6);
    const int64_t stride = static_cast<int64_t>(gridDim.x) * waves_per_block * RPW;

    for (int64_t row0 = wave * RPW; row0 < rows; row0 += stride) {
        const int64_t row = row0 + sub;
        const bool row_ok = row < rows;
        const typename Io<IO>::elem *src = in + row * cols;
        int vlen = cols;
        if constexpr (MASKED) {
            // The rows of a wavefront are consecutive and start at a wave-uniform row: their sequence lengths are
            // fetched with wave-uniform addresses (scalar loads through the constant cache, which the 6144 rows
            // of a sequence keep hitting) instead of one vector load per lane, whose latency would stand in front
            // of the row loads.
            const uint64_t r0 = static_cast<uint64_t>(row0);
            const int64_t first_row = static_cast<int64_t>(
                (static_cast<uint64_t>(static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(r0 >> 32)))) << 32) |
                static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(r0))));
#pragma unroll
            for (int r = 0; r < RPW; ++r) {
                const int64_t rr = first_row + r;
                if (rr < rows) {
                    const int len = clamp_len(valid_len[rr / rows_per_seq], cols);
                    if (sub == r) vlen = len;
                }
            }
        }

        // All of the lane's loads go out first and are unpacked and masked afterwards: with the unpacking inside
        // the same branch as its load, each load would be waited for before the next one is issued.
        typename Io<IO>::raw loaded[VPL];
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = l + k * LPR;
            loaded[k] = typename Io<IO>::raw{};
            if (row_ok && j < nvec) loaded[k] = fetch_row_vec<IO, MASKED, NT>(src + E * j, j, vlen);
        }
        float v[VPL][E];
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = l + k * LPR;
            finish_row_vec<IO, MASKED>(loaded[k], j, vlen, v[k]);
            if (!(row_ok && j < nvec)) {
#pragma unroll
                for (int e = 0; e < E; ++e) v[k][e] = -INFINITY;
            }
        }

        float m = -FLT_MAX;
#pragma unroll
        for (int k = 0; k < VPL; ++k) m = vec_max<E>(v[k], m);
        m = wave::allreduce<LPR, wave::Max>(m);

        // Vectors wholly inside the padding hold -10000; once the row maximum is more than 128 above
        // that, their exponentials are exactly zero in fp32 and need not be computed.
        const bool pad_is_zero = MASKED && m > kMaskValue + 128.0f;
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            if (pad_is_zero && E * (l + k * LPR) >= vlen) {
#pragma unroll
                for (int e = 0; e < E; ++e) v[k][e] = 0.0f;
            } else {
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    v[k][e] = exp_for_storage<IO>(v[k][e] - m);
                    s += v[k][e];
                }
            }
        }
        s = wave::allreduce<LPR, wave::Sum>(s);
        const float inv = 1.0f / s;

        // streaming stores: wave-uniform base (the wavefront's first row) + per-lane byte offset; written through
        // at once only when rows are whole 64-byte lines (see store_row_vec)
        typename Io<IO>::elem *dst0 = out + row0 * cols;
        const uint32_t sub_off = static_cast<uint32_t>(sub) * static_cast<uint32_t>(cols) * sizeof(typename Io<IO>::elem);
        const bool whole_lines = rows_are_whole_lines<IO>(cols);
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = l + k * LPR;
            if (row_ok && j < nvec) {
#pragma unroll
                for (int e = 0; e < E; ++e) v[k][e] *= inv;
                if constexpr (NT) {
                    store_row_vec<IO>(whole_lines, dst0, sub_off + Io<IO>::kBytes * j, v[k]);
                } else {
                    Io<IO>::template store<false>(dst0 + static_cast<int64_t>(sub) * cols + E * j, v[k]);
                }
            }
        }
    }
}

// --------------------------------------------------------------- BLOCK policy
// Workgroup-wide all-reduce: wave all-reduce, then every thread folds the per-wave
// partials from LDS in the same order (bit-identical result in every thread).
template <int THREADS, class Op>
__device__ __forceinline__ float block_allreduce(float v, float *lds, float identity) {
    constexpr int WAVES = THREADS / 64;
    v = wave::allreduce<64, Op>(v);
    if constexpr (WAVES == 1) return v;
    __syncthreads();  // previous use of lds finished
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = identity;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) r = Op()(r, lds[w]);
    return r;
}

// One barrier per reduction: `slot` holds this reduction's partials and is not written again before every
// wave has passed the workgroup's next barrier (the caller alternates between two slots).
template <int THREADS, class Op>
__device__ __forceinline__ float block_allreduce_slot(float v, float *slot, float identity) {
    constexpr int WAVES = THREADS / 64;
    v = wave::allreduce<64, Op>(v);
    if constexpr (WAVES == 1) return v;
    if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = identity;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) r = Op()(r, slot[w]);
    return r;
}

// One workgroup per row, the row held on chip between its single read and its single write.  Loads and
// stores bypass the caches' retention (nontemporal): every byte is touched once, and on rows of 16 to 128 KB
// that measured 9 % faster than cached accesses.  Issuing the next row's loads ahead of the reductions
// measured no different: two or more resident workgroups already cover each other's reductions.
// VPL vectors per thread live in registers.  LV more live in LDS (vector k of thread t at tail[k][t], filled by
// direct-to-LDS loads, so they cost no registers on the way): a 1024-thread workgroup alone on a CU has 128
// registers per thread, of which 96 can hold row values, and 9 x 16 KB of the CU's 160 KB of LDS hold the rest
// of rows up to 135168 fp32 columns, which would otherwise be read twice.  fp32 storage writes the exponentials
// back into the tail; 16-bit storage keeps the inputs there (eight values per 16 bytes) and takes the
// exponential again on the way out.
template <int IO, int THREADS, int VPL, bool MASKED, int LV = 0>
__global__ __launch_bounds__(THREADS) void softmax_block_kernel(const typename Io<IO>::elem *in,
                                                                typename Io<IO>::elem *out, int64_t rows,
                                                                int cols,
                                                                const int32_t *__restrict__ valid_len,
                                                                int64_t rows_per_seq) {
    constexpr int E = Io<IO>::E;
    static_assert(LV == 0 || !MASKED, "the LDS tail is built for rows without a mask");
    typedef typename Io<IO>::raw Raw;
    __shared__ float lds[2][16];
    extern __shared__ __attribute__((aligned(16))) char tail_bytes[];  // Raw tail[LV][THREADS]
    Raw *tail = reinterpret_cast<Raw *>(tail_bytes);
    const int nvec = cols / E;
    // Byte offset of this thread's first vector in a row (vector k lies k * THREADS * 16 bytes further); passed
    // through an empty asm per row so that addresses are formed per use from the uniform row pointer and this
    // one register rather than kept as VPL pointer pairs.
    uint32_t first = threadIdx.x * Io<IO>::kBytes;
    constexpr uint32_t kStep = THREADS * Io<IO>::kBytes;
    static_assert(LV == 0 || Io<IO>::kBytes == 16, "the LDS tail is filled 16 bytes per lane");
    const bool whole_lines = rows_are_whole_lines<IO>(cols);
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        asm volatile("" : "+v"(first));
        const typename Io<IO>::elem *src = in + row * cols;
        int vlen = cols;
        if constexpr (MASKED) vlen = clamp_len(valid_len[row / rows_per_seq], cols);
        float v[VPL][E];
        if constexpr (IO == IO_F32 && !MASKED) {
            // nothing to unpack or mask: the loaded registers are the values (the two-step form below costs ten
            // registers more here, and with them the second resident workgroup at 32768 columns)
#pragma unroll
            for (int k = 0; k < VPL; ++k) {
                const int j = threadIdx.x + k * THREADS;
                if (j < nvec) {
                    Io<IO>::template load<true>(at_bytes(src, first + k * kStep), v[k]);
                } else {
#pragma unroll
                    for (int e = 0; e < E; ++e) v[k][e] = -INFINITY;
                }
            }
        }
        typename Io<IO>::raw loaded[(IO == IO_F32 && !MASKED) ? 1 : VPL];
        if constexpr (!(IO == IO_F32 && !MASKED)) {
#pragma unroll
            for (int k = 0; k < VPL; ++k) {
                const int j = threadIdx.x + k * THREADS;
                loaded[k] = typename Io<IO>::raw{};
                if (j < nvec) loaded[k] = fetch_row_vec<IO, MASKED, true>(at_bytes(src, first + k * kStep), j, vlen);
            }
        }
        if constexpr (LV > 0) {
            // the tail goes from global memory straight into LDS: each lane's 16 bytes land at the wave's base
            // plus 16 x lane, i.e. at tail[k][thread]; lanes past the end of the row write nothing
#pragma unroll
            for (int k = 0; k < LV; ++k) {
                const int j = threadIdx.x + (VPL + k) * THREADS;
                if (j < nvec)
                    __builtin_amdgcn_global_load_lds(
                        (const __attribute__((address_space(1))) void *)at_bytes(src, first + (VPL + k) * kStep),
                        (__attribute__((address_space(3))) void *)(tail + k * THREADS + (threadIdx.x & ~63u)), 16, 0, 0);
            }
        }
        if constexpr (!(IO == IO_F32 && !MASKED)) {
#pragma unroll
            for (int k = 0; k < VPL; ++k) {
                const int j = threadIdx.x + k * THREADS;
                finish_row_vec<IO, MASKED>(loaded[k], j, vlen, v[k]);
                if (j >= nvec) {
#pragma unroll
                    for (int e = 0; e < E; ++e) v[k][e] = -INFINITY;
                }
            }
        }
        float m = -FLT_MAX;
#pragma unroll
        for (int k = 0; k < VPL; ++k) m = vec_max<E>(v[k], m);
#pragma unroll
        for (int k = 0; k < LV; ++k) {
            if (static_cast<int>(threadIdx.x) + (VPL + k) * THREADS < nvec) {
                float x[E];
                Io<IO>::unpack(tail[k * THREADS + threadIdx.x], x);
                m = vec_max<E>(x, m);
            }
        }
        m = block_allreduce_slot<THREADS, wave::Max>(m, lds[0], -FLT_MAX);
        const bool pad_is_zero = MASKED && m > kMaskValue + 128.0f;  // see the wave kernel
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            if (pad_is_zero && E * (static_cast<int>(threadIdx.x) + k * THREADS) >= vlen) {
#pragma unroll
                for (int e = 0; e < E; ++e) v[k][e] = 0.0f;
            } else {
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    v[k][e] = exp_for_storage<IO>(v[k][e] - m);
                    s += v[k][e];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < LV; ++k) {
            if (static_cast<int>(threadIdx.x) + (VPL + k) * THREADS < nvec) {
                float x[E];
                Io<IO>::unpack(tail[k * THREADS + threadIdx.x], x);
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    x[e] = exp_for_storage<IO>(x[e] - m);
                    s += x[e];
                }
                if constexpr (IO == IO_F32) tail[k * THREADS + threadIdx.x] = Raw{x[0], x[1], x[2], x[3]};
            }
        }
        s = block_allreduce_slot<THREADS, wave::Sum>(s, lds[1], 0.0f);
        const float inv = 1.0f / s;
        typename Io<IO>::elem *dst = out + row * cols;
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
            const int j = threadIdx.x + k * THREADS;
            if (j < nvec) {
#pragma unroll
                for (int e = 0; e < E; ++e) v[k][e] *= inv;
                store_row_vec<IO>(whole_lines, dst, first + k * kStep, v[k]);
            }
        }
#pragma unroll
        for (int k = 0; k < LV; ++k) {
            if (static_cast<int>(threadIdx.x) + (VPL + k) * THREADS < nvec) {
                float x[E];
                Io<IO>::unpack(tail[k * THREADS + threadIdx.x], x);
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    if constexpr (IO != IO_F32) x[e] = exp_for_storage<IO>(x[e] - m);
                    x[e] *= inv;
                }
                store_row_vec<IO>(whole_lines, dst, first + (VPL + k) * kStep, x);
            }
        }
    }
}

// ------------------------------------------------------- BLOCK_NOCACHE policy
// Online pair (m, s): s = sum exp(x - m) over the elements seen so far.
__device__ __forceinline__ void online_add(float &m, float &s, float x) {
    if (x > m) {
        s = s * exp_nonpositive(m - x) + 1.0f;
        m = x;
    } else {
        s += exp_nonpositive(x - m);
    }
}

template <int IO, int THREADS, bool MASKED>
__global__ __launch_bounds__(THREADS) void softmax_nocache_kernel(const typename Io<IO>::elem *in,
                                                                  typename Io<IO>::elem *out,
                                                                  int64_t rows, int cols,
                                                                  const int32_t *__restrict__ valid_len,
                                                                  int64_t rows_per_seq) {
    constexpr int E = Io<IO>::E;
    __shared__ float lds[16];
    const int nvec = cols / E;
    const bool whole_lines = rows_are_whole_lines<IO>(cols);
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const typename Io<IO>::elem *src = in + row * cols;
        int vlen = cols;
        if constexpr (MASKED) vlen = clamp_len(valid_len[row / rows_per_seq], cols);
        float m = -FLT_MAX, s = 0.0f;
        // UNROLL vectors per thread and trip: their loads are issued together, so that a workgroup keeps
        // enough bytes in flight to cover the memory latency
        constexpr int UNROLL = 4;
        for (int j0 = threadIdx.x; j0 < nvec; j0 += THREADS * UNROLL) {
            float x[UNROLL][E];
            typename Io<IO>::raw loaded[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int j = j0 + u * THREADS;
                loaded[u] = typename Io<IO>::raw{};
                if (j < nvec) loaded[u] = fetch_row_vec<IO, MASKED, false>(src + E * j, j, vlen);
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) finish_row_vec<IO, MASKED>(loaded[u], j0 + u * THREADS, vlen, x[u]);
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                if (j0 + u * THREADS >= nvec) break;
#pragma unroll
                for (int e = 0; e < E; ++e) online_add(m, s, x[u][e]);
            }
        }
        const float gm = block_allreduce<THREADS, wave::Max>(m, lds, -FLT_MAX);
        s *= exp_nonpositive(m - gm);  // threads that saw nothing: s = 0
        const float gs = block_allreduce<THREADS, wave::Sum>(s, lds, 0.0f);
        const float inv = 1.0f / gs;
        typename Io<IO>::elem *dst = out + row * cols;
        // Second pass from the row's end backwards: what the first pass read last is the likeliest to be in a
        // cache still (measured 5 % faster at 65536 columns, no different at 131072).  Nontemporal accesses from
        // here on: nothing is touched again (19 % faster than cached ones at 131072 columns).
        const int trips = (nvec + THREADS * UNROLL - 1) / (THREADS * UNROLL);
        for (int t = 0; t < trips; ++t) {
            const int j0 = threadIdx.x + (trips - 1 - t) * (THREADS * UNROLL);
            float x[UNROLL][E];
            typename Io<IO>::raw loaded[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int j = j0 + u * THREADS;
                loaded[u] = typename Io<IO>::raw{};
                if (j < nvec) loaded[u] = fetch_row_vec<IO, MASKED, true>(src + E * j, j, vlen);
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) finish_row_vec<IO, MASKED>(loaded[u], j0 + u * THREADS, vlen, x[u]);
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int j = j0 + u * THREADS;
                if (j >= nvec) break;
#pragma unroll
                for (int e = 0; e < E; ++e) x[u][e] = exp_for_storage<IO>(x[u][e] - gm) * inv;
                store_row_vec<IO>(whole_lines, dst, Io<IO>::kBytes * j, x[u]);
            }
        }
    }
}

// ------------------------------------------- few rows: a row split over workgroups
// With fewer rows than compute units (the softmax over a vocabulary for a batch of a few dozen rows) one workgroup
// per row leaves most of the chip idle.  Such rows are cut into `parts` pieces of `piece` vectors each, one
// workgroup per piece, in two launches with nothing but the kernel boundary between them: the first leaves every
// piece's (maximum, sum of exponentials against that maximum) in a workspace, the second folds a row's pairs - in
// piece order, every workgroup the same way, so the result is the same bits from call to call - and writes its
// piece of the output, reading the piece a second time (it is the only traffic that is added; a tensor of a few
// rows sits in the last-level cache).  blockIdx.x = piece, blockIdx.y = row.
struct PiecePair {
    float m, s;
};

template <int IO, int THREADS, bool MASKED>
__global__ __launch_bounds__(THREADS) void softmax_pieces_stats_kernel(const typename Io<IO>::elem *in, int cols,
                                                                       const int32_t *__restrict__ valid_len,
                                                                       int64_t rows_per_seq, int piece,
                                                                       PiecePair *__restrict__ pairs) {
    constexpr int E = Io<IO>::E;
    constexpr int UNROLL = 4;
    __shared__ float lds[16];
    const int nvec = cols / E;
    const int64_t row = blockIdx.y;
    const int lo = static_cast<int>(blockIdx.x) * piece;
    const int hi = lo + piece < nvec ? lo + piece : nvec;
    const typename Io<IO>::elem *src = in + row * cols;
    int vlen = cols;
    if constexpr (MASKED) vlen = clamp_len(valid_len[row / rows_per_seq], cols);
    float m = -FLT_MAX, s = 0.0f;
    for (int j0 = lo + threadIdx.x; j0 < hi; j0 += THREADS * UNROLL) {
        float x[UNROLL][E];
        typename Io<IO>::raw loaded[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int j = j0 + u * THREADS;
            loaded[u] = typename Io<IO>::raw{};
            if (j < hi) loaded[u] = fetch_row_vec<IO, MASKED, false>(src + E * j, j, vlen);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) finish_row_vec<IO, MASKED>(loaded[u], j0 + u * THREADS, vlen, x[u]);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (j0 + u * THREADS >= hi) break;
#pragma unroll
            for (int e = 0; e < E; ++e) online_add(m, s, x[u][e]);
        }
    }
    const float gm = block_allreduce<THREADS, wave::Max>(m, lds, -FLT_MAX);
    s *= exp_nonpositive(m - gm);  // threads that saw nothing: s = 0
    const float gs = block_allreduce<THREADS, wave::Sum>(s, lds, 0.0f);
    if (threadIdx.x == 0) pairs[row * gridDim.x + blockIdx.x] = PiecePair{gm, gs};
}

template <int IO, int THREADS, bool MASKED>
__global__ __launch_bounds__(THREADS) void softmax_pieces_apply_kernel(const typename Io<IO>::elem *in,
                                                                       typename Io<IO>::elem *out, int cols,
                                                                       const int32_t *__restrict__ valid_len,
                                                                       int64_t rows_per_seq, int piece,
                                                                       const PiecePair *__restrict__ pairs) {
    constexpr int E = Io<IO>::E;
    constexpr int UNROLL = 4;
    const int nvec = cols / E;
    const int64_t row = blockIdx.y;
    const int parts = static_cast<int>(gridDim.x);
    const int lo = static_cast<int>(blockIdx.x) * piece;
    const int hi = lo + piece < nvec ? lo + piece : nvec;
    const typename Io<IO>::elem *src = in + row * cols;
    int vlen = cols;
    if constexpr (MASKED) vlen = clamp_len(valid_len[row / rows_per_seq], cols);
    // the row's maximum and sum from its pieces' pairs, folded in piece order (wave-uniform loads)
    const PiecePair *mine = pairs + row * parts;
    float gm = -FLT_MAX;
    for (int i = 0; i < parts; ++i) gm = fmaxf(gm, mine[i].m);
    float gs = 0.0f;
    for (int i = 0; i < parts; ++i) gs += mine[i].s * exp_nonpositive(mine[i].m - gm);
    const float inv = 1.0f / gs;
    typename Io<IO>::elem *dst = out + row * cols;
    const bool whole_lines = rows_are_whole_lines<IO>(cols);
    for (int j0 = lo + threadIdx.x; j0 < hi; j0 += THREADS * UNROLL) {
        float x[UNROLL][E];
        typename Io<IO>::raw loaded[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int j = j0 + u * THREADS;
            loaded[u] = typename Io<IO>::raw{};
            if (j < hi) loaded[u] = fetch_row_vec<IO, MASKED, true>(src + E * j, j, vlen);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) finish_row_vec<IO, MASKED>(loaded[u], j0 + u * THREADS, vlen, x[u]);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int j = j0 + u * THREADS;
            if (j >= hi) break;
#pragma unroll
            for (int e = 0; e < E; ++e) x[u][e] = exp_for_storage<IO>(x[u][e] - gm) * inv;
            store_row_vec<IO>(whole_lines, dst, Io<IO>::kBytes * j, x[u]);
        }
    }
}

// ------------------------------------------------------------------ dispatch
template <int IO>
struct Args {
    const typename Io<IO>::elem *in;
    typename Io<IO>::elem *out;
    int64_t rows;
    int cols;
    const int32_t *valid_len;
    int64_t rows_per_seq;
    hipStream_t stream;
};

template <int IO, int LPR, int VPL, bool MASKED, bool NT>
int launch_wave(const Args<IO> &a) {
    constexpr int RPW = 64 / LPR;
    // Single-wavefront workgroups by default (measured 1-4 % faster than 256 threads: the dispatcher
    // places waves more freely); the knob selects 128 or 256.
    int kThreads = tuning(knob_softmax_wave_threads);
    if (kThreads != 128 && kThreads != 256) kThreads = 64;
    const int64_t rows_per_block = RPW * (kThreads / 64);
    const int64_t needed = (a.rows + rows_per_block - 1) / rows_per_block;
    // One row batch per wavefront by default (measured faster than a persistent grid-stride
    // launch: the hardware keeps more loads in flight); a positive knob caps the grid instead.
    int64_t grid = needed;
    const int per_cu = tuning(knob_softmax_blocks_per_cu);
    if (per_cu > 0 && grid > static_cast<int64_t>(compute_units()) * per_cu)
        grid = static_cast<int64_t>(compute_units()) * per_cu;
    if (grid > 0x7fffffff) grid = 0x7fffffff;
    // Residency cap (see lds_pad_for_residency): 40 KB of row loads in flight per CU; with a mask about a third
    // of the nominal row bytes are never loaded, hence 64 KB of nominal bytes.  Knob: bytes, or -1 for none.
    int lds = tuning(knob_softmax_wave_lds);
    if (lds == 0 && kThreads == 64)
        lds = lds_pad_for_residency(static_cast<int64_t>(RPW) * a.cols * sizeof(typename Io<IO>::elem),
                                    (MASKED ? 64 : 40) * 1024);
    if (lds < 0) lds = 0;
    softmax_wave_kernel<IO, LPR, VPL, MASKED, NT><<<dim3(static_cast<unsigned>(grid)), dim3(kThreads), lds, a.stream>>>(
        a.in, a.out, a.rows, a.cols, a.valid_len, a.rows_per_seq);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <int IO, int LPR, bool MASKED, bool NT>
int launch_wave_vpl(const Args<IO> &a, int vpl) {
    switch (vpl) {
        case 1: return launch_wave<IO, LPR, 1, MASKED, NT>(a);
        case 2: return launch_wave<IO, LPR, 2, MASKED, NT>(a);
        case 3: return launch_wave<IO, LPR, 3, MASKED, NT>(a);
        case 4: return launch_wave<IO, LPR, 4, MASKED, NT>(a);
        case 5:
        case 6: return launch_wave<IO, LPR, 6, MASKED, NT>(a);
        default: return launch_wave<IO, LPR, 8, MASKED, NT>(a);
    }
}

template <int IO, bool MASKED, bool NT>
int launch_wave_lpr(const Args<IO> &a, int lpr) {
    const int nvec = a.cols / Io<IO>::E;
    const int vpl = (nvec + lpr - 1) / lpr;
    if constexpr (!MASKED) {
        // Rows of one to four vectors (the softmax over 8 or 16 experts for every token): 1, 2 or 4 lanes per row
        // with one vector each, 16 to 64 rows per wavefront, whose one load still covers a contiguous stretch of
        // memory ([16777216, 4]: 466 -> 83 us, the time of the same-bytes copy).  More vectors per lane of such
        // a small group would stride through memory (three vectors of one lane each: [8388608, 12] 236 -> 356 us).
        if (lpr == 1 && vpl == 1) return launch_wave<IO, 1, 1, false, true>(a);
        if (lpr == 2 && vpl == 1) return launch_wave<IO, 2, 1, false, true>(a);
        if (lpr == 4 && vpl == 1) return launch_wave<IO, 4, 1, false, true>(a);
    }
    switch (lpr) {
        case 8: return launch_wave_vpl<IO, 8, MASKED, NT>(a, vpl);
        case 16: return launch_wave_vpl<IO, 16, MASKED, NT>(a, vpl);
        case 32: return launch_wave_vpl<IO, 32, MASKED, NT>(a, vpl);
        default: return launch_wave_vpl<IO, 64, MASKED, NT>(a, vpl);
    }
}

constexpr int kWaveMaxVpl = 8;
// Longest row per policy, in 16-byte vectors: 512 per wavefront, 8192 per workgroup
// (fp32: 2048 and 32768 columns; 16-bit: twice that).
constexpr int kWaveMaxVecs = 64 * kWaveMaxVpl;
// BLOCK policy: at most 96 values per thread of a 1024-thread workgroup in registers (98304 columns) and, without
// a mask, nine more 16-byte vectors per thread in LDS (135168 fp32 or 172032 16-bit columns).  With a mask the
// kernels past 64 values per thread spill registers, and AUTO leaves those rows to the re-reading policy.
constexpr int kTailMaxVecs = 9;  // of 16 KB each per 1024-thread workgroup, in the 160 KB of LDS of a CU
template <int IO>
constexpr int kBlockMaxVecs = 1024 * (96 / Io<IO>::E + kTailMaxVecs);
template <int IO>
constexpr int kBlockMaxVecsMasked = 1024 * (64 / Io<IO>::E);
// AUTO goes to the re-reading policy from five LDS vectors on: with one workgroup per CU either way, nine of them
// cost about what the second read does ([1024, 131072]: 244 against 238 us; [1170, 114688], four: 218 against 236).
template <int IO>
constexpr int kBlockAutoMaxVecs = 1024 * (96 / Io<IO>::E + 4);

// Lanes per row for the WARP policy.  A group of LPR lanes holds a row in VPL vectors per lane, VPL from
// {1, 2, 3, 4, 6, 8}; the choice wastes the fewest vector slots (idle lanes still cost issue cycles
// and a wavefront's worth of latency), and among equals takes the widest group: one load instruction
// of the group then covers the longest contiguous piece of the row.  With a padding mask at least two
// vectors per lane are preferred: a lane whose only vector lies in the padding idles through the whole
// row (measured on [786432, 512] binary16, mean valid length 288: 64 x 1 309 us, 32 x 2 230 us).
int default_lanes_per_row(int nvec, bool masked, int masked_min_vpl) {
    int best = 64, best_waste = 1 << 30;
    // (groups of 1, 2 and 4 lanes: without a mask, one vector per lane)
    for (int lpr = masked ? 8 : 1; lpr <= 64; lpr <<= 1) {
        int vpl = (nvec + lpr - 1) / lpr;
        if (vpl > (lpr < 8 ? 1 : 8)) continue;
        if (vpl == 5) vpl = 6;
        if (vpl == 7) vpl = 8;
        const int waste = lpr * vpl - nvec;
        // with a mask, four vectors per lane before two (fp32 [786432, 512]: 32 x 4 391 us, 64 x 2 395 us)
        if (waste < best_waste || (waste == best_waste && !(masked && vpl < masked_min_vpl))) {
            best_waste = waste;
            best = lpr;
        }
    }
    return best;
}

template <int IO, bool MASKED>
int launch_wave_any(const Args<IO> &a) {
    const int nvec = a.cols / Io<IO>::E;
    int lpr = tuning(knob_softmax_lanes_per_row);
    if (lpr != 8 && lpr != 16 && lpr != 32 && lpr != 64) lpr = default_lanes_per_row(nvec, MASKED, IO == IO_F32 ? 4 : 2);
    while (lpr < 64 && (nvec + lpr - 1) / lpr > (lpr < 8 ? 1 : kWaveMaxVpl)) lpr <<= 1;
    // Streaming (non-temporal) accesses by default: every byte is touched once.  Knob: 2 = off
    // (fp32 storage only; the 16-bit kernels are built with streaming accesses).
    if constexpr (IO == IO_F32) {
        if (tuning(knob_softmax_nontemporal) == 2) return launch_wave_lpr<IO, MASKED, false>(a, lpr);
    }
    return launch_wave_lpr<IO, MASKED, true>(a, lpr);
}

template <int IO, int THREADS, bool MASKED>
int launch_block_threads(const Args<IO> &a) {
    const int nvec = a.cols / Io<IO>::E;
    const int vpl = (nvec + THREADS - 1) / THREADS;
    int64_t grid = static_cast<int64_t>(compute_units()) * (2048 / THREADS) * 2;
    // one workgroup per row for rows of at most two vectors per thread (see launch_block); knob: 1 always, 2 never
    const int grid_knob = tuning(knob_rows_block_grid);
    if (grid_knob == 1 || (grid_knob != 2 && vpl <= 2 && THREADS >= 512)) grid = a.rows;
    if (grid > a.rows) grid = a.rows;
    if (grid > 0x7fffffff) grid = 0x7fffffff;
    dim3 g(static_cast<unsigned>(grid)), b(THREADS);
#define KO_SM_BLOCK(V)                                                                         \
    softmax_block_kernel<IO, THREADS, V, MASKED><<<g, b, 0, a.stream>>>(                         \
        a.in, a.out, a.rows, a.cols, a.valid_len, a.rows_per_seq)
    constexpr int E = Io<IO>::E;
    if (vpl <= 1) KO_SM_BLOCK(1);
    else if (vpl <= 2) KO_SM_BLOCK(2);
    else if (vpl <= 4) KO_SM_BLOCK(4);
    else if (vpl <= 8) KO_SM_BLOCK(8);
    else if constexpr (THREADS == 1024) {
        // a single resident workgroup of 1024 threads has 128 registers per thread: up to 96 hold the row
        constexpr int kRegs = 96 / E;  // vectors per thread held in registers
        if constexpr (E == 4) {
            if (vpl <= 12) KO_SM_BLOCK(12);
            else if (vpl <= 16) KO_SM_BLOCK(16);
            else if (vpl <= 20) KO_SM_BLOCK(20);
            else if (vpl <= 24) KO_SM_BLOCK(24);
        } else if (vpl <= 10) KO_SM_BLOCK(10);
        else if (vpl <= 12) KO_SM_BLOCK(12);
        if constexpr (!MASKED) {
            // longer rows: the rest of the row in LDS (4 or 9 vectors of 16 KB per workgroup)
            if (vpl > kRegs) {
                const int lv = vpl - kRegs <= 4 ? 4 : kTailMaxVecs;
                const void *fn = lv == 4 ? reinterpret_cast<const void *>(softmax_block_kernel<IO, THREADS, kRegs, false, 4>)
                                         : reinterpret_cast<const void *>(softmax_block_kernel<IO, THREADS, kRegs, false, kTailMaxVecs>);
                static std::atomic<uint64_t> done4{0}, done9{0};
                if (const int rc = allow_dynamic_lds(fn, 160 * 1024 - 256, lv == 4 ? done4 : done9); rc != KO_OK) return rc;
                const size_t bytes = static_cast<size_t>(lv) * THREADS * 16;
                if (lv == 4)
                    softmax_block_kernel<IO, THREADS, kRegs, false, 4><<<g, b, bytes, a.stream>>>(
                        a.in, a.out, a.rows, a.cols, a.valid_len, a.rows_per_seq);
                else
                    softmax_block_kernel<IO, THREADS, kRegs, false, kTailMaxVecs><<<g, b, bytes, a.stream>>>(
                        a.in, a.out, a.rows, a.cols, a.valid_len, a.rows_per_seq);
            }
        }
    }
#undef KO_SM_BLOCK
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <int IO, bool MASKED>
int launch_block(const Args<IO> &a) {
    const int nvec = a.cols / Io<IO>::E;
    int threads = tuning(knob_softmax_block_threads);
    if (threads != 256 && threads != 512 && threads != 1024) {
        // Rows of up to two vectors per thread of a big workgroup: 512 or 1024 threads and one workgroup per row,
        // dispatched in row order (like the wave kernels and the plain copy, a one-shot launch beats a grid that
        // walks the rows: [32768, 4096] 183 -> 164 us = 0.98 of the same-bytes copy, [16384, 8192] 188 -> 168 us).
        // Longer rows: up to four vectors per thread before the workgroup grows, and a grid of two workgroups
        // per resident slot walking the rows.
        if (nvec <= 1024) threads = 512;
        else if (nvec <= 2048) threads = 1024;
        else {
            threads = 256;
            while (threads < 1024 && (nvec + threads - 1) / threads > 4) threads <<= 1;
        }
    }
    while (threads < 1024 && (nvec + threads - 1) / threads > 8) threads <<= 1;
    if (threads == 256) return launch_block_threads<IO, 256, MASKED>(a);
    if (threads == 512) return launch_block_threads<IO, 512, MASKED>(a);
    return launch_block_threads<IO, 1024, MASKED>(a);
}

template <int IO, int THREADS, bool MASKED>
int launch_nocache_threads(const Args<IO> &a) {
    int64_t grid = static_cast<int64_t>(compute_units()) * (2048 / THREADS) * 2;
    if (tuning(knob_rows_block_grid) == 1) grid = a.rows;  // one workgroup per row
    if (grid > a.rows) grid = a.rows;
    if (grid > 0x7fffffff) grid = 0x7fffffff;
    softmax_nocache_kernel<IO, THREADS, MASKED><<<dim3(static_cast<unsigned>(grid)), dim3(THREADS), 0, a.stream>>>(
        a.in, a.out, a.rows, a.cols, a.valid_len, a.rows_per_seq);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

// Workgroup size by row length: a thread should have several trips of four vectors to make.
template <int IO, bool MASKED>
int launch_nocache(const Args<IO> &a) {
    const int nvec = a.cols / Io<IO>::E;
    if (nvec <= 2048) return launch_nocache_threads<IO, 256, MASKED>(a);
    if (nvec <= 8192) return launch_nocache_threads<IO, 512, MASKED>(a);
    return launch_nocache_threads<IO, 1024, MASKED>(a);
}

// A row of up to 1024 * VPL columns in the registers of one 1024-thread workgroup, element by element.
template <int IO, int VPL, bool MASKED>
int launch_block_by_element(const Args<IO> &a) {
    int64_t grid = static_cast<int64_t>(compute_units()) * 4;  // two workgroups per resident slot walk the rows
    if (grid > a.rows) grid = a.rows;
    softmax_block_kernel<IO, 1024, VPL, MASKED><<<dim3(static_cast<unsigned>(grid)), dim3(1024), 0, a.stream>>>(
        a.in, a.out, a.rows, a.cols, a.valid_len, a.rows_per_seq);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

// Rows walked element by element (IO is one of the *_1 kinds): up to 2048 columns a row sits in the registers of
// 16 or 64 lanes (column j in lane j % lanes, slot j / lanes), up to 65536 in those of a workgroup, and is read
// once; longer rows are read twice.
// An explicit policy is honoured: WARP takes the wavefront kernels (up to 2048 columns here), BLOCK the workgroup
// kernel (up to 65536 columns), BLOCK_NOCACHE the one that reads twice; AUTO the first that holds the row.
template <int IO, bool MASKED>
int launch_by_element(const Args<IO> &a, int policy) {
    static_assert(Io<IO>::E == 1, "");
    const int cols = a.cols;
    if (policy == KO_POLICY_BLOCK_NOCACHE) return launch_nocache<IO, MASKED>(a);
    if (policy == KO_POLICY_WARP && cols > 2048)
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "softmax: WARP policy holds at most 2048 columns of a row walked element "
                                              "by element, got %d", cols);
    if (policy == KO_POLICY_BLOCK) {
        if (cols <= 4096) return launch_block_by_element<IO, 4, MASKED>(a);
        if (cols <= 8192) return launch_block_by_element<IO, 8, MASKED>(a);
        if (cols <= 16384) return launch_block_by_element<IO, 16, MASKED>(a);
        if (cols <= 32768) return launch_block_by_element<IO, 32, MASKED>(a);
        if (cols <= 65536) return launch_block_by_element<IO, 64, MASKED>(a);
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "softmax: BLOCK policy holds at most 65536 columns of a row walked "
                                              "element by element, got %d", cols);
    }
    if constexpr (!MASKED) {  // rows of a few columns: as many lanes as columns, up to 64 rows per wavefront
        if (cols <= 1) return launch_wave<IO, 1, 1, false, true>(a);
        if (cols <= 2) return launch_wave<IO, 2, 1, false, true>(a);
        if (cols <= 4) return launch_wave<IO, 4, 1, false, true>(a);
        if (cols <= 8) return launch_wave<IO, 8, 1, false, true>(a);
    }
    if (cols <= 16) return launch_wave<IO, 16, 1, MASKED, true>(a);
    if (cols <= 32) return launch_wave<IO, 16, 2, MASKED, true>(a);
    if (cols <= 64) return launch_wave<IO, 16, 4, MASKED, true>(a);
    if (cols <= 128) return launch_wave<IO, 64, 2, MASKED, true>(a);
    if (cols <= 256) return launch_wave<IO, 64, 4, MASKED, true>(a);
    if (cols <= 512) return launch_wave<IO, 64, 8, MASKED, true>(a);
    if (cols <= 1024) return launch_wave<IO, 64, 16, MASKED, true>(a);
    if (cols <= 2048) return launch_wave<IO, 64, 32, MASKED, true>(a);
    if (cols <= 4096) return launch_block_by_element<IO, 4, MASKED>(a);
    if (cols <= 8192) return launch_block_by_element<IO, 8, MASKED>(a);
    if (cols <= 16384) return launch_block_by_element<IO, 16, MASKED>(a);
    if (cols <= 32768) return launch_block_by_element<IO, 32, MASKED>(a);
    if (cols <= 65536) return launch_block_by_element<IO, 64, MASKED>(a);
    return launch_nocache<IO, MASKED>(a);
}

// Few long rows (see softmax_pieces_stats_kernel).  Pieces of at least 1024 vectors (16 KB), two workgroups per
// compute unit in all.  Returns -1 when the
// shape is left to the one-workgroup-per-row kernels, or when the stream has no workspace to be had (inside a
// graph capture on a stream that never ran a call that needs one).
template <int IO, bool MASKED>
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
    if (workspace == nullptr || static_cast<size_t>(a.rows) * parts * sizeof(PiecePair) > kStreamSmallWorkspaceBytes) return -1;
    PiecePair *pairs = static_cast<PiecePair *>(workspace);
    const dim3 grid(static_cast<unsigned>(parts), static_cast<unsigned>(a.rows));
    softmax_pieces_stats_kernel<IO, THREADS, MASKED><<<grid, dim3(THREADS), 0, a.stream>>>(a.in, a.cols, a.valid_len,
                                                                                          a.rows_per_seq, piece, pairs);
    KO_CHECK_LAUNCH();
    softmax_pieces_apply_kernel<IO, THREADS, MASKED><<<grid, dim3(THREADS), 0, a.stream>>>(
        a.in, a.out, a.cols, a.valid_len, a.rows_per_seq, piece, pairs);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <int IO, bool MASKED>
int dispatch(const Args<IO> &a, int policy) {
    constexpr int E = Io<IO>::E;
    const int nvec = a.cols / E;
    if (policy == KO_POLICY_AUTO) {
        if (const int st = launch_pieces<IO, MASKED>(a); st != -1) return st;
        // (with at most one row per compute unit nothing competes for the memory system and the row held on chip
        // wins up to its full length: [128, 128256] 35 us against 46 us read twice)
        const int block_max = MASKED ? kBlockMaxVecsMasked<IO> : a.rows <= compute_units() ? kBlockMaxVecs<IO> : kBlockAutoMaxVecs<IO>;
        policy = nvec <= kWaveMaxVecs ? KO_POLICY_WARP : nvec <= block_max ? KO_POLICY_BLOCK : KO_POLICY_BLOCK_NOCACHE;
    }
    switch (policy) {
        case KO_POLICY_WARP:
            if (nvec > kWaveMaxVecs)
                return fail(KO_ERR_UNSUPPORTED_SHAPE,
                            "softmax: WARP policy holds at most %d columns per row, got %d", kWaveMaxVecs * E,
                            a.cols);
            return launch_wave_any<IO, MASKED>(a);
        case KO_POLICY_BLOCK:
            // with a mask the row has to fit the registers (no LDS tail)
            if (nvec > (MASKED ? 1024 * (96 / E) : kBlockMaxVecs<IO>))
                return fail(KO_ERR_UNSUPPORTED_SHAPE,
                            "softmax: BLOCK policy holds at most %d columns per row%s, got %d",
                            (MASKED ? 1024 * (96 / E) : kBlockMaxVecs<IO>) * E, MASKED ? " with a mask" : "", a.cols);
            return launch_block<IO, MASKED>(a);
        case KO_POLICY_BLOCK_NOCACHE: return launch_nocache<IO, MASKED>(a);
        default: return fail(KO_ERR_INVALID_ARGUMENT, "softmax: unknown policy %d", policy);
    }
}

template <int IO>
int entry(const void *in, void *out, int64_t rows, int64_t cols, const int32_t *valid_len, int64_t rows_per_seq,
          int policy, ko_stream_t stream) {
    constexpr int E = Io<IO>::E;
    if (rows < 0 || cols <= 0)
        return fail(KO_ERR_INVALID_ARGUMENT, "softmax: rows=%lld cols=%lld", (long long)rows, (long long)cols);
    if (cols > (1 << 30)) return fail(KO_ERR_UNSUPPORTED_SHAPE, "softmax: cols=%lld too large", (long long)cols);
    if (rows == 0) return KO_OK;
    if (!in || !out) return fail(KO_ERR_INVALID_ARGUMENT, "softmax: null in/out pointer");
    const uintptr_t addresses = reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out);
    if (addresses & (sizeof(typename Io<IO>::elem) - 1))
        return fail(KO_ERR_INVALID_ARGUMENT, "softmax: in/out must be aligned to their element type");
    if (valid_len && rows_per_seq <= 0)
        return fail(KO_ERR_INVALID_ARGUMENT, "softmax: valid_len given but rows_per_seq=%lld", (long long)rows_per_seq);
    if (cols % E != 0 || (addresses & 15) != 0) {
        // Rows that do not start on 16-byte boundaries (the reference's descriptors with vec_len = 1 or 2, or a
        // tensor that starts off one): every policy walks such a row element by element (launch_by_element); the
        // policies' row limits stay.
        constexpr int BY_ELEMENT = io_by_element(IO);
        const int64_t nvec = (cols + E - 1) / E;
        if (policy != KO_POLICY_AUTO && policy != KO_POLICY_WARP && policy != KO_POLICY_BLOCK && policy != KO_POLICY_BLOCK_NOCACHE)
            return fail(KO_ERR_INVALID_ARGUMENT, "softmax: unknown policy %d", policy);
        if (policy == KO_POLICY_WARP && nvec > kWaveMaxVecs)
            return fail(KO_ERR_UNSUPPORTED_SHAPE, "softmax: WARP policy holds at most %d columns per row, got %lld",
                        kWaveMaxVecs * E, (long long)cols);
        if (policy == KO_POLICY_BLOCK && nvec > (valid_len ? 1024 * (96 / E) : kBlockMaxVecs<IO>))
            return fail(KO_ERR_UNSUPPORTED_SHAPE, "softmax: BLOCK policy holds at most %d columns per row%s, got %lld",
                        (valid_len ? 1024 * (96 / E) : kBlockMaxVecs<IO>) * E, valid_len ? " with a mask" : "", (long long)cols);
        Args<BY_ELEMENT> a{static_cast<const typename Io<IO>::elem *>(in), static_cast<typename Io<IO>::elem *>(out), rows,
                           static_cast<int>(cols), valid_len, rows_per_seq, as_stream(stream)};
        return valid_len ? launch_by_element<BY_ELEMENT, true>(a, policy) : launch_by_element<BY_ELEMENT, false>(a, policy);
    }
    Args<IO> a{static_cast<const typename Io<IO>::elem *>(in), static_cast<typename Io<IO>::elem *>(out), rows,
               static_cast<int>(cols), valid_len, rows_per_seq, as_stream(stream)};
    return valid_len ? dispatch<IO, true>(a, policy) : dispatch<IO, false>(a, policy);
}

}  // namespace
}  // namespace ko

KO_EXPORT int ko_softmax_f32_policy(const float *in, float *out, int64_t rows, int64_t cols,
                                    const int32_t *valid_len, int64_t rows_per_seq, int policy,
                                    ko_stream_t stream) {
    return ko::entry<ko::IO_F32>(in, out, rows, cols, valid_len, rows_per_seq, policy, stream);
}

KO_EXPORT int ko_softmax_f32(const float *in, float *out, int64_t rows, int64_t cols,
                             const int32_t *valid_len, int64_t rows_per_seq, ko_stream_t stream) {
    return ko_softmax_f32_policy(in, out, rows, cols, valid_len, rows_per_seq, KO_POLICY_AUTO, stream);
}

KO_EXPORT int ko_softmax_16(const void *in, void *out, int64_t rows, int64_t cols, const int32_t *valid_len,
                            int64_t rows_per_seq, int dtype, int policy, ko_stream_t stream) {
    if (dtype == KO_F16) return ko::entry<ko::IO_F16>(in, out, rows, cols, valid_len, rows_per_seq, policy, stream);
    if (dtype == KO_BF16) return ko::entry<ko::IO_BF16>(in, out, rows, cols, valid_len, rows_per_seq, policy, stream);
    return ko::fail(KO_ERR_INVALID_ARGUMENT, "softmax: dtype=%d is neither KO_F16 nor KO_BF16", dtype);
}
