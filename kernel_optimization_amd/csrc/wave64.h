// Cross-lane primitives for 64-wide wavefronts on gfx950.
//
// The reference reduces over 32-lane warps with a __shfl_down_sync tree whose
// result is valid in lane 0 and is then broadcast with __shfl_sync
// (common/common.h:37-46, nn_operators/softmax/softmax.h:41-42).  Here every
// step is a symmetric exchange (lane i pairs with a lane j that pairs back
// with i), so after log2(G) steps every lane of a G-lane group holds the same
// bits and no broadcast is needed:
//   xor 1, xor 2        DPP quad_perm          (inside a quad)
//   i <-> 7-i           DPP row_half_mirror    (quad 0 <-> quad 1 of an 8-lane half row)
//   i <-> 15-i          DPP row_mirror         (the two halves of a 16-lane row)
//   row 2k <-> row 2k+1 v_permlane16_swap      (gfx950)
//   lanes 0-31 <-> 32-63 v_permlane32_swap     (gfx950)
// No LDS is touched.
#pragma once

#include <hip/hip_runtime.h>

namespace ko {
namespace wave {

constexpr int kDppQuadXor1 = 0xB1;      // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;      // quad_perm:[2,3,0,1]
constexpr int kDppRowMirror = 0x140;
constexpr int kDppRowHalfMirror = 0x141;

template <int Ctrl>
__device__ __forceinline__ float dpp(float v) {
    int i = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(i, i, Ctrl, 0xf, 0xf, true));
}

// Partner value across adjacent 16-lane rows (row 0 <-> 1, row 2 <-> 3).
// v_permlane16_swap exchanges the odd rows of its first operand with the even
// rows of its second; starting from two copies of v, the first operand ends up
// holding the even row of each pair in both rows, the second the odd row in both.
// Written as inline assembly: with this compiler the two results of
// __builtin_amdgcn_permlane16_swap / permlane32_swap come back in one register.
// The s_nop before covers the wait states the instruction needs after a VALU write
// of its operands (the compiler cannot see inside the asm to insert them).
__device__ __forceinline__ void swap16(float v, float &even_rows, float &odd_rows) {
    float a = v, b = v;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    even_rows = a;
    odd_rows = b;
}

// Same for the two 32-lane halves: first result = lower half's values in both
// halves, second = upper half's.
__device__ __forceinline__ void swap32(float v, float &lower, float &upper) {
    float a = v, b = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    lower = a;
    upper = b;
}

// Value held by the first lane of each aligned group of G lanes, in every lane of the group.
template <int G>
__device__ __forceinline__ float broadcast_group_first(float v) {
    const int bits = __builtin_bit_cast(int, v);
    if constexpr (G == 64) {
        return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(bits));
    } else {
        const int lane = static_cast<int>(threadIdx.x) & 63;
        return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane & ~(G - 1)) << 2, bits));
    }
}

struct Max {
    __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};
struct Sum {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};

// All-reduce over aligned groups of G lanes (G in {1,2,4,8,16,32,64}).  Op must be
// commutative; the result is bit-identical in every lane of the group.
template <int G, class Op>
__device__ __forceinline__ float allreduce(float v, Op op = Op()) {
    static_assert(G == 1 || G == 2 || G == 4 || G == 8 || G == 16 || G == 32 || G == 64, "");
    if constexpr (G >= 2) v = op(v, dpp<kDppQuadXor1>(v));
    if constexpr (G >= 4) v = op(v, dpp<kDppQuadXor2>(v));
    if constexpr (G >= 8) v = op(v, dpp<kDppRowHalfMirror>(v));
    if constexpr (G >= 16) v = op(v, dpp<kDppRowMirror>(v));
    if constexpr (G >= 32) {
        float a, b;
        swap16(v, a, b);
        v = op(a, b);
    }
    if constexpr (G >= 64) {
        float a, b;
        swap32(v, a, b);
        v = op(a, b);
    }
    return v;
}

// Welford triplet (count, mean, M2).  The merge is Chan's pairwise update
// (nn_operators/layernorm/layernorm.h:36-47, without the division of M2 by
// count-1 at :48), written so that merge(a,b) and merge(b,a) give the same bits:
//   n = na + nb;  mean = (na*ma + nb*mb)/n;  M2 = (M2a + M2b) + (mb-ma)^2 * na*nb/n
// An empty side (count 0) is the identity; two empty sides stay empty.
struct Welford {
    float count, mean, m2;
};

__device__ __forceinline__ Welford welford_merge(const Welford &a, const Welford &b) {
    Welford r;
    r.count = a.count + b.count;
    // 1/n from the hardware reciprocal (1 ulp; two correctly rounded divisions cost ten instructions each, and
    // a workgroup-wide all-reduce makes ten merges per row).  Both sides empty: n = 1 keeps the triplet at zero.
    const float inv_n = __builtin_amdgcn_rcpf(r.count > 0.0f ? r.count : 1.0f);
    r.mean = (a.count * a.mean + b.count * b.mean) * inv_n;
    const float d = b.mean - a.mean;
    r.m2 = (a.m2 + b.m2) + d * d * (a.count * b.count * inv_n);
    return r;
}

template <int Ctrl>
__device__ __forceinline__ Welford welford_dpp_step(const Welford &w) {
    Welford o{dpp<Ctrl>(w.count), dpp<Ctrl>(w.mean), dpp<Ctrl>(w.m2)};
    return welford_merge(w, o);
}

template <int G>
__device__ __forceinline__ Welford welford_allreduce(Welford w) {
    static_assert(G == 1 || G == 2 || G == 4 || G == 8 || G == 16 || G == 32 || G == 64, "");
    if constexpr (G >= 2) w = welford_dpp_step<kDppQuadXor1>(w);
    if constexpr (G >= 4) w = welford_dpp_step<kDppQuadXor2>(w);
    if constexpr (G >= 8) w = welford_dpp_step<kDppRowHalfMirror>(w);
    if constexpr (G >= 16) w = welford_dpp_step<kDppRowMirror>(w);
    if constexpr (G >= 32) {
        Welford a, b;
        swap16(w.count, a.count, b.count);
        swap16(w.mean, a.mean, b.mean);
        swap16(w.m2, a.m2, b.m2);
        w = welford_merge(a, b);
    }
    if constexpr (G >= 64) {
        Welford a, b;
        swap32(w.count, a.count, b.count);
        swap32(w.mean, a.mean, b.mean);
        swap32(w.m2, a.m2, b.m2);
        w = welford_merge(a, b);
    }
    return w;
}

// The same all-reduce when every lane of the group enters with the same count c (rows whose length is a
// whole number of vectors per lane): n = 2c at every step, so mean = (ma + mb) / 2 and
// M2 = (M2a + M2b) + (mb - ma)^2 * c / 2 - Chan's merge with the counts folded into constants, no
// division, and only two values to exchange.  Symmetric in a and b like the general form.
__device__ __forceinline__ void welford_merge_equal(float &mean, float &m2, float pmean, float pm2, float half_c) {
    const float d = pmean - mean;
    mean = 0.5f * (mean + pmean);
    m2 = __builtin_fmaf(d * d, half_c, m2 + pm2);
}

template <int G>
__device__ __forceinline__ Welford welford_allreduce_equal(Welford w) {
    static_assert(G == 1 || G == 2 || G == 4 || G == 8 || G == 16 || G == 32 || G == 64, "");
    float half_c = 0.5f * w.count;
    if constexpr (G >= 2) {
        welford_merge_equal(w.mean, w.m2, dpp<kDppQuadXor1>(w.mean), dpp<kDppQuadXor1>(w.m2), half_c);
        half_c *= 2.0f;
    }
    if constexpr (G >= 4) {
        welford_merge_equal(w.mean, w.m2, dpp<kDppQuadXor2>(w.mean), dpp<kDppQuadXor2>(w.m2), half_c);
        half_c *= 2.0f;
    }
    if constexpr (G >= 8) {
        welford_merge_equal(w.mean, w.m2, dpp<kDppRowHalfMirror>(w.mean), dpp<kDppRowHalfMirror>(w.m2), half_c);
        half_c *= 2.0f;
    }
    if constexpr (G >= 16) {
        welford_merge_equal(w.mean, w.m2, dpp<kDppRowMirror>(w.mean), dpp<kDppRowMirror>(w.m2), half_c);
        half_c *= 2.0f;
    }
    if constexpr (G >= 32) {
        float am, bm, a2, b2;
        swap16(w.mean, am, bm);
        swap16(w.m2, a2, b2);
        welford_merge_equal(am, a2, bm, b2, half_c);
        w.mean = am;
        w.m2 = a2;
        half_c *= 2.0f;
    }
    if constexpr (G >= 64) {
        float am, bm, a2, b2;
        swap32(w.mean, am, bm);
        swap32(w.m2, a2, b2);
        welford_merge_equal(am, a2, bm, b2, half_c);
        w.mean = am;
        w.m2 = a2;
    }
    w.count *= static_cast<float>(G);
    return w;
}

}  // namespace wave

// 128-bit global accesses, optionally non-temporal (streaming: data is touched once).
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

template <bool NT>
__device__ __forceinline__ float4v load4(const float *p) {
    const float4v *q = reinterpret_cast<const float4v *>(p);
    if constexpr (NT) return __builtin_nontemporal_load(q);
    return *q;
}

// Streaming store of 16 bytes: written through the XCD's L2 at once (sc1: device scope) and marked
// non-temporal, so the line does not wait in L2 as a dirty line to be evicted later.  Measured on 1 GiB
// streams on MI355X: write-only 7.18 TB/s against 6.73 TB/s with `nt` alone and 6.90 TB/s with plain stores;
// copy 6.85 against 6.65 TB/s.  The compiler has no spelling for the sc1 bit on a plain store, hence the
// inline assembly; it needs no "memory" clobber for the callers here: what a thread stores it never reads
// back, and a row's loads are complete (their values are used) before its first store.
// The s_nop behind the store is required: a store of more than 64 bits reads its data registers over several
// cycles, and a vector-ALU write to them within the next two wait states would change what is stored.  The
// compiler inserts those wait states for its own stores but does not look inside inline assembly.
// The address is a wave-uniform base (in scalar registers) plus a 32-bit byte offset per lane: with a 64-bit
// address per lane the register allocator, which cannot move or merge inline assembly, spilled in the kernels
// that hold 96 row values per thread.  `uniform_base` MUST have the same value in every lane of the wavefront
// (the compiler reads it from the first active lane if it cannot prove that).
template <class V>
__device__ __forceinline__ void stream_store16(void *uniform_base, uint32_t byte_offset, V v) {
    static_assert(sizeof(V) == 16, "");
    // through readfirstlane: the "s" constraint alone does not move a value the compiler holds in vector
    // registers (a row pointer derived from threadIdx.x >> 6, say) into scalar ones
    const uint64_t b = reinterpret_cast<uint64_t>(uniform_base);
    // (the builtin returns int: each half goes through uint32_t, or the low half would be sign-extended)
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b >> 32)));
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b)));
    const uint64_t base = (static_cast<uint64_t>(hi) << 32) | lo;
    // s_nop 4 in front: the base reaches its scalar registers through v_readfirstlane, a vector-ALU write of
    // scalar registers, and a memory instruction may read such a register only five wait states later.  The
    // compiler keeps that distance for its own instructions but cannot see that this assembly reads them.
    asm volatile("s_nop 4\n\tglobal_store_dwordx4 %0, %1, %2 sc1 nt\n\ts_nop 1" ::"v"(byte_offset), "v"(v), "s"(base));
}

template <bool NT>
__device__ __forceinline__ void store4(float *p, float4v v) {
    float4v *q = reinterpret_cast<float4v *>(p);
    if constexpr (NT) __builtin_nontemporal_store(v, q);
    else *q = v;
}

// Storage types of the row operators.  The arithmetic is always fp32; a 16-byte vector holds
// E = 4 floats or E = 8 binary16 / bfloat16 values, converted on load and rounded (to nearest
// even) once on store.  The reference carries half specialisations of its functors for the same
// purpose (common/functors.h:71-77,105-111, common/common.h:171-177).
// The *_1 kinds move one element per access (E = 1): rows whose length is not a multiple of the 16-byte vector
// start at element alignment, and the kernels that walk a row vector by vector (the re-reading ones) walk it
// element by element instead - what the reference's descriptors do with vec_len = 1.
enum { IO_F32 = 0, IO_F16 = 1, IO_BF16 = 2, IO_F32_1 = 3, IO_F16_1 = 4, IO_BF16_1 = 5 };
// the one-element kind of a storage type, and the storage type of any kind
constexpr int io_by_element(int io) { return io % 3 + 3; }
constexpr int io_storage(int io) { return io % 3; }

template <int IO>
struct Io;

template <>
struct Io<IO_F32> {
    typedef float elem;
    static constexpr int E = 4;
    typedef float4v raw;  // one 16-byte vector as loaded, before conversion
    static constexpr uint32_t kBytes = sizeof(raw);  // between consecutive vectors of a row
    template <bool NT>
    static __device__ __forceinline__ raw load_raw(const elem *p) {
        return load4<NT>(p);
    }
    static __device__ __forceinline__ void unpack(raw x, float (&v)[E]) {
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] = x[e];
    }
    template <bool NT>
    static __device__ __forceinline__ void load(const elem *p, float (&v)[E]) {
        unpack(load_raw<NT>(p), v);
    }
    template <bool NT>
    static __device__ __forceinline__ void store(elem *p, const float (&v)[E]) {
        store4<NT>(p, float4v{v[0], v[1], v[2], v[3]});
    }
    // streaming store of one vector at uniform_base + byte_offset (see stream_store16)
    static __device__ __forceinline__ void store_stream(elem *uniform_base, uint32_t byte_offset, const float (&v)[E]) {
        stream_store16(uniform_base, byte_offset, float4v{v[0], v[1], v[2], v[3]});
    }
    static __device__ __forceinline__ float scalar(const elem *p) { return *p; }
};

template <bool NT>
__device__ __forceinline__ uint4v load_bits16(const uint16_t *p) {
    const uint4v *q = reinterpret_cast<const uint4v *>(p);
    if constexpr (NT) return __builtin_nontemporal_load(q);
    return *q;
}

template <bool NT>
__device__ __forceinline__ void store_bits16(uint16_t *p, uint4v v) {
    uint4v *q = reinterpret_cast<uint4v *>(p);
    if constexpr (NT) __builtin_nontemporal_store(v, q);
    else *q = v;
}

template <>
struct Io<IO_F16> {
    typedef uint16_t elem;
    static constexpr int E = 8;
    typedef _Float16 half8 __attribute__((ext_vector_type(8)));
    typedef uint4v raw;
    static constexpr uint32_t kBytes = sizeof(raw);
    template <bool NT>
    static __device__ __forceinline__ raw load_raw(const elem *p) {
        return load_bits16<NT>(p);
    }
    static __device__ __forceinline__ void unpack(raw x, float (&v)[E]) {
        const half8 h = __builtin_bit_cast(half8, x);
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] = static_cast<float>(h[e]);
    }
    template <bool NT>
    static __device__ __forceinline__ void load(const elem *p, float (&v)[E]) {
        unpack(load_raw<NT>(p), v);
    }
    template <bool NT>
    static __device__ __forceinline__ void store(elem *p, const float (&v)[E]) {
        half8 h;
#pragma unroll
        for (int e = 0; e < E; ++e) h[e] = static_cast<_Float16>(v[e]);
        store_bits16<NT>(p, __builtin_bit_cast(uint4v, h));
    }
    static __device__ __forceinline__ void store_stream(elem *uniform_base, uint32_t byte_offset, const float (&v)[E]) {
        half8 h;
#pragma unroll
        for (int e = 0; e < E; ++e) h[e] = static_cast<_Float16>(v[e]);
        stream_store16(uniform_base, byte_offset, __builtin_bit_cast(uint4v, h));
    }
    static __device__ __forceinline__ float scalar(const elem *p) {
        return static_cast<float>(__builtin_bit_cast(_Float16, *p));
    }
};

template <>
struct Io<IO_BF16> {
    typedef uint16_t elem;
    static constexpr int E = 8;
    typedef uint4v raw;
    static constexpr uint32_t kBytes = sizeof(raw);
    template <bool NT>
    static __device__ __forceinline__ raw load_raw(const elem *p) {
        return load_bits16<NT>(p);
    }
    static __device__ __forceinline__ void unpack(raw x, float (&v)[E]) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[2 * e] = __builtin_bit_cast(float, x[e] << 16);
            v[2 * e + 1] = __builtin_bit_cast(float, x[e] & 0xffff0000u);
        }
    }
    template <bool NT>
    static __device__ __forceinline__ void load(const elem *p, float (&v)[E]) {
        unpack(load_raw<NT>(p), v);
    }
    template <bool NT>
    static __device__ __forceinline__ void store(elem *p, const float (&v)[E]) {
        // float -> bfloat16, round to nearest even: v_cvt_pk_bf16_f32, two values per instruction
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        typedef float float2v __attribute__((ext_vector_type(2)));
        uint4v x;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            x[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(float2v{v[2 * e], v[2 * e + 1]}, bf16x2));
        store_bits16<NT>(p, x);
    }
    static __device__ __forceinline__ void store_stream(elem *uniform_base, uint32_t byte_offset, const float (&v)[E]) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        typedef float float2v __attribute__((ext_vector_type(2)));
        uint4v x;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            x[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(float2v{v[2 * e], v[2 * e + 1]}, bf16x2));
        stream_store16(uniform_base, byte_offset, x);
    }
    static __device__ __forceinline__ float scalar(const elem *p) {
        return __builtin_bit_cast(float, static_cast<uint32_t>(*p) << 16);
    }
};

// One element per access.  CONVERT supplies the storage type's conversions (float <-> bits).
template <class Elem, class Convert>
struct IoByElement {
    typedef Elem elem;
    static constexpr int E = 1;
    typedef Elem raw;
    static constexpr uint32_t kBytes = sizeof(raw);
    template <bool NT>
    static __device__ __forceinline__ raw load_raw(const elem *p) {
        if constexpr (NT) return __builtin_nontemporal_load(p);
        return *p;
    }
    static __device__ __forceinline__ void unpack(raw x, float (&v)[E]) { v[0] = Convert::to_float(x); }
    template <bool NT>
    static __device__ __forceinline__ void load(const elem *p, float (&v)[E]) {
        unpack(load_raw<NT>(p), v);
    }
    template <bool NT>
    static __device__ __forceinline__ void store(elem *p, const float (&v)[E]) {
        if constexpr (NT) __builtin_nontemporal_store(Convert::from_float(v[0]), p);
        else *p = Convert::from_float(v[0]);
    }
    static __device__ __forceinline__ void store_stream(elem *base, uint32_t byte_offset, const float (&v)[E]) {
        __builtin_nontemporal_store(Convert::from_float(v[0]),
                                    reinterpret_cast<elem *>(reinterpret_cast<char *>(base) + byte_offset));
    }
    static __device__ __forceinline__ float scalar(const elem *p) { return Convert::to_float(*p); }
};
struct ConvertF32 {
    static __device__ __forceinline__ float to_float(float x) { return x; }
    static __device__ __forceinline__ float from_float(float x) { return x; }
};
struct ConvertF16 {
    static __device__ __forceinline__ float to_float(uint16_t x) { return static_cast<float>(__builtin_bit_cast(_Float16, x)); }
    static __device__ __forceinline__ uint16_t from_float(float x) {  // round to nearest even
        return __builtin_bit_cast(uint16_t, static_cast<_Float16>(x));
    }
};
struct ConvertBF16 {
    static __device__ __forceinline__ float to_float(uint16_t x) { return __builtin_bit_cast(float, static_cast<uint32_t>(x) << 16); }
    static __device__ __forceinline__ uint16_t from_float(float x) {  // round to nearest even, as the vector kind does
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        typedef float float2v __attribute__((ext_vector_type(2)));
        return static_cast<uint16_t>(__builtin_bit_cast(uint32_t, __builtin_convertvector(float2v{x, 0.0f}, bf16x2)));
    }
};
template <>
struct Io<IO_F32_1> : IoByElement<float, ConvertF32> {};
template <>
struct Io<IO_F16_1> : IoByElement<uint16_t, ConvertF16> {};
template <>
struct Io<IO_BF16_1> : IoByElement<uint16_t, ConvertBF16> {};

// One vector of an output row, at uniform_base + byte_offset.  Rows that are whole 64-byte lines are written through
// at once (stream_store16).  A row that ends inside a line would send that line out twice, half-filled each time,
// and written through the halves reach the memory side separately: such rows are stored with the non-temporal
// hint alone and left to the L2 to put together (softmax [49152, 1000]: 75.5 us written through, 64.8 us this way;
// [32768, 2052] in the workgroup kernel 104 us against 2304 columns' 95 us).
template <int IO>
__device__ __forceinline__ void store_row_vec(bool whole_lines, typename Io<IO>::elem *uniform_base, uint32_t byte_offset,
                                              const float (&v)[Io<IO>::E]) {
    if (whole_lines) {
        Io<IO>::store_stream(uniform_base, byte_offset, v);
    } else {
        Io<IO>::template store<true>(
            reinterpret_cast<typename Io<IO>::elem *>(reinterpret_cast<char *>(uniform_base) + byte_offset), v);
    }
}
// whether rows of `cols` elements are whole 64-byte lines
template <int IO>
__device__ __forceinline__ bool rows_are_whole_lines(int cols) {
    return (static_cast<uint32_t>(cols) * static_cast<uint32_t>(sizeof(typename Io<IO>::elem))) % 64u == 0;
}

// exp(d) for d <= 0, within 2 ulp: 2^y (1 + r ln 2), where y = d * log2(e) is the rounded product, r its exact
// residual plus d times the low part of log2(e) (|r| <= 2^-24 |y|, so the first-order term is all that matters),
// and 2^y is the hardware base-2 exponential (v_exp_f32: 1 ulp over its whole range; results below 2^-126 are
// flushed to zero, which no gate here can see: they are below FLT_MIN relative to a sum of at least 1).  Eight
// vector-ALU operations per value; splitting off the integer part and applying it with ldexp took twelve, and on
// rows that fill a workgroup's registers that arithmetic is time during which the compute unit requests no memory.
// Arguments below -128 (minus infinity included) are clamped: the result is 0 either way.  A NaN argument gives
// NaN - the clamp is a compare and select, not fmaxf, which would return the clamp value for a NaN - so that a NaN
// or a +inf element (inf - inf) poisons its row's sum as it does with expf in the reference
// (nn_operators/softmax/softmax.h:46).
__device__ __forceinline__ float exp_nonpositive(float d) {
    const float kLog2eHi = 0x1.715476p+0f;
    const float kLog2eLo = 0x1.4ae0cp-26f;
    const float kLn2 = 0x1.62e43p-1f;
    d = d < -128.0f ? -128.0f : d;
    const float y = d * kLog2eHi;
    float r = __builtin_fmaf(d, kLog2eHi, -y);
    r = __builtin_fmaf(d, kLog2eLo, r);
    const float e = __builtin_amdgcn_exp2f(y);
    return __builtin_fmaf(e * r, kLn2, e);
}

// exp(d) for d <= 0 where the result is rounded to bfloat16 afterwards (which keeps fp32's exponent range, so
// results below 2^-126 matter): 2^(d log2(e) + 64) from the bare instruction, in the normal range for every
// result that is not zero in the end, times 2^-64 by a multiplication, which produces subnormal results
// correctly.  The rounded fused multiply-add costs 2^-18 absolute in the exponent, 2.6e-6 relative in the
// result: far inside half an ulp of bfloat16 (3.9e-3).  No clamp: the instruction returns 0 for arguments below
// -126 (minus infinity included) and NaN for NaN.
__device__ __forceinline__ float exp_nonpositive_fast(float d) {
    return __builtin_amdgcn_exp2f(__builtin_fmaf(d, 0x1.715476p+0f, 64.0f)) * 0x1p-64f;
}

// The same for binary16 storage: everything below 2^-25 rounds to zero there, so the bare instruction is used
// as it is (it flushes results below the normal range to zero; the compiler's exp2f would rescale them: a
// compare, two selects and an ldexp per value, a third of this kernel's vector ALU work).
__device__ __forceinline__ float exp_nonpositive_f16(float d) {
    return __builtin_amdgcn_exp2f(d * 0x1.715476p+0f);
}

template <int IO>
__device__ __forceinline__ float exp_for_storage(float d) {
    if constexpr (io_storage(IO) == IO_F32) return exp_nonpositive(d);
    else if constexpr (io_storage(IO) == IO_F16) return exp_nonpositive_f16(d);
    else return exp_nonpositive_fast(d);
}

}  // namespace ko
