// Row softmax: the reference's descriptor types (nn_operators/softmax/softmax.h) and its
// kernel entry, as host-side types over the C ABI.
//
// Reference:   softmax<K><<<grid_dim, block_dim, K::smem_in_bytes, stream>>>(in, out);
// Here:        softmax<K>(grid_dim, block_dim, K::smem_in_bytes, stream, in, out);
//
// num_row, num_column and the policy come from the descriptor, as in the reference.
// grid_dim, block_dim and the shared-memory size are accepted and ignored (the library
// sizes its launch for gfx950).  An overload adds the per-sequence padding mask.
#ifndef KERNEL_OPTIMIZATION_SOFTMAX_H
#define KERNEL_OPTIMIZATION_SOFTMAX_H

#include <type_traits>

#include "../../common/common.h"

// Row per (sub-)wavefront, row in registers (reference: row per 32-lane warp, softmax.h:11-60).
template <typename _T, int _vec_len, int _num_row, int _num_column>
struct SoftMaxWarpImpl {
    static const int smem_in_bytes = 0;
    using T = _T;
    static const int vec_len = _vec_len;
    static const int num_row = _num_row;
    static const int num_column = _num_column;
    static const int policy = KO_POLICY_WARP;
    static_assert(_num_column % _vec_len == 0, "Unaligned vectorized access");
};

// Row per workgroup, row kept on chip (reference: row cached in shared memory, softmax.h:62-113).
template <typename _T, int _vec_len, int _num_row, int _num_column>
struct SoftMaxBlockImpl {
    using T = _T;
    static const int vec_len = _vec_len;
    static const int num_row = _num_row;
    static const int num_column = _num_column;
    static const int smem_in_bytes = num_column * sizeof(T) + 32 * sizeof(T);
    static const int policy = KO_POLICY_BLOCK;
    static_assert(_num_column % _vec_len == 0, "Unaligned vectorized access");
};

// Row per workgroup, row re-read from global memory (softmax.h:116-166).
template <typename _T, int _vec_len, int _num_row, int _num_column>
struct SoftMaxBlockNoCacheImpl {
    using T = _T;
    static const int vec_len = _vec_len;
    static const int num_row = _num_row;
    static const int num_column = _num_column;
    static const int smem_in_bytes = 32 * sizeof(T);
    static const int policy = KO_POLICY_BLOCK_NOCACHE;
    static_assert(_num_column % _vec_len == 0, "Unaligned vectorized access");
};

// T = float, half (ko_half) or ko_bfloat16; the 16-bit types are storage types, the arithmetic is fp32
// (the reference instantiates the same template with its half functors, common/functors.h:71-77).
template <typename SoftMaxKernel>
void softmax(int grid_dim, int block_dim, int smem_in_bytes, ko_stream_t stream, typename SoftMaxKernel::T *in_data,
             typename SoftMaxKernel::T *out_data, const int32_t *valid_len = nullptr, int64_t rows_per_seq = 0) {
    using T = typename SoftMaxKernel::T;
    static_assert(std::is_same<T, float>::value || std::is_same<T, ko_half>::value ||
                      std::is_same<T, ko_bfloat16>::value,
                  "libko provides softmax on float, half and bfloat16 storage");
    (void)grid_dim;
    (void)block_dim;
    (void)smem_in_bytes;
    if constexpr (std::is_same<T, float>::value) {
        checkKoErrors(ko_softmax_f32_policy(in_data, out_data, SoftMaxKernel::num_row, SoftMaxKernel::num_column,
                                            valid_len, rows_per_seq, SoftMaxKernel::policy, stream));
    } else {
        checkKoErrors(ko_softmax_16(in_data, out_data, SoftMaxKernel::num_row, SoftMaxKernel::num_column, valid_len,
                                    rows_per_seq, std::is_same<T, ko_half>::value ? KO_F16 : KO_BF16,
                                    SoftMaxKernel::policy, stream));
    }
}

#endif  // KERNEL_OPTIMIZATION_SOFTMAX_H
