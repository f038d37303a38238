// LayerNorm: the reference's descriptor types (nn_operators/layernorm/layernorm.h:145-300)
// and its kernel entry (:302-312) as host-side types over the C ABI.
//
// Reference:   layer_normalization<K><<<grid, block, K::smem_in_bytes, stream>>>(in, out, epsilon, gamma, beta);
// Here:        layer_normalization<K>(grid, block, K::smem_in_bytes, stream, in, out, epsilon, gamma, beta);
//
// With K::elementwise_affine == false gamma and beta are not applied, as in the reference
// (layernorm.h:189).  The extended overload also returns the per-row mean and rstd and
// selects the variance denominator (N by default; N-1 is what layernorm.h:48 aims at).
#ifndef KERNEL_OPTIMIZATION_LAYERNORM_H
#define KERNEL_OPTIMIZATION_LAYERNORM_H

#include <type_traits>

#include "../../common/common.h"

#define KO_LAYERNORM_DESCRIPTOR(NAME, POLICY, SMEM)                                                      \
    template <typename _Element, int _vec_len, int _num_row, int _num_column, bool _elementwise_affine> \
    struct NAME {                                                                                        \
        using Element = _Element;                                                                        \
        static const int vec_len = _vec_len;                                                             \
        static const int num_row = _num_row;                                                             \
        static const int num_column = _num_column;                                                       \
        static const bool elementwise_affine = _elementwise_affine;                                      \
        static const int smem_in_bytes = (SMEM);                                                         \
        static const int policy = (POLICY);                                                              \
        static_assert(_num_column % _vec_len == 0, "Unaligned vectorized access");                       \
    }

KO_LAYERNORM_DESCRIPTOR(LayerNormWarpImpl, KO_POLICY_WARP, 0);                                                 // :145-201
KO_LAYERNORM_DESCRIPTOR(LayerNormBlockImpl, KO_POLICY_BLOCK,
                        _num_column * sizeof(_Element) + 32 * 3 * sizeof(_Element));                            // :204-252
KO_LAYERNORM_DESCRIPTOR(LayerNormBlockNoCacheImpl, KO_POLICY_BLOCK_NOCACHE, 32 * 3 * sizeof(_Element));         // :254-300
#undef KO_LAYERNORM_DESCRIPTOR

// Element = float, half (ko_half) or ko_bfloat16 (storage of in, out, gamma, beta; fp32 arithmetic;
// mean and rstd are always float).
// Variance divisor: `unbiased = false` (the default) divides the sum of squared deviations by num_column, what
// BERT and every framework's LayerNorm compute; `unbiased = true` divides by num_column - 1, which is what
// the reference's merge is written to do (layernorm.h:48).  A driver ported verbatim from the reference therefore
// gets the population variance unless it passes `true` here; the two differ by a factor num_column/(num_column-1)
// in the variance (1.3e-3 at 768 columns).
template <typename LayerNormKernel>
void layer_normalization(int grid_dim, int block_dim, int smem_in_bytes, ko_stream_t stream,
                         typename LayerNormKernel::Element *in_data, typename LayerNormKernel::Element *out_data,
                         typename LayerNormKernel::Element epsilon,
                         typename LayerNormKernel::Element *gamma = nullptr,
                         typename LayerNormKernel::Element *beta = nullptr, float *mean = nullptr,
                         float *rstd = nullptr, bool unbiased = false) {
    using Element = typename LayerNormKernel::Element;
    static_assert(std::is_same<Element, float>::value || std::is_same<Element, ko_half>::value ||
                      std::is_same<Element, ko_bfloat16>::value,
                  "libko provides LayerNorm on float, half and bfloat16 storage");
    (void)grid_dim;
    (void)block_dim;
    (void)smem_in_bytes;
    const bool affine = LayerNormKernel::elementwise_affine;
    if constexpr (std::is_same<Element, float>::value) {
        checkKoErrors(ko_layernorm_f32_policy(in_data, out_data, mean, rstd, affine ? gamma : nullptr,
                                              affine ? beta : nullptr, LayerNormKernel::num_row,
                                              LayerNormKernel::num_column, epsilon, unbiased ? 1 : 0,
                                              LayerNormKernel::policy, stream));
    } else {
        checkKoErrors(ko_layernorm_16(in_data, out_data, mean, rstd, affine ? gamma : nullptr, affine ? beta : nullptr,
                                      LayerNormKernel::num_row, LayerNormKernel::num_column,
                                      static_cast<float>(epsilon), unbiased ? 1 : 0,
                                      std::is_same<Element, ko_half>::value ? KO_F16 : KO_BF16,
                                      LayerNormKernel::policy, stream));
    }
}

#endif  // KERNEL_OPTIMIZATION_LAYERNORM_H
