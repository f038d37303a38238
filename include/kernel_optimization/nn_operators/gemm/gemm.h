// GEMM: the reference's two kernel descriptors (nn_operators/gemm/simt_gemm.h:46-103,
// tensor_core_gemm.h:101-160) and its kernel entry (gemm.h:11-21) as host-side types over
// the C ABI.
//
// Reference:   gemm<K><<<grid, K::thread_per_block, K::smem_total_size_in_bytes, stream>>>(problem_size, A, B, C, D);
// Here:        gemm<K>(grid, K::thread_per_block, K::smem_total_size_in_bytes, stream, problem_size, A, B, C, D);
//
// Semantics as in the reference's epilogue (simt_gemm.h:325-373): D = A*B + C when C is
// given, D = A*B when it is null; all matrices row-major (B is [K,N]).  The tile shapes
// of the descriptor are T4 tuning parameters: they are kept as types and constants, and
// the library chooses its own gfx950 tiling.  The extended overload exposes alpha, beta
// and a column-major B.
#ifndef KERNEL_OPTIMIZATION_GEMM_H
#define KERNEL_OPTIMIZATION_GEMM_H

#include <type_traits>

#include "../../common/common.h"

template <typename _ElementA, typename _ElementB, typename _ElementC, typename _ThreadBlockShape,
          typename _WarpShape, int AlignmentA, int AlignmentB, int AlignmentC>
struct GemmKernelSimt {
    using ElementA = _ElementA;
    using ElementB = _ElementB;
    using ElementC = _ElementC;
    using ThreadBlockShape = _ThreadBlockShape;
    using WarpShape = _WarpShape;
    static const bool tensor_core = false;

    static_assert(ThreadBlockShape::kK % AlignmentA == 0, "");
    static_assert(ThreadBlockShape::kN % AlignmentB == 0, "");
    static_assert(ThreadBlockShape::kN % AlignmentC == 0, "");

    // Same formulas as simt_gemm.h:66-74 (wavefronts are 64 wide here).
    static const int smem_A_total_size_in_bytes = ThreadBlockShape::kM * (ThreadBlockShape::kK + 1) * sizeof(ElementA) * 2;
    static const int smem_B_total_size_in_bytes = ThreadBlockShape::kKN * sizeof(ElementB) * 2;
    static const int smem_total_size_in_bytes = smem_A_total_size_in_bytes + smem_B_total_size_in_bytes;
    static const int warp_count_m = ThreadBlockShape::kM / WarpShape::kM;
    static const int warp_count_n = ThreadBlockShape::kN / WarpShape::kN;
    static const int warp_count = warp_count_m * warp_count_n;
    static const int thread_per_block = warp_count * 64;
};

template <typename _ElementA, typename _ElementB, typename _ElementC, typename _ThreadBlockShape,
          typename _WarpShape, typename _InstructionShape, int AlignmentA, int AlignmentB, int AlignmentC>
struct GemmKernelTensorCore {
    using ElementA = _ElementA;
    using ElementB = _ElementB;
    using ElementC = _ElementC;
    using ThreadBlockShape = _ThreadBlockShape;
    using WarpShape = _WarpShape;
    using InstructionShape = _InstructionShape;
    static const bool tensor_core = true;

    static_assert(ThreadBlockShape::kK % AlignmentA == 0, "");
    static_assert(ThreadBlockShape::kN % AlignmentB == 0, "");
    static_assert(ThreadBlockShape::kN % AlignmentC == 0, "");

    // tensor_core_gemm.h:122-131
    static const int smem_A_total_size_in_bytes = ThreadBlockShape::kMK * sizeof(ElementA) * 2;
    static const int smem_B_total_size_in_bytes = ThreadBlockShape::kKN * sizeof(ElementB) * 2;
    static const int smem_total_size_in_bytes = smem_A_total_size_in_bytes + smem_B_total_size_in_bytes;
    static const int warp_count_m = ThreadBlockShape::kM / WarpShape::kM;
    static const int warp_count_n = ThreadBlockShape::kN / WarpShape::kN;
    static const int warp_count = warp_count_m * warp_count_n;
    static const int thread_per_block = warp_count * 64;
};

namespace ko_detail {
template <typename K, bool TensorCore = K::tensor_core>
struct GemmDispatch;

template <typename K>
struct GemmDispatch<K, false> {
    static int run(const shape::GemmCoord &ps, float alpha, const typename K::ElementA *A, const typename K::ElementB *B,
                   int b_layout, float beta, const typename K::ElementC *C, typename K::ElementC *D, ko_stream_t stream) {
        static_assert(std::is_same<typename K::ElementA, float>::value && std::is_same<typename K::ElementB, float>::value &&
                          std::is_same<typename K::ElementC, float>::value,
                      "GemmKernelSimt is the fp32 path");
        if (b_layout != KO_ROW_MAJOR) return KO_ERR_UNSUPPORTED_SHAPE;
        return ko_sgemm_f32(ps.m(), ps.n(), ps.k(), alpha, A, B, beta, C, D, stream);
    }
};

template <typename K>
struct GemmDispatch<K, true> {
    static int run(const shape::GemmCoord &ps, float alpha, const typename K::ElementA *A, const typename K::ElementB *B,
                   int b_layout, float beta, const typename K::ElementC *C, typename K::ElementC *D, ko_stream_t stream) {
        static_assert(sizeof(typename K::ElementA) == 2 && sizeof(typename K::ElementB) == 2 &&
                          sizeof(typename K::ElementC) == 2,
                      "GemmKernelTensorCore is the 16-bit path");
        const int dtype = std::is_same<typename K::ElementA, ko_bfloat16>::value ? KO_BF16 : KO_F16;
        return ko_gemm_f16f32acc(ps.m(), ps.n(), ps.k(), alpha, A, B, b_layout, beta, C, D, dtype, stream);
    }
};
}  // namespace ko_detail

// Reference semantics: D = A*B (+ C).
template <typename GemmKernel>
void gemm(int grid_dim, int block_dim, int smem_in_bytes, ko_stream_t stream, const shape::GemmCoord problem_size,
          typename GemmKernel::ElementA *ptr_A, typename GemmKernel::ElementB *ptr_B,
          typename GemmKernel::ElementC *ptr_C, typename GemmKernel::ElementC *ptr_D) {
    (void)grid_dim;
    (void)block_dim;
    (void)smem_in_bytes;
    checkKoErrors(ko_detail::GemmDispatch<GemmKernel>::run(problem_size, 1.0f, ptr_A, ptr_B, KO_ROW_MAJOR,
                                                           ptr_C ? 1.0f : 0.0f, ptr_C, ptr_D, stream));
}

// Extended: D = alpha*A*B + beta*C, B row-major [K,N] or column-major (memory [N][K]; 16-bit path only).
template <typename GemmKernel>
void gemm(int grid_dim, int block_dim, int smem_in_bytes, ko_stream_t stream, const shape::GemmCoord problem_size,
          float alpha, typename GemmKernel::ElementA *ptr_A, typename GemmKernel::ElementB *ptr_B, int b_layout,
          float beta, typename GemmKernel::ElementC *ptr_C, typename GemmKernel::ElementC *ptr_D) {
    (void)grid_dim;
    (void)block_dim;
    (void)smem_in_bytes;
    checkKoErrors(ko_detail::GemmDispatch<GemmKernel>::run(problem_size, alpha, ptr_A, ptr_B, b_layout, beta, ptr_C,
                                                           ptr_D, stream));
}

#endif  // KERNEL_OPTIMIZATION_GEMM_H
