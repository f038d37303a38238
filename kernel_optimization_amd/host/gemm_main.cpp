// GEMM benchmark driver: the counterpart of nn_operators/gemm/main.cu (benchmark :25-177,
// tensor_core_benchmark :189-339, main :341-346) written against the C ABI.  The
// reference validates against cuBLAS with |err| <= 1e-3 (:157-174); this driver validates
// against the sequential-k CPU loop the reference keeps commented out (:162-167), in double,
// on sampled rows, with the same gate for the fp32 path and its known-answer inputs
// (A[idx] = idx/1024, B = I, C = 0; :219,226,233) for the 16-bit path.
#include <cmath>
#include <cstdio>
#include <iostream>

#include "kernel_optimization/common/common.h"
#include "kernel_optimization/common/random.h"
#include "kernel_optimization/common/tensor.h"
#include "kernel_optimization/nn_operators/gemm/gemm.h"

template <typename GemmKernel>
float time_gemm(ko_stream_t stream, const shape::GemmCoord &problem_size, Tensor &A, Tensor &B, Tensor *C, Tensor &D,
                int grid_dim) {
    using EA = typename GemmKernel::ElementA;
    using EB = typename GemmKernel::ElementB;
    using EC = typename GemmKernel::ElementC;
    ko_event_t _start, _stop;
    checkKoErrors(ko_event_create(&_start));
    checkKoErrors(ko_event_create(&_stop));
    const int n_warm = 3, n_iter = 20;
    auto launch = [&]() {
        gemm<GemmKernel>(grid_dim, GemmKernel::thread_per_block, GemmKernel::smem_total_size_in_bytes, stream,
                         problem_size, A.template device_ref<EA>(), B.template device_ref<EB>(),
                         C ? C->template device_ref<EC>() : nullptr, D.template device_ref<EC>());
    };
    for (int i = 0; i < n_warm; ++i) launch();
    checkKoErrors(ko_event_record(_start, stream));
    for (int i = 0; i < n_iter; ++i) launch();
    checkKoErrors(ko_event_record(_stop, stream));
    checkKoErrors(ko_event_synchronize(_stop));
    float ms = 0;
    checkKoErrors(ko_event_elapsed_ms(&ms, _start, _stop));
    checkKoErrors(ko_event_destroy(_start));
    checkKoErrors(ko_event_destroy(_stop));
    return ms / n_iter;
}

template <typename ElementA, typename ElementB, typename ElementC, typename ThreadBlockShape, typename WarpShape,
          int AlignmentA, int AlignmentB, int AlignmentC>
void benchmark(const shape::GemmCoord &problem_size) {
    using GemmKernel = GemmKernelSimt<ElementA, ElementB, ElementC, ThreadBlockShape, WarpShape, AlignmentA, AlignmentB,
                                      AlignmentC>;
    Tensor A(problem_size.mk() * sizeof(ElementA));
    Tensor B(problem_size.kn() * sizeof(ElementB));
    Tensor C(problem_size.mn() * sizeof(ElementC));
    Tensor D(problem_size.mn() * sizeof(ElementC));

    ko_stream_t stream;
    checkKoErrors(ko_stream_create(&stream));
    for (size_t idx = 0; idx < problem_size.mk(); ++idx)
        A.template host_ref<ElementA>()[idx] = ElementA(ko_random::uniform(ko_random::tensor_seed(3, 0), idx, -1, 1));
    for (size_t idx = 0; idx < problem_size.kn(); ++idx)
        B.template host_ref<ElementB>()[idx] = ElementB(ko_random::uniform(ko_random::tensor_seed(3, 1), idx, -1, 1));
    for (size_t idx = 0; idx < problem_size.mn(); ++idx)
        C.template host_ref<ElementC>()[idx] = ElementC(ko_random::normal(ko_random::tensor_seed(3, 2), idx, 0, 1));
    A.host_to_device_async(stream);
    B.host_to_device_async(stream);
    C.host_to_device_async(stream);
    checkKoErrors(ko_stream_synchronize(stream));

    std::cout << "SmemA bytes: " << GemmKernel::smem_A_total_size_in_bytes
              << ". SmemB bytes: " << GemmKernel::smem_B_total_size_in_bytes << std::endl;
    std::cout << "Total smem bytes: " << GemmKernel::smem_total_size_in_bytes << std::endl;

    const int grid_dim = (problem_size.m() / ThreadBlockShape::kM) * (problem_size.n() / ThreadBlockShape::kN);
    const float ms = time_gemm<GemmKernel>(stream, problem_size, A, B, &C, D, grid_dim);

    printf("======Problem size %s block shape: %s warp shape %s======\n", problem_size.to_string().c_str(),
           ThreadBlockShape::to_string().c_str(), WarpShape::to_string().c_str());
    printf("Average time %.2fms\n", ms);
    printf("%.1f TFLOP/s\n", 2.0 * problem_size.mnk() / (ms * 1e-3) / 1e12);

    D.device_to_host_async(stream);
    checkKoErrors(ko_stream_synchronize(stream));
    for (size_t row = 0; row < problem_size.m(); row += 37) {
        for (size_t col = 0; col < problem_size.n(); ++col) {
            double ref_value = 0;
            for (size_t k = 0; k < problem_size.k(); ++k)
                ref_value += double(A.template host_ref<ElementA>()[row * problem_size.k() + k]) *
                             double(B.template host_ref<ElementB>()[k * problem_size.n() + col]);
            ref_value += C.template host_ref<ElementC>()[row * problem_size.n() + col];
            const double cal_value = D.template host_ref<ElementC>()[row * problem_size.n() + col];
            if (std::fabs(cal_value - ref_value) > 1e-3) {
                printf("Error at row %zu, col %zu, reference=%.2f, got %.2f\n", row, col, ref_value, cal_value);
                exit(-1);
            }
        }
    }
    printf("Passed.\n");
    checkKoErrors(ko_stream_destroy(stream));
}

template <typename ElementA, typename ElementB, typename ElementC, typename ThreadBlockShape, typename WarpShape,
          typename InstructionShape, int AlignmentA, int AlignmentB, int AlignmentC>
void tensor_core_benchmark(const shape::GemmCoord &problem_size) {
    using GemmKernel = GemmKernelTensorCore<ElementA, ElementB, ElementC, ThreadBlockShape, WarpShape, InstructionShape,
                                            AlignmentA, AlignmentB, AlignmentC>;
    Tensor A(problem_size.mk() * sizeof(ElementA));
    Tensor B(problem_size.kn() * sizeof(ElementB));
    Tensor C(problem_size.mn() * sizeof(ElementC));
    Tensor D(problem_size.mn() * sizeof(ElementC));

    ko_stream_t stream;
    checkKoErrors(ko_stream_create(&stream));
    for (size_t idx = 0; idx < problem_size.mk(); ++idx) A.template host_ref<ElementA>()[idx] = ElementA(int(idx / 1024));
    for (size_t idx = 0; idx < problem_size.kn(); ++idx) {
        const size_t r = idx / problem_size.n(), c = idx % problem_size.n();
        B.template host_ref<ElementB>()[idx] = ElementB(r == c ? 1 : 0);
    }
    for (size_t idx = 0; idx < problem_size.mn(); ++idx) C.template host_ref<ElementC>()[idx] = ElementC(0);
    A.host_to_device_async(stream);
    B.host_to_device_async(stream);
    C.host_to_device_async(stream);
    checkKoErrors(ko_stream_synchronize(stream));

    const int grid_dim = (problem_size.m() / ThreadBlockShape::kM) * (problem_size.n() / ThreadBlockShape::kN);
    const float ms = time_gemm<GemmKernel>(stream, problem_size, A, B, &C, D, grid_dim);

    printf("======Problem size %s block shape: %s warp shape %s======\n", problem_size.to_string().c_str(),
           ThreadBlockShape::to_string().c_str(), WarpShape::to_string().c_str());
    printf("Average time %.2fms\n", ms);
    printf("%.1f TFLOP/s\n", 2.0 * problem_size.mnk() / (ms * 1e-3) / 1e12);

    D.device_to_host_async(stream);
    checkKoErrors(ko_stream_synchronize(stream));
    for (size_t idx = 0; idx < problem_size.mn(); ++idx) {
        // A * I = A (k == n here)
        const double cal_value = double(float(D.template host_ref<ElementC>()[idx]));
        const double ref_value = double(float(A.template host_ref<ElementA>()[idx]));
        if (std::fabs(cal_value - ref_value) > 1e-3) {
            printf("Error at row %zu, col %zu, reference=%.2f, got %.2f\n", idx / problem_size.n(), idx % problem_size.n(),
                   ref_value, cal_value);
            exit(-1);
        }
    }
    printf("Passed.\n");
    checkKoErrors(ko_stream_destroy(stream));
}

int main() {
    benchmark<float, float, float, shape::GemmShape<64, 64, 8>, shape::GemmShape<32, 32, 8>, 4, 4, 4>({1024, 1024, 1024});
    tensor_core_benchmark<half, half, half, shape::GemmShape<128, 128, 32>, shape::GemmShape<64, 64, 32>,
                          shape::GemmShape<16, 8, 8>, 8, 8, 8>({1024, 1024, 1024});
    return 0;
}
