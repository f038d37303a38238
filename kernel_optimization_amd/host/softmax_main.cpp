// Softmax benchmark driver: the counterpart of the reference's nn_operators/softmax/main.cu
// (run_benchmark :22-74, main :76-81) written against the C ABI.  Same flow - fill on the
// host, copy to the device, time the launch with an event pair on a non-blocking stream,
// print the same two lines - plus warm-up, repetitions and the achieved bandwidth.
#include <cstdio>
#include <vector>

#include "kernel_optimization/common/common.h"
#include "kernel_optimization/common/random.h"
#include "kernel_optimization/common/tensor.h"
#include "kernel_optimization/nn_operators/softmax/softmax.h"

template <int grid_dim, int block_dim, typename T, template <typename, int, int, int> class SoftMax, int vec_len,
          int num_row, int num_column>
void run_benchmark(int cfg, int n_seq = 0, int rows_per_seq = 0) {
    using SoftMaxKernel = SoftMax<T, vec_len, num_row, num_column>;
    const size_t count = static_cast<size_t>(num_row) * num_column;

    Tensor in_data(count * sizeof(T));
    Tensor out_data(count * sizeof(T));
    Tensor lengths(static_cast<size_t>(n_seq > 0 ? n_seq : 1) * sizeof(int32_t));

    ko_stream_t stream;
    checkKoErrors(ko_stream_create(&stream));

    for (size_t idx = 0; idx < count; ++idx)
        in_data.template host_ref<T>()[idx] = T(ko_random::normal(ko_random::tensor_seed(cfg, 0), idx, 0.0, 4.0));
    for (int s = 0; s < n_seq; ++s)
        lengths.template host_ref<int32_t>()[s] =
            64 + static_cast<int32_t>(449.0 * ko_random::unit(ko_random::tensor_seed(cfg, 1), s));

    in_data.host_to_device_async(stream);
    lengths.host_to_device_async(stream);
    checkKoErrors(ko_stream_synchronize(stream));

    ko_event_t _start, _stop;
    checkKoErrors(ko_event_create(&_start));
    checkKoErrors(ko_event_create(&_stop));

    const int n_warm = 3, n_iter = 20;
    const int32_t *valid_len = n_seq > 0 ? lengths.template device_ref<int32_t>() : nullptr;
    for (int idx = 0; idx < n_warm; ++idx)
        softmax<SoftMaxKernel>(grid_dim, block_dim, SoftMaxKernel::smem_in_bytes, stream,
                               in_data.template device_ref<T>(), out_data.template device_ref<T>(), valid_len,
                               rows_per_seq);
    checkKoErrors(ko_event_record(_start, stream));
    for (int idx = 0; idx < n_iter; ++idx)
        softmax<SoftMaxKernel>(grid_dim, block_dim, SoftMaxKernel::smem_in_bytes, stream,
                               in_data.template device_ref<T>(), out_data.template device_ref<T>(), valid_len,
                               rows_per_seq);
    checkKoErrors(ko_event_record(_stop, stream));
    checkKoErrors(ko_event_synchronize(_stop));
    float time_in_ms = 0;
    checkKoErrors(ko_event_elapsed_ms(&time_in_ms, _start, _stop));
    checkKoErrors(ko_stream_synchronize(stream));

    printf("======Num row %d, num column %d======\n", num_row, num_column);
    printf("Average time %.2fms\n", time_in_ms / n_iter);
    printf("Algorithmic bandwidth %.0f GB/s (read + write of %zu bytes each)\n",
           2.0 * count * sizeof(T) / (time_in_ms / n_iter * 1e-3) / 1e9, count * sizeof(T));

    // Every row sums to one: a check the reference never makes (it prints the time only).
    out_data.device_to_host_async(stream);
    checkKoErrors(ko_stream_synchronize(stream));
    double worst = 0;
    for (int r = 0; r < num_row; r += 997) {
        double s = 0;
        for (int c = 0; c < num_column; ++c) s += out_data.template host_ref<T>()[static_cast<size_t>(r) * num_column + c];
        worst = std::fabs(s - 1.0) > worst ? std::fabs(s - 1.0) : worst;
    }
    printf("max |row sum - 1| over sampled rows: %.3g %s\n", worst, worst < 1e-5 ? "Passed." : "FAILED");

    checkKoErrors(ko_event_destroy(_start));
    checkKoErrors(ko_event_destroy(_stop));
    checkKoErrors(ko_stream_destroy(stream));
    if (worst >= 1e-5) exit(-1);
}

int main() {
    run_benchmark<40 * 8, 128, float, SoftMaxWarpImpl, 4, 128 * 12 * 128, 128>(1);
    run_benchmark<40 * 8, 128, float, SoftMaxBlockImpl, 4, 49152, 1024>(1);
    run_benchmark<40 * 8, 128, float, SoftMaxBlockNoCacheImpl, 4, 49152, 1024>(1);
    run_benchmark<40 * 8, 128, float, SoftMaxWarpImpl, 4, 128 * 12 * 512, 512>(5, 128, 12 * 512);
    return 0;
}
