// Host-layer self test (no GPU needed for part 1): the 16-bit conversions, the shape types
// and AlignedArray.  With "gpu" as argument it also exercises Tensor and the three launch
// wrappers on tiny problems.  Prints "host selftest ok" and exits 0 on success.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "kernel_optimization/common/common.h"
#include "kernel_optimization/common/tensor.h"
#include "kernel_optimization/nn_operators/gemm/gemm.h"
#include "kernel_optimization/nn_operators/layernorm/layernorm.h"
#include "kernel_optimization/nn_operators/softmax/softmax.h"

#define REQUIRE(cond)                                                     \
    do {                                                                  \
        if (!(cond)) {                                                    \
            printf("FAILED %s at %s:%d\n", #cond, __FILE__, __LINE__);   \
            return 1;                                                     \
        }                                                                 \
    } while (0)

static int cpu_part(const char *dump_path) {
    // half <-> float: every half value round-trips; dump float->half of a sweep for an outside check
    for (uint32_t h = 0; h < 65536; ++h) {
        ko_half x;
        x.bits = static_cast<uint16_t>(h);
        const float f = float(x);
        if (std::isnan(f)) continue;
        REQUIRE(ko_half(f).bits == h);
    }
    REQUIRE(ko_half(1.0f).bits == 0x3c00 && ko_half(-2.0f).bits == 0xc000 && ko_half(65504.0f).bits == 0x7bff);
    REQUIRE(ko_half(65520.0f).bits == 0x7c00 && ko_half(5.9604645e-8f).bits == 0x0001 && ko_half(2.9802322e-8f).bits == 0);
    REQUIRE(float(ko_bfloat16(1.0f)) == 1.0f && ko_bfloat16(1.00390625f).bits == 0x3f80);  // tie -> even
    if (dump_path) {
        FILE *f = fopen(dump_path, "wb");
        REQUIRE(f != nullptr);
        for (uint32_t i = 0; i < (1u << 20); ++i) {
            uint32_t u = i * 4099u + 12345u;
            u = (u & 0x807fffffu) | (((u >> 23) % 48 + 100) << 23);  // exponents -27..20
            float x;
            std::memcpy(&x, &u, 4);
            uint16_t b = ko_half(x).bits;
            fwrite(&u, 4, 1, f);
            fwrite(&b, 2, 1, f);
        }
        fclose(f);
    }
    shape::GemmCoord ps(3, 5, 7);
    REQUIRE(ps.mk() == 21 && ps.kn() == 35 && ps.mn() == 15 && ps.mnk() == 105 && ps.to_string() == "{3,5,7}");
    using S = shape::GemmShape<64, 32, 8>;
    REQUIRE(S::kMN == 2048 && S::kMK == 512 && S::kKN == 256 && S::kMNK == 16384 && S::to_string() == "{64,32,8}");
    AlignedArray<float, 4> v(2.0f);
    REQUIRE(alignof(decltype(v)) == 16 && v[3] == 2.0f);
    v.clear();
    REQUIRE(v.at(0) == 0.0f);
    using K = GemmKernelSimt<float, float, float, shape::GemmShape<64, 64, 8>, shape::GemmShape<32, 32, 8>, 4, 4, 4>;
    REQUIRE(K::warp_count == 4 && K::thread_per_block == 256 && K::smem_A_total_size_in_bytes == 4608 &&
            K::smem_B_total_size_in_bytes == 4096);
    REQUIRE((SoftMaxBlockImpl<float, 4, 8, 1024>::smem_in_bytes == 1024 * 4 + 128));
    REQUIRE((LayerNormBlockImpl<float, 4, 8, 768, false>::smem_in_bytes == 768 * 4 + 384));
    return 0;
}

static int gpu_part() {
    ko_stream_t stream;
    checkKoErrors(ko_stream_create(&stream));
    {
        constexpr int R = 8, C = 128;
        Tensor in(std::vector<size_t>{R, C}, sizeof(float)), out(R * C * sizeof(float));
        REQUIRE(in.size() == R * C * 4);
        for (int i = 0; i < R * C; ++i) in.host_ref<float>()[i] = 1.5f;
        in.host_to_device_async(stream);
        softmax<SoftMaxWarpImpl<float, 4, R, C>>(320, 128, 0, stream, in.device_ref<float>(), out.device_ref<float>());
        out.device_to_host_async(stream);
        checkKoErrors(ko_stream_synchronize(stream));
        for (int i = 0; i < R * C; ++i) REQUIRE(out.host_ref<float>()[i] == 1.0f / C);
        Tensor moved(16);
        moved = std::move(out);  // move assignment releases the old buffers and carries the size
        REQUIRE(moved.size() == R * C * 4 && moved.host_ref<float>()[0] == 1.0f / C);
    }
    {
        constexpr int R = 4, C = 768;
        Tensor in(R * C * 4), out(R * C * 4), mean(R * 4), rstd(R * 4);
        for (int i = 0; i < R * C; ++i) in.host_ref<float>()[i] = float(i % C);
        in.host_to_device();
        layer_normalization<LayerNormWarpImpl<float, 4, R, C, false>>(320, 128, 0, stream, in.device_ref<float>(),
                                                                       out.device_ref<float>(), 0.0f, nullptr, nullptr,
                                                                       mean.device_ref<float>(), rstd.device_ref<float>());
        checkKoErrors(ko_stream_synchronize(stream));
        mean.device_to_host();
        rstd.device_to_host();
        REQUIRE(std::fabs(mean.host_ref<float>()[2] - 383.5f) < 1e-3f);
        REQUIRE(std::fabs(rstd.host_ref<float>()[1] - 1.0 / std::sqrt((768.0 * 768.0 - 1) / 12)) < 1e-8);
    }
    {
        // 16-bit storage through the same templates: constant rows give exactly 1/C (softmax) and beta (LayerNorm)
        constexpr int R = 8, C = 128;
        Tensor in(R * C * 2), out(R * C * 2), beta(C * 2), mean(R * 4);
        for (int i = 0; i < R * C; ++i) in.host_ref<half>()[i] = half(1.5f);
        for (int i = 0; i < C; ++i) beta.host_ref<half>()[i] = half(float(i) / 8);
        in.host_to_device();
        beta.host_to_device();
        softmax<SoftMaxWarpImpl<half, 8, R, C>>(320, 128, 0, stream, in.device_ref<half>(), out.device_ref<half>());
        checkKoErrors(ko_stream_synchronize(stream));
        out.device_to_host();
        for (int i = 0; i < R * C; ++i) REQUIRE(float(out.host_ref<half>()[i]) == 1.0f / C);
        layer_normalization<LayerNormWarpImpl<half, 8, R, C, true>>(320, 128, 0, stream, in.device_ref<half>(),
                                                                    out.device_ref<half>(), half(1e-5f), nullptr,
                                                                    beta.device_ref<half>(), mean.device_ref<float>());
        checkKoErrors(ko_stream_synchronize(stream));
        out.device_to_host();
        mean.device_to_host();
        for (int i = 0; i < R * C; ++i) REQUIRE(float(out.host_ref<half>()[i]) == float(i % C) / 8);
        REQUIRE(mean.host_ref<float>()[3] == 1.5f);
        Tensor inb(R * C * 2), outb(R * C * 2);
        for (int i = 0; i < R * C; ++i) inb.host_ref<ko_bfloat16>()[i] = ko_bfloat16(-2.0f);
        inb.host_to_device();
        softmax<SoftMaxBlockImpl<ko_bfloat16, 8, R, C>>(320, 128, 0, stream, inb.device_ref<ko_bfloat16>(),
                                                        outb.device_ref<ko_bfloat16>());
        checkKoErrors(ko_stream_synchronize(stream));
        outb.device_to_host();
        for (int i = 0; i < R * C; ++i) REQUIRE(float(outb.host_ref<ko_bfloat16>()[i]) == 1.0f / C);
    }
    {
        // vec_len = 1: the reference's descriptors take any row length that way (softmax.h:72, layernorm.h:215);
        // 197 columns put every row but the first off a 16-byte boundary
        constexpr int R = 6, C = 197;
        Tensor in(R * C * 4), out(R * C * 4), mean(R * 4), rstd(R * 4);
        for (int i = 0; i < R * C; ++i) in.host_ref<float>()[i] = (i % C == i / C) ? 3.0f : 3.0f - 100.0f;
        in.host_to_device();
        softmax<SoftMaxBlockImpl<float, 1, R, C>>(R, 128, SoftMaxBlockImpl<float, 1, R, C>::smem_in_bytes, stream,
                                                  in.device_ref<float>(), out.device_ref<float>());
        checkKoErrors(ko_stream_synchronize(stream));
        out.device_to_host();
        for (int i = 0; i < R * C; ++i)  // exp(-100) is below half an ulp of 1: the row's own column gets all of it
            REQUIRE(std::fabs(out.host_ref<float>()[i] - ((i % C == i / C) ? 1.0f : 3.72e-44f)) < 1e-6f);
        for (int i = 0; i < R * C; ++i) in.host_ref<float>()[i] = float(i % C);
        in.host_to_device();
        layer_normalization<LayerNormBlockImpl<float, 1, R, C, false>>(R, 128, 0, stream, in.device_ref<float>(),
                                                                        out.device_ref<float>(), 0.0f, nullptr, nullptr,
                                                                        mean.device_ref<float>(), rstd.device_ref<float>());
        checkKoErrors(ko_stream_synchronize(stream));
        mean.device_to_host();
        rstd.device_to_host();
        REQUIRE(std::fabs(mean.host_ref<float>()[5] - 98.0f) < 1e-3f);
        REQUIRE(std::fabs(rstd.host_ref<float>()[4] - 1.0 / std::sqrt((197.0 * 197.0 - 1) / 12)) < 1e-7);
    }
    {
        constexpr int N = 128;
        Tensor A(N * N * 4), B(N * N * 4), C(N * N * 4), D(N * N * 4);
        for (int i = 0; i < N * N; ++i) {
            A.host_ref<float>()[i] = float(i / 64);
            B.host_ref<float>()[i] = (i / N == i % N) ? 1.0f : 0.0f;
            C.host_ref<float>()[i] = 0.5f;
        }
        A.host_to_device();
        B.host_to_device();
        C.host_to_device();
        using K = GemmKernelSimt<float, float, float, shape::GemmShape<64, 64, 8>, shape::GemmShape<32, 32, 8>, 4, 4, 4>;
        gemm<K>(4, K::thread_per_block, K::smem_total_size_in_bytes, stream, {N, N, N}, A.device_ref<float>(),
                B.device_ref<float>(), C.device_ref<float>(), D.device_ref<float>());
        checkKoErrors(ko_stream_synchronize(stream));
        D.device_to_host();
        for (int i = 0; i < N * N; ++i) REQUIRE(D.host_ref<float>()[i] == float(i / 64) + 0.5f);  // D = A*I + C
        gemm<K>(4, K::thread_per_block, K::smem_total_size_in_bytes, stream, {N, N, N}, A.device_ref<float>(),
                B.device_ref<float>(), nullptr, D.device_ref<float>());
        checkKoErrors(ko_stream_synchronize(stream));
        D.device_to_host();
        for (int i = 0; i < N * N; ++i) REQUIRE(D.host_ref<float>()[i] == float(i / 64));  // C null: D = A*I

        Tensor Ah(N * N * 2), Bh(N * N * 2), Dh(N * N * 2);
        for (int i = 0; i < N * N; ++i) {
            Ah.host_ref<half>()[i] = half(i / 64);
            Bh.host_ref<half>()[i] = half((i / N == i % N) ? 1 : 0);
        }
        Ah.host_to_device();
        Bh.host_to_device();
        using KT = GemmKernelTensorCore<half, half, half, shape::GemmShape<128, 128, 32>, shape::GemmShape<64, 64, 32>,
                                        shape::GemmShape<16, 8, 8>, 8, 8, 8>;
        gemm<KT>(1, KT::thread_per_block, KT::smem_total_size_in_bytes, stream, {N, N, N}, Ah.device_ref<half>(),
                 Bh.device_ref<half>(), nullptr, Dh.device_ref<half>());
        checkKoErrors(ko_stream_synchronize(stream));
        Dh.device_to_host();
        for (int i = 0; i < N * N; ++i) REQUIRE(float(Dh.host_ref<half>()[i]) == float(i / 64));
    }
    checkKoErrors(ko_stream_destroy(stream));
    return 0;
}

int main(int argc, char **argv) {
    const char *dump = nullptr;
    bool gpu = false;
    for (int i = 1; i < argc; ++i) {
        if (!std::strcmp(argv[i], "gpu")) gpu = true;
        else dump = argv[i];
    }
    if (int rc = cpu_part(dump)) return rc;
    if (gpu)
        if (int rc = gpu_part()) return rc;
    printf("host selftest ok%s\n", gpu ? " (with gpu)" : "");
    return 0;
}
