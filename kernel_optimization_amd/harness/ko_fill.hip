// Seeded device fills and the plain copy kernel of the measurement harness.
//
// The fills replace the host RNG loops of the reference's benchmark drivers
// (nn_operators/softmax/main.cu:31-36, nn_operators/gemm/main.cu:46-66), which
// draw from a default-seeded std::default_random_engine and so are not
// reproducible across standard libraries.  The generator here is counter based
// (splitmix64 of seed and element index), evaluated in double and rounded once
// to the storage type, so host code can produce the same tensor element by
// element.
#include "ko_internal.h"
#include "wave64.h"


namespace ko {
namespace {

__device__ __forceinline__ uint64_t splitmix64(uint64_t seed, uint64_t ctr) {
    uint64_t z = seed + (ctr + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__device__ __forceinline__ double unit_double(uint64_t seed, uint64_t ctr) {
    return static_cast<double>(splitmix64(seed, ctr) >> 11) * 0x1.0p-53;
}

__device__ __forceinline__ double normal_double(uint64_t seed, uint64_t i) {
    const double u1 = unit_double(seed, 2 * i);
    const double u2 = unit_double(seed, 2 * i + 1);
    const double r = sqrt(-2.0 * log(1.0 - u1));
    return r * cos(2.0 * 3.14159265358979323846 * u2);
}

__global__ void fill_normal_f32_kernel(float *out, int64_t n, uint64_t seed, double mean, double std,
                                       int64_t first) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n; i += stride)
        out[i] = static_cast<float>(mean + std * normal_double(seed, static_cast<uint64_t>(first + i)));
}

__global__ void fill_uniform_f32_kernel(float *out, int64_t n, uint64_t seed, double lo, double hi,
                                        int64_t first) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n; i += stride)
        out[i] = static_cast<float>(lo + (hi - lo) * unit_double(seed, static_cast<uint64_t>(first + i)));
}

// double -> binary16 with one rounding (nearest even): round to the target's ulp in
// double arithmetic first, so the hardware double->float->half conversions are exact.
__device__ __forceinline__ double round_to_f16_grid(double v) {
    const double a = fabs(v);
    if (a == 0.0 || a >= 65520.0) return v;
    int e = ilogb(a);
    if (e < -14) e = -14;
    const double ulp = ldexp(1.0, e - 10);
    return rint(v / ulp) * ulp;
}

__global__ void fill_uniform_16_kernel(uint16_t *out, int64_t n, uint64_t seed, double lo, double hi,
                                       int64_t first, int dtype) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n; i += stride) {
        const double v = lo + (hi - lo) * unit_double(seed, static_cast<uint64_t>(first + i));
        uint16_t bits;
        if (dtype == KO_F16) {
            const _Float16 h = static_cast<_Float16>(static_cast<float>(round_to_f16_grid(v)));
            bits = __builtin_bit_cast(uint16_t, h);
        } else {
            // bfloat16: double -> float (nearest even) -> bfloat16 (nearest even)
            const uint32_t u = __builtin_bit_cast(uint32_t, static_cast<float>(v));
            bits = static_cast<uint16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
        }
        out[i] = bits;
    }
}

__global__ void fill_lengths_kernel(int32_t *out, int64_t n, uint64_t seed, int32_t lo, int32_t hi) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n; i += stride)
        out[i] = static_cast<int32_t>(static_cast<int64_t>(lo) +
                                      static_cast<int64_t>(floor((static_cast<double>(hi) - static_cast<double>(lo) + 1.0) *
                                                                 unit_double(seed, static_cast<uint64_t>(i)))));
}

template <bool NT>
__global__ __launch_bounds__(128) void copy_f32_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                       int64_t nvec, int64_t n) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    // NT: non-temporal loads and streaming (sc1 nt) stores, addressed as the workgroup's uniform chunk base plus
    // 16 bytes per thread
    for (int64_t i0 = blockIdx.x * static_cast<int64_t>(blockDim.x); i0 < nvec; i0 += stride) {
        const int64_t i = i0 + threadIdx.x;
        if (i < nvec) {
            const float4v v = load4<NT>(in + 4 * i);
            if constexpr (NT) stream_store16(out + 4 * i0, threadIdx.x * 16u, v);
            else store4<false>(out + 4 * i, v);
        }
    }
    // tail (n not a multiple of 4)
    const int64_t t = nvec * 4 + blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
    if (t < n) out[t] = in[t];
}

int fill_grid(int64_t n) {
    int64_t blocks = (n + 255) / 256;
    const int64_t cap = static_cast<int64_t>(compute_units()) * 16;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return static_cast<int>(blocks);
}

}  // namespace
}  // namespace ko

KO_EXPORT int ko_fill_normal_f32(float *out, int64_t n, uint64_t seed, double mean, double std,
                                 int64_t first, ko_stream_t stream) {
    if (n < 0 || first < 0) return ko::fail(KO_ERR_INVALID_ARGUMENT, "fill_normal_f32: negative size");
    if (n == 0) return KO_OK;
    if (!out) return ko::fail(KO_ERR_INVALID_ARGUMENT, "fill_normal_f32: null pointer");
    ko::fill_normal_f32_kernel<<<ko::fill_grid(n), 256, 0, ko::as_stream(stream)>>>(out, n, seed, mean, std, first);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

KO_EXPORT int ko_fill_uniform_f32(float *out, int64_t n, uint64_t seed, double lo, double hi,
                                  int64_t first, ko_stream_t stream) {
    if (n < 0 || first < 0) return ko::fail(KO_ERR_INVALID_ARGUMENT, "fill_uniform_f32: negative size");
    if (n == 0) return KO_OK;
    if (!out) return ko::fail(KO_ERR_INVALID_ARGUMENT, "fill_uniform_f32: null pointer");
    ko::fill_uniform_f32_kernel<<<ko::fill_grid(n), 256, 0, ko::as_stream(stream)>>>(out, n, seed, lo, hi, first);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

KO_EXPORT int ko_fill_uniform_16(void *out, int64_t n, uint64_t seed, double lo, double hi,
                                 int64_t first, int dtype, ko_stream_t stream) {
    if (n < 0 || first < 0) return ko::fail(KO_ERR_INVALID_ARGUMENT, "fill_uniform_16: negative size");
    if (dtype != KO_F16 && dtype != KO_BF16)
        return ko::fail(KO_ERR_INVALID_ARGUMENT, "fill_uniform_16: dtype=%d", dtype);
    if (n == 0) return KO_OK;
    if (!out) return ko::fail(KO_ERR_INVALID_ARGUMENT, "fill_uniform_16: null pointer");
    ko::fill_uniform_16_kernel<<<ko::fill_grid(n), 256, 0, ko::as_stream(stream)>>>(
        static_cast<uint16_t *>(out), n, seed, lo, hi, first, dtype);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

KO_EXPORT int ko_fill_lengths_i32(int32_t *out, int64_t n, uint64_t seed, int32_t lo, int32_t hi,
                                  ko_stream_t stream) {
    if (n < 0 || hi < lo) return ko::fail(KO_ERR_INVALID_ARGUMENT, "fill_lengths_i32: bad range");
    if (n == 0) return KO_OK;
    if (!out) return ko::fail(KO_ERR_INVALID_ARGUMENT, "fill_lengths_i32: null pointer");
    ko::fill_lengths_kernel<<<ko::fill_grid(n), 256, 0, ko::as_stream(stream)>>>(out, n, seed, lo, hi);
    KO_CHECK_LAUNCH();
    return KO_OK;
}

KO_EXPORT int ko_copy_f32(const float *in, float *out, int64_t n, ko_stream_t stream) {
    if (n < 0) return ko::fail(KO_ERR_INVALID_ARGUMENT, "copy_f32: negative size");
    if (n == 0) return KO_OK;
    if (!in || !out) return ko::fail(KO_ERR_INVALID_ARGUMENT, "copy_f32: null pointer");
    if ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15)
        return ko::fail(KO_ERR_INVALID_ARGUMENT, "copy_f32: pointers must be 16-byte aligned");
    const int64_t nvec = n / 4;
    // 128 threads, one vector per thread, non-temporal loads and sc1 nt stores: the fastest copy of the streaming
    // probe's sweep on MI355X (1 GiB: 6.85 TB/s; 256 threads 6.75, two vectors per thread 6.3)
    const int64_t needed = (nvec + 127) / 128 > 0 ? (nvec + 127) / 128 : 1;
    int64_t grid = needed;  // one vector per thread unless the knob caps the grid
    const int per_cu = ko::tuning(ko::knob_copy_blocks_per_cu);
    if (per_cu > 0 && grid > static_cast<int64_t>(ko::compute_units()) * per_cu)
        grid = static_cast<int64_t>(ko::compute_units()) * per_cu;
    if (grid > 0x7fffffff) grid = 0x7fffffff;
    hipStream_t s = ko::as_stream(stream);
    if (ko::tuning(ko::knob_copy_nontemporal) == 2)
        ko::copy_f32_kernel<false><<<dim3(static_cast<unsigned>(grid)), 128, 0, s>>>(in, out, nvec, n);
    else
        ko::copy_f32_kernel<true><<<dim3(static_cast<unsigned>(grid)), 128, 0, s>>>(in, out, nvec, n);
    KO_CHECK_LAUNCH();
    return KO_OK;
}
