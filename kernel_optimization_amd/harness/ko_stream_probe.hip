// Streaming-rate probe of the measurement harness: write-only, read-only, copy and partial-read copy kernels
// over a buffer pair, with the launch shape and the cache-policy bits of the accesses as arguments.  It exists
// to establish, on the device at hand, what a read stream, a write stream and a read+write stream reach at
// best, so that the bandwidth-bound operators (row softmax, LayerNorm) are judged against a measured ceiling
// and not only against the data-sheet peak.  It has no counterpart in the reference, whose benchmark drivers
// report one effective bandwidth per operator (nn_operators/softmax/main.cu:70-73).
#include "ko_internal.h"
#include "wave64.h"

namespace ko {
namespace {

enum { LOAD_PLAIN = 0, LOAD_NT = 1 };
enum { STORE_PLAIN = 0, STORE_NT = 1, STORE_SC1 = 2, STORE_SC1_NT = 3, STORE_SC0_SC1_NT = 4 };
enum { MODE_WRITE = 0, MODE_READ = 1, MODE_COPY = 2, MODE_PARTIAL = 3 };

template <int LP>
__device__ __forceinline__ float4v probe_load(const float4v *p) {
    if constexpr (LP == LOAD_NT) return __builtin_nontemporal_load(p);
    return *p;
}

// The cache-policy bits of a store have no spelling in the language beyond `nt`; the others are inline
// assembly, each followed by the two wait states a store of more than 64 bits needs before its data registers
// may be overwritten.
template <int SP>
__device__ __forceinline__ void probe_store(float4v *p, float4v v) {
    if constexpr (SP == STORE_PLAIN) *p = v;
    if constexpr (SP == STORE_NT) __builtin_nontemporal_store(v, p);
    if constexpr (SP == STORE_SC1) asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
    if constexpr (SP == STORE_SC1_NT)
        asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
    if constexpr (SP == STORE_SC0_SC1_NT)
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}

// A workgroup of T threads handles chunks of T * VPT vectors (thread t: vectors t, t + T, ...), chunk index =
// workgroup index, stride = grid size.  MODE_PARTIAL reads only the vectors whose index modulo 128 is below
// `read_of_128` (the shape of a 512-column fp32 row whose tail is padding) and writes all of them.
template <int MODE, int VPT, int LP, int SP>
__global__ __launch_bounds__(1024) void stream_probe_kernel(const float4v *__restrict__ in, float4v *__restrict__ out,
                                                            int64_t nchunks, int read_of_128, float *sink) {
    extern __shared__ float residency_pad[];  // never touched: its size caps the resident workgroups per CU
    const int T = blockDim.x;
    float4v acc = {0.f, 0.f, 0.f, 0.f};
    for (int64_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
        const int64_t base = c * static_cast<int64_t>(T) * VPT + threadIdx.x;
        float4v v[VPT];
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            const int64_t i = base + static_cast<int64_t>(j) * T;
            v[j] = float4v{1.f, 2.f, 3.f, static_cast<float>(j)};
            if (MODE == MODE_READ || MODE == MODE_COPY) v[j] = probe_load<LP>(in + i);
            if (MODE == MODE_PARTIAL && static_cast<int>(i & 127) < read_of_128) v[j] = probe_load<LP>(in + i);
        }
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            if (MODE == MODE_READ) acc += v[j];
            else probe_store<SP>(out + base + static_cast<int64_t>(j) * T, v[j]);
        }
    }
    if (MODE == MODE_READ && acc.x == 12345.f && sink) sink[0] = acc.y;  // keeps the loads alive
}

template <int MODE, int VPT, int LP>
int launch_sp(int sp, dim3 grid, dim3 block, int lds, hipStream_t s, const float4v *in, float4v *out, int64_t nchunks,
              int read_of_128) {
#define KO_PROBE(SP)                                                                                          \
    case SP: {                                                                                                \
        static std::atomic<uint64_t> done{0};                                                                 \
        if (lds > 48 * 1024) {                                                                                \
            const int rc = allow_dynamic_lds(reinterpret_cast<const void *>(stream_probe_kernel<MODE, VPT, LP, SP>), \
                                             160 * 1024, done);                                               \
            if (rc != KO_OK) return rc;                                                                       \
        }                                                                                                     \
        stream_probe_kernel<MODE, VPT, LP, SP><<<grid, block, lds, s>>>(in, out, nchunks, read_of_128, nullptr); \
        break;                                                                                                \
    }
    switch (sp) {
        KO_PROBE(STORE_PLAIN)
        KO_PROBE(STORE_NT)
        KO_PROBE(STORE_SC1)
        KO_PROBE(STORE_SC1_NT)
        KO_PROBE(STORE_SC0_SC1_NT)
        default: return fail(KO_ERR_INVALID_ARGUMENT, "stream_probe: store_policy=%d", sp);
    }
#undef KO_PROBE
    KO_CHECK_LAUNCH();
    return KO_OK;
}

template <int MODE, int VPT>
int launch_lp(int lp, int sp, dim3 grid, dim3 block, int lds, hipStream_t s, const float4v *in, float4v *out,
              int64_t nchunks, int read_of_128) {
    if (MODE == MODE_WRITE || lp == LOAD_PLAIN)
        return launch_sp<MODE, VPT, LOAD_PLAIN>(MODE == MODE_READ ? STORE_PLAIN : sp, grid, block, lds, s, in, out,
                                                nchunks, read_of_128);
    if (lp == LOAD_NT)
        return launch_sp<MODE, VPT, LOAD_NT>(MODE == MODE_READ ? STORE_PLAIN : sp, grid, block, lds, s, in, out, nchunks,
                                             read_of_128);
    return fail(KO_ERR_INVALID_ARGUMENT, "stream_probe: load_policy=%d", lp);
}

template <int MODE>
int launch_vpt(int vpt, int lp, int sp, dim3 grid, dim3 block, int lds, hipStream_t s, const float4v *in, float4v *out,
               int64_t nchunks, int read_of_128) {
    switch (vpt) {
        case 1: return launch_lp<MODE, 1>(lp, sp, grid, block, lds, s, in, out, nchunks, read_of_128);
        case 2: return launch_lp<MODE, 2>(lp, sp, grid, block, lds, s, in, out, nchunks, read_of_128);
        case 4: return launch_lp<MODE, 4>(lp, sp, grid, block, lds, s, in, out, nchunks, read_of_128);
        default: return fail(KO_ERR_INVALID_ARGUMENT, "stream_probe: vectors_per_thread=%d (1, 2 or 4)", vpt);
    }
}

}  // namespace
}  // namespace ko

KO_EXPORT int ko_stream_probe(const void *in, void *out, int64_t nbytes, int mode, int vectors_per_thread,
                              int threads, int blocks_per_cu, int load_policy, int store_policy,
                              int read_of_128, int lds_pad_bytes, ko_stream_t stream) {
    using namespace ko;
    if (nbytes < 0) return fail(KO_ERR_INVALID_ARGUMENT, "stream_probe: negative size");
    if (threads < 64 || threads > 1024 || (threads & 63))
        return fail(KO_ERR_INVALID_ARGUMENT, "stream_probe: threads=%d (a multiple of 64 up to 1024)", threads);
    if (vectors_per_thread != 1 && vectors_per_thread != 2 && vectors_per_thread != 4)
        return fail(KO_ERR_INVALID_ARGUMENT, "stream_probe: vectors_per_thread=%d (1, 2 or 4)", vectors_per_thread);
    const int64_t chunk_bytes = static_cast<int64_t>(threads) * vectors_per_thread * 16;
    if (nbytes % chunk_bytes)
        return fail(KO_ERR_UNSUPPORTED_SHAPE, "stream_probe: %lld bytes are not whole chunks of %lld", (long long)nbytes,
                    (long long)chunk_bytes);
    if (lds_pad_bytes < 0 || lds_pad_bytes > 160 * 1024 || blocks_per_cu < 0 || read_of_128 < 0 || read_of_128 > 128)
        return fail(KO_ERR_INVALID_ARGUMENT, "stream_probe: bad lds_pad_bytes, blocks_per_cu or read_of_128");
    if (nbytes == 0) return KO_OK;
    if ((mode != MODE_WRITE && !in) || (mode != MODE_READ && !out))
        return fail(KO_ERR_INVALID_ARGUMENT, "stream_probe: null pointer");
    if ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15)
        return fail(KO_ERR_INVALID_ARGUMENT, "stream_probe: pointers must be 16-byte aligned");
    const int64_t nchunks = nbytes / chunk_bytes;
    int64_t grid = nchunks;
    if (blocks_per_cu > 0 && grid > static_cast<int64_t>(compute_units()) * blocks_per_cu)
        grid = static_cast<int64_t>(compute_units()) * blocks_per_cu;
    if (grid > 0x7fffffff) grid = 0x7fffffff;
    const dim3 g(static_cast<unsigned>(grid)), b(static_cast<unsigned>(threads));
    const float4v *src = static_cast<const float4v *>(in);
    float4v *dst = static_cast<float4v *>(out);
    hipStream_t s = as_stream(stream);
    switch (mode) {
        case MODE_WRITE:
            return launch_vpt<MODE_WRITE>(vectors_per_thread, load_policy, store_policy, g, b, lds_pad_bytes, s, src, dst, nchunks, read_of_128);
        case MODE_READ:
            return launch_vpt<MODE_READ>(vectors_per_thread, load_policy, store_policy, g, b, lds_pad_bytes, s, src, dst, nchunks, read_of_128);
        case MODE_COPY:
            return launch_vpt<MODE_COPY>(vectors_per_thread, load_policy, store_policy, g, b, lds_pad_bytes, s, src, dst, nchunks, read_of_128);
        case MODE_PARTIAL:
            return launch_vpt<MODE_PARTIAL>(vectors_per_thread, load_policy, store_policy, g, b, lds_pad_bytes, s, src, dst, nchunks, read_of_128);
        default: return fail(KO_ERR_INVALID_ARGUMENT, "stream_probe: mode=%d", mode);
    }
}
