// Host-side counterpart of the reference's common/common.h: the error-check macro,
// the 128-bit vector type and the GEMM shape types, with the same names and members.
// Device-side pieces of that header (WarpReduce, BlockReduce, to_scalar, limits;
// common/common.h:37-65,138-178) live inside libko.so as wave64 primitives and are
// not part of the host interface.
#ifndef KERNEL_OPTIMIZATION_COMMON_H
#define KERNEL_OPTIMIZATION_COMMON_H

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "../../ko.h"

// checkCudaErrors of the reference (common/common.h:16-25): same message layout, same
// exit(EXIT_FAILURE); the code is a ko_status and the detail comes from the library.
inline void ko_check(int result, char const *const func, const char *const file, int const line) {
    if (result) {
        fprintf(stderr, "KO error at %s:%d code=%d(%s) \"%s\" : %s\n", file, line, result, ko_status_name(result),
                func, ko_last_error_string());
        exit(EXIT_FAILURE);
    }
}
#define checkKoErrors(val) ko_check((val), #val, __FILE__, __LINE__)

// 16-bit storage types for the tensor-core path (the reference uses CUDA's `half`).
// Conversions are software, round-to-nearest-even; arithmetic happens on the device.
struct ko_half {
    uint16_t bits;
    ko_half() : bits(0) {}
    ko_half(float f) : bits(from_float(f)) {}
    ko_half(double f) : bits(from_float(static_cast<float>(f))) {}
    ko_half(int i) : bits(from_float(static_cast<float>(i))) {}
    operator float() const { return to_float(bits); }

    static uint16_t from_float(float f) {
        uint32_t u;
        std::memcpy(&u, &f, 4);
        const uint32_t sign = (u >> 16) & 0x8000u;
        u &= 0x7fffffffu;
        if (u > 0x7f800000u) return static_cast<uint16_t>(sign | 0x7e00u);          // NaN
        if (u >= 0x477ff000u) return static_cast<uint16_t>(sign | 0x7c00u);         // rounds to inf
        if (u < 0x33000001u) return static_cast<uint16_t>(sign);                     // rounds to zero
        int e = static_cast<int>(u >> 23) - 127;
        uint32_t m = (u & 0x7fffffu) | 0x800000u;
        int shift = e < -14 ? (13 + (-14 - e)) : 13;                                 // subnormal: shift more
        uint32_t half_m = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_m & 1u))) ++half_m;
        uint32_t out = e < -14 ? half_m : ((static_cast<uint32_t>(e + 15) << 10) + (half_m - 0x400u));
        return static_cast<uint16_t>(sign | out);
    }
    static float to_float(uint16_t h) {
        const uint32_t sign = (h & 0x8000u) << 16;
        uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu, u;
        if (e == 0) {
            if (m == 0) {
                u = sign;
            } else {
                int s = 0;
                while (!(m & 0x400u)) { m <<= 1; ++s; }
                u = sign | (static_cast<uint32_t>(113 - s) << 23) | ((m & 0x3ffu) << 13);
            }
        } else if (e == 31) {
            u = sign | 0x7f800000u | (m << 13);
        } else {
            u = sign | ((e + 112) << 23) | (m << 13);
        }
        float f;
        std::memcpy(&f, &u, 4);
        return f;
    }
};

struct ko_bfloat16 {
    uint16_t bits;
    ko_bfloat16() : bits(0) {}
    ko_bfloat16(float f) {
        uint32_t u;
        std::memcpy(&u, &f, 4);
        if ((u & 0x7fffffffu) > 0x7f800000u) bits = static_cast<uint16_t>((u >> 16) | 0x40u);
        else bits = static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
    }
    operator float() const {
        uint32_t u = static_cast<uint32_t>(bits) << 16;
        float f;
        std::memcpy(&f, &u, 4);
        return f;
    }
};

#ifndef KO_NO_GLOBAL_HALF
using half = ko_half;  // the reference's drivers spell the type `half`
#endif

// common/common.h:67-130: N elements of T aligned for one 128-bit access.
template <typename T, int N>
struct alignas(sizeof(T) * N) AlignedArray {
    using Element = T;
    static const int kElements = N;

    AlignedArray() {}
    AlignedArray(const T &rhs) {
        for (int idx = 0; idx < kElements; ++idx) this->at(idx) = rhs;
    }
    T &operator[](int offset) { return this->buffer[offset]; }
    const T &operator[](int offset) const { return this->buffer[offset]; }
    T &at(int offset) { return this->buffer[offset]; }
    const T &at(int offset) const { return this->buffer[offset]; }
    void clear() {
        for (int idx = 0; idx < kElements; ++idx) this->at(idx) = Element(0);
    }

    Element buffer[N];
};

// common/common.h:180-231
namespace shape {
class GemmCoord {
public:
    GemmCoord(size_t _m, size_t _n, size_t _k) : _m(_m), _n(_n), _k(_k) {}

    size_t m() const { return this->_m; }
    size_t n() const { return this->_n; }
    size_t k() const { return this->_k; }
    size_t mk() const { return this->_m * this->_k; }
    size_t kn() const { return this->_k * this->_n; }
    size_t mn() const { return this->_m * this->_n; }
    size_t mnk() const { return this->_m * this->_n * this->_k; }

    std::string to_string() const {
        return std::string("{") + std::to_string(this->m()) + "," + std::to_string(this->n()) + "," +
               std::to_string(this->k()) + "}";
    }

private:
    size_t _m, _n, _k;
};

template <int _M, int _N>
struct MatrixShape {
    static const int kM = _M;
    static const int kN = _N;
};

template <int _M, int _N, int _K>
struct GemmShape {
    static const int kM = _M;
    static const int kN = _N;
    static const int kK = _K;

    static const int kMN = kM * kN;
    static const int kMK = kM * kK;
    static const int kKN = kK * kN;

    static const int kMNK = kM * kN * kK;

    static std::string to_string() {
        return std::string("{") + std::to_string(kM) + "," + std::to_string(kN) + "," + std::to_string(kK) + "}";
    }
};
}  // namespace shape

// Launch geometry as the reference passes it in <<<grid, block, smem, stream>>>.  The
// values the reference uses are tuned for a 40-SM T4 (e.g. 40*8 blocks of 128 threads,
// nn_operators/softmax/main.cu:77); on gfx950 the library sizes its own grid for 256
// CUs and 64-lane wavefronts, so these are accepted and ignored.
struct LaunchHint {
    int grid_dim;
    int block_dim;
    int smem_in_bytes;
};

#endif  // KERNEL_OPTIMIZATION_COMMON_H
