// Seeded host-side input generator for the benchmark drivers.  The reference fills its
// tensors from a default-seeded std::default_random_engine + std::normal_distribution
// (nn_operators/softmax/main.cu:31-36), which differs between standard libraries; this
// generator is counter based, so element i of a tensor depends only on (seed, i) and the
// device fills of the C ABI (ko_fill_*) produce the same values.
#ifndef KERNEL_OPTIMIZATION_RANDOM_H
#define KERNEL_OPTIMIZATION_RANDOM_H

#include <cmath>
#include <cstdint>

namespace ko_random {

inline uint64_t splitmix64(uint64_t seed, uint64_t ctr) {
    uint64_t z = seed + (ctr + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline double unit(uint64_t seed, uint64_t ctr) { return static_cast<double>(splitmix64(seed, ctr) >> 11) * 0x1.0p-53; }

inline double uniform(uint64_t seed, uint64_t i, double lo, double hi) { return lo + (hi - lo) * unit(seed, i); }

inline double normal(uint64_t seed, uint64_t i, double mean, double std) {
    const double u1 = unit(seed, 2 * i), u2 = unit(seed, 2 * i + 1);
    return mean + std * (std::sqrt(-2.0 * std::log(1.0 - u1)) * std::cos(2.0 * 3.14159265358979323846 * u2));
}

inline uint64_t tensor_seed(int cfg, int tensor_index) { return 20220513ull * 1000ull + 10ull * cfg + tensor_index; }

}  // namespace ko_random

#endif  // KERNEL_OPTIMIZATION_RANDOM_H
