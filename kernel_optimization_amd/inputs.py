"""Seeded, portable input generators (host side, numpy).

The reference fills its buffers from a default-seeded
``std::default_random_engine`` + ``std::normal_distribution``
(nn_operators/softmax/main.cu:31-36, nn_operators/gemm/main.cu:46-66), which is
standard-library specific and so cannot give identical inputs on two machines.
These generators are counter based and element addressable instead, so the
host (this module) and the device fill kernels (``ko_fill_*`` in the C ABI)
produce the same tensors from the same seed:

    z = seed + (ctr + 1) * 0x9E3779B97F4A7C15          (splitmix64)
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9
    z = (z ^ (z >> 27)) * 0x94D049BB133111EB
    z =  z ^ (z >> 31)
    u = (z >> 11) * 2**-53                              in [0, 1)

    uniform(a, b)[i] = a + (b - a) * u(i)
    normal(mu, s)[i] = mu + s * sqrt(-2 ln(1 - u(2i))) * cos(2 pi u(2i + 1))

evaluated in double and rounded once to the storage type.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)

BASE_SEED = 20220513 * 1000
MASK_VALUE = -10000.0


def tensor_seed(cfg, tensor_index):
    """One seed per tensor of a benchmark configuration (cfg is 1-based)."""
    return BASE_SEED + 10 * int(cfg) + int(tensor_index)


def splitmix64(seed, ctr):
    """ctr: uint64 array of counters -> uint64 array of outputs."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (np.asarray(ctr, dtype=np.uint64) + np.uint64(1)) * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        z = z ^ (z >> np.uint64(31))
    return z


def unit_double(seed, ctr):
    return (splitmix64(seed, ctr) >> np.uint64(11)).astype(np.float64) * 2.0 ** -53


def uniform_f64(n, seed, lo, hi, start=0):
    ctr = np.arange(start, start + n, dtype=np.uint64)
    return lo + (hi - lo) * unit_double(seed, ctr)


def normal_f64(n, seed, mean, std, start=0):
    i = np.arange(start, start + n, dtype=np.uint64)
    u1 = unit_double(seed, np.uint64(2) * i)
    u2 = unit_double(seed, np.uint64(2) * i + np.uint64(1))
    r = np.sqrt(-2.0 * np.log(1.0 - u1))
    return mean + std * (r * np.cos(2.0 * np.pi * u2))


def uniform_f32(shape, seed, lo=-1.0, hi=1.0):
    n = int(np.prod(shape))
    return uniform_f64(n, seed, lo, hi).astype(np.float32).reshape(shape)


def normal_f32(shape, seed, mean=0.0, std=1.0):
    n = int(np.prod(shape))
    return normal_f64(n, seed, mean, std).astype(np.float32).reshape(shape)


def uniform_f16(shape, seed, lo=-1.0, hi=1.0):
    """float16 array; the double is rounded once to binary16 (numpy rounds to nearest even)."""
    n = int(np.prod(shape))
    return uniform_f64(n, seed, lo, hi).astype(np.float16).reshape(shape)


def f32_to_bf16_bits(x):
    """float32 -> bfloat16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    rounded = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return (rounded >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_f32(bits):
    return (np.ascontiguousarray(bits, np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def uniform_bf16_bits(shape, seed, lo=-1.0, hi=1.0):
    """bfloat16 bit patterns: double -> float32 -> bfloat16 (both nearest even)."""
    return f32_to_bf16_bits(uniform_f32(shape, seed, lo, hi)).reshape(shape)


def valid_lengths(n_seq, seed, lo=64, hi=512):
    """int32 lengths lo + floor((hi - lo + 1) * u), i.e. uniform on [lo, hi]."""
    u = unit_double(seed, np.arange(n_seq, dtype=np.uint64))
    return (lo + np.floor((hi - lo + 1) * u)).astype(np.int32)


# ---------------------------------------------------------------------------
# The five benchmark configurations
# ---------------------------------------------------------------------------

CONFIGS = {
    1: dict(name="softmax_f32_196608x128", op="softmax", rows=196608, cols=128),
    2: dict(name="layernorm_f32_16384x768", op="layernorm", rows=16384, cols=768, eps=1e-5),
    3: dict(name="sgemm_f32_1024x1024x1024", op="sgemm", m=1024, n=1024, k=1024),
    4: dict(name="gemm_f16_16384x3072x768", op="gemm16", m=16384, n=3072, k=768),
    5: dict(name="masked_softmax_f32_786432x512", op="softmax", rows=786432, cols=512,
            n_seq=128, rows_per_seq=6144, len_lo=64, len_hi=512),
}


def algorithmic_work(cfg):
    """Bytes (softmax/LayerNorm) or flops (GEMM) one launch is credited with."""
    c = CONFIGS[cfg]
    if c["op"] == "softmax":
        return 2 * c["rows"] * c["cols"] * 4
    if c["op"] == "layernorm":
        return 2 * c["rows"] * c["cols"] * 4 + 2 * c["cols"] * 4 + 2 * c["rows"] * 4
    return 2 * c["m"] * c["n"] * c["k"]


def make_inputs(cfg, rows=None):
    """Host inputs of a configuration, optionally cut to the first `rows` rows (M for GEMMs)."""
    c = CONFIGS[cfg]
    if c["op"] == "softmax":
        r = c["rows"] if rows is None else rows
        out = dict(x=normal_f32((r, c["cols"]), tensor_seed(cfg, 0), 0.0, 4.0))
        if "n_seq" in c:
            out["valid_len"] = valid_lengths(c["n_seq"], tensor_seed(cfg, 1), c["len_lo"], c["len_hi"])
            out["rows_per_seq"] = c["rows_per_seq"]
        return out
    if c["op"] == "layernorm":
        r = c["rows"] if rows is None else rows
        return dict(x=normal_f32((r, c["cols"]), tensor_seed(cfg, 0), 0.5, 2.0),
                    gamma=normal_f32((c["cols"],), tensor_seed(cfg, 1), 1.0, 0.1),
                    beta=normal_f32((c["cols"],), tensor_seed(cfg, 2), 0.0, 0.1),
                    eps=c["eps"])
    if c["op"] == "sgemm":
        m = c["m"] if rows is None else rows
        return dict(A=uniform_f32((m, c["k"]), tensor_seed(cfg, 0)),
                    B=uniform_f32((c["k"], c["n"]), tensor_seed(cfg, 1)))
    m = c["m"] if rows is None else rows
    return dict(A=uniform_f16((m, c["k"]), tensor_seed(cfg, 0)),
                B=uniform_f16((c["n"], c["k"]), tensor_seed(cfg, 1)))  # column-major B: memory [N][K]
