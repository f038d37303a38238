"""kernel_optimization_amd - MI355X (gfx950) row softmax, LayerNorm and GEMM kernels
behind a C ABI (include/ko.h), with a thin ctypes front end.

The compute path is libko.so (hand-written HIP).  There is no CPU fallback: if the
library has not been built, or no GPU is visible, calls raise.
"""
import ctypes
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libko.so")
HARNESS_PATH = os.path.join(_PKG, "lib", "libko_harness.so")

KO_OK = 0
KO_ERR_INVALID_ARGUMENT = 1
KO_ERR_UNSUPPORTED_SHAPE = 2
KO_ERR_RUNTIME = 3
KO_ERR_OUT_OF_MEMORY = 4
KO_ERR_NO_DEVICE = 5

POLICY_AUTO, POLICY_WARP, POLICY_BLOCK, POLICY_BLOCK_NOCACHE = 0, 1, 2, 3
F16, BF16 = 0, 1
ACT_NONE, ACT_GELU_ERF, ACT_GELU_TANH = 0, 1, 2
ROW_MAJOR, COL_MAJOR = 0, 1

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_u64 = ctypes.c_uint64
_int = ctypes.c_int
_f = ctypes.c_float
_d = ctypes.c_double
_sz = ctypes.c_size_t


class DeviceInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 256), ("arch", ctypes.c_char * 64),
                ("compute_units", _int), ("wavefront_size", _int), ("clock_khz", _int),
                ("memory_clock_khz", _int), ("memory_bus_bits", _int), ("l2_bytes", _int),
                ("lds_bytes_per_workgroup", _int), ("hbm_bytes", _sz)]


# name -> (restype, argtypes); every symbol include/ko.h declares
SIGNATURES = {
    "ko_last_error_string": (ctypes.c_char_p, []),
    "ko_status_name": (ctypes.c_char_p, [_int]),
    "ko_device_info": (_int, [ctypes.POINTER(DeviceInfo)]),
    "ko_malloc": (_int, [ctypes.POINTER(_vp), _sz]),
    "ko_free": (_int, [_vp]),
    "ko_memset_async": (_int, [_vp, _int, _sz, _vp]),
    "ko_memcpy_h2d": (_int, [_vp, _vp, _sz]),
    "ko_memcpy_h2d_async": (_int, [_vp, _vp, _sz, _vp]),
    "ko_memcpy_d2h": (_int, [_vp, _vp, _sz]),
    "ko_memcpy_d2h_async": (_int, [_vp, _vp, _sz, _vp]),
    "ko_memcpy_d2d_async": (_int, [_vp, _vp, _sz, _vp]),
    "ko_stream_create": (_int, [ctypes.POINTER(_vp)]),
    "ko_stream_destroy": (_int, [_vp]),
    "ko_stream_synchronize": (_int, [_vp]),
    "ko_device_synchronize": (_int, []),
    "ko_event_create": (_int, [ctypes.POINTER(_vp)]),
    "ko_event_record": (_int, [_vp, _vp]),
    "ko_event_synchronize": (_int, [_vp]),
    "ko_event_elapsed_ms": (_int, [ctypes.POINTER(_f), _vp, _vp]),
    "ko_event_destroy": (_int, [_vp]),
    "ko_softmax_f32": (_int, [_vp, _vp, _i64, _i64, _vp, _i64, _vp]),
    "ko_softmax_f32_policy": (_int, [_vp, _vp, _i64, _i64, _vp, _i64, _int, _vp]),
    "ko_layernorm_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f, _int, _vp]),
    "ko_layernorm_f32_policy": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f, _int, _int, _vp]),
    "ko_softmax_16": (_int, [_vp, _vp, _i64, _i64, _vp, _i64, _int, _int, _vp]),
    "ko_layernorm_16": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f, _int, _int, _int, _vp]),
    "ko_sgemm_f32": (_int, [_i64, _i64, _i64, _f, _vp, _vp, _f, _vp, _vp, _vp]),
    "ko_sgemm_f32_static_scratch": (_int, [_i64, _i64, _i64, _f, _vp, _vp, _f, _vp, _vp, _vp]),
    "ko_gemm_f16f32acc": (_int, [_i64, _i64, _i64, _f, _vp, _vp, _int, _f, _vp, _vp, _int, _vp]),
    "ko_gemm_f16f32acc_bias_act": (_int, [_i64, _i64, _i64, _f, _vp, _vp, _int, _f, _vp, _vp, _int, _vp, _int, _vp]),
}

# every symbol of libko_harness.so that include/ko_harness.h declares (tests and benchmark only)
HARNESS_SIGNATURES = {
    "ko_fill_normal_f32": (_int, [_vp, _i64, _u64, _d, _d, _i64, _vp]),
    "ko_fill_uniform_f32": (_int, [_vp, _i64, _u64, _d, _d, _i64, _vp]),
    "ko_fill_uniform_16": (_int, [_vp, _i64, _u64, _d, _d, _i64, _int, _vp]),
    "ko_fill_lengths_i32": (_int, [_vp, _i64, _u64, ctypes.c_int32, ctypes.c_int32, _vp]),
    "ko_copy_f32": (_int, [_vp, _vp, _i64, _vp]),
    "ko_stream_probe": (_int, [_vp, _vp, _i64, _int, _int, _int, _int, _int, _int, _int, _int, _vp]),
    "ko_set_tuning": (_int, [ctypes.c_char_p, _int]),
    "ko_get_tuning": (_int, [ctypes.c_char_p, ctypes.POINTER(_int)]),
    "ko_debug_wave_allreduce": (_int, [_vp, _vp, _int, _int, _vp]),
    "ko_debug_stream_workspace_count": (_int, [ctypes.POINTER(_int)]),
    "ko_time_gemm16_sets": (_int, [_i64, _i64, _i64, ctypes.POINTER(_vp), ctypes.POINTER(_vp), ctypes.POINTER(_vp), _int,
                                   _int, _int, _int, _int, _int, ctypes.POINTER(ctypes.c_float)]),
    "ko_debug_sgemm_plan": (_int, [_i64, _i64, _i64, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                                   ctypes.POINTER(ctypes.c_int)]),
    "ko_debug_gemm16_plan": (_int, [_i64, _i64, _i64, _int, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                                    ctypes.POINTER(ctypes.c_int)]),
}

_lib = None
_harness = None


class KoError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("%s (status %d): %s" % (status_name(status), status, message))
        self.status = status


def lib():
    """Loads libko.so (built in-tree by kernel_optimization_amd.build).  Raises if it is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libko.so is not built: run `python -m kernel_optimization_amd.build` "
                               "(expected %s).  There is no CPU fallback." % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def harness():
    """Loads libko_harness.so (fills, probes, tuning knobs, debug views): what tests and the benchmark use beside
    the operator library.  Raises if it is missing."""
    global _harness
    if _harness is None:
        lib()
        if not os.path.exists(HARNESS_PATH):
            raise RuntimeError("libko_harness.so is not built: run `python -m kernel_optimization_amd.build` "
                               "(expected %s)." % HARNESS_PATH)
        H = ctypes.CDLL(HARNESS_PATH)
        for name, (res, args) in HARNESS_SIGNATURES.items():
            fn = getattr(H, name)
            fn.restype = res
            fn.argtypes = args
        _harness = H
    return _harness


def status_name(status):
    return lib().ko_status_name(int(status)).decode()


def last_error():
    return lib().ko_last_error_string().decode()


def check(status):
    if status != KO_OK:
        raise KoError(status, last_error())


def device_info():
    info = DeviceInfo()
    check(lib().ko_device_info(ctypes.byref(info)))
    return {k: (getattr(info, k).decode() if isinstance(getattr(info, k), bytes) else getattr(info, k))
            for k, _ in DeviceInfo._fields_}


def device_available():
    info = DeviceInfo()
    return lib().ko_device_info(ctypes.byref(info)) == KO_OK


def set_tuning(name, value):
    check(harness().ko_set_tuning(name.encode(), int(value)))


def get_tuning(name):
    v = _int(0)
    check(harness().ko_get_tuning(name.encode(), ctypes.byref(v)))
    return v.value


def synchronize():
    check(lib().ko_device_synchronize())


class Stream:
    def __init__(self):
        h = _vp()
        check(lib().ko_stream_create(ctypes.byref(h)))
        self.handle = h

    def synchronize(self):
        check(lib().ko_stream_synchronize(self.handle))

    def close(self):
        if self.handle is not None:
            lib().ko_stream_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Event:
    def __init__(self):
        h = _vp()
        check(lib().ko_event_create(ctypes.byref(h)))
        self.handle = h

    def record(self, stream=None):
        check(lib().ko_event_record(self.handle, _h(stream)))

    def synchronize(self):
        check(lib().ko_event_synchronize(self.handle))

    def elapsed_ms(self, stop):
        ms = _f(0)
        check(lib().ko_event_elapsed_ms(ctypes.byref(ms), self.handle, stop.handle))
        return ms.value

    def __del__(self):
        try:
            if self.handle is not None:
                lib().ko_event_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


def _h(stream):
    if stream is None:
        return None
    if isinstance(stream, Stream):
        return stream.handle
    return _vp(int(stream))  # raw hipStream_t value, e.g. torch.cuda.current_stream().cuda_stream


class DeviceBuffer:
    """Device allocation owned by Python (ko_malloc / ko_free)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = _vp()
        check(lib().ko_malloc(ctypes.byref(p), self.nbytes))
        self.ptr = p.value or 0

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        buf.upload(a)
        return buf

    def upload(self, a):
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.nbytes
        check(lib().ko_memcpy_h2d(self.ptr, a.ctypes.data, a.nbytes))

    def download(self, dtype, shape, offset_bytes=0):
        out = np.empty(shape, dtype=dtype)
        assert offset_bytes + out.nbytes <= self.nbytes
        check(lib().ko_memcpy_d2h(out.ctypes.data, self.ptr + offset_bytes, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            lib().ko_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _p(x):
    """DeviceBuffer | int address | None -> pointer argument."""
    if x is None:
        return None
    if isinstance(x, DeviceBuffer):
        return x.ptr
    return int(x)


# ---- operators on device pointers ------------------------------------------------------------

def softmax(inp, out, rows, cols, valid_len=None, rows_per_seq=0, policy=POLICY_AUTO, stream=None):
    check(lib().ko_softmax_f32_policy(_p(inp), _p(out), rows, cols, _p(valid_len), rows_per_seq,
                                      policy, _h(stream)))


def layernorm(inp, out, rows, cols, mean=None, rstd=None, gamma=None, beta=None, eps=1e-5,
              unbiased=False, policy=POLICY_AUTO, stream=None):
    check(lib().ko_layernorm_f32_policy(_p(inp), _p(out), _p(mean), _p(rstd), _p(gamma), _p(beta),
                                        rows, cols, eps, int(bool(unbiased)), policy, _h(stream)))


def softmax16(inp, out, rows, cols, valid_len=None, rows_per_seq=0, dtype=F16, policy=POLICY_AUTO, stream=None):
    check(lib().ko_softmax_16(_p(inp), _p(out), rows, cols, _p(valid_len), rows_per_seq, dtype, policy,
                              _h(stream)))


def layernorm16(inp, out, rows, cols, mean=None, rstd=None, gamma=None, beta=None, eps=1e-5,
                unbiased=False, dtype=F16, policy=POLICY_AUTO, stream=None):
    check(lib().ko_layernorm_16(_p(inp), _p(out), _p(mean), _p(rstd), _p(gamma), _p(beta), rows, cols, eps,
                                int(bool(unbiased)), dtype, policy, _h(stream)))


def sgemm(m, n, k, A, B, D, C=None, alpha=1.0, beta=0.0, stream=None):
    check(lib().ko_sgemm_f32(m, n, k, alpha, _p(A), _p(B), beta, _p(C), _p(D), _h(stream)))


def gemm_plan(m, n, k, sixteen_bit=False, b_layout=COL_MAJOR):
    """(slices, k_slice, tiling) the host-side planner of the SGEMM or the 16-bit GEMM (with B in b_layout) decides
    for a shape; (1, 0, 1000 * rows + columns) is the 16-bit GEMM's one launch whose workgroups own one output tile of
    that size and split K over their waves (32 x 32 to 64 x 64) or walk it through a deep ring of LDS stages (64 x 128
    to 128 x 128)."""
    a, b, c = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    if sixteen_bit:
        check(harness().ko_debug_gemm16_plan(m, n, k, b_layout, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)))
    else:
        check(harness().ko_debug_sgemm_plan(m, n, k, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)))
    return a.value, b.value, c.value


def time_gemm16_sets(m, n, k, As, Bs, Ds, b_layout=COL_MAJOR, dtype=F16, warmup=100, reps=30, batches=3):
    """Microseconds per ko_gemm_f16f32acc launch, timed from a host loop in C (the median of `batches` batches of
    `reps` launches after `warmup` launches), launch i on the operand set i % len(As)."""
    arr = lambda bufs: (ctypes.c_void_p * len(bufs))(*[b.ptr for b in bufs])
    us = ctypes.c_float()
    check(harness().ko_time_gemm16_sets(m, n, k, arr(As), arr(Bs), arr(Ds), len(As), b_layout, dtype, warmup, reps,
                                        batches, ctypes.byref(us)))
    return us.value


def sgemm_static_scratch(m, n, k, A, B, D, C=None, alpha=1.0, beta=0.0, stream=None):
    """ko_sgemm_f32 for callers that cannot allocate: partial products in the library's static device array."""
    check(lib().ko_sgemm_f32_static_scratch(m, n, k, alpha, _p(A), _p(B), beta, _p(C), _p(D), _h(stream)))


def gemm16(m, n, k, A, B, D, C=None, alpha=1.0, beta=0.0, b_layout=COL_MAJOR, dtype=F16,
           stream=None, bias=None, act=ACT_NONE):
    if bias is None and act == ACT_NONE:
        check(lib().ko_gemm_f16f32acc(m, n, k, alpha, _p(A), _p(B), b_layout, beta, _p(C), _p(D),
                                      dtype, _h(stream)))
    else:
        check(lib().ko_gemm_f16f32acc_bias_act(m, n, k, alpha, _p(A), _p(B), b_layout, beta, _p(C), _p(bias), act,
                                               _p(D), dtype, _h(stream)))


def fill_normal_f32(out, n, seed, mean=0.0, std=1.0, first=0, stream=None):
    check(harness().ko_fill_normal_f32(_p(out), n, seed, mean, std, first, _h(stream)))


def fill_uniform_f32(out, n, seed, lo=-1.0, hi=1.0, first=0, stream=None):
    check(harness().ko_fill_uniform_f32(_p(out), n, seed, lo, hi, first, _h(stream)))


def fill_uniform_16(out, n, seed, lo=-1.0, hi=1.0, first=0, dtype=F16, stream=None):
    check(harness().ko_fill_uniform_16(_p(out), n, seed, lo, hi, first, dtype, _h(stream)))


def fill_lengths_i32(out, n, seed, lo, hi, stream=None):
    check(harness().ko_fill_lengths_i32(_p(out), n, seed, lo, hi, _h(stream)))


def copy_f32(inp, out, n, stream=None):
    check(harness().ko_copy_f32(_p(inp), _p(out), n, _h(stream)))


PROBE_WRITE, PROBE_READ, PROBE_COPY, PROBE_PARTIAL = 0, 1, 2, 3
LOAD_POLICIES = {"plain": 0, "nt": 1}
STORE_POLICIES = {"plain": 0, "nt": 1, "sc1": 2, "sc1 nt": 3, "sc0 sc1 nt": 4}


def stream_probe(inp, out, nbytes, mode, vectors_per_thread=1, threads=128, blocks_per_cu=0, load_policy=1,
                 store_policy=3, read_of_128=128, lds_pad_bytes=0, stream=None):
    check(harness().ko_stream_probe(_p(inp), _p(out), nbytes, mode, vectors_per_thread, threads, blocks_per_cu,
                                load_policy, store_policy, read_of_128, lds_pad_bytes, _h(stream)))


def memcpy_d2d(dst, src, nbytes, stream=None):
    check(lib().ko_memcpy_d2d_async(_p(dst), _p(src), nbytes, _h(stream)))


def memset(dst, value, nbytes, stream=None):
    check(lib().ko_memset_async(_p(dst), value, nbytes, _h(stream)))


# ---- host-array conveniences (upload, run, download): used by tests and examples --------------

def softmax_host(x, valid_len=None, rows_per_seq=0, policy=POLICY_AUTO, in_place=False):
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    dx = DeviceBuffer.from_numpy(x)
    dy = dx if in_place else DeviceBuffer(x.nbytes)
    dv = None if valid_len is None else DeviceBuffer.from_numpy(np.ascontiguousarray(valid_len, np.int32))
    softmax(dx, dy, rows, cols, dv, rows_per_seq, policy)
    synchronize()
    return dy.download(np.float32, x.shape)


def softmax16_host(x_bits, valid_len=None, rows_per_seq=0, dtype=F16, policy=POLICY_AUTO, in_place=False):
    """x_bits: uint16 bit patterns [rows, cols]; returns uint16 [rows, cols]."""
    x_bits = np.ascontiguousarray(x_bits).view(np.uint16)
    rows, cols = x_bits.shape
    dx = DeviceBuffer.from_numpy(x_bits)
    dy = dx if in_place else DeviceBuffer(x_bits.nbytes)
    dv = None if valid_len is None else DeviceBuffer.from_numpy(np.ascontiguousarray(valid_len, np.int32))
    softmax16(dx, dy, rows, cols, dv, rows_per_seq, dtype, policy)
    synchronize()
    return dy.download(np.uint16, x_bits.shape)


def layernorm16_host(x_bits, gamma_bits=None, beta_bits=None, eps=1e-5, unbiased=False, dtype=F16,
                     policy=POLICY_AUTO, in_place=False):
    """16-bit storage; returns (y uint16 [rows, cols], mean float32 [rows], rstd float32 [rows])."""
    x_bits = np.ascontiguousarray(x_bits).view(np.uint16)
    rows, cols = x_bits.shape
    dx = DeviceBuffer.from_numpy(x_bits)
    dy = dx if in_place else DeviceBuffer(x_bits.nbytes)
    dg = None if gamma_bits is None else DeviceBuffer.from_numpy(np.ascontiguousarray(gamma_bits).view(np.uint16))
    db = None if beta_bits is None else DeviceBuffer.from_numpy(np.ascontiguousarray(beta_bits).view(np.uint16))
    dm, dr = DeviceBuffer(rows * 4), DeviceBuffer(rows * 4)
    layernorm16(dx, dy, rows, cols, dm, dr, dg, db, eps, unbiased, dtype, policy)
    synchronize()
    return dy.download(np.uint16, x_bits.shape), dm.download(np.float32, (rows,)), dr.download(np.float32, (rows,))


def layernorm_host(x, gamma=None, beta=None, eps=1e-5, unbiased=False, policy=POLICY_AUTO,
                   want_stats=True, in_place=False):
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    dx = DeviceBuffer.from_numpy(x)
    dy = dx if in_place else DeviceBuffer(x.nbytes)
    dg = None if gamma is None else DeviceBuffer.from_numpy(np.ascontiguousarray(gamma, np.float32))
    db = None if beta is None else DeviceBuffer.from_numpy(np.ascontiguousarray(beta, np.float32))
    dm = DeviceBuffer(rows * 4) if want_stats else None
    dr = DeviceBuffer(rows * 4) if want_stats else None
    layernorm(dx, dy, rows, cols, dm, dr, dg, db, eps, unbiased, policy)
    synchronize()
    y = dy.download(np.float32, x.shape)
    if not want_stats:
        return y
    return y, dm.download(np.float32, (rows,)), dr.download(np.float32, (rows,))


def sgemm_host(A, B, C=None, alpha=1.0, beta=0.0):
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    m, k = A.shape
    k2, n = B.shape
    assert k == k2
    dA, dB = DeviceBuffer.from_numpy(A), DeviceBuffer.from_numpy(B)
    dC = None if C is None else DeviceBuffer.from_numpy(np.ascontiguousarray(C, np.float32))
    dD = DeviceBuffer(max(m * n * 4, 4))
    sgemm(m, n, k, dA, dB, dD, dC, alpha, beta)
    synchronize()
    return dD.download(np.float32, (m, n))


def gemm16_host(A_bits, B_bits, m, n, k, C_bits=None, alpha=1.0, beta=0.0, b_layout=COL_MAJOR,
                dtype=F16, bias_bits=None, act=ACT_NONE):
    """Operands as uint16 bit patterns (binary16 or bfloat16); returns uint16 [m, n]."""
    A_bits = np.ascontiguousarray(A_bits).view(np.uint16)
    B_bits = np.ascontiguousarray(B_bits).view(np.uint16)
    assert A_bits.size == m * k and B_bits.size == n * k
    dA, dB = DeviceBuffer.from_numpy(A_bits), DeviceBuffer.from_numpy(B_bits)
    dC = None if C_bits is None else DeviceBuffer.from_numpy(np.ascontiguousarray(C_bits).view(np.uint16))
    dbias = None if bias_bits is None else DeviceBuffer.from_numpy(np.ascontiguousarray(bias_bits).view(np.uint16))
    dD = DeviceBuffer(max(m * n * 2, 8))
    gemm16(m, n, k, dA, dB, dD, dC, alpha, beta, b_layout, dtype, bias=dbias, act=act)
    synchronize()
    return dD.download(np.uint16, (m, n))
