#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--all/--no-all]

A step is one launch of the operator over one batch of synthetic, seeded input that is
already resident in HBM.  The headline workload is the masked row softmax
[786432, 512] (3.2 GB of traffic: past the 256 MB Infinity Cache by itself); the other four
configurations are measured as well (rotating buffer sets so that they, too, run out of
HBM rather than out of the cache) and reported under "workloads".

Prints ONE JSON line.  `value` is algorithmic bytes per second over the wall-clock of the K
timed steps; `roofline.achieved` is the same algorithmic bytes over the average launch
duration measured with HIP events on the launch stream.
"""
import argparse
import ctypes
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import kernel_optimization_amd as ko  # noqa: E402
from kernel_optimization_amd import inputs  # noqa: E402

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_PEAK_TFLOPS = {"f32": 157.3, "f16": 2500.0}
WORKLOADS = {c["name"]: k for k, c in inputs.CONFIGS.items()}
HEADLINE = 5


def _traffic_table():
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


def _traffic(name):
    """HBM bytes per launch measured offline with rocprofv3 --pmc (profiles/hbm_traffic.json), or None.  The
    counters cannot be read from inside this process, so the figure is the one of the profiled commit."""
    return _traffic_table().get(name, {}).get("traffic_bytes")


def _roofline(bound, achieved, peak, unit, name, launch_s=None):
    """launch_s: the average launch duration the figure was taken over; with it and a counter-traffic entry the
    HBM bytes that really moved are priced against the HBM peak as well (frac_on_traffic)."""
    roof = dict(bound=bound, achieved=achieved, peak=peak, unit=unit, frac=achieved / peak, traffic=_traffic(name))
    if roof["traffic"] is not None:
        roof["traffic_source"] = "profiles/hbm_traffic.json @ %s (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE)" % \
            _traffic_table().get("_measured_at_commit", "unknown commit")
        if launch_s and bound == "hbm":
            roof["frac_on_traffic"] = roof["traffic"] / launch_s / 1e9 / HBM_PEAK_GBS
    return roof


SECONDARY_MIN_WARMUP = 300


def _time_steps(launch, steps, warmup):
    """warmup untimed launches, then `steps` launches: wall clock bracketed by device syncs, and a
    HIP event pair on the launch stream around the same launches."""
    for i in range(warmup):
        launch(i)
    ko.synchronize()
    e0, e1 = ko.Event(), ko.Event()
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        launch(warmup + i)
    e1.record()
    ko.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) / steps, e0.elapsed_ms(e1) * 1e-3 / steps


def _vendor():
    path = os.path.join(ROOT, "kernel_optimization_amd", "lib", "libko_vendor.so")
    if not os.path.exists(path):
        return None
    V = ctypes.CDLL(path)
    i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
    V.kov_gemm16.argtypes = [i64, i64, i64, vp, vp, ci, vp, ci, ci, ci, ctypes.POINTER(ctypes.c_float),
                             ctypes.POINTER(ci)]
    V.kov_sgemm.argtypes = [i64, i64, i64, vp, vp, vp, ci, ci, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ci)]
    pp = ctypes.POINTER(vp)
    V.kov_gemm16_sets.argtypes = [i64, i64, i64, pp, pp, ci, pp, ci, ci, ci, ci, ctypes.POINTER(ctypes.c_float),
                                  ctypes.POINTER(ci)]
    V.kov_gemm16_bias_gelu_sets.argtypes = [i64, i64, i64, pp, pp, vp, ci, pp, ci, ci, ci, ci,
                                            ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ci)]
    V.kov_sgemm_sets.argtypes = [i64, i64, i64, pp, pp, pp, ci, ci, ci, ctypes.POINTER(ctypes.c_float),
                                 ctypes.POINTER(ci)]
    if hasattr(V, "kov_rocblas_sgemm_sets"):
        V.kov_rocblas_sgemm_sets.argtypes = [i64, i64, i64, pp, pp, pp, ci, ci, ctypes.POINTER(ctypes.c_float)]
    return V


def _ptr_array(buffers):
    return (ctypes.c_void_p * len(buffers))(*[b.ptr for b in buffers])


# ------------------------------------------------------------------------------ workloads

def _copy_floor_us(xs, ys, n_f32, steps, warmup):
    """Times the plain copy kernel over the same buffers (same bytes in, same bytes out, same rotation): what a
    read+write stream of this size reaches on the device, launch ramp included.  Overwrites ys: call it
    before the operator that is being measured."""
    nsets = len(xs)
    _, dev = _time_steps(lambda i: ko.copy_f32(xs[i % nsets], ys[i % nsets], n_f32), steps, warmup)
    return dev * 1e6


def _add_copy_floor(res, floor_us):
    res["copy_same_bytes_us"] = floor_us
    res["vs_copy_same_bytes"] = floor_us / res["kernel_us"]


def _masked_bytes(vl, n_seq, rows_per_seq, rows, cols, elem_bytes):
    """Bytes a masked row softmax has to move: every column written, the valid columns read, the lengths read."""
    lens = np.minimum(vl.download(np.int32, (n_seq,)).astype(np.int64), cols)
    seq_rows = np.minimum(rows_per_seq, rows - rows_per_seq * np.arange(n_seq, dtype=np.int64)).clip(min=0)
    return int(elem_bytes * (rows * cols + (lens * seq_rows).sum()) + 4 * n_seq)


def bench_softmax(cfg, steps, warmup, unmasked=False):
    """Configurations 1 and 5.  unmasked: the shape of the masked configuration without its mask, so that every
    algorithmic byte really moves (with the mask a third of the reads is skipped)."""
    c = dict(inputs.CONFIGS[cfg])
    if unmasked:
        c["name"] = c["name"].replace("masked_", "") + "_unmasked"
        for key in ("n_seq", "rows_per_seq", "len_lo", "len_hi"):
            c.pop(key, None)
    rows, cols = c["rows"], c["cols"]
    n = rows * cols
    work = inputs.algorithmic_work(cfg)
    nsets = max(1, -(-(1 << 30) // work))  # rotate through > 1 GiB of buffers unless one set is that big
    xs = [ko.DeviceBuffer(n * 4) for _ in range(nsets)]
    ys = [ko.DeviceBuffer(n * 4) for _ in range(nsets)]
    for x in xs:
        ko.fill_normal_f32(x, n, inputs.tensor_seed(cfg, 0), 0.0, 4.0)
    vl, rps = None, 0
    if "n_seq" in c:
        vl, rps = ko.DeviceBuffer(c["n_seq"] * 4), c["rows_per_seq"]
        ko.fill_lengths_i32(vl, c["n_seq"], inputs.tensor_seed(cfg, 1), c["len_lo"], c["len_hi"])
    floor_us = _copy_floor_us(xs, ys, n, steps, warmup)
    wall, dev = _time_steps(lambda i: ko.softmax(xs[i % nsets], ys[i % nsets], rows, cols, vl, rps), steps, warmup)
    full = work
    if vl is not None:
        # A padded column takes the value -10000 whatever the tensor holds, so the operator has to read only the
        # valid columns; every column is written.  These are the bytes the roofline figure is taken over: counting
        # the padded reads as well (as 2 R C 4 does) credits the kernel with bytes that nothing has to move, and
        # puts the "fraction of peak" above 1.
        work = _masked_bytes(vl, c["n_seq"], rps, rows, cols, 4)
    res = dict(workload=c["name"], metric="hbm_gbytes_per_s", unit="GB/s", value=work / wall / 1e9,
               ms_per_step=wall * 1e3, dtype="f32", buffer_sets=nsets,
               roofline=_roofline("hbm", work / dev / 1e9, HBM_PEAK_GBS, "GB/s", c["name"], dev),
               algorithmic_bytes=work, kernel_us=dev * 1e6)
    if vl is not None:
        res["bytes_basis"] = "every column written, valid columns read (padded columns need no read)"
        res["roofline"]["frac_counting_padded_reads"] = full / dev / 1e9 / HBM_PEAK_GBS
        res["bytes_counting_padded_reads"] = full
    _add_copy_floor(res, floor_us)
    keep = dict(x=xs[0], y=ys[0], vl=vl, rows=rows, cols=cols, rps=rps, work=work)
    return res, keep


def bench_layernorm(cfg, steps, warmup):
    c = inputs.CONFIGS[cfg]
    rows, cols = c["rows"], c["cols"]
    n = rows * cols
    work = inputs.algorithmic_work(cfg)
    nsets = max(1, -(-(1 << 30) // work))
    xs = [ko.DeviceBuffer(n * 4) for _ in range(nsets)]
    ys = [ko.DeviceBuffer(n * 4) for _ in range(nsets)]
    ms = [ko.DeviceBuffer(rows * 4) for _ in range(nsets)]
    rs = [ko.DeviceBuffer(rows * 4) for _ in range(nsets)]
    g, b = ko.DeviceBuffer(cols * 4), ko.DeviceBuffer(cols * 4)
    for x in xs:
        ko.fill_normal_f32(x, n, inputs.tensor_seed(cfg, 0), 0.5, 2.0)
    ko.fill_normal_f32(g, cols, inputs.tensor_seed(cfg, 1), 1.0, 0.1)
    ko.fill_normal_f32(b, cols, inputs.tensor_seed(cfg, 2), 0.0, 0.1)
    floor_us = _copy_floor_us(xs, ys, n, steps, warmup)
    wall, dev = _time_steps(lambda i: ko.layernorm(xs[i % nsets], ys[i % nsets], rows, cols, ms[i % nsets],
                                                   rs[i % nsets], g, b, c["eps"]), steps, warmup)
    res = dict(workload=c["name"], metric="hbm_gbytes_per_s", unit="GB/s", value=work / wall / 1e9,
               ms_per_step=wall * 1e3, dtype="f32", buffer_sets=nsets,
               roofline=_roofline("hbm", work / dev / 1e9, HBM_PEAK_GBS, "GB/s", c["name"], dev),
               algorithmic_bytes=work, kernel_us=dev * 1e6)
    _add_copy_floor(res, floor_us)
    keep = dict(x=xs[0], y=ys[0], mean=ms[0], rstd=rs[0], g=g, b=b, rows=rows, cols=cols, eps=c["eps"])
    return res, keep


def bench_sgemm(cfg, steps, warmup, vendor, shape=None):
    """Configuration 3, or with shape = (m, n, k) the same operator on a shape that does not fill its tiles."""
    c = inputs.CONFIGS[cfg]
    m, n, k = shape or (c["m"], c["n"], c["k"])
    flops = 2 * m * n * k
    nsets = 32 if shape is None else 2  # 12 MB per set: rotate through 400 MB (192 MB per set at 4000^3)
    wname = c["name"] if shape is None else "sgemm_f32_%dx%dx%d" % (m, n, k)
    As = [ko.DeviceBuffer(m * k * 4) for _ in range(nsets)]
    Bs = [ko.DeviceBuffer(k * n * 4) for _ in range(nsets)]
    Ds = [ko.DeviceBuffer(m * n * 4) for _ in range(nsets)]
    for a, b in zip(As, Bs):
        ko.fill_uniform_f32(a, m * k, inputs.tensor_seed(cfg, 0))
        ko.fill_uniform_f32(b, k * n, inputs.tensor_seed(cfg, 1))
    wall, dev = _time_steps(lambda i: ko.sgemm(m, n, k, As[i % nsets], Bs[i % nsets], Ds[i % nsets]), steps, warmup)
    res = dict(workload=wname, metric="tflops", unit="TFLOP/s", value=flops / wall / 1e12,
               ms_per_step=wall * 1e3, dtype="f32", buffer_sets=nsets,
               roofline=_roofline("mfma", flops / dev / 1e12, MFMA_PEAK_TFLOPS["f32"], "TFLOP/s", wname, dev),
               flops=flops, kernel_us=dev * 1e6)
    if vendor is not None:
        us, na = ctypes.c_float(), ctypes.c_int()
        # the vendor library rotates through the same operand sets (its own output buffers)
        Vs = [ko.DeviceBuffer(m * n * 4) for _ in range(nsets)]
        tmp = Vs[0]
        if vendor.kov_sgemm_sets(m, n, k, _ptr_array(As), _ptr_array(Bs), _ptr_array(Vs), nsets, 16, 2 * nsets,
                                 ctypes.byref(us), ctypes.byref(na)) == 0:
            res["hipblaslt_tflops"] = flops / us.value / 1e6
            res["vs_hipblaslt"] = (flops / dev / 1e12) / res["hipblaslt_tflops"]
            ref = tmp.download(np.float32, (m, n))
            res["max_abs_diff_vs_hipblaslt"] = float(np.abs(Ds[0].download(np.float32, (m, n)) - ref).max())
        # rocblas_sgemm: the call-for-call counterpart of the reference's cublasSgemm check (gemm/main.cu:146-150)
        if hasattr(vendor, "kov_rocblas_sgemm_sets") and vendor.kov_rocblas_sgemm_sets(
                m, n, k, _ptr_array(As), _ptr_array(Bs), _ptr_array(Vs), nsets, 2 * nsets, ctypes.byref(us)) == 0:
            res["rocblas_tflops"] = flops / us.value / 1e6
            res["vs_rocblas"] = (flops / dev / 1e12) / res["rocblas_tflops"]
            ref = tmp.download(np.float32, (m, n))
            res["max_abs_diff_vs_rocblas"] = float(np.abs(Ds[0].download(np.float32, (m, n)) - ref).max())
    keep = dict(A=As[0], B=Bs[0], D=Ds[0], m=m, n=n, k=k) if shape is None else None
    return res, keep


def bench_gemm16(cfg, steps, warmup, vendor, b_row_major=False, shape=None, c_loop=False):
    """Configuration 4 (B column-major, both operands K-contiguous) or, with b_row_major, the same product with B
    handed over as [K][N], the layout of the reference's own tensor-core kernel (tensor_core_gemm.h:178)."""
    c = inputs.CONFIGS[cfg]
    m, n, k = shape or (c["m"], c["n"], c["k"])  # shape: the same operator on a row count that does not fill its tiles
    flops = 2 * m * n * k
    nsets = 4  # 130 MB per set
    As = [ko.DeviceBuffer(m * k * 2) for _ in range(nsets)]
    Bs = [ko.DeviceBuffer(k * n * 2) for _ in range(nsets)]
    Ds = [ko.DeviceBuffer(m * n * 2) for _ in range(nsets)]
    for a, b in zip(As, Bs):
        ko.fill_uniform_16(a, m * k, inputs.tensor_seed(cfg, 0))
        ko.fill_uniform_16(b, k * n, inputs.tensor_seed(cfg, 1))
    layout = ko.ROW_MAJOR if b_row_major else ko.COL_MAJOR
    wall, dev = _time_steps(lambda i: ko.gemm16(m, n, k, As[i % nsets], Bs[i % nsets], Ds[i % nsets], b_layout=layout),
                            steps, warmup)
    if c_loop:
        # kernels of a few microseconds: launched from a loop in C, as the vendor library's are below (a Python loop
        # launches one every 4-8 us); the median of three batches
        dev = ko.time_gemm16_sets(m, n, k, As, Bs, Ds, b_layout=layout, warmup=warmup, reps=steps, batches=3) * 1e-6
    name = c["name"] if shape is None else "gemm_f16_%dx%dx%d" % (m, n, k)
    if b_row_major:
        name = name.replace("gemm_f16_", "gemm_f16_rowmajorB_")
    # below the ridge of the roofline (flops per byte of A, B and D under MFMA peak / HBM peak) the bound is HBM
    nbytes = 2 * (m * k + k * n + m * n)
    if flops / nbytes < MFMA_PEAK_TFLOPS["f16"] * 1e12 / (HBM_PEAK_GBS * 1e9):
        roof = _roofline("hbm", nbytes / dev / 1e9, HBM_PEAK_GBS, "GB/s", name, dev)
    else:
        roof = _roofline("mfma", flops / dev / 1e12, MFMA_PEAK_TFLOPS["f16"], "TFLOP/s", name, dev)
    res = dict(workload=name, metric="tflops", unit="TFLOP/s", value=flops / wall / 1e12,
               ms_per_step=wall * 1e3, dtype="f16", buffer_sets=nsets, roofline=roof,
               flops=flops, kernel_us=dev * 1e6)
    if vendor is not None:
        us, na = ctypes.c_float(), ctypes.c_int()
        Vs = [ko.DeviceBuffer(m * n * 2) for _ in range(nsets)]
        tmp = Vs[0]
        if vendor.kov_gemm16_sets(m, n, k, _ptr_array(As), _ptr_array(Bs), 0 if b_row_major else 1, _ptr_array(Vs), nsets,
                                  0, 16, 20, ctypes.byref(us), ctypes.byref(na)) == 0:
            res["hipblaslt_tflops"] = flops / us.value / 1e6
            res["vs_hipblaslt"] = (flops / dev / 1e12) / res["hipblaslt_tflops"]
            ref = tmp.download(np.uint16, (m, n)).view(np.float16).astype(np.float32)
            got = Ds[0].download(np.uint16, (m, n)).view(np.float16).astype(np.float32)
            res["max_abs_diff_vs_hipblaslt"] = float(np.abs(got - ref).max())
    keep = dict(A=As[0], B=Bs[0], D=Ds[0], m=m, n=n, k=k, b_row_major=b_row_major) if shape is None else None
    return res, keep


def bench_gemm16_bias_gelu(steps, warmup, vendor):
    """The feed-forward up-projection whole: D = gelu(A B + bias) (tanh form) at the shape of configuration 4,
    next to the vendor library's fused GELU_BIAS epilogue on the same buffers."""
    c = inputs.CONFIGS[4]
    m, n, k = c["m"], c["n"], c["k"]
    flops = inputs.algorithmic_work(4)
    nsets = 4
    As = [ko.DeviceBuffer(m * k * 2) for _ in range(nsets)]
    Bs = [ko.DeviceBuffer(k * n * 2) for _ in range(nsets)]
    Ds = [ko.DeviceBuffer(m * n * 2) for _ in range(nsets)]
    bias = ko.DeviceBuffer(n * 2)
    ko.fill_uniform_16(bias, n, inputs.tensor_seed(4, 2))
    for a, b in zip(As, Bs):
        ko.fill_uniform_16(a, m * k, inputs.tensor_seed(4, 0))
        ko.fill_uniform_16(b, k * n, inputs.tensor_seed(4, 1))
    wall, dev = _time_steps(lambda i: ko.gemm16(m, n, k, As[i % nsets], Bs[i % nsets], Ds[i % nsets], bias=bias,
                                                act=ko.ACT_GELU_TANH), steps, warmup)
    res_name = "gemm_f16_bias_gelu_%dx%dx%d" % (m, n, k)
    res = dict(workload=res_name, metric="tflops", unit="TFLOP/s",
               value=flops / wall / 1e12, ms_per_step=wall * 1e3, dtype="f16", buffer_sets=nsets,
               roofline=_roofline("mfma", flops / dev / 1e12, MFMA_PEAK_TFLOPS["f16"], "TFLOP/s", res_name, dev),
               flops=flops, kernel_us=dev * 1e6)
    if vendor is not None:
        us, na = ctypes.c_float(), ctypes.c_int()
        Vs = [ko.DeviceBuffer(m * n * 2) for _ in range(nsets)]
        if vendor.kov_gemm16_bias_gelu_sets(m, n, k, _ptr_array(As), _ptr_array(Bs), bias.ptr, 1, _ptr_array(Vs), nsets,
                                            0, 16, 20, ctypes.byref(us), ctypes.byref(na)) == 0:
            res["hipblaslt_tflops"] = flops / us.value / 1e6
            res["vs_hipblaslt"] = (flops / dev / 1e12) / res["hipblaslt_tflops"]
            ref = Vs[0].download(np.uint16, (m, n)).view(np.float16).astype(np.float32)
            got = Ds[0].download(np.uint16, (m, n)).view(np.float16).astype(np.float32)
            res["max_abs_diff_vs_hipblaslt"] = float(np.abs(got - ref).max())
    return res


def bench_copy(steps, warmup, nbytes=1 << 30):
    """Plain out[i] = in[i] copy of `nbytes` in and `nbytes` out: the practical ceiling of a read+write
    stream on this device, and the calibration kernel for the HBM traffic counters."""
    n = nbytes // 4
    x, y = ko.DeviceBuffer(n * 4), ko.DeviceBuffer(n * 4)
    ko.fill_uniform_f32(x, n, 1)
    wall, dev = _time_steps(lambda i: ko.copy_f32(x, y, n), steps, warmup)
    return dict(workload="copy_f32_%dMiB" % (nbytes >> 20), metric="hbm_gbytes_per_s", unit="GB/s",
                value=2 * n * 4 / wall / 1e9, ms_per_step=wall * 1e3, dtype="f32", buffer_sets=1,
                roofline=dict(bound="hbm", achieved=2 * n * 4 / dev / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                              frac=2 * n * 4 / dev / 1e9 / HBM_PEAK_GBS, traffic=None),
                algorithmic_bytes=2 * n * 4, kernel_us=dev * 1e6)


def bench_long_rows(op, rows, cols, policy, steps, warmup):
    """Row lengths past what one wavefront holds: the row-per-workgroup (BLOCK) and re-read (BLOCK_NOCACHE) policies,
    and the reference's commented-out [49152, 1024] run (nn_operators/softmax/main.cu:78-79)."""
    n = rows * cols
    if op == "softmax":
        work = 2 * n * 4
    else:
        work = 2 * n * 4 + 2 * cols * 4 + 2 * rows * 4
    nsets = max(1, -(-(1 << 30) // work))
    xs = [ko.DeviceBuffer(n * 4) for _ in range(nsets)]
    ys = [ko.DeviceBuffer(n * 4) for _ in range(nsets)]
    for x in xs:
        ko.fill_normal_f32(x, n, 11, 0.0, 4.0)
    floor_us = _copy_floor_us(xs, ys, n, steps, warmup)
    if op == "softmax":
        launch = lambda i: ko.softmax(xs[i % nsets], ys[i % nsets], rows, cols, None, 0, policy)
    else:
        g, b = ko.DeviceBuffer(cols * 4), ko.DeviceBuffer(cols * 4)
        ko.fill_normal_f32(g, cols, 12, 1.0, 0.1)
        ko.fill_normal_f32(b, cols, 13, 0.0, 0.1)
        m, r = ko.DeviceBuffer(rows * 4), ko.DeviceBuffer(rows * 4)
        launch = lambda i: ko.layernorm(xs[i % nsets], ys[i % nsets], rows, cols, m, r, g, b, 1e-5, False, policy)
    wall, dev = _time_steps(launch, steps, warmup)
    names = {ko.POLICY_AUTO: "auto", ko.POLICY_WARP: "warp", ko.POLICY_BLOCK: "block", ko.POLICY_BLOCK_NOCACHE: "nocache"}
    res_name = "%s_f32_%dx%d_%s" % (op, rows, cols, names[policy])
    res = dict(workload=res_name, metric="hbm_gbytes_per_s", unit="GB/s",
               value=work / wall / 1e9, ms_per_step=wall * 1e3, dtype="f32", buffer_sets=nsets,
               roofline=_roofline("hbm", work / dev / 1e9, HBM_PEAK_GBS, "GB/s", res_name, dev),
               algorithmic_bytes=work, kernel_us=dev * 1e6)
    _add_copy_floor(res, floor_us)
    return res


def bench_rows16(kind, dtype_name, steps, warmup):
    """The two row operators on 16-bit storage at the shapes of the masked-softmax and LayerNorm configurations
    (half the bytes per element; fp32 arithmetic).  Inputs: uniform fills of the storage type."""
    dtype = ko.BF16 if dtype_name == "bf16" else ko.F16
    if kind == "softmax":
        c = inputs.CONFIGS[5]
        rows, cols = c["rows"], c["cols"]
        work = 2 * rows * cols * 2
    else:
        c = inputs.CONFIGS[2]
        rows, cols = c["rows"], c["cols"]
        work = 2 * rows * cols * 2 + 2 * cols * 2 + 2 * rows * 4
    n = rows * cols
    nsets = max(1, -(-(1 << 30) // work))
    xs = [ko.DeviceBuffer(n * 2) for _ in range(nsets)]
    ys = [ko.DeviceBuffer(n * 2) for _ in range(nsets)]
    for x in xs:
        ko.fill_uniform_16(x, n, 7, -8.0, 8.0, dtype=dtype)
    if kind == "softmax":
        vl = ko.DeviceBuffer(c["n_seq"] * 4)
        ko.fill_lengths_i32(vl, c["n_seq"], inputs.tensor_seed(5, 1), c["len_lo"], c["len_hi"])
        launch = lambda i: ko.softmax16(xs[i % nsets], ys[i % nsets], rows, cols, vl, c["rows_per_seq"], dtype)
        name = "masked_softmax_%s_%dx%d" % (dtype_name, rows, cols)
    else:
        g, b = ko.DeviceBuffer(cols * 2), ko.DeviceBuffer(cols * 2)
        ko.fill_uniform_16(g, cols, 8, 0.8, 1.2, dtype=dtype)
        ko.fill_uniform_16(b, cols, 9, -0.2, 0.2, dtype=dtype)
        ms = [ko.DeviceBuffer(rows * 4) for _ in range(nsets)]
        rs = [ko.DeviceBuffer(rows * 4) for _ in range(nsets)]
        launch = lambda i: ko.layernorm16(xs[i % nsets], ys[i % nsets], rows, cols, ms[i % nsets], rs[i % nsets], g, b,
                                          c["eps"], False, dtype)
        name = "layernorm_%s_%dx%d" % (dtype_name, rows, cols)
    floor_us = _copy_floor_us(xs, ys, n // 2, steps, warmup)
    wall, dev = _time_steps(launch, steps, warmup)
    full = work
    if kind == "softmax":
        work = _masked_bytes(vl, c["n_seq"], c["rows_per_seq"], rows, cols, 2)
    res_name = name
    res = dict(workload=name, metric="hbm_gbytes_per_s", unit="GB/s", value=work / wall / 1e9,
               ms_per_step=wall * 1e3, dtype=dtype_name + " storage, f32 arithmetic", buffer_sets=nsets,
               roofline=_roofline("hbm", work / dev / 1e9, HBM_PEAK_GBS, "GB/s", res_name, dev),
               algorithmic_bytes=work, kernel_us=dev * 1e6)
    if kind == "softmax":
        res["roofline"]["frac_counting_padded_reads"] = full / dev / 1e9 / HBM_PEAK_GBS
    _add_copy_floor(res, floor_us)
    return res


def bench_short_kernels(steps, warmup):
    """Where the time of the two short configurations goes: the row count of softmax [196608, 128] and LayerNorm
    [16384, 768] times 1, 2, 4, 8 and 16 next to the plain copy of the same bytes, with the straight line through
    the five points (intercept: what a launch costs whatever its size; slope: the rate the kernel streams at), the
    price of gamma and beta, and what a plain copy reaches when a wavefront holds as many bytes as a row."""
    out = dict(steps=steps, warmup=warmup, lines={}, points=[])

    def median_us(launch):
        runs = []
        for _ in range(5):
            _, dev = _time_steps(launch, steps, warmup)
            runs.append(dev * 1e6)
        return float(np.median(runs))

    def sets(nbytes):
        nsets = max(2, -(-(1 << 30) // (2 * nbytes)))
        xs = [ko.DeviceBuffer(nbytes) for _ in range(nsets)]
        ys = [ko.DeviceBuffer(nbytes) for _ in range(nsets)]
        for x in xs:
            ko.fill_normal_f32(x, nbytes // 4, 1, 0.5, 2.0)
        return xs, ys, nsets

    for op, rows0, cols in (("softmax", 196608, 128), ("layernorm", 16384, 768)):
        g, b = ko.DeviceBuffer(cols * 4), ko.DeviceBuffer(cols * 4)
        ko.fill_normal_f32(g, cols, 2, 1.0, 0.1)
        ko.fill_normal_f32(b, cols, 3, 0.0, 0.1)
        for kind in (op, "copy") + (("layernorm_no_gamma_beta",) if op == "layernorm" else ()):
            pts = []
            for mult in (1, 2, 4, 8, 16):
                rows = rows0 * mult
                n = rows * cols
                xs, ys, ns = sets(n * 4)
                m, r = ko.DeviceBuffer(rows * 4), ko.DeviceBuffer(rows * 4)
                if kind == "copy":
                    us = median_us(lambda i: ko.copy_f32(xs[i % ns], ys[i % ns], n))
                elif kind == "softmax":
                    us = median_us(lambda i: ko.softmax(xs[i % ns], ys[i % ns], rows, cols))
                elif kind == "layernorm":
                    us = median_us(lambda i: ko.layernorm(xs[i % ns], ys[i % ns], rows, cols, m, r, g, b, 1e-5))
                else:
                    us = median_us(lambda i: ko.layernorm(xs[i % ns], ys[i % ns], rows, cols, m, r, None, None, 1e-5))
                pts.append((2 * n * 4, us))
                out["points"].append(dict(kernel=kind, rows=rows, cols=cols, bytes=2 * n * 4, us=us,
                                          gbps=2 * n * 4 / us / 1e3))
                del xs, ys
            slope, intercept = np.polyfit([p[0] for p in pts], [p[1] for p in pts], 1)
            out["lines"]["%s_%dcols" % (kind, cols)] = dict(intercept_us=float(intercept), slope_gbps=float(1e-3 / slope))
    # a plain copy whose wavefronts hold 1, 2 and 4 vectors per lane, and whose workgroups hold 3 KB and 6 KB
    n = 262144 * 768
    xs, ys, ns = sets(n * 4)
    out["copy_by_footprint"] = []
    for threads, vpt in ((64, 1), (64, 2), (64, 4), (128, 1), (192, 1), (256, 1), (384, 1)):
        for pad in (0, 10240):
            us = median_us(lambda i: ko.stream_probe(xs[i % ns], ys[i % ns], n * 4, ko.PROBE_COPY, vectors_per_thread=vpt,
                                                     threads=threads, load_policy=1, store_policy=3, lds_pad_bytes=pad))
            out["copy_by_footprint"].append(dict(threads=threads, vectors_per_thread=vpt, lds_pad_bytes=pad, us=us,
                                                 gbps=2 * n * 4 / us / 1e3))
    return out


MIDSIZE_ROWS = (100, 256, 512, 1000, 2048, 3000, 4096, 6000, 8192, 12000, 20000)
MIDSIZE_WEIGHTS = ((3072, 768), (768, 3072), (2304, 768), (4096, 4096), (1024, 1024), (4096, 1024), (1024, 4096))


def bench_gemm16_midsize(steps, warmup, vendor):
    """The 16-bit GEMM on token counts from 100 to 20000 against transformer weight shapes (N x K), next to
    hipBLASLt on the same buffers: time, ratio, and what the host-side planner decided (K slices and their tiling)."""
    rows = []
    for n, k in MIDSIZE_WEIGHTS:
        for m in MIDSIZE_ROWS:
            res, _ = bench_gemm16(4, steps, warmup, vendor, shape=(m, n, k), c_loop=True)
            slices, k_slice, tile = ko.gemm_plan(m, n, k, sixteen_bit=True)
            rows.append(dict(m=m, n=n, k=k, us=res["kernel_us"], tflops=res["roofline"]["achieved"]
                             if res["roofline"]["unit"] == "TFLOP/s" else res["flops"] / res["kernel_us"] / 1e6,
                             hipblaslt_us=res["flops"] / res["hipblaslt_tflops"] / 1e6 if "hipblaslt_tflops" in res else None,
                             vs_hipblaslt=res.get("vs_hipblaslt"), k_slices=slices, k_slice=k_slice, slice_tile=tile,
                             tiles_256=-(-m // 256) * -(-n // 256)))
    ratios = sorted(r["vs_hipblaslt"] for r in rows if r["vs_hipblaslt"])
    return dict(steps=steps, warmup=warmup, shapes=len(rows), median_vs_hipblaslt=ratios[len(ratios) // 2] if ratios else None,
                min_vs_hipblaslt=ratios[0] if ratios else None, max_vs_hipblaslt=ratios[-1] if ratios else None, rows=rows)


# weight-gradient shapes: a layer's weight (M x N) against batch x sequence (K), and a decoding step's few rows
DEEP_K_SHAPES = ((768, 768, 16384), (768, 3072, 16384), (3072, 768, 16384), (768, 2304, 16384), (1024, 1024, 16384),
                 (1024, 4096, 16384), (4096, 1024, 16384), (4096, 4096, 16384), (1024, 3072, 12288), (2048, 4096, 16384),
                 (1536, 2304, 16384), (2048, 2048, 32768), (512, 512, 32768), (256, 1024, 16384), (1024, 4096, 8192),
                 (8, 8192, 8192), (32, 8192, 8192), (8, 4096, 4096), (8, 28672, 4096), (32, 32000, 4096), (8, 128256, 4096))


def bench_gemm16_deep_k(steps, warmup, vendor):
    """The 16-bit GEMM on a deep K against few or mid-size outputs (weight gradients), and on a handful of rows against
    large weights (decoding), next to hipBLASLt on the same buffers; with the planner's decision."""
    rows = []
    for m, n, k in DEEP_K_SHAPES:
        res, _ = bench_gemm16(4, steps, warmup, vendor, shape=(m, n, k), c_loop=True)
        slices, k_slice, tile = ko.gemm_plan(m, n, k, sixteen_bit=True)
        rows.append(dict(m=m, n=n, k=k, us=res["kernel_us"], tflops=res["flops"] / res["kernel_us"] / 1e6,
                         hipblaslt_us=res["flops"] / res["hipblaslt_tflops"] / 1e6 if "hipblaslt_tflops" in res else None,
                         vs_hipblaslt=res.get("vs_hipblaslt"), k_slices=slices, k_slice=k_slice, slice_tile=tile))
    ratios = sorted(r["vs_hipblaslt"] for r in rows if r["vs_hipblaslt"])
    return dict(steps=steps, warmup=warmup, shapes=len(rows), median_vs_hipblaslt=ratios[len(ratios) // 2] if ratios else None,
                min_vs_hipblaslt=ratios[0] if ratios else None, max_vs_hipblaslt=ratios[-1] if ratios else None, rows=rows)


def bench_gemm16_active_cus(steps, warmup):
    """Time per K tile of the 256 x 256 kernel of the 16-bit GEMM by how many compute units have a tile: K = 4096
    (64 K tiles per output tile), N = 3072 (12 tile columns), M from 256 to 16384."""
    out = []
    ko.set_tuning("gemm16.variant", 53)  # the 256 x 256 pinned kernel whatever the dispatch would pick
    for m in (256, 512, 1024, 2048, 4096, 5376, 10752, 16384):
        n, k = 3072, 4096
        res, _ = bench_gemm16(4, steps, warmup, None, shape=(m, n, k))
        tiles = (m // 256) * (n // 256)
        cus = ko.device_info()["compute_units"]
        rounds = -(-tiles // cus)
        out.append(dict(m=m, n=n, k=k, tiles=tiles, busy_compute_units=min(tiles, cus), tiles_per_compute_unit=rounds,
                        us=res["kernel_us"], us_per_k_tile=res["kernel_us"] / (rounds * k / 64),
                        tflops=res["flops"] / res["kernel_us"] / 1e6))
    ko.set_tuning("gemm16.variant", 0)
    return dict(steps=steps, warmup=warmup, rows=out)


def run_workload(cfg, steps, warmup, vendor):
    op = inputs.CONFIGS[cfg]["op"]
    if op == "softmax":
        return bench_softmax(cfg, steps, warmup)
    if op == "layernorm":
        return bench_layernorm(cfg, steps, warmup)
    if op == "sgemm":
        return bench_sgemm(cfg, steps, warmup, vendor)
    return bench_gemm16(cfg, steps, warmup, vendor)


# ---------------------------------------------------------------------------- CPU baseline

def cpu_baseline_softmax(keep, cfg):
    """The CPU oracle (a port: the reference has no CPU softmax) on the rows the GPU just processed, all
    host threads, best of 3 (about 15-25 core-seconds in all); also checks the GPU rows against it."""
    import oracle  # test infrastructure: used here as the timed CPU baseline and checker only
    c = inputs.CONFIGS[cfg]
    rows = keep["rows"]
    if keep["rps"]:
        rows -= rows % keep["rps"]
    cols = keep["cols"]
    x = keep["x"].download(np.float32, (rows, cols))
    y = keep["y"].download(np.float32, (rows, cols))
    vl = keep["vl"].download(np.int32, (c["n_seq"],)) if keep["vl"] is not None else None
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        ref = oracle.softmax(x, vl, keep["rps"])
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    # one thread, on the first sixteenth of the rows (whole sequences): the scalar port's own speed
    nthreads = oracle.max_threads()
    rows1 = max(keep["rps"] or 1, (rows // 16) // (keep["rps"] or 1) * (keep["rps"] or 1))
    oracle.set_threads(1)
    t0 = time.perf_counter()
    oracle.softmax(x[:rows1], vl, keep["rps"])
    single = time.perf_counter() - t0
    oracle.set_threads(nthreads)
    d = np.abs(y.astype(np.float64) - ref)
    sel = ref >= np.finfo(np.float32).tiny
    parity = dict(rows_checked=rows, max_abs_err=float(d.max()), max_rel_err=float((d[sel] / ref[sel]).max()),
                  gate="abs<=1e-6 and rel<=1e-5", ok=bool(d.max() <= 1e-6 and (d[sel] / ref[sel]).max() <= 1e-5))
    work = keep.get("work", 2 * rows * cols * 4)  # the byte count the GPU figure is taken over
    return dict(value=work / best / 1e9, unit="GB/s", cores=oracle.max_threads(), kind="port",
                sample="all %d rows x %d cols of the same device-resident input, %d threads, best of 3; "
                       "host cpus visible: %d" % (rows, cols, oracle.max_threads(), os.cpu_count() or 0),
                seconds=best,
                single_thread=dict(value=work * rows1 / rows / single / 1e9, unit="GB/s", cores=1,
                                   sample="first %d rows, 1 thread, one run" % rows1, seconds=single)), parity


def cpu_baseline_layernorm(keep):
    """The CPU oracle's LayerNorm on the rows the GPU just processed: all host threads, best of 3, and one thread
    on a sixteenth of the rows; also checks y, mean and rstd of the GPU against it."""
    import oracle
    rows, cols = keep["rows"], keep["cols"]
    x = keep["x"].download(np.float32, (rows, cols))
    g, b = keep["g"].download(np.float32, (cols,)), keep["b"].download(np.float32, (cols,))
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        ry, rm, rr = oracle.layernorm(x, g, b, eps=keep["eps"])
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    nthreads = oracle.max_threads()
    rows1 = max(1, rows // 16)
    oracle.set_threads(1)
    t0 = time.perf_counter()
    oracle.layernorm(x[:rows1], g, b, eps=keep["eps"])
    single = time.perf_counter() - t0
    oracle.set_threads(nthreads)
    y = keep["y"].download(np.float32, (rows, cols)).astype(np.float64)
    mean = keep["mean"].download(np.float32, (rows,)).astype(np.float64)
    rstd = keep["rstd"].download(np.float32, (rows,)).astype(np.float64)
    ey = float((np.abs(y - ry) / np.maximum(np.abs(ry), 1.0)).max())
    er = float((np.abs(rstd - rr) / rr).max())
    em = float((np.abs(mean - rm) / np.maximum(np.abs(rm), 1.0 / rr)).max())
    # not gated: the elementwise-relative worst cases, which no fp32 evaluation keeps below 1e-5 where x - mean
    # (for y) or the sum of the row (for mean) cancels; printed so that what the gates give up can be seen
    big = np.abs(ry) >= 1e-2
    ey_pure = float((np.abs(y - ry)[big] / np.abs(ry)[big]).max())
    em_pure = float((np.abs(mean - rm) / np.maximum(np.abs(rm), 1e-3)).max())
    parity = dict(rows_checked=rows, max_y_err=ey, max_rstd_rel_err=er, max_mean_err=em,
                  gate="|dy| <= 1e-5 max(|y|, 1); rstd 1e-5 relative; mean 1e-5 of max(|mean|, std)",
                  ok=bool(ey <= 1e-5 and er <= 1e-5 and em <= 1e-5),
                  ungated=dict(max_y_rel_err_where_y_ge_1e_2=ey_pure, max_mean_err_over_max_mean_1e_3=em_pure))
    work = 2 * rows * cols * 4
    return dict(value=work / best / 1e9, unit="GB/s", cores=nthreads, kind="port",
                sample="all %d rows x %d cols, %d threads, best of 3; host cpus visible: %d" % (
                    rows, cols, nthreads, os.cpu_count() or 0), seconds=best,
                single_thread=dict(value=2 * rows1 * cols * 4 / single / 1e9, unit="GB/s", cores=1,
                                   sample="first %d rows, 1 thread, one run" % rows1, seconds=single)), parity


def cpu_baseline_sgemm(keep):
    """The CPU oracle's SGEMM - the reference's commented-out CPU loop (nn_operators/gemm/main.cu:162-167) with a
    double accumulator - on the same operands, all host threads, best of 3; checks the GPU's D against it."""
    import oracle
    m, n, k = keep["m"], keep["n"], keep["k"]
    A, B = keep["A"].download(np.float32, (m, k)), keep["B"].download(np.float32, (k, n))
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        ref, ap = oracle.sgemm(A, B, want_absprod=True)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    d = np.abs(keep["D"].download(np.float32, (m, n)).astype(np.float64) - ref)
    worst = float((d / (2.0 * k * 2.0 ** -24 * ap + 1e-30)).max())
    parity = dict(elements_checked=m * n, max_abs_err=float(d.max()), worst_over_bound=worst,
                  gate="|d| <= 2 K 2^-24 sum|a||b| and |d| <= 1e-3 (gemm/main.cu:169-170)",
                  ok=bool(worst <= 1.0 and d.max() <= 1e-3))
    return dict(value=2.0 * m * n * k / best / 1e12, unit="TFLOP/s", cores=oracle.max_threads(), kind="port",
                sample="the whole %dx%dx%d product, %d threads, best of 3" % (m, n, k, oracle.max_threads()),
                seconds=best), parity


def cpu_baseline_gemm16(keep, sample_rows=1024):
    """The CPU oracle's 16-bit GEMM on the first `sample_rows` rows of A (the operator is independent per output
    row; the whole product would take about a minute of host time), all host threads, one run; checks those rows of
    the GPU's D against it."""
    import oracle
    m, n, k = keep["m"], keep["n"], keep["k"]
    ms = min(m, sample_rows)
    A = keep["A"].download(np.uint16, (ms, k))
    B = keep["B"].download(np.uint16, (k, n) if keep["b_row_major"] else (n, k))
    t0 = time.perf_counter()
    _, ref64, ap = oracle.gemm16(A, B, ms, n, k, b_col_major=not keep["b_row_major"])
    dt = time.perf_counter() - t0
    got = oracle.f16_to_f64(keep["D"].download(np.uint16, (ms, n)))
    d = np.abs(got - ref64)
    worst = float((d / (2.0 ** -11 * np.abs(ref64) + k * 2.0 ** -24 * ap + 2.0 ** -24)).max())
    parity = dict(elements_checked=ms * n, max_abs_err=float(d.max()), worst_over_bound=worst,
                  gate="|d| <= 2^-11 |ref| + K 2^-24 sum|a||b| + 2^-24", ok=bool(worst <= 1.0))
    return dict(value=2.0 * ms * n * k / dt / 1e12, unit="TFLOP/s", cores=oracle.max_threads(), kind="port",
                sample="first %d of %d rows of A (x %d x %d), %d threads, one run" % (ms, m, n, k, oracle.max_threads()),
                seconds=dt), parity


def cpu_baseline(cfg, keep):
    op = inputs.CONFIGS[cfg]["op"]
    if op == "softmax":
        return cpu_baseline_softmax(keep, cfg)
    if op == "layernorm":
        return cpu_baseline_layernorm(keep)
    if op == "sgemm":
        return cpu_baseline_sgemm(keep)
    return cpu_baseline_gemm16(keep)


# ------------------------------------------------------------------------- streaming ceilings

def _probe_rate(nbytes, moved, launch, steps, warmup):
    _, dev = _time_steps(launch, steps, warmup)
    return dict(us=dev * 1e6, gbps=moved / dev / 1e9, frac_of_peak=moved / dev / 1e9 / HBM_PEAK_GBS)


def bench_ceilings(steps, warmup, nbytes=1 << 30, full=False):
    """What a read stream, a write stream and a read+write stream reach on this device, from independent sources
    in the same run: the runtime's own device-to-device copy and memset, and the streaming probe kernel in the
    launch shapes that matter (workgroup size, vectors per thread, cache-policy bits of the stores, residency cap).
    full: the whole sweep (for profiles/), else the handful of shapes that bracket the best."""
    x, y = ko.DeviceBuffer(nbytes), ko.DeviceBuffer(nbytes)
    ko.fill_uniform_f32(x, nbytes // 4, 1)
    out = dict(bytes_per_direction=nbytes, steps=steps, warmup=warmup)
    out["runtime_memcpy_d2d"] = _probe_rate(nbytes, 2 * nbytes, lambda i: ko.memcpy_d2d(y, x, nbytes), steps, warmup)
    out["runtime_memset"] = _probe_rate(nbytes, nbytes, lambda i: ko.memset(y, 0, nbytes), steps, warmup)
    out["copy_f32_kernel"] = _probe_rate(nbytes, 2 * nbytes, lambda i: ko.copy_f32(x, y, nbytes // 4), steps, warmup)
    rows = []

    def probe(mode, name, moved, **kw):
        r = _probe_rate(nbytes, moved, lambda i: ko.stream_probe(x, y, nbytes, mode, **kw), steps, warmup)
        r.update(kind=name, **kw)
        rows.append(r)
        return r

    lp, sp = ko.LOAD_POLICIES, ko.STORE_POLICIES
    threads_list = (64, 128, 256, 512, 1024) if full else (128, 256)
    vpts = (1, 2, 4) if full else (1, 2)
    grids = (0, 2, 8) if full else (0,)
    for t in threads_list:
        for v in vpts:
            for g in grids:
                for l in ((lp["plain"], lp["nt"]) if full else (lp["nt"],)):
                    probe(ko.PROBE_READ, "read", nbytes, threads=t, vectors_per_thread=v, blocks_per_cu=g, load_policy=l)
                for st in (sp.values() if full else (sp["nt"], sp["sc1 nt"])):
                    probe(ko.PROBE_WRITE, "write", nbytes, threads=t, vectors_per_thread=v, blocks_per_cu=g, store_policy=st)
                    probe(ko.PROBE_COPY, "copy", 2 * nbytes, threads=t, vectors_per_thread=v, blocks_per_cu=g,
                          load_policy=lp["nt"], store_policy=st)
                if full:
                    probe(ko.PROBE_COPY, "copy", 2 * nbytes, threads=t, vectors_per_thread=v, blocks_per_cu=g,
                          load_policy=lp["plain"], store_policy=sp["plain"])
    # residency cap: two vectors per thread with all 32 wavefronts of a CU resident, and with 16
    for pad in ((0, 5120, 10240, 20480, 40960) if full else (0, 10240)):
        for v in (1, 2, 4):
            probe(ko.PROBE_COPY, "copy", 2 * nbytes, threads=64, vectors_per_thread=v, load_policy=lp["nt"],
                  store_policy=sp["sc1 nt"], lds_pad_bytes=pad)
    # the traffic mix of the masked-softmax configuration: every vector written, 81 of 128 read
    for t in ((64, 128, 256) if full else (128,)):
        for st in ((sp["nt"], sp["sc1 nt"]) if full else (sp["sc1 nt"],)):
            probe(ko.PROBE_PARTIAL, "copy reading 81/128", nbytes + nbytes * 81 // 128, threads=t, vectors_per_thread=1,
                  load_policy=lp["nt"], store_policy=st, read_of_128=81)
    for kind in ("read", "write", "copy", "copy reading 81/128"):
        best = max((r for r in rows if r["kind"] == kind), key=lambda r: r["gbps"])
        out["best_" + kind.replace(" ", "_").replace("/", "_of_")] = best
    if full:
        out["rows"] = rows
    return out


# ------------------------------------------------------------------------------ the record

MAX_LINE_BYTES = 4096
CONFIG_LINES = ("softmax_f32_196608x128", "layernorm_f32_16384x768", "sgemm_f32_1024x1024x1024",
                "gemm_f16_16384x3072x768", "masked_softmax_f32_786432x512", "softmax_f32_786432x512_unmasked",
                "gemm_f16_bias_gelu_16384x3072x768")


def _sig(v, digits=4):
    return None if v is None else float("%.*g" % (digits, v))


def _compact(res):
    """The handful of numbers of one workload that go into the one-line record."""
    roof = res["roofline"]
    out = {"name": res["workload"], "value": _sig(res["value"]), "unit": res["unit"],
           "kernel_us": _sig(res["kernel_us"]), "bound": roof["bound"], "frac": _sig(roof["frac"])}
    if roof.get("frac_on_traffic") is not None:
        out["frac_on_traffic"] = _sig(roof["frac_on_traffic"])
    for key in ("vs_hipblaslt", "vs_rocblas", "vs_copy_same_bytes"):
        if key in res:
            out[key] = _sig(res[key])
    if res.get("parity") is not None:
        out["parity_ok"] = res["parity"]["ok"]
    if res.get("cpu_baseline") is not None:
        out["cpu"] = _sig(res["cpu_baseline"]["value"])
        out["cpu_cores"] = res["cpu_baseline"]["cores"]
    return out


def headline_line(head, cpu, parity, others, copy, info, steps, warmup, midsize=None, deep_k=None):
    """The record: one JSON object of at most MAX_LINE_BYTES characters, printed as the last line of stdout.  It
    carries the headline workload in full (roofline, CPU baseline, parity) and six numbers for each of the other
    configurations; everything else goes to gpurun_out/bench_workloads.json and to earlier lines."""
    roof = {k: (_sig(v, 5) if isinstance(v, float) else v) for k, v in head["roofline"].items()}
    line = {
        "metric": head["metric"], "value": _sig(head["value"], 6), "unit": head["unit"], "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": _sig(head["ms_per_step"], 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"],
        "data": "synthetic (seeded counter-based generator, filled on the device)",
        "config": {"workload": head["workload"], "buffer_sets": head["buffer_sets"],
                   "device": info["name"] or info["arch"], "compute_units": info["compute_units"]},
        "roofline": roof,
        "cpu_baseline": None if cpu is None else {
            "value": _sig(cpu["value"]), "unit": cpu["unit"], "cores": cpu["cores"], "kind": cpu["kind"],
            "sample": cpu["sample"], "seconds": _sig(cpu.get("seconds"))},
        "parity": None if parity is None else {k: (_sig(v) if isinstance(v, float) else v)
                                               for k, v in parity.items() if k != "ungated"},
        "kernel_us": _sig(head["kernel_us"], 5),
    }
    if "bytes_basis" in head:
        line["config"]["bytes_basis"] = head["bytes_basis"]
    if head.get("copy_same_bytes_us") is not None:
        line["copy_same_bytes_us"] = _sig(head["copy_same_bytes_us"], 5)
    if copy is not None:
        line["copy_ceiling_frac"] = _sig(copy["roofline"]["frac"])
    for key in ("hipblaslt_tflops", "vs_hipblaslt", "max_abs_diff_vs_hipblaslt"):
        if key in head:
            line[key] = _sig(head[key])
    by_name = {r["workload"]: r for r in others}
    line["configs"] = [_compact(by_name[n]) for n in CONFIG_LINES if n in by_name]
    if midsize is not None:  # the 16-bit GEMM on 77 mid-size shapes next to hipBLASLt (rows in the details file)
        line["gemm16_midsize"] = {"shapes": midsize["shapes"], "median_vs_hipblaslt": _sig(midsize["median_vs_hipblaslt"]),
                                  "min_vs_hipblaslt": _sig(midsize["min_vs_hipblaslt"])}
    if deep_k is not None:  # and on weight-gradient and decoding shapes
        line["gemm16_deep_k"] = {"shapes": deep_k["shapes"], "median_vs_hipblaslt": _sig(deep_k["median_vs_hipblaslt"]),
                                 "min_vs_hipblaslt": _sig(deep_k["min_vs_hipblaslt"])}
    line["details_file"] = "gpurun_out/bench_workloads.json"
    # never let the record outgrow what a reader of the last line keeps: shed the optional parts first
    for key in ("details_file", "copy_ceiling_frac", "copy_same_bytes_us", "max_abs_diff_vs_hipblaslt", "gemm16_deep_k",
                "gemm16_midsize"):
        if len(json.dumps(line)) <= MAX_LINE_BYTES:
            break
        line.pop(key, None)
    while len(json.dumps(line)) > MAX_LINE_BYTES and line["configs"]:
        line["configs"].pop()
    return line




def emit_record(head, cpu, parity, others, copy, ceilings, info, steps, warmup, out_dir=None, midsize=None, deep_k=None):
    """Writes everything that was measured to <out_dir>/bench_workloads.json, prints one short line per secondary
    workload, and prints the record as the LAST line of stdout."""
    line = headline_line(head, cpu, parity, others, copy, info, steps, warmup, midsize, deep_k)
    details = dict(line)
    if midsize is not None:
        details["gemm16_midsize"] = midsize
    if deep_k is not None:
        details["gemm16_deep_k"] = deep_k
    details["copy_ceiling"] = None if copy is None else {
        "GB/s": copy["roofline"]["achieved"], "frac_of_peak": copy["roofline"]["frac"], "workload": copy["workload"],
        "independent_sources": ceilings}
    details["headline"] = dict(head, cpu_baseline=cpu, parity=parity)
    details["workloads"] = others
    out_dir = out_dir or os.path.join(ROOT, "gpurun_out")
    try:
        os.makedirs(out_dir, exist_ok=True)
        with open(os.path.join(out_dir, "bench_workloads.json"), "w") as f:
            json.dump(details, f, indent=1)
    except OSError:
        line.pop("details_file", None)
    for res in others:
        print(json.dumps(_compact(res)))
    sys.stdout.flush()
    print(json.dumps(line))
    sys.stdout.flush()
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=100,
                    help="untimed launches before the timed ones; the device takes a few hundred short launches "
                         "to settle its clocks, so the microsecond-scale secondary workloads use at least 300")
    ap.add_argument("--workload", default=inputs.CONFIGS[HEADLINE]["name"],
                    help="one of %s, copy_f32, hbm_ceilings, short_kernels, gemm16_midsize, gemm16_deep_k, gemm16_active_cus, softmax_f32_786432x512_unmasked, or a long-row line by name: "
                         "(softmax|layernorm)_f32_<rows>x<cols>_(auto|warp|block|nocache); or one 16-bit GEMM shape: gemm_f16_<m>x<n>x<k>" % ", ".join(sorted(WORKLOADS)))
    ap.add_argument("--all", dest="all", action="store_true", default=True,
                    help="also measure the other four configurations (default)")
    ap.add_argument("--no-all", dest="all", action="store_false")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (every operator here shards by rows with no "
                 "communication); run with --gpus 1")
    ko.lib()
    info = ko.device_info()  # raises without a GPU: there is no CPU fallback
    vendor = _vendor()

    if args.workload == "copy_f32":  # calibration run for the traffic counters
        print(json.dumps(bench_copy(args.steps, args.warmup)))
        return
    if args.workload == "hbm_ceilings":  # the whole streaming sweep, for profiles/
        print(json.dumps(bench_ceilings(min(args.steps, 10), 3, full=True)))
        return
    if args.workload == "gemm16_deep_k":  # the sweep behind profiles/gemm16_deep_k.md
        print(json.dumps(bench_gemm16_deep_k(min(args.steps, 30), max(args.warmup, 60), vendor)))
        return
    if args.workload == "gemm16_midsize":  # the sweep behind profiles/gemm16_midsize.md
        print(json.dumps(bench_gemm16_midsize(min(args.steps, 30), max(args.warmup, 100), vendor)))
        return
    if args.workload == "gemm16_active_cus":  # time per K tile by the number of busy compute units, for profiles/
        print(json.dumps(bench_gemm16_active_cus(min(args.steps, 30), max(args.warmup, 100))))
        return
    if args.workload == "short_kernels":  # intercept and slope of the two short configurations, for profiles/
        print(json.dumps(bench_short_kernels(min(args.steps, 30), max(args.warmup, 100))))
        return
    if args.workload == "softmax_f32_786432x512_unmasked":  # for the traffic counters and traces
        res, _ = bench_softmax(5, args.steps, args.warmup, unmasked=True)
        print(json.dumps(res))
        return
    gemm_line = re.fullmatch(r"gemm_f16_(\d+)x(\d+)x(\d+)", args.workload)
    if gemm_line and args.workload not in WORKLOADS:  # one 16-bit GEMM shape alone (B column-major), for traces
        m, n, k = (int(g) for g in gemm_line.groups())
        res, _ = bench_gemm16(4, min(args.steps, 30), max(args.warmup, 100), vendor, shape=(m, n, k), c_loop=True)
        res["plan"] = ko.gemm_plan(m, n, k, sixteen_bit=True)
        print(json.dumps(res))
        return
    row_line = re.fullmatch(r"(softmax|layernorm)_f32_(\d+)x(\d+)_(auto|warp|block|nocache)", args.workload)
    if row_line and args.workload not in WORKLOADS:  # one of the long-row lines alone, for counters and traces
        policy = {"auto": ko.POLICY_AUTO, "warp": ko.POLICY_WARP, "block": ko.POLICY_BLOCK,
                  "nocache": ko.POLICY_BLOCK_NOCACHE}[row_line.group(4)]
        print(json.dumps(bench_long_rows(row_line.group(1), int(row_line.group(2)), int(row_line.group(3)), policy,
                                         args.steps, args.warmup)))
        return
    if args.workload not in WORKLOADS:
        sys.exit("bench.py: unknown workload %r (see --help)" % args.workload)
    cfg = WORKLOADS[args.workload]

    def headline():
        head, keep = run_workload(cfg, args.steps, args.warmup, vendor)
        cpu, parity = (None, None)
        if not args.no_cpu and keep is not None:
            cpu, parity = cpu_baseline(cfg, keep)
        return head, cpu, parity

    # With --all the headline is measured last, with its own W warm-up and K timed steps like any other run of it: the
    # first workload of a process meets a device that has just woken up (the masked softmax: 424 us per launch as the
    # first workload with 5 warm-up launches, 400 us once the device has worked for a second), and the order of the
    # workloads is the one free choice that does not touch W or K.
    if not args.all:
        head, cpu, parity = headline()
    others = []
    copy = None
    ceilings = None
    midsize = deep_k = None
    if args.all:
        copy = bench_copy(args.steps, args.warmup)
        ceilings = bench_ceilings(min(args.steps, 10), 3)
        for other in sorted(inputs.CONFIGS):
            if other == cfg:
                continue
            warm = max(args.warmup, SECONDARY_MIN_WARMUP)
            res, k2 = run_workload(other, args.steps, warm, vendor)
            if not args.no_cpu and k2 is not None:
                res["cpu_baseline"], res["parity"] = cpu_baseline(other, k2)
            del k2
            res["steps"], res["warmup"] = args.steps, warm
            others.append(res)
        # the masked configuration's shape without the mask: every algorithmic byte moves
        res, k2 = bench_softmax(5, args.steps, args.warmup, unmasked=True)
        del k2
        res["steps"], res["warmup"] = args.steps, args.warmup
        others.append(res)
        for op, rows, cols, policy in (("softmax", 49152, 1024, ko.POLICY_WARP), ("softmax", 32768, 4096, ko.POLICY_BLOCK),
                                       ("softmax", 8192, 16384, ko.POLICY_BLOCK),
                                       ("softmax", 2048, 65536, ko.POLICY_BLOCK),
                                       ("softmax", 1024, 131072, ko.POLICY_BLOCK_NOCACHE),
                                       ("layernorm", 32768, 4096, ko.POLICY_BLOCK),
                                       ("layernorm", 8192, 16384, ko.POLICY_BLOCK),
                                       ("layernorm", 2048, 65536, ko.POLICY_BLOCK),
                                       ("layernorm", 1024, 131072, ko.POLICY_BLOCK),
                                       ("layernorm", 1024, 131072, ko.POLICY_BLOCK_NOCACHE),
                                       # a vocabulary for a batch of 32 rows: each row cut into pieces (two launches)
                                       ("softmax", 32, 128256, ko.POLICY_AUTO)):
            res = bench_long_rows(op, rows, cols, policy, args.steps, args.warmup)
            res["steps"], res["warmup"] = args.steps, args.warmup
            others.append(res)
        res, _ = bench_gemm16(4, args.steps, max(args.warmup, SECONDARY_MIN_WARMUP), vendor, b_row_major=True)
        res["steps"], res["warmup"] = args.steps, max(args.warmup, SECONDARY_MIN_WARMUP)
        others.append(res)
        # shapes that do not fill their tiles: fp32 4000^3 (edge form of the kernel), 16-bit with 16000 rows (the
        # last 128 rows go out as a launch of their own)
        res, _ = bench_sgemm(3, args.steps, args.warmup, vendor, shape=(4000, 4000, 4000))
        res["steps"], res["warmup"] = args.steps, args.warmup
        others.append(res)
        # a deep K on few tiles: K cut into slices that run side by side, partial products summed by a second kernel
        res, _ = bench_sgemm(3, args.steps, max(args.warmup, SECONDARY_MIN_WARMUP), vendor, shape=(256, 256, 2048))
        res["steps"], res["warmup"] = args.steps, max(args.warmup, SECONDARY_MIN_WARMUP)
        others.append(res)
        # a weight-gradient shape: 144 tiles of 64 x 64 would leave 112 compute units idle; the planner takes
        # 36 tiles of 128 x 128 in seven slices of K
        res, _ = bench_sgemm(3, args.steps, args.warmup, vendor, shape=(768, 768, 16384))
        res["steps"], res["warmup"] = args.steps, args.warmup
        others.append(res)
        res, _ = bench_gemm16(4, args.steps, max(args.warmup, SECONDARY_MIN_WARMUP), vendor, shape=(16000, 3072, 768))
        res["steps"], res["warmup"] = args.steps, max(args.warmup, SECONDARY_MIN_WARMUP)
        others.append(res)
        # K off the K tile: padded with zeros inside the pinned kernel
        res, _ = bench_gemm16(4, args.steps, max(args.warmup, SECONDARY_MIN_WARMUP), vendor, shape=(16384, 3072, 760))
        res["steps"], res["warmup"] = args.steps, max(args.warmup, SECONDARY_MIN_WARMUP)
        others.append(res)
        # a vocabulary projection: 30522 columns put the rows of D off 16-byte boundaries (full tile columns on the
        # pinned kernel, the last 58 columns as a launch of their own)
        res, _ = bench_gemm16(4, args.steps, max(args.warmup, SECONDARY_MIN_WARMUP), vendor, shape=(4096, 30522, 768))
        res["steps"], res["warmup"] = args.steps, max(args.warmup, SECONDARY_MIN_WARMUP)
        others.append(res)
        # a batch of eight rows against a weight matrix: 32 x 256 tiles in slices of K, every compute unit streaming
        # its share of B
        res, _ = bench_gemm16(4, args.steps, max(args.warmup, SECONDARY_MIN_WARMUP), vendor, shape=(8, 8192, 8192))
        res["steps"], res["warmup"] = args.steps, max(args.warmup, SECONDARY_MIN_WARMUP)
        others.append(res)
        # a 16-bit weight-gradient shape: 36 tiles of 128 x 128 in seven slices of K
        res, _ = bench_gemm16(4, args.steps, max(args.warmup, SECONDARY_MIN_WARMUP), vendor, shape=(768, 768, 16384))
        res["steps"], res["warmup"] = args.steps, max(args.warmup, SECONDARY_MIN_WARMUP)
        others.append(res)
        res = bench_gemm16_bias_gelu(args.steps, max(args.warmup, SECONDARY_MIN_WARMUP), vendor)
        res["steps"], res["warmup"] = args.steps, max(args.warmup, SECONDARY_MIN_WARMUP)
        others.append(res)
        for kind, dt in (("softmax", "f16"), ("layernorm", "bf16")):
            warm = max(args.warmup, SECONDARY_MIN_WARMUP if kind == "layernorm" else 0)
            res = bench_rows16(kind, dt, args.steps, warm)
            res["steps"], res["warmup"] = args.steps, warm
            others.append(res)

        # token counts from 100 to 20000 against transformer weight shapes, next to hipBLASLt (launch loops in C on both
        # sides; about ten seconds): the summary goes into the record, the rows into the details file
        if vendor is not None:
            midsize = bench_gemm16_midsize(min(args.steps, 30), 100, vendor)
            deep_k = bench_gemm16_deep_k(min(args.steps, 30), 60, vendor)

        head, cpu, parity = headline()
    emit_record(head, cpu, parity, others, copy, ceilings, info, args.steps, args.warmup, midsize=midsize, deep_k=deep_k)


if __name__ == "__main__":
    main()
