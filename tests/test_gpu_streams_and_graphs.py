"""The operators are plain kernel launches on the caller's stream, so a caller can capture them into a HIP graph
(the reference's drivers launch on one non-blocking stream as well, softmax/main.cu:28-29).  This test captures a
softmax -> LayerNorm -> 16-bit GEMM -> SGEMM -> 16-bit GEMM (persistent kernel) -> K-sliced SGEMM and 16-bit GEMM -> softmax and LayerNorm of a few long rows (cut into pieces) sequence with the HIP runtime that libko.so itself is linked against,
replays the graph several times with eager work and synchronisations in between, and compares every replay bit
for bit with the eager results.  One eager pass comes first: the library's one-time set-up (device properties,
kernel attributes) is not stream work and belongs in front of a capture."""
import ctypes
import re

import numpy as np
import pytest

from kernel_optimization_amd import inputs

pytestmark = pytest.mark.gpu


def _hip_runtime():
    """The libamdhip64 this process already has loaded (through libko.so)."""
    with open("/proc/self/maps") as f:
        paths = sorted(set(re.findall(r"(/\S*libamdhip64\.so[\w.]*)", f.read())))
    assert paths, "libko.so is loaded, so the HIP runtime must be mapped"
    hip = ctypes.CDLL(paths[0])
    vp = ctypes.c_void_p
    hip.hipStreamBeginCapture.argtypes = [vp, ctypes.c_int]
    hip.hipStreamEndCapture.argtypes = [vp, ctypes.POINTER(vp)]
    hip.hipGraphInstantiate.argtypes = [ctypes.POINTER(vp), vp, vp, vp, ctypes.c_size_t]
    hip.hipGraphLaunch.argtypes = [vp, vp]
    hip.hipGraphExecDestroy.argtypes = [vp]
    hip.hipGraphDestroy.argtypes = [vp]
    return hip


def test_operators_replay_from_a_hip_graph(ko):
    ko.lib()
    hip = _hip_runtime()
    stream = ko.Stream()
    rows, cols = 1024, 768
    m, n, k = 512, 768, 256  # the 16-bit GEMM splits K over the waves of its workgroups here
    x = inputs.normal_f32((rows, cols), 501, 0.0, 4.0)
    g = inputs.normal_f32((cols,), 502, 1.0, 0.1)
    vl = np.array([700, 13, 768, 0], np.int32)
    dx, dg, dvl = ko.DeviceBuffer.from_numpy(x), ko.DeviceBuffer.from_numpy(g), ko.DeviceBuffer.from_numpy(vl)
    ds, dl = ko.DeviceBuffer(rows * cols * 4), ko.DeviceBuffer(rows * cols * 4)
    dmean, drstd = ko.DeviceBuffer(rows * 4), ko.DeviceBuffer(rows * 4)
    a16, b16, d16 = ko.DeviceBuffer(m * k * 2), ko.DeviceBuffer(n * k * 2), ko.DeviceBuffer(m * n * 2)
    a32, b32, d32 = ko.DeviceBuffer(m * k * 4), ko.DeviceBuffer(k * n * 4), ko.DeviceBuffer(m * n * 4)
    m2, n2, k2 = 4096, 2048, 256  # 128 tiles of 256 x 256: the persistent direct-to-LDS kernel
    a2, b2, d2 = ko.DeviceBuffer(m2 * k2 * 2), ko.DeviceBuffer(n2 * k2 * 2), ko.DeviceBuffer(m2 * n2 * 2)
    m3, n3, k3 = 8000, 2312, 256  # cut along columns and twice along rows: the most launches behind one call
    a3, b3, d3 = ko.DeviceBuffer(m3 * k3 * 2), ko.DeviceBuffer(n3 * k3 * 2), ko.DeviceBuffer(m3 * n3 * 2)
    m4, n4, k4 = 256, 256, 2048  # few tiles, deep K: slices of K into the stream's workspace, then their sum
    a4, b4, d4 = ko.DeviceBuffer(m4 * k4 * 4), ko.DeviceBuffer(k4 * n4 * 4), ko.DeviceBuffer(m4 * n4 * 4)
    ko.fill_uniform_f32(a4, m4 * k4, 511)
    ko.fill_uniform_f32(b4, k4 * n4, 512)
    m5, n5, k5 = 256, 384, 4096  # 16-bit, few tiles and a deep K: slices of K as well (with gemm16.wave_k = 1)
    a5, b5, d5 = ko.DeviceBuffer(m5 * k5 * 2), ko.DeviceBuffer(n5 * k5 * 2), ko.DeviceBuffer(m5 * n5 * 2)
    ko.fill_uniform_16(a5, m5 * k5, 513)
    ko.fill_uniform_16(b5, n5 * k5, 514)
    m7, n7, k7 = 1000, 1280, 8200  # 16-bit, a mid-size output and K beyond 8192: the pinned kernel's tiles in K slices
    a7, b7, d7 = ko.DeviceBuffer(m7 * k7 * 2), ko.DeviceBuffer(n7 * k7 * 2), ko.DeviceBuffer(m7 * n7 * 2)
    ko.fill_uniform_16(a7, m7 * k7, 516)
    ko.fill_uniform_16(b7, n7 * k7, 517)
    assert ko.gemm_plan(m7, n7, k7, sixteen_bit=True)[2] == 256
    rows6, cols6 = 8, 131072  # a few long rows: cut into pieces that hand partial results over through the workspace
    x6 = ko.DeviceBuffer.from_numpy(inputs.normal_f32((rows6, cols6), 515, 0.0, 4.0))
    s6, l6 = ko.DeviceBuffer(rows6 * cols6 * 4), ko.DeviceBuffer(rows6 * cols6 * 4)
    ko.fill_uniform_16(a3, m3 * k3, 509)
    ko.fill_uniform_16(b3, n3 * k3, 510)
    ko.fill_uniform_16(a2, m2 * k2, 507)
    ko.fill_uniform_16(b2, n2 * k2, 508)
    ko.fill_uniform_16(a16, m * k, 503)
    ko.fill_uniform_16(b16, n * k, 504)
    ko.fill_uniform_f32(a32, m * k, 505)
    ko.fill_uniform_f32(b32, k * n, 506)
    ko.synchronize()

    def chain():
        ko.softmax(dx, ds, rows, cols, dvl, rows // 4, stream=stream)
        ko.layernorm(ds, dl, rows, cols, dmean, drstd, dg, None, 1e-5, False, stream=stream)
        ko.gemm16(m, n, k, a16, b16, d16, stream=stream)
        ko.sgemm(m, n, k, a32, b32, d32, stream=stream)
        ko.gemm16(m2, n2, k2, a2, b2, d2, stream=stream)
        ko.gemm16(m3, n3, k3, a3, b3, d3, stream=stream)
        ko.sgemm(m4, n4, k4, a4, b4, d4, stream=stream)
        ko.set_tuning("gemm16.wave_k", 1)
        ko.gemm16(m5, n5, k5, a5, b5, d5, stream=stream)
        ko.set_tuning("gemm16.wave_k", 0)
        ko.softmax(x6, s6, rows6, cols6, stream=stream)
        ko.layernorm(s6, l6, rows6, cols6, stream=stream)
        ko.gemm16(m7, n7, k7, a7, b7, d7, stream=stream)

    def outputs():
        return (dl.download(np.uint32, (rows, cols)), dmean.download(np.uint32, (rows,)),
                d16.download(np.uint16, (m, n)), d32.download(np.uint32, (m, n)), d2.download(np.uint16, (m2, n2)),
                d3.download(np.uint16, (m3, n3)), d4.download(np.uint32, (m4, n4)), d5.download(np.uint16, (m5, n5)),
                l6.download(np.uint32, (rows6, cols6)), d7.download(np.uint16, (m7, n7)))

    def clear():
        for buf, nbytes in ((ds, rows * cols * 4), (dl, rows * cols * 4), (dmean, rows * 4), (d16, m * n * 2), (d32, m * n * 4),
                            (d2, m2 * n2 * 2), (d3, m3 * n3 * 2), (d4, m4 * n4 * 4), (d5, m5 * n5 * 2),
                            (s6, rows6 * cols6 * 4), (l6, rows6 * cols6 * 4), (d7, m7 * n7 * 2)):
            buf.upload(np.zeros(nbytes, np.uint8))

    chain()
    stream.synchronize()
    want = outputs()
    assert want[0].any() and want[2].any() and want[3].any() and want[6].any() and want[7].any() and want[8].any() and want[9].any()

    graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream.handle, 0) == 0  # hipStreamCaptureModeGlobal
    try:
        chain()
    finally:
        rc = hip.hipStreamEndCapture(stream.handle, ctypes.byref(graph))
    assert rc == 0 and graph.value
    assert hip.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, 0) == 0
    try:
        for replay in range(3):
            clear()
            ko.synchronize()
            assert hip.hipGraphLaunch(graph_exec, stream.handle) == 0
            stream.synchronize()
            got = outputs()
            for w, gt in zip(want, got):
                np.testing.assert_array_equal(gt, w, err_msg="replay %d" % replay)
            # eager work between replays, on the same stream and on the default one
            ko.softmax(dx, ds, rows, cols, None, 0, stream=stream)
            ko.copy_f32(dx, dl, rows * cols)
            stream.synchronize()
            ko.synchronize()
    finally:
        hip.hipGraphExecDestroy(graph_exec)
        hip.hipGraphDestroy(graph)


def test_sgemm_whose_first_sliced_call_is_captured_allocates_nothing(ko):
    """The workspace of the K-sliced SGEMM belongs to a stream and is allocated by the first sliced call on it.
    Inside a capture nothing may be allocated: a stream that has no workspace yet takes the unsliced kernels
    there.  Small integers make both paths exact, so the replayed result is checked against the exact product."""
    ko.lib()
    hip = _hip_runtime()
    stream = ko.Stream()
    m, n, k = 128, 192, 3072
    rng = np.random.default_rng(77)
    A = rng.integers(-4, 5, (m, k)).astype(np.float32)
    B = rng.integers(-4, 5, (k, n)).astype(np.float32)
    dA, dB, dD = ko.DeviceBuffer.from_numpy(A), ko.DeviceBuffer.from_numpy(B), ko.DeviceBuffer(m * n * 4)
    ko.set_tuning("sgemm.k_slices", 1)  # one-time set-up of the unsliced kernel in front of the capture, no workspace yet
    try:
        ko.sgemm(m, n, k, dA, dB, dD, stream=stream)
    finally:
        ko.set_tuning("sgemm.k_slices", 0)
    stream.synchronize()
    graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream.handle, 0) == 0
    try:
        ko.sgemm(m, n, k, dA, dB, dD, stream=stream)
    finally:
        rc = hip.hipStreamEndCapture(stream.handle, ctypes.byref(graph))
    assert rc == 0 and graph.value
    assert hip.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, 0) == 0
    try:
        for replay in range(2):
            dD.upload(np.zeros(m * n * 4, np.uint8))
            assert hip.hipGraphLaunch(graph_exec, stream.handle) == 0
            stream.synchronize()
            np.testing.assert_array_equal(dD.download(np.float32, (m, n)), A.astype(np.float64) @ B.astype(np.float64))
    finally:
        hip.hipGraphExecDestroy(graph_exec)
        hip.hipGraphDestroy(graph)
    # the same call outside a capture gets the stream its workspace and slices K
    ko.sgemm(m, n, k, dA, dB, dD, stream=stream)
    stream.synchronize()
    np.testing.assert_array_equal(dD.download(np.float32, (m, n)), A.astype(np.float64) @ B.astype(np.float64))


def _workspaces(ko):
    n = ctypes.c_int()
    ko.check(ko.harness().ko_debug_stream_workspace_count(ctypes.byref(n)))
    return n.value


def test_stream_destroy_releases_the_workspace(ko):
    """ko_stream_destroy frees the workspace a K-sliced call gave the stream: a process that creates and
    destroys more streams than the workspace table has entries (64) keeps the sliced path - same bits as on the
    first stream - and holds no more workspaces afterwards than before."""
    ko.set_tuning("gemm16.wave_k", 1)  # (by default the 16-bit GEMM splits K over the waves of a workgroup here, in one launch)
    try:
        _stream_destroy_releases_the_workspace(ko)
    finally:
        ko.set_tuning("gemm16.wave_k", 0)


def _stream_destroy_releases_the_workspace(ko):
    m, n, k = 256, 256, 2048
    assert ko.gemm_plan(m, n, k)[0] > 1 and ko.gemm_plan(m, n, k, sixteen_bit=True)[0] > 1
    A, B = inputs.uniform_f32((m, k), 41), inputs.uniform_f32((k, n), 42)
    dA, dB = ko.DeviceBuffer.from_numpy(A), ko.DeviceBuffer.from_numpy(B)
    A16 = inputs.uniform_f16((m, k), 43).view(np.uint16)
    B16 = inputs.uniform_f16((n, k), 44).view(np.uint16)
    dA16, dB16 = ko.DeviceBuffer.from_numpy(A16), ko.DeviceBuffer.from_numpy(B16)
    ko.set_tuning("sgemm.k_slices", 1)
    try:
        unsliced = ko.DeviceBuffer(m * n * 4)
        ko.sgemm(m, n, k, dA, dB, unsliced)
        ko.synchronize()
        unsliced = unsliced.download(np.uint32, (m, n))
    finally:
        ko.set_tuning("sgemm.k_slices", 0)
    base = _workspaces(ko)
    first = first16 = None
    for i in range(70):
        stream = ko.Stream()
        dD, dD16 = ko.DeviceBuffer(m * n * 4), ko.DeviceBuffer(m * n * 2)
        ko.sgemm(m, n, k, dA, dB, dD, stream=stream)
        assert _workspaces(ko) == base + 1, i
        ko.gemm16(m, n, k, dA16, dB16, dD16, stream=stream)
        assert _workspaces(ko) == base + 1, i
        stream.close()  # waits for the work, then frees the workspace
        assert _workspaces(ko) == base, i
        got, got16 = dD.download(np.uint32, (m, n)), dD16.download(np.uint16, (m, n))
        if first is None:
            first, first16 = got, got16
            assert not np.array_equal(first, unsliced)  # the sliced sum rounds differently: that path really ran
        np.testing.assert_array_equal(got, first, err_msg="stream %d" % i)
        np.testing.assert_array_equal(got16, first16, err_msg="stream %d" % i)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    assert np.abs(first.view(np.float32) - ref).max() <= 2 * k * 2.0 ** -24 * (np.abs(A) @ np.abs(B)).max()


def test_row_operators_hold_a_small_workspace_of_their_own(ko):
    """A stream that only ever cuts a few long rows into pieces holds 1 MiB, not the GEMMs' 64 MiB: free device memory
    drops by a few MiB at most on the first such call, by the large workspace when a K-sliced GEMM follows on the
    same stream (the table still counts one pair), and ko_stream_destroy gives both back."""
    hip = _hip_runtime()
    hip.hipMemGetInfo.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    rows, cols = 8, 131072
    x = ko.DeviceBuffer.from_numpy(inputs.normal_f32((rows, cols), 611, 0.0, 4.0))
    y, z = ko.DeviceBuffer(rows * cols * 4), ko.DeviceBuffer(rows * cols * 4)
    m, n, k = 256, 256, 2048
    assert ko.gemm_plan(m, n, k)[0] > 1
    dA, dB, dD = ko.DeviceBuffer(m * k * 4), ko.DeviceBuffer(k * n * 4), ko.DeviceBuffer(m * n * 4)
    ko.fill_uniform_f32(dA, m * k, 612)
    ko.fill_uniform_f32(dB, k * n, 613)
    ko.softmax(x, y, rows, cols)           # the default stream: the reference result, in pieces as well
    ko.synchronize()
    want = y.download(np.uint32, (rows, cols))
    stream = ko.Stream()
    ko.synchronize()
    base, free0 = _workspaces(ko), free_bytes()
    ko.softmax(x, z, rows, cols, stream=stream)
    ko.layernorm(z, y, rows, cols, stream=stream)
    stream.synchronize()
    assert _workspaces(ko) == base + 1
    free1 = free_bytes()
    assert free0 - free1 <= 8 << 20, "the row operators took %d bytes" % (free0 - free1)
    np.testing.assert_array_equal(z.download(np.uint32, (rows, cols)), want)
    ko.sgemm(m, n, k, dA, dB, dD, stream=stream)
    stream.synchronize()
    assert _workspaces(ko) == base + 1
    assert free1 - free_bytes() >= 60 << 20
    stream.close()
    assert _workspaces(ko) == base
    assert free_bytes() >= free0 - (1 << 20)


def test_operators_from_two_threads_on_two_streams(ko):
    """Thread-compatible entry points: two host threads, each with its own stream and buffers, run the row
    operators and the GEMMs at the same time; every result equals the single-threaded one bit for bit."""
    import threading
    ko.lib()
    rows, cols = 2048, 512
    m, n, k = 512, 512, 128

    def work(seed, stream, out):
        x = inputs.normal_f32((rows, cols), seed, 0.0, 4.0)
        dx, dy, dl = ko.DeviceBuffer.from_numpy(x), ko.DeviceBuffer(rows * cols * 4), ko.DeviceBuffer(rows * cols * 4)
        a, b, d = ko.DeviceBuffer(m * k * 4), ko.DeviceBuffer(k * n * 4), ko.DeviceBuffer(m * n * 4)
        a16, b16, d16 = ko.DeviceBuffer(m * k * 2), ko.DeviceBuffer(n * k * 2), ko.DeviceBuffer(m * n * 2)
        ms, ns, ks = 128, 128, 2048  # K-sliced: each stream sums its partial products in a workspace of its own
        a_s, b_s, d_s = ko.DeviceBuffer(ms * ks * 4), ko.DeviceBuffer(ks * ns * 4), ko.DeviceBuffer(ms * ns * 4)
        ko.fill_uniform_f32(a_s, ms * ks, seed + 5, stream=stream)
        ko.fill_uniform_f32(b_s, ks * ns, seed + 6, stream=stream)
        ko.fill_uniform_f32(a, m * k, seed + 1, stream=stream)
        ko.fill_uniform_f32(b, k * n, seed + 2, stream=stream)
        ko.fill_uniform_16(a16, m * k, seed + 3, stream=stream)
        ko.fill_uniform_16(b16, n * k, seed + 4, stream=stream)
        for _ in range(20):
            ko.softmax(dx, dy, rows, cols, stream=stream)
            ko.layernorm(dy, dl, rows, cols, stream=stream)
            ko.sgemm(m, n, k, a, b, d, stream=stream)
            ko.gemm16(m, n, k, a16, b16, d16, stream=stream)
            ko.sgemm(ms, ns, ks, a_s, b_s, d_s, stream=stream)
        if stream is not None:
            stream.synchronize()
        else:
            ko.synchronize()
        out[seed] = (dy.download(np.uint32, (rows, cols)), dl.download(np.uint32, (rows, cols)),
                     d.download(np.uint32, (m, n)), d16.download(np.uint16, (m, n)), d_s.download(np.uint32, (ms, ns)))

    want = {}
    for seed in (610, 620):
        work(seed, None, want)
    got, errors = {}, []

    def guarded(seed):
        try:
            work(seed, ko.Stream(), got)
        except Exception as e:  # surfaced below: an exception in a thread would otherwise be lost
            errors.append(e)

    threads = [threading.Thread(target=guarded, args=(seed,)) for seed in (610, 620)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(60)
    assert not errors, errors
    for seed in (610, 620):
        for w, g in zip(want[seed], got[seed]):
            np.testing.assert_array_equal(g, w)
