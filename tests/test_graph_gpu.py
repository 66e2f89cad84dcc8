"""Recording a sequence of library calls into a graph and replaying it (och_stream_begin_capture /
och_stream_end_capture / och_graph_launch) gives, at every replay, bit for bit what the same calls give when they are
launched one by one. The sequence is the small-operation pattern of a modified Gram-Schmidt sweep (dot product into a
device scalar, rank-1 update that reads it) followed by an elementwise operation, a byte fill, a full reduction into
device memory and an axis reduction. The program's own eager work and synchronisations run between the replays."""
import ctypes as C

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

orc = H.orc

pytestmark = pytest.mark.gpu


def test_graph_replays_equal_eager_launches(hip, stream):
    lib, h = oh.lib, stream.handle
    rng = np.random.default_rng(31)
    m, ncol = 1024, 6
    q0 = rng.uniform(-1, 1, (ncol, m))                     # column-major m x ncol
    x0 = rng.uniform(-1, 1, (64, 96))
    dq, dx = oh.to_device(q0, stream), oh.to_device(x0, stream)
    dr = oh.DeviceBuffer(8 * ncol * ncol, stream)
    dz, dw = oh.DeviceBuffer(x0.nbytes, stream), oh.DeviceBuffer(1000, stream)
    dsum, dax = oh.DeviceBuffer(64, stream), oh.DeviceBuffer(8 * 96, stream)
    consts = oh.to_device(np.array([1.0, 0.0, -1.0]), stream)
    one, zero, minus = [C.c_void_p(consts.address + 8 * i) for i in range(3)]
    col = lambda j: C.c_void_p(dq.address + 8 * m * j)
    rij = lambda i, j: C.c_void_p(dr.address + 8 * (i + ncol * j))
    shape, st = oh.sizes([96, 64]), oh.strides([8, 8 * 96])
    cfg = oh.ReduceAxisConfig()
    cfg.ndims, cfg.rdims = 1, 1
    cfg.size[0], cfg.strides1[0], cfg.strides2[0] = 96, 8, 8
    cfg.rsize[0], cfg.rstrides[0] = 64, 8 * 96
    cfg.ptr1, cfg.ptr2, cfg.stream = dz.ptr.value, dax.ptr.value, h

    def sequence():
        for j in range(1, ncol):
            for i in range(j):
                oh.check(lib.och_gemm(H.DOUBLE, b"T", b"N", 1, 1, m, minus, col(i), m, col(j), m, zero, rij(i, j), 1, 0, h))
                oh.check(lib.och_gemm(H.DOUBLE, b"N", b"N", m, 1, 1, one, col(i), m, rij(i, j), 1, one, col(j), m, 0, h))
        oh.check(lib.och_binary(oh.B["add"], H.DOUBLE, 2, shape, st, dx.ptr, st, dx.ptr, st, dz.ptr, h))
        oh.check(lib.och_binary(oh.B["multiply"], H.DOUBLE, 2, shape, st, dz.ptr, st, dx.ptr, st, dx.ptr, h))      # state that changes per run
        oh.check(lib.och_memset_async(dw.ptr, 0x3C, 1000, h))
        oh.check(lib.och_reduce_all_device(oh.R["sum"], H.DOUBLE, 2, shape, st, dz.ptr, None, None, 0.0, dsum.ptr, None, h))
        oh.check(lib.och_reduce_axis(oh.R["maximum"], H.DOUBLE, C.byref(cfg), 0.0))

    def snapshot():
        stream.synchronize()
        return [b.download(np.uint8).copy() for b in (dq, dx, dr, dz, dw, dsum, dax)]

    def reset():
        dq.upload(q0); dx.upload(x0)
        for b in (dr, dz, dw, dsum, dax):
            oh.check(lib.och_memset_async(b.ptr, 0, b.nbytes, h))
        stream.synchronize()

    reset()
    eager = []
    for _ in range(3):
        sequence()
        eager.append(snapshot())
    assert not np.array_equal(eager[0][1], eager[1][1])            # the runs really differ

    reset()
    oh.check(lib.och_stream_begin_capture(h))
    sequence()
    graph = C.c_void_p()
    oh.check(lib.och_stream_end_capture(h, C.byref(graph)))
    assert np.array_equal(dx.download(np.float64, x0.size).reshape(x0.shape), x0)       # recording executed nothing
    scratch = oh.to_device(x0, stream)
    for k in range(3):
        oh.check(lib.och_graph_launch(graph, h))
        got = snapshot()
        for g, e, name in zip(got, eager[k], ("Q", "x", "R", "z", "w", "sum", "axis")):
            assert np.array_equal(g, e), "replay %d: %s differs from the eager launches" % (k, name)
        # unrelated eager work and a synchronisation between the replays
        oh.check(lib.och_binary(oh.B["add"], H.DOUBLE, 2, shape, st, scratch.ptr, st, scratch.ptr, st, scratch.ptr, h))
        stream.synchronize()
    # a graph replays on its recording stream only: its reductions use that stream's partial slots and counter
    other = oh.Stream()
    assert lib.och_graph_launch(graph, other.handle) == -1 and "stream that recorded it" in lib.och_last_error().decode()
    assert lib.och_graph_launch(graph, None) == -1
    other.destroy()
    oh.check(lib.och_graph_destroy(graph))
    # recording on the default stream is refused, as is a second end without a begin
    with pytest.raises(oh.OceanHipError):
        oh.check(lib.och_stream_begin_capture(None))
    for b in (dq, dx, dr, dz, dw, dsum, dax, consts, scratch):
        b.free()


def test_graph_with_half_gemm_split_k_projection_and_gather(hip, stream):
    """The entries added after the first recording test are recordable too: the half-precision MFMA product (a kernel with
    more than 64 KB of LDS), a product cut along K (partial sums in the stream's workspace, which begin_capture creates),
    the fused Gram-Schmidt projection and a gather through an offset table. Every replay must equal the eager run."""
    lib, h = oh.lib, stream.handle
    rng = np.random.default_rng(32)
    M = N = 512; K = 128
    a16 = rng.standard_normal(M * K).astype(np.float16); b16 = rng.standard_normal(K * N).astype(np.float16)
    dA, dB, dC = oh.to_device(a16, stream), oh.to_device(b16, stream), oh.DeviceBuffer(2 * M * N, stream)
    long_a = rng.uniform(-1, 1, 64 * 16384); long_b = rng.uniform(-1, 1, 16384 * 64)
    dLA, dLB, dLC = oh.to_device(long_a, stream), oh.to_device(long_b, stream), oh.DeviceBuffer(8 * 64 * 64, stream)
    n, k = 2000, 5
    q = rng.uniform(-1, 1, n * (k + 1)) / 40
    dQ, dR = oh.to_device(q, stream), oh.DeviceBuffer(8 * k, stream)
    rows = rng.permutation(64)[:20].astype(np.int64) * (8 * 64)
    dtab = oh.to_device(rows, stream)
    import index_cases as IC
    table = IC.pointer_table([None, dtab], lambda b: b.address)
    dG = oh.DeviceBuffer(8 * 64 * 20, stream)
    one16, zero16 = np.array([0x3C00], np.uint16), np.array([0], np.uint16)
    one, zero = np.array([1.0]), np.array([0.0])

    def sequence():
        oh.check(lib.och_gemm(H.HALF, b"N", b"T", M, N, K, one16.ctypes.data_as(C.c_void_p), dA.ptr, M, dB.ptr, N, zero16.ctypes.data_as(C.c_void_p), dC.ptr, M, 1, h))
        oh.check(lib.och_gemm(H.DOUBLE, b"N", b"N", 64, 64, 16384, one.ctypes.data_as(C.c_void_p), dLA.ptr, 64, dLB.ptr, 16384, zero.ctypes.data_as(C.c_void_p), dLC.ptr, 64, 1, h))
        oh.check(lib.och_mgs_project(H.DOUBLE, n, k, dQ.ptr, n, C.c_void_p(dQ.address + 8 * n * k), dR.ptr, h))        # the last column changes per run
        oh.check(lib.och_get_index(H.DOUBLE, 2, oh.sizes([64, 20]), table, oh.strides([8, 0]), dLC.ptr, oh.strides([8, 8 * 64]), dG.ptr, h))

    outputs = (dC, dLC, dQ, dR, dG)
    def snapshot():
        stream.synchronize()
        return [b.download(np.uint8).copy() for b in outputs]
    def reset():
        dQ.upload(q)
        for b in (dC, dLC, dR, dG):
            oh.check(lib.och_memset_async(b.ptr, 0, b.nbytes, h))
        stream.synchronize()

    reset()
    eager = []
    for _ in range(3):
        sequence(); eager.append(snapshot())
    assert not np.array_equal(eager[0][2], eager[1][2])
    reset()
    oh.check(lib.och_stream_begin_capture(h))
    sequence()
    graph = C.c_void_p()
    oh.check(lib.och_stream_end_capture(h, C.byref(graph)))
    for r in range(3):
        oh.check(lib.och_graph_launch(graph, h))
        for g, e, name in zip(snapshot(), eager[r], ("half product", "split product", "Q", "r", "gather")):
            assert np.array_equal(g, e), "replay %d: %s differs from the eager launches" % (r, name)
    oh.check(lib.och_graph_destroy(graph))
    for b in (dA, dB, dC, dLA, dLB, dLC, dQ, dR, dtab, dG):
        b.free()


def test_graph_with_pipelined_gemm(hip, stream):
    """The pipelined float and double kernels in a recorded sequence: more than 64 KB of LDS, loads straight to LDS, and (for
    the float product, 320 tiles on 256 compute units) the last round cut along K with its shares in the stream's workspace
    and the kernel that adds them. Every replay equals the eager run of the same number, bit for bit; C accumulates
    (beta = 1), so the runs differ."""
    # (the sizes are chosen for 256 compute units; on another device the planner cuts differently or not at all, and the
    #  results are checked all the same)
    lib, h = oh.lib, stream.handle
    rng = np.random.default_rng(41)
    M, N, K = 2560, 2048, 17 * 32
    a32, b32 = rng.uniform(-1, 1, M * K).astype(np.float32), rng.uniform(-1, 1, K * N).astype(np.float32)
    a64, b64 = rng.uniform(-1, 1, 384 * 64), rng.uniform(-1, 1, 64 * 258)
    dA, dB, dC = oh.to_device(a32, stream), oh.to_device(b32, stream), oh.DeviceBuffer(4 * M * N, stream)
    eA, eB, eC = oh.to_device(a64, stream), oh.to_device(b64, stream), oh.DeviceBuffer(8 * 384 * 258, stream)
    half32, one32, half64, one64 = np.float32([0.5]), np.float32([1.0]), np.float64([0.5]), np.float64([1.0])
    p = lambda x: x.ctypes.data_as(C.c_void_p)

    def sequence():
        oh.check(lib.och_gemm(H.FLOAT, b"N", b"N", M, N, K, p(half32), dA.ptr, M, dB.ptr, K, p(one32), dC.ptr, M, 1, h))
        oh.check(lib.och_gemm(H.DOUBLE, b"T", b"N", 384, 258, 64, p(half64), eA.ptr, 64, eB.ptr, 64, p(one64), eC.ptr, 384, 1, h))

    def snapshot():
        stream.synchronize()
        return [dC.download(np.uint8).copy(), eC.download(np.uint8).copy()]

    def reset():
        for b in (dC, eC):
            oh.check(lib.och_memset_async(b.ptr, 0, b.nbytes, h))
        stream.synchronize()

    oh.check(lib.och_gemm_set_kernel_choice(2))
    try:
        reset()
        eager = []
        for _ in range(3):
            sequence()
            eager.append(snapshot())
        assert not np.array_equal(eager[0][0], eager[1][0])
        # the float product against numpy, to a float bound
        want = 0.5 * (a32.reshape(K, M).T.astype(np.float64) @ b32.reshape(N, K).T.astype(np.float64))
        got = eager[0][0].view(np.float32).reshape(N, M).T
        assert np.abs(got - want).max() <= 1e-5 * K
        reset()
        oh.check(lib.och_stream_begin_capture(h))
        sequence()
        graph = C.c_void_p()
        oh.check(lib.och_stream_end_capture(h, C.byref(graph)))
        assert not eC.download(np.uint8).any()                                      # recording executed nothing
        for k in range(3):
            oh.check(lib.och_graph_launch(graph, h))
            got = snapshot()
            assert np.array_equal(got[0], eager[k][0]) and np.array_equal(got[1], eager[k][1]), "replay %d differs from the eager run" % k
            stream.synchronize()
        oh.check(lib.och_graph_destroy(graph))
    finally:
        oh.check(lib.och_gemm_set_kernel_choice(0))
    for b in (dA, dB, dC, eA, eB, eC):
        b.free()


def test_first_error_is_kept_until_it_is_checked(hip, stream):
    """The status protocol of src/core/gpu/cuda.c:84-120: the first failing runtime call is remembered, later ones do not
    replace it, och_status_check reports it once and forgets it. The failures are host-side argument errors."""
    lib = oh.lib
    lib.och_status_clear()
    assert lib.och_status_check() == 0
    stream.synchronize()
    assert lib.och_status_check() == 0                              # waiting on healthy work notes nothing
    count = C.c_int()
    oh.check(lib.och_device_count(C.byref(count)))
    assert lib.och_device_set(count.value + 100) == -1               # hipErrorInvalidDevice
    first = lib.och_last_error().decode()
    graph = C.c_void_p()
    assert lib.och_stream_end_capture(stream.handle, C.byref(graph)) == -1     # a different error: the stream records nothing
    assert lib.och_status_check() == -1
    msg = lib.och_last_error().decode()
    assert msg.startswith("HIP error: ") and msg[len("HIP error: "):] in first
    assert lib.och_status_check() == 0
    oh.check(lib.och_device_set(0))
    # the stream still works
    x = oh.to_device(np.arange(8, dtype=np.float64), stream)
    out = np.zeros(1)
    oh.check(lib.och_reduce_all(oh.R["sum"], H.DOUBLE, 1, oh.sizes([8]), oh.strides([8]), x.ptr, None, None, 0.0, orc.ptr(out), None, stream.handle))
    assert out[0] == 28.0
    x.free()
