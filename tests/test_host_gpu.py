"""The GPU device module driven through Ocean's module table and a small front end, the way
Ocean's interface layer drives it (OcInitGPU -> OcModuleCore table -> OcTensorGPU_* -> device
library). Mirrors examples/python/gpu/tensors/tensor_add_02.py (transposed + broadcast add),
tensor_dtype_cast_01.py / tensor_copy_0x.py (casting and strided copies between devices),
ocean_sum_02.py, ocean_axis_reduce_04.py, ocean_gemm_01.py, and benchmark configuration 2
end to end: Z = (A.T + r + I) * F with automatic type promotion and a byte-swapped operand.

Expected values come from numpy, which fixes them independently: every step of the float64
expression is a single correctly rounded IEEE operation or an exact conversion, so the result is
bit-identical; reductions and GEMM use the tolerances of the other GPU tests.
"""
import ctypes as C

import numpy as np
import pytest

import ocean_host as host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    return host.gpu_device(0)


def binary(op, a, b, out=None):
    dst = host.TP() if out is None else out
    host.check(host.lib.OcTensor_binary(op, a, b, C.byref(dst)))
    return dst


ADD, SUB, SCALE, LT, BITSHIFT_LEFT, POWER = 0, 1, 2, 13, 25, 6


def test_init_and_table(gpu):
    assert host.lib.OcInitGPU() == 0 and host.lib.OcInitGPU() == 0           # idempotent
    assert host.lib.OcDeviceGPUCount() >= 1


@pytest.mark.parametrize("n", [96, 4096])
def test_configuration2_through_the_front_end(gpu, n):
    rng = np.random.default_rng(2024)
    A = rng.uniform(-10, 10, (n, n))
    r = rng.uniform(-10, 10, (n, 1))                                          # Ocean shape (1, n): a row
    I = rng.integers(-10, 10, (n, n), endpoint=True).astype(np.int32)
    F = rng.uniform(-10, 10, (n, n)).astype(np.float32)
    tA = host.from_numpy(A, host.DOUBLE, gpu)
    tr = host.from_numpy(r, host.DOUBLE, gpu)
    tI = host.from_numpy(I, host.INT32, gpu)
    tF = host.from_numpy(F.byteswap(), host.FLOAT, gpu, byteswapped=True)
    tAt = host.lib.OcTensor_transpose(tA)
    z = binary(ADD, tAt, tr)                       # transposed view + zero-stride broadcast
    z2 = binary(ADD, z, tI)                        # int32 operand promoted to float64 by a converting copy
    z3 = binary(SCALE, z2, tF)                     # byte-swapped float32 operand normalised and widened
    assert z3.contents.dtype == host.DOUBLE and host.shape_of(z3) == [n, n]
    want = ((A.T + r) + I.astype(np.float64)) * F.astype(np.float64)
    got = host.to_numpy(z3)
    assert got.tobytes() == want.tobytes()
    # in place: z3 += A.T
    binary(ADD, z3, tAt, out=z3)
    assert host.to_numpy(z3).tobytes() == (want + A.T).tobytes()
    for t in (tA, tr, tI, tF, tAt, z, z2, z3):
        host.lib.OcDecrefTensor(t)


def test_promotion_compare_shift_power(gpu):
    rng = np.random.default_rng(5)
    a = rng.integers(-100, 100, (7, 33)).astype(np.int16)
    b = rng.uniform(-100, 100, (7, 33)).astype(np.float32)
    ta, tb = host.from_numpy(a, host.INT16, gpu), host.from_numpy(b, host.FLOAT, gpu)
    s = binary(ADD, ta, tb)
    assert s.contents.dtype == host.FLOAT
    assert np.array_equal(host.to_numpy(s), a.astype(np.float32) + b)
    lt = binary(LT, ta, tb)
    assert lt.contents.dtype == host.BOOL and np.array_equal(host.to_numpy(lt), (a.astype(np.float32) < b).astype(np.uint8))
    cnt = rng.integers(0, 8, (7, 33)).astype(np.int32)
    tc = host.from_numpy(cnt, host.INT32, gpu)
    sh = binary(BITSHIFT_LEFT, ta, tc)             # counts are converted to int8 on the way in
    assert sh.contents.dtype == host.INT16 and np.array_equal(host.to_numpy(sh), (a.astype(np.int32) << cnt).astype(np.int16))
    e = rng.integers(0, 4, (7, 33)).astype(np.int64)
    te = host.from_numpy(e, host.INT64, gpu)
    small = host.from_numpy((a % 7).astype(np.int16), host.INT16, gpu)
    pw = binary(POWER, small, te)
    # an integer base keeps its type and the exponent is taken as int16 (OcTensor_power, tensor_itf.c:4753-4756)
    assert pw.contents.dtype == host.INT16 and np.array_equal(host.to_numpy(pw), ((a % 7).astype(np.int64) ** e).astype(np.int16))
    tf = host.from_numpy(np.full((7, 33), 0.5, np.float32), host.FLOAT, gpu)
    pf = binary(POWER, small, tf)                   # a floating exponent: both operands in the common type
    assert pf.contents.dtype == host.FLOAT and np.allclose(host.to_numpy(pf), np.sqrt((a % 7).astype(np.float32)), rtol=1e-6)
    # destination of another type: computed in the common type, then converted
    out = host.create([33, 7], host.DOUBLE, gpu)
    binary(ADD, ta, tb, out=out)
    assert np.array_equal(host.to_numpy(out), (a.astype(np.float32) + b).astype(np.float64))
    # incompatible shapes are reported, not computed
    bad = host.from_numpy(np.zeros((7, 5), np.float32), host.FLOAT, gpu)
    with pytest.raises(host.OceanError, match="not compatible"):
        binary(ADD, ta, bad)


def test_copy_between_devices_with_cast_strides_and_byte_order(gpu):
    rng = np.random.default_rng(6)
    cpu = host.cpu_device()
    src = rng.integers(-32768, 32767, (64, 40, 66), dtype=np.int16, endpoint=True)
    ts = host.from_numpy(src.byteswap(), host.INT16, None, byteswapped=True)       # host tensor, other byte order
    view = host.lib.OcTensor_slice(ts, 0, 1, 32, 2)                                  # every second element of dimension 0
    d = host.create([32, 40, 64], host.FLOAT, gpu)
    host.check(host.lib.OcTensor_copy(view, d))                                      # upload raw, swap + cast + gather on the device
    want = src[:, :, 1:65:2].astype(np.float32)
    assert np.array_equal(host.to_numpy(d), want)
    # back into a strided, byte-swapped host tensor of another type
    back = host.create([64, 40, 64], host.DOUBLE, cpu)
    C.memset(host.data_address(back), 0, back.contents.storage.contents.size)
    bview = host.lib.OcTensor_slice(back, 0, 0, 32, 2)
    host.lib.OcTensor_setByteswapped(bview, 1)
    host.check(host.lib.OcTensor_copy(d, bview))
    raw = np.empty((64, 40, 64), np.float64)
    C.memmove(raw.ctypes.data, host.data_address(back), raw.nbytes)
    assert np.array_equal(raw[:, :, 0::2].byteswap(), want.astype(np.float64))
    assert not raw[:, :, 1::2].any()                                                 # the gaps were not touched


def test_reductions_and_axis_reductions(gpu):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((50, 70, 90)).astype(np.float32)
    t = host.from_numpy(x, host.FLOAT, gpu)
    s = host.Scalar()
    host.check(host.lib.OcTensor_reduceAll(15, t, 0.0, C.byref(s)))
    assert s.dtype == host.FLOAT and abs(s.get() - x.astype(np.float64).sum()) <= 1e-5 * np.abs(x).sum()
    host.check(host.lib.OcTensor_reduceAll(21, t, 0.0, C.byref(s)))
    assert s.get() == x.max()
    host.check(host.lib.OcTensor_reduceAll(27, t, 0.0, C.byref(s)))
    assert abs(s.get() - np.linalg.norm(x.astype(np.float64))) <= 1e-5 * np.linalg.norm(x)
    xi = rng.integers(-100, 100, (50, 70, 90)).astype(np.int8)
    ti = host.from_numpy(xi, host.INT8, gpu)
    host.check(host.lib.OcTensor_reduceAll(15, ti, 0.0, C.byref(s)))
    assert s.dtype == host.INT64 and s.get() == int(xi.astype(np.int64).sum())
    # a strided view: every second row, reversed along the last Ocean dimension
    v = host.lib.OcTensor_slice(t, 1, 1, 30, 2)                 # Ocean dims (90, 70, 50) -> (90, 30, 50)
    v2 = host.lib.OcTensor_slice(v, 2, 49, 50, -1)
    xv = x[::-1, 1:61:2, :]
    for axes, keep in (([0], 0), ([1], 1), ([0, 2], 0), ([2], 0), ([0, 1, 2], 1)):
        dst = host.TP()
        host.check(host.lib.OcTensor_axisReduce(15, v2, len(axes), (C.c_int * len(axes))(*axes), keep, 0.0, C.byref(dst)))
        np_axes = tuple(2 - a for a in axes)
        want = xv.astype(np.float64).sum(axis=np_axes, keepdims=bool(keep))
        got = host.to_numpy(dst)
        assert got.shape == want.shape
        assert np.allclose(got, want, rtol=0, atol=1e-5 * np.abs(xv).sum(axis=np_axes, keepdims=bool(keep)).max())
        dmin = host.TP()
        host.check(host.lib.OcTensor_axisReduce(22, v2, len(axes), (C.c_int * len(axes))(*axes), keep, 0.0, C.byref(dmin)))
        assert np.array_equal(host.to_numpy(dmin), xv.min(axis=np_axes, keepdims=bool(keep)))
    with pytest.raises(host.OceanError, match="Repeated axis"):
        host.check(host.lib.OcTensor_axisReduce(15, t, 2, (C.c_int * 2)(1, 1), 0, 0.0, C.byref(host.TP())))


def test_gemm_through_the_front_end(gpu):
    rng = np.random.default_rng(9)
    m, n, k = 150, 70, 90
    A = rng.uniform(-1, 1, (k, m))                 # Ocean (m, k), column-major
    B = rng.uniform(-1, 1, (n, k))                 # Ocean (k, n)
    tA, tB = host.from_numpy(A, host.DOUBLE, gpu), host.from_numpy(B, host.DOUBLE, gpu)
    c = host.TP()
    host.check(host.lib.OcTensor_mtimes(tA, tB, C.byref(c)))
    want = (A.T @ B.T).T                           # numpy layout of the Ocean (m, n) result
    assert host.shape_of(c) == [m, n]
    assert np.linalg.norm(host.to_numpy(c) - want) <= 1e-13 * np.linalg.norm(np.abs(A.T) @ np.abs(B.T))
    # transposed views are used through the opposite mode instead of being copied: (A')' * B
    At = host.from_numpy(np.ascontiguousarray(A.T), host.DOUBLE, gpu)        # Ocean (k, m)
    v = host.lib.OcTensor_transpose(At)                                      # Ocean (m, k), rows contiguous
    c2 = host.TP()
    alpha, beta = host.scalar(host.DOUBLE, 2.0), host.scalar(host.DOUBLE, -1.0)
    c0 = rng.uniform(-1, 1, (n, m))
    c2 = host.from_numpy(c0, host.DOUBLE, gpu)
    host.check(host.lib.OcTensor_gemm(C.byref(alpha), v, b"N", tB, b"N", C.byref(beta), C.byref(c2)))
    want2 = 2.0 * want - c0
    assert np.linalg.norm(host.to_numpy(c2) - want2) <= 1e-13 * (2 * np.linalg.norm(np.abs(A.T) @ np.abs(B.T)) + np.linalg.norm(c0))
    # mixed types promote: int32 x float32 -> double; integer product is exact
    Ai = rng.integers(-5, 5, (k, m)).astype(np.int32); Bi = rng.integers(-5, 5, (n, k)).astype(np.int32)
    ci = host.TP()
    host.check(host.lib.OcTensor_mtimes(host.from_numpy(Ai, host.INT32, gpu), host.from_numpy(Bi, host.INT32, gpu), C.byref(ci)))
    assert ci.contents.dtype == host.INT32 and np.array_equal(host.to_numpy(ci), (Ai.T @ Bi.T).T)
    with pytest.raises(host.OceanError, match="Inner dimensions"):
        host.check(host.lib.OcTensor_mtimes(tA, tA, C.byref(host.TP())))


def test_unary_and_fill(gpu):
    rng = np.random.default_rng(10)
    x = rng.uniform(0.5, 9, (12, 31))
    t = host.from_numpy(x, host.DOUBLE, gpu)
    out = host.TP()
    host.check(host.lib.OcTensor_unary(17, t, C.byref(out)))               # sqrt
    assert np.array_equal(host.to_numpy(out), np.sqrt(x))
    isn = host.TP()
    host.check(host.lib.OcTensor_unary(36, t, C.byref(isn)))               # isnan -> bool
    assert isn.contents.dtype == host.BOOL and not host.to_numpy(isn).any()
    val = host.scalar(host.DOUBLE, 3.25)
    host.check(host.lib.OcTensor_fill(t, C.byref(val)))
    assert (host.to_numpy(t) == 3.25).all()


def test_masked_fill_fill_nan_and_steps_through_the_table(gpu):
    """Tensor_maskedFill, Tensor_fillNaN, Tensor_stepsInt64 and Tensor_stepsDouble reached the way Ocean's interface
    reaches them (tensor_itf.c:2788-2908, 2965-3075): the value converted to the tensor's type, the mask of another
    type and shape brought to bool and broadcast. Expected values: numpy.where and offset + i * step."""
    rng = np.random.default_rng(77)
    x = rng.uniform(-5, 5, (20, 33)).astype(np.float32)                       # Ocean shape (33, 20)
    t = host.from_numpy(x, host.FLOAT, gpu)
    mask = (rng.random((20, 33)) < 0.4).astype(np.uint8)
    tm = host.from_numpy(mask, host.BOOL, gpu)
    val = host.scalar(host.DOUBLE, 2.5)                                       # a double scalar into a float tensor
    host.check(host.lib.OcTensor_maskedFill(t, tm, C.byref(val)))
    want = np.where(mask != 0, np.float32(2.5), x)
    assert host.to_numpy(t).tobytes() == want.tobytes()
    # an int32 mask on the HOST with one row (Ocean shape (33, 1)), broadcast along the second dimension
    row = rng.integers(-1, 2, (1, 33)).astype(np.int32)
    trow = host.from_numpy(row, host.INT32)
    val = host.scalar(host.INT64, -7)
    host.check(host.lib.OcTensor_maskedFill(t, trow, C.byref(val)))
    want = np.where(np.broadcast_to(row != 0, (20, 33)), np.float32(-7), want)
    assert host.to_numpy(t).tobytes() == want.tobytes()
    # a transposed view as destination: the mask follows the view's shape
    tt = host.lib.OcTensor_transpose(t)                                       # Ocean shape (20, 33)
    mask2 = (rng.random((33, 20)) < 0.3).astype(np.uint8)
    tm2 = host.from_numpy(mask2, host.BOOL, gpu)
    val = host.scalar(host.FLOAT, 0.125)
    host.check(host.lib.OcTensor_maskedFill(tt, tm2, C.byref(val)))
    want = np.where(mask2.T != 0, np.float32(0.125), want)
    assert host.to_numpy(t).tobytes() == want.tobytes()
    # a mask of the wrong shape is refused
    bad = host.from_numpy(np.zeros((3, 5), np.uint8), host.BOOL, gpu)
    assert host.lib.OcTensor_maskedFill(t, bad, C.byref(val)) != 0
    # integer destination: the value is converted with C's rule
    xi = rng.integers(-100, 100, (7, 9)).astype(np.int16)
    ti = host.from_numpy(xi, host.INT16, gpu)
    mi = (rng.random((7, 9)) < 0.5).astype(np.uint8)
    val = host.scalar(host.DOUBLE, -3.75)
    host.check(host.lib.OcTensor_maskedFill(ti, host.from_numpy(mi, host.BOOL, gpu), C.byref(val)))
    assert np.array_equal(host.to_numpy(ti), np.where(mi != 0, np.int16(-3), xi))
    # fillNaN
    y = rng.uniform(-1, 1, (6, 11)); y[rng.random((6, 11)) < 0.3] = np.nan
    ty = host.from_numpy(y, host.DOUBLE, gpu)
    val = host.scalar(host.FLOAT, 9.5)
    host.check(host.lib.OcTensor_fillNaN(ty, C.byref(val)))
    assert host.to_numpy(ty).tobytes() == np.where(np.isnan(y), 9.5, y).tobytes()
    host.check(host.lib.OcTensor_fillNaN(ti, C.byref(val)))                   # integers hold no NaN: untouched
    assert np.array_equal(host.to_numpy(ti), np.where(mi != 0, np.int16(-3), xi))
    # steps: the flat index runs over Ocean's first dimension fastest = numpy's C order of the reversed shape
    ts = host.create([5, 4, 3], host.INT32, gpu)
    host.check(host.lib.OcTensor_stepsInt64(ts, -4, 3))
    assert np.array_equal(host.to_numpy(ts), (-4 + 3 * np.arange(60)).reshape(3, 4, 5).astype(np.int32))
    td = host.create([8, 5], host.FLOAT, gpu)
    host.check(host.lib.OcTensor_stepsDouble(td, 0.1, 0.3))
    assert host.to_numpy(td).tobytes() == (0.1 + np.arange(40).astype(np.float64) * 0.3).astype(np.float32).reshape(5, 8).tobytes()
    tdt = host.lib.OcTensor_transpose(td)                                     # Ocean shape (5, 8) over the same memory
    host.check(host.lib.OcTensor_stepsInt64(tdt, 100, 1))
    assert np.array_equal(host.to_numpy(td), (100 + np.arange(40)).reshape(8, 5).T.astype(np.float32))


def test_public_device_object_and_reference_named_helpers(gpu):
    """OcDeviceGPU_updateProperties (device_gpu.c:620-637) refreshes freeGlobalMem inside the device object, whose public
    part carries the reference's field names; the buffer functions are callable under the reference's names."""
    pub = host.gpu_public_properties(gpu)
    assert pub.warpSize == 64 and pub.multiProcessorCount >= 64 and pub.totalGlobalMem >= (1 << 30)
    assert pub.maxWarpsPerMultiProcessor * 64 == pub.maxThreadsPerMultiProcessor and pub.major >= 9
    before = host.gpu_public_properties(gpu, update=True).freeGlobalMem
    assert 0 < before <= pub.totalGlobalMem
    big = host.create([1 << 26], host.DOUBLE, gpu)
    after = host.gpu_public_properties(gpu, update=True).freeGlobalMem
    assert after <= before - (1 << 28)
    cpu_dev = host.cpu_device()
    host.lib.OcDeviceGPU_updateProperties.argtypes = [C.c_void_p]
    assert host.lib.OcDeviceGPU_updateProperties(cpu_dev) == -1               # not a GPU device
    # OcBufferGPU_copyHostToStorage / copyStorageToHost / zero on the storage of `big` (storage_gpu.c:252-302)
    st = big.contents.storage
    data = np.arange(1000, dtype=np.float64)
    back = np.zeros(1000)
    for fn in (host.lib.OcBufferGPU_copyHostToStorage, host.lib.OcBufferGPU_copyStorageToHost):
        fn.argtypes = [C.POINTER(host.Storage), C.c_ssize_t, C.c_ssize_t, C.c_void_p]
    host.lib.OcBufferGPU_zero.argtypes = [C.POINTER(host.Storage), C.c_void_p, C.c_int, C.c_ssize_t]
    host.check(host.lib.OcBufferGPU_copyHostToStorage(st, 4096, data.nbytes, data.ctypes.data))
    host.check(host.lib.OcBufferGPU_copyStorageToHost(st, 4096, back.nbytes, back.ctypes.data))
    assert np.array_equal(back, data)
    host.check(host.lib.OcBufferGPU_zero(st, st.contents.data + 4096 + 80, host.DOUBLE, 500))
    host.check(host.lib.OcBufferGPU_copyStorageToHost(st, 4096, back.nbytes, back.ctypes.data))
    assert np.array_equal(back[:10], data[:10]) and not back[10:510].any() and np.array_equal(back[510:], data[510:])
    host.lib.OcDecrefTensor(big)
    # the registration pieces fill a caller's table: the same entries as the registered one
    table = (C.c_void_p * 256)()
    host.lib.OcRegisterStorageGPU.argtypes = [C.c_void_p]; host.lib.OcRegisterTensorGPU.argtypes = [C.c_void_p]
    assert host.lib.OcRegisterStorageGPU(table) == 0 and host.lib.OcRegisterTensorGPU(table) == 0
    assert sum(1 for v in table if v) > 120


def test_find_and_mask_to_offset_through_the_table(gpu):
    rng = np.random.default_rng(12)
    mask = (rng.random((9, 40, 33)) < 0.2).astype(np.uint8)                 # Ocean dims (33, 40, 9)
    t = host.from_numpy(mask, host.BOOL, gpu)
    idx = host.lib.OcTensor_find(t)
    assert idx and idx.contents.dtype == host.INT64
    got = host.to_numpy(idx)                                                # numpy (nnz, ndims)
    want = np.stack(np.nonzero(mask), axis=1)[:, ::-1]                      # C-order walk = Ocean dimension 0 fastest
    assert np.array_equal(got, want)
    strides = host._arr([8, 8 * 33, 8 * 33 * 40])
    off = host.lib.OcTensor_maskToOffset(t, strides)
    assert np.array_equal(host.to_numpy(off), want @ np.array([8, 8 * 33, 8 * 33 * 40]))
    f = host.from_numpy(np.zeros((3, 3), np.float32), host.FLOAT, gpu)
    assert not host.lib.OcTensor_find(f) and b"Boolean" in host.lib.OcError_lastMessage()


def test_batched_gemm_with_broadcast_through_the_front_end(gpu):
    """Dimensions beyond the second index independent products (tensor_blas_gpu.c:171-252); here one batched launch.
    A is (m, k, 3, 2), B is (k, n, 1, 2): B is shared along dimension 2."""
    rng = np.random.default_rng(21)
    m, n, k = 40, 30, 50
    A = rng.uniform(-1, 1, (2, 3, k, m))           # numpy axes are Ocean's reversed
    B = rng.uniform(-1, 1, (2, 1, n, k))
    tA, tB = host.from_numpy(A, host.DOUBLE, gpu), host.from_numpy(B, host.DOUBLE, gpu)
    c = host.TP()
    host.check(host.lib.OcTensor_mtimes(tA, tB, C.byref(c)))
    assert host.shape_of(c) == [m, n, 3, 2]
    want = np.einsum("xykm,xznk->xynm", A, np.broadcast_to(B, (2, 1, n, k)))
    got = host.to_numpy(c)
    assert got.shape == want.shape
    assert np.linalg.norm(got - want) <= 1e-13 * np.linalg.norm(np.einsum("xykm,xznk->xynm", np.abs(A), np.abs(B)))
    # accumulate into an existing destination: C <- 2 * A * B - C, integers, exact
    Ai = rng.integers(-4, 4, (3, k, m)).astype(np.int64); Bi = rng.integers(-4, 4, (3, n, k)).astype(np.int64)
    C0 = rng.integers(-9, 9, (3, n, m)).astype(np.int64)
    tc = host.from_numpy(C0, host.INT64, gpu)
    alpha, beta = host.scalar(host.INT64, 2), host.scalar(host.INT64, -1)
    host.check(host.lib.OcTensor_gemm(C.byref(alpha), host.from_numpy(Ai, host.INT64, gpu), b"N", host.from_numpy(Bi, host.INT64, gpu), b"N",
                                      C.byref(beta), C.byref(tc)))
    assert np.array_equal(host.to_numpy(tc), 2 * np.einsum("xkm,xnk->xnm", Ai, Bi) - C0)
    with pytest.raises(host.OceanError, match="not compatible"):
        host.check(host.lib.OcTensor_mtimes(tA, host.from_numpy(rng.uniform(-1, 1, (2, 2, n, k)), host.DOUBLE, gpu), C.byref(host.TP())))


def test_gram_schmidt_with_the_fused_projection(gpu):
    """A modified Gram-Schmidt factorisation A = Q R through the front end: every column is made orthogonal to the finished
    ones by OcTensorGPU_projectColumns (one launch; the reference's example issues a dot product and an update per pair),
    normalised with norm2 and a scale. Checked through what a QR factorisation must satisfy: Q'Q = I, Q R = A, R upper
    triangular with the norms on its diagonal; and against numpy's QR up to the signs of the columns."""
    rng = np.random.default_rng(21)
    n, k = 300, 24
    A = rng.uniform(-1, 1, (k, n))                      # numpy (k, n) = Ocean (n, k): columns contiguous
    tA = host.from_numpy(A, host.DOUBLE, gpu)
    tR = host.from_numpy(np.zeros((k, k)), host.DOUBLE, gpu)
    NORM2, DIVIDE = 27, 3
    for j in range(k):
        colj = host.lib.OcTensor_slice(tA, 1, j, 1, 1)               # Ocean (n, 1)
        vj = host.lib.OcTensor_slice(tA, 1, j, 1, 1)
        vj.contents.ndims = 1                                        # the column as a vector
        if j > 0:
            Qj = host.lib.OcTensor_slice(tA, 1, 0, j, 1)
            rj = host.lib.OcTensor_slice(tR, 1, j, 1, 1); rj.contents.ndims = 1; rj.contents.size[0] = j; rj.contents.nelem = j
            host.check(host.lib.OcTensorGPU_projectColumns(Qj, vj, rj))
        nrm = host.Scalar()
        host.check(host.lib.OcTensor_reduceAll(NORM2, vj, 0.0, C.byref(nrm)))
        d = nrm.get()
        host.check(host.lib.OcTensor_fill(host.lib.OcTensor_slice(host.lib.OcTensor_slice(tR, 1, j, 1, 1), 0, j, 1, 1), C.byref(host.scalar(host.DOUBLE, d))))
        inv = host.from_numpy(np.array([1.0 / d]), host.DOUBLE, gpu)
        out = vj
        host.check(host.lib.OcTensor_binary(SCALE, vj, host.lib.OcTensor_broadcastTo(inv, 1, host._arr([n])), C.byref(out)))
    Q = host.to_numpy(tA).T                              # (n, k)
    R = host.to_numpy(tR).T                              # (k, k): column j holds the coefficients of column j
    assert np.allclose(np.tril(R, -1), 0)
    assert np.linalg.norm(Q.T @ Q - np.eye(k)) < 1e-12
    assert np.linalg.norm(Q @ R - A.T) < 1e-12 * np.linalg.norm(A)
    qn, rn = np.linalg.qr(A.T)
    sign = np.sign(np.diag(rn))
    assert np.linalg.norm(Q - qn * sign) < 1e-10 and np.linalg.norm(R - (rn.T * sign).T) < 1e-10
    # argument checks
    with pytest.raises(host.OceanError, match="same GPU"):
        host.check(host.lib.OcTensorGPU_projectColumns(tA, host.from_numpy(np.zeros(n), host.DOUBLE), None))
    with pytest.raises(host.OceanError, match="data types"):
        host.check(host.lib.OcTensorGPU_projectColumns(tA, host.from_numpy(np.zeros(n, np.float32), host.FLOAT, gpu), None))
    with pytest.raises(host.OceanError, match="sizes"):
        host.check(host.lib.OcTensorGPU_projectColumns(tA, host.from_numpy(np.zeros(n + 1), host.DOUBLE, gpu), None))


def test_complex_half_product_falls_back_to_complex_float(gpu):
    """The device module multiplies half but not complex-half matrices (Tensor_gemmSupportedOn); for complex-half the front
    end computes in complex-float and converts the result back, as tensor_itf.c:6388-6400 and 6756-6758 do."""
    rng = np.random.default_rng(17)
    m, n, k = 40, 24, 56
    A = (rng.integers(-4, 5, (k, m)) + 1j * rng.integers(-4, 5, (k, m))).astype(np.complex64)       # Ocean (m, k)
    B = (rng.integers(-4, 5, (n, k)) + 1j * rng.integers(-4, 5, (n, k))).astype(np.complex64)       # Ocean (k, n)
    host.lib.OcTensor_ensure.argtypes = [C.POINTER(host.TP), C.c_int, C.c_void_p]
    tA, tB = host.from_numpy(A, host.CFLOAT, gpu), host.from_numpy(B, host.CFLOAT, gpu)
    host.check(host.lib.OcTensor_ensure(C.byref(tA), host.CHALF, gpu)); host.check(host.lib.OcTensor_ensure(C.byref(tB), host.CHALF, gpu))
    assert tA.contents.dtype == host.CHALF
    c = host.TP()
    host.check(host.lib.OcTensor_mtimes(tA, tB, C.byref(c)))
    assert c.contents.dtype == host.CHALF and host.shape_of(c) == [m, n]
    host.check(host.lib.OcTensor_ensure(C.byref(c), host.CFLOAT, gpu))
    want = (A.T @ B.T).T                                   # small integers: every partial sum is exact in float, results below 2048 exact in half
    got = host.to_numpy(c)
    assert np.abs(want).max() < 2048 and np.array_equal(got, want)
    # half itself runs on the device module directly
    hA, hB = host.from_numpy(A.real.copy(), host.FLOAT, gpu), host.from_numpy(B.real.copy(), host.FLOAT, gpu)
    host.check(host.lib.OcTensor_ensure(C.byref(hA), host.HALF, gpu)); host.check(host.lib.OcTensor_ensure(C.byref(hB), host.HALF, gpu))
    ch = host.TP()
    host.check(host.lib.OcTensor_mtimes(hA, hB, C.byref(ch)))
    assert ch.contents.dtype == host.HALF
    host.check(host.lib.OcTensor_ensure(C.byref(ch), host.FLOAT, gpu))
    assert np.array_equal(host.to_numpy(ch), (A.real.T @ B.real.T).T)


def test_negative_of_unsigned_takes_the_signed_type(gpu):
    """-arange(5, uint8) is an int16 tensor 0 -1 -2 -3 -4 (examples/python/cpu/tensors/tensor_negative_01.ref; the
    interface casts to the signed type before it calls the module, tensor_itf.c:3637-3651); uint64 goes to double."""
    import ocean_hip as oh
    for dt, np_t, want_dt, want_np in ((host.UINT8, np.uint8, host.INT16, np.int16), (host.UINT16, np.uint16, host.INT32, np.int32),
                                       (host.UINT32, np.uint32, host.INT64, np.int64), (host.UINT64, np.uint64, host.DOUBLE, np.float64),
                                       (host.INT8, np.int8, host.INT8, np.int8)):
        t = host.from_numpy(np.arange(5, dtype=np_t), dt, gpu)
        out = host.TP()
        host.check(host.lib.OcTensor_unary(oh.U["negative"], t, C.byref(out)))
        assert out.contents.dtype == want_dt
        assert np.array_equal(host.to_numpy(out), -np.arange(5).astype(want_np))


def _activity(gpu):
    rec, wait, streams = C.c_long(), C.c_long(), C.c_long()
    host.check(host.lib.OcDeviceGPU_activity(gpu, C.byref(rec), C.byref(wait), C.byref(streams)))
    return rec.value, wait.value, streams.value


def test_every_storage_has_its_own_stream_and_operations_are_ordered_by_events(gpu):
    """The reference gives every GPU storage a stream of its own (no default stream on GPU devices, storage.c:94-103)
    and orders operations by the read / write protocol alone (storage.c:141-222). Here the operands of a binary
    operation, a copy, an axis reduction and a GEMM all live on different streams, and every step is followed at once
    by an operation on ANOTHER stream that overwrites one of its inputs: without the event protocol (startRead /
    update / finishRead) the overwrite overtakes the reader and the results below are wrong. Sizes are large enough
    (64 MB per tensor) that the readers are still running when the overwrites are issued."""
    rng = np.random.default_rng(31)
    n = 2896                                                                    # n * n doubles = 64 MB
    X, Y = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    rec0, wait0, _ = _activity(gpu)
    tx, ty = host.from_numpy(X, host.DOUBLE, gpu), host.from_numpy(Y, host.DOUBLE, gpu)
    streams = {tx.contents.storage.contents.stream, ty.contents.storage.contents.stream}
    assert None not in streams and len(streams) == 2
    seven, three = host.scalar(host.DOUBLE, 7.0), host.scalar(host.DOUBLE, 3.0)
    for rep in range(3):
        # binary operation on z's stream, then its first input overwritten on that input's own stream
        z = binary(ADD, tx, ty)
        assert z.contents.storage.contents.stream not in streams
        host.check(host.lib.OcTensor_fill(tx, C.byref(seven)))
        # copy (with a cast) out of z on the copy's stream, then z overwritten
        c = host.create([n, n], host.FLOAT, gpu)
        host.check(host.lib.OcTensor_copy(z, c))
        host.check(host.lib.OcTensor_fill(z, C.byref(three)))
        # axis reduction of the copy into a tensor on yet another stream, then the copy overwritten
        r = host.TP()
        host.check(host.lib.OcTensor_axisReduce(15, c, 1, (C.c_int * 1)(0), 0, 0.0, C.byref(r)))
        host.check(host.lib.OcTensor_fill(c, C.byref(host.scalar(host.FLOAT, 1.0))))
        z32 = (X + Y).astype(np.float32)                                         # the cast is exact arithmetic: one rounding
        ref = z32.sum(axis=1, dtype=np.float64)
        assert np.abs(host.to_numpy(r) - ref).max() <= 1e-5 * np.abs(z32).sum(axis=1, dtype=np.float64).max()
        assert host.to_numpy(z).min() == 3.0 and host.to_numpy(tx).max() == 7.0 and host.to_numpy(c).max() == 1.0
        # restore x for the next round (upload waits for the storage's outstanding work)
        host.lib.OcDecrefTensor(tx)
        tx = host.from_numpy(X, host.DOUBLE, gpu)
        for t in (z, c, r):
            host.lib.OcDecrefTensor(t)
    # GEMM: C on its own stream reads A and B, which are overwritten right after the call
    m = 1024
    A, B = rng.uniform(-1, 1, (m, m)), rng.uniform(-1, 1, (m, m))
    ta, tb = host.from_numpy(A, host.DOUBLE, gpu), host.from_numpy(B, host.DOUBLE, gpu)
    c = host.TP()
    host.check(host.lib.OcTensor_mtimes(ta, tb, C.byref(c)))
    host.check(host.lib.OcTensor_fill(ta, C.byref(seven))); host.check(host.lib.OcTensor_fill(tb, C.byref(seven)))
    want = (A.T @ B.T).T
    assert np.linalg.norm(host.to_numpy(c) - want) <= 1e-13 * m * np.linalg.norm(want)
    rec1, wait1, _ = _activity(gpu)
    assert rec1 - rec0 >= 30 and wait1 - wait0 >= 30                            # the protocol really ran
    for t in (tx, ty, ta, tb, c):
        host.lib.OcDecrefTensor(t)


def test_index_tables_on_their_own_streams(gpu):
    """Gather and scatter through offset tables that were written just before, on storages (and streams) of their own,
    by addIfNegative + indexToOffset: the gather must wait for the tables (tensor_index_gpu.c:155-172, 199-216)."""
    rng = np.random.default_rng(32)
    rows, cols, picks = 4096, 2048, 1 << 15
    T = rng.uniform(-1, 1, (cols, rows))                                        # Ocean shape (rows, cols): dimension 0 fastest
    idx = np.stack([rng.integers(-rows, rows, picks), rng.integers(-cols, cols, picks)], axis=1).astype(np.int64)   # Ocean [2, picks]
    host.lib.OcTensor_getIndexed.argtypes = [host.TP, host.TP, C.POINTER(host.TP)]
    host.lib.OcTensor_setIndexed.argtypes = [host.TP, host.TP, host.TP]
    t, ti = host.from_numpy(T, host.DOUBLE, gpu), host.from_numpy(idx, host.INT64, gpu)
    out = host.TP()
    host.check(host.lib.OcTensor_getIndexed(t, ti, C.byref(out)))
    got = host.to_numpy(out)
    assert got.shape == (picks,) and np.array_equal(got, T[idx[:, 1], idx[:, 0]])
    # scatter: distinct positions, so the result does not depend on the order of the writes
    flat = rng.choice(rows * cols, picks, replace=False)
    idx2 = np.stack([flat % rows, flat // rows], axis=1).astype(np.int64)
    vals = rng.uniform(5, 6, picks)
    ti2, tv = host.from_numpy(idx2, host.INT64, gpu), host.from_numpy(vals, host.DOUBLE, gpu)
    host.check(host.lib.OcTensor_setIndexed(t, ti2, tv))
    want = T.copy(); want[idx2[:, 1], idx2[:, 0]] = vals
    assert np.array_equal(host.to_numpy(t), want)
    # one indexed dimension, the rest of the tensor whole: rows of a matrix picked by (negative) column numbers
    pick = np.array([[-1], [0], [5], [-cols]], dtype=np.int64)                  # Ocean [1, 4] ... indexes dimension 0
    tp = host.from_numpy(pick, host.INT64, gpu)
    out2 = host.TP()
    host.check(host.lib.OcTensor_getIndexed(t, tp, C.byref(out2)))
    sel = [rows - 1, 0, 5, rows - cols]
    assert np.array_equal(host.to_numpy(out2), want[:, sel])
    # indices outside [-size, size) are refused before anything is addressed through them (index_itf.c:1311-1336): the
    # call returns the reference's error, launches no gather or scatter, and leaves the tensor as it was
    before = host.to_numpy(t)
    for bad_value, dim in ((rows, 0), (-rows - 1, 0), (cols, 1), (-cols - 1, 1), (1 << 40, 0)):
        bad = idx2.copy()
        bad[picks // 2, dim] = bad_value
        tb = host.from_numpy(bad, host.INT64, gpu)
        out3 = host.TP()
        assert host.lib.OcTensor_getIndexed(t, tb, C.byref(out3)) == -1 and not out3
        msg = host.lib.OcError_lastMessage().decode()
        assert "out of range" in msg and "(%d)" % bad_value in msg and "dimension %d" % dim in msg, msg
        assert host.lib.OcTensor_setIndexed(t, tb, tv) == -1
        host.lib.OcDecrefTensor(tb)
    assert np.array_equal(host.to_numpy(t), before)
    for x in (t, ti, out, ti2, tv, tp, out2):
        host.lib.OcDecrefTensor(x)


def test_temporaries_come_from_the_ring(gpu):
    """Converted operands of a binary operation live in the device's ring of three temporary storages
    (storage_itf.c:61-121): a long sequence of promoting operations creates no new streams once the ring is warm."""
    rng = np.random.default_rng(33)
    a = rng.integers(-100, 100, (512, 512)).astype(np.int32)
    b = rng.uniform(-1, 1, (512, 512))
    ta, tb = host.from_numpy(a, host.INT32, gpu), host.from_numpy(b, host.DOUBLE, gpu)
    z = binary(ADD, ta, tb)
    host.lib.OcDecrefTensor(z)
    for _ in range(4):                                                         # warm the three slots
        z = binary(ADD, ta, tb); host.lib.OcDecrefTensor(z)
    _, _, streams0 = _activity(gpu)
    for _ in range(60):
        z = binary(ADD, ta, tb)
        assert np.array_equal(host.to_numpy(z), a + b)
        host.lib.OcDecrefTensor(z)
    _, _, streams1 = _activity(gpu)
    assert streams1 == streams0                                                # streams come back from the free list, temporaries from the ring
    host.lib.OcDecrefTensor(ta); host.lib.OcDecrefTensor(tb)
