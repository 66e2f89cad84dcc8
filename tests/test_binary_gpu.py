"""Parity of the binary elementwise kernels (och_binary) with the CPU oracle.

Mirrors the reference's own GPU tests, which run the same expression on the CPU and the
GPU device and compare (examples/python/gpu/tensors/tensor_add_02.py, tensor_multiply_01.py,
tensor_divide_01.py, ocean_power_01..03.py, ocean_bitshift_01/02.py, ocean_{and,or,xor}_01.py),
extended to every (operation, type) pair, broadcast / transposed / sliced operands and the
benchmark shapes. Results must be bit-identical; the only exception is `power` on floating
and complex types, which calls pow/exp/log/sin/cos (host libm and device library differ in
the last bits): tolerance 4 ulp (float, double evaluates pow in single precision on the CPU)
and 1e-5 relative for complex.
"""
import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

pytestmark = pytest.mark.gpu

N = 4099     # odd: exercises the vector body plus the scalar tail


def operand2_data(op, dtype, n, rng):
    name = oh.BINARY_OPS[op]
    if name in ("bitshift_left", "bitshift_right"):
        lim = 63 if oh.TYPE_SIZE[dtype] == 8 else 31
        if dtype == H.BOOL:
            lim = 3
        return H.INT8, rng.integers(-lim, lim, size=n, endpoint=True).astype(np.int8)
    if name == "power" and dtype <= H.INT64:
        return H.INT16, rng.integers(-2, 6, size=n, endpoint=True).astype(np.int16)
    kind = "general"
    if name == "power":
        kind = "small"
    data = H.random_data(dtype, n, rng, kind)
    if dtype in H.INT_TYPES and name in ("divide", "true_divide", "floor_divide", "mod", "fmod"):
        data[:: 7] = 0                                   # division by zero is defined as 0
        if np.iinfo(data.dtype).min < 0 and data.dtype.itemsize <= 2:
            data[3:: 11] = -1
    return dtype, data


def operand1_data(op, dtype, n, rng):
    name = oh.BINARY_OPS[op]
    if dtype in (H.INT8, H.INT16, H.UINT8, H.UINT16):
        return H.random_data(dtype, n, rng, "full")      # 8/16-bit arithmetic is fully defined: whole range
    if name == "power":
        return H.random_data(dtype, n, rng, "positive" if dtype in H.FLOAT_TYPES else "small")
    if dtype in H.FLOAT_TYPES + H.COMPLEX_TYPES and name not in ("mod", "fmod", "floor_divide"):
        return H.random_data(dtype, n, rng, "special")
    return H.random_data(dtype, n, rng, "general")


def compare(op, dtype, got, want, rdtype):
    name = oh.BINARY_OPS[op]
    if name == "power" and dtype in H.FLOAT_TYPES + H.COMPLEX_TYPES:
        if dtype in (H.HALF, H.CHALF):
            g = got.view(np.uint16).astype(np.int32)
            w = want.view(np.uint16).astype(np.int32)
            assert np.max(np.abs(g - w)) <= 1, "half power differs by more than one code"
        elif dtype == H.DOUBLE:
            # the CPU table evaluates double pow with powf: compare at single precision
            assert H.max_ulp_diff(got.astype(np.float32), want.astype(np.float32)) <= 4
        elif dtype in H.FLOAT_TYPES:
            assert H.max_ulp_diff(got, want) <= 4
        else:
            ok = np.isclose(got, want, rtol=1e-5, atol=1e-6, equal_nan=True)
            assert ok.all()
        return
    H.assert_same_bytes(got, want, "%s %s" % (name, H.NAMES[dtype]))


CASES = [(op, dt) for op in range(len(oh.BINARY_OPS)) for dt in H.ALL_TYPES]


@pytest.mark.parametrize("op,dtype", CASES, ids=["%s-%s" % (oh.BINARY_OPS[o], H.NAMES[d]) for o, d in CASES])
def test_binary_contiguous(hip, stream, op, dtype):
    sup_gpu = bool(oh.lib.och_binary_supported(op, dtype))
    sup_cpu = bool(H.orc.lib.oracle_binary_supported(op, dtype))
    assert sup_gpu == sup_cpu, "support tables disagree"
    if not sup_gpu:
        status = oh.lib.och_binary(op, dtype, 1, oh.sizes([1]), oh.strides([0]), None, oh.strides([0]), None,
                                   oh.strides([0]), None, stream.handle)
        assert status == -1 and b"not available" in oh.lib.och_last_error()
        return
    rng = np.random.default_rng(1000 + op * 16 + dtype)
    dt2, ydata = operand2_data(op, dtype, N, rng)
    assert dt2 == oh.lib.och_binary_operand2_dtype(op, dtype)
    rdtype = oh.lib.och_binary_result_dtype(op, dtype)
    x = H.Operand.contiguous(operand1_data(op, dtype, N, rng), dtype).upload(stream)
    y = H.Operand.contiguous(ydata, dt2).upload(stream)
    z = H.Operand.contiguous(np.zeros(N, dtype=H.storage(rdtype)), rdtype).upload(stream)
    H.gpu_binary(stream, op, dtype, x, y, z)
    want = z.parent.copy()
    H.cpu_binary(op, dtype, x, y, z, want)
    got = z.download()
    for t in (x, y, z):
        t.free()
    compare(op, dtype, got, want, rdtype)


LAYOUT_OPS = ["add", "multiply", "true_divide", "lt", "max"]
LAYOUT_TYPES = [H.BOOL, H.INT8, H.INT16, H.INT32, H.UINT64, H.HALF, H.FLOAT, H.DOUBLE, H.CFLOAT, H.CDOUBLE]


@pytest.mark.parametrize("opname", LAYOUT_OPS)
@pytest.mark.parametrize("dtype", LAYOUT_TYPES, ids=[H.NAMES[d] for d in LAYOUT_TYPES])
def test_binary_layouts(hip, stream, opname, dtype):
    """Transposed, broadcast (zero stride), sliced (step 2, negative step) and 4-D operands."""
    op = oh.B[opname]
    rdtype = oh.lib.och_binary_result_dtype(op, dtype)
    rng = np.random.default_rng(77 + dtype)
    st = H.storage(dtype)
    layouts = []
    # (shape, maker of x view, maker of y view, maker of z view) on parents of the given sizes
    m, n = 67, 36
    A = H.random_data(dtype, m * n, rng).reshape(n, m)            # numpy row-major parent
    Bm = H.random_data(dtype, m * n, rng).reshape(m, n)
    row = H.random_data(dtype, m, rng).reshape(1, m)
    Z = np.zeros((n, m), dtype=H.storage(rdtype))
    layouts.append(("transposed", A, A, Bm, Bm.T, Z, Z))
    layouts.append(("row-broadcast", A, A, row, np.broadcast_to(row, (n, m)), Z, Z))
    col = H.random_data(dtype, n, rng).reshape(n, 1)
    layouts.append(("col-broadcast", A, A, col, np.broadcast_to(col, (n, m)), Z, Z))
    A2 = H.random_data(dtype, 2 * m * n, rng).reshape(n, 2 * m)
    layouts.append(("step2", A2, A2[:, ::2], Bm, Bm.T, Z, Z))
    layouts.append(("negative-step", A, A[::-1, ::-1], Bm, Bm.T[:, ::-1], Z, Z))
    Z2 = np.zeros((n, 2 * m), dtype=H.storage(rdtype))
    layouts.append(("strided-dst", A, A, Bm, Bm.T, Z2, Z2[:, 1::2]))
    P = H.random_data(dtype, 3 * 4 * 5 * 6, rng).reshape(3, 4, 5, 6)
    Q = H.random_data(dtype, 3 * 4 * 5 * 6, rng).reshape(6, 5, 4, 3)
    Z4 = np.zeros((3, 4, 5, 6), dtype=H.storage(rdtype))
    layouts.append(("4d-permuted", P, P, Q, Q.transpose(3, 2, 1, 0), Z4, Z4))
    scalar = H.random_data(dtype, 1, rng).reshape(1, 1)
    layouts.append(("scalar-broadcast", A, A, scalar, np.broadcast_to(scalar, (n, m)), Z, Z))
    for name, xp, xv, yp, yv, zp, zv in layouts:
        zp[...] = 0
        x = H.Operand(xp, xv, dtype).upload(stream)
        y = H.Operand(yp, yv, dtype).upload(stream)
        z = H.Operand(zp, zv, rdtype).upload(stream)
        H.gpu_binary(stream, op, dtype, x, y, z)
        want = zp.copy()
        H.cpu_binary(op, dtype, x, y, z, want)
        got = z.download()
        for t in (x, y, z):
            t.free()
        H.assert_same_bytes(got, want, "%s %s %s" % (opname, H.NAMES[dtype], name))


def test_binary_in_place_and_empty(hip, stream):
    rng = np.random.default_rng(5)
    xd = H.random_data(H.FLOAT, 1000, rng)
    yd = H.random_data(H.FLOAT, 1000, rng)
    x = H.Operand.contiguous(xd.copy(), H.FLOAT).upload(stream)
    y = H.Operand.contiguous(yd, H.FLOAT).upload(stream)
    oh.check(oh.lib.och_binary(oh.B["subtract"], H.FLOAT, 1, oh.sizes([1000]), oh.strides([4]), x.dptr(),
                               oh.strides([4]), y.dptr(), None, None, stream.handle))
    H.assert_same_bytes(x.download(), xd - yd, "in-place subtract")
    # empty tensor: nothing is launched, nothing is touched
    oh.check(oh.lib.och_binary(oh.B["add"], H.FLOAT, 2, oh.sizes([0, 5]), oh.strides([4, 0]), x.dptr(),
                               oh.strides([4, 0]), y.dptr(), oh.strides([4, 0]), x.dptr(), stream.handle))
    H.assert_same_bytes(x.download(), xd - yd, "empty add")
    # comparison cannot run in place
    st = oh.lib.och_binary(oh.B["lt"], H.FLOAT, 1, oh.sizes([10]), oh.strides([4]), x.dptr(), oh.strides([4]), y.dptr(),
                           None, None, stream.handle)
    assert st == -1
    x.free(); y.free()


def test_config1_scale_add_fp32(hip, stream):
    """benchmark configuration 1: z = x*y + x on contiguous float32 vectors of 2^24 elements, U(-1,1),
    as two table calls (scale, then add); bit-exact against the CPU path."""
    n = 1 << 24
    rng = np.random.default_rng(1234)
    xd = rng.uniform(-1, 1, n).astype(np.float32)
    yd = rng.uniform(-1, 1, n).astype(np.float32)
    x = H.Operand.contiguous(xd, H.FLOAT).upload(stream)
    y = H.Operand.contiguous(yd, H.FLOAT).upload(stream)
    t = H.Operand.contiguous(np.zeros(n, np.float32), H.FLOAT).upload(stream)
    z = H.Operand.contiguous(np.zeros(n, np.float32), H.FLOAT).upload(stream)
    H.gpu_binary(stream, oh.B["multiply"], H.FLOAT, x, y, t)
    H.gpu_binary(stream, oh.B["add"], H.FLOAT, t, x, z)
    tw, zw = t.parent.copy(), z.parent.copy()
    H.cpu_binary(oh.B["multiply"], H.FLOAT, x, y, t, tw)
    tt = H.Operand.contiguous(tw, H.FLOAT)
    H.cpu_binary(oh.B["add"], H.FLOAT, tt, x, z, zw)
    got = z.download()
    for o in (x, y, t, z):
        o.free()
    H.assert_same_bytes(got, zw, "config 1")
    # closed form: two separately rounded IEEE operations
    H.assert_same_bytes(got, (xd * yd) + xd, "config 1 vs numpy")


@pytest.mark.parametrize("dtype", [H.INT8, H.INT16, H.FLOAT, H.DOUBLE, H.CFLOAT], ids=lambda d: H.NAMES[d])
def test_binary_first_dimension_equals_access_width(hip, stream, dtype):
    """Rows of exactly one 128-bit access (16 int8, 8 int16, 4 float, 2 double, 2 cfloat elements) with a
    padded pitch: one group per row, so the group index is divided by one."""
    op = oh.B["add"]
    rng = np.random.default_rng(4242 + dtype)
    w = 16 // oh.TYPE_SIZE[dtype]
    for rows in (5, 64, 1000):
        A = H.random_data(dtype, rows * 2 * w, rng).reshape(rows, 2 * w)
        Bm = H.random_data(dtype, rows * 3 * w, rng).reshape(rows, 3 * w)
        Z = np.zeros((rows, 2 * w), dtype=H.storage(dtype))
        x = H.Operand(A, A[:, :w], dtype).upload(stream)
        y = H.Operand(Bm, Bm[:, w:2 * w], dtype).upload(stream)
        z = H.Operand(Z, Z[:, :w], dtype).upload(stream)
        H.gpu_binary(stream, op, dtype, x, y, z)
        want = Z.copy()
        H.cpu_binary(op, dtype, x, y, z, want)
        got = z.download()
        for t in (x, y, z):
            t.free()
        H.assert_same_bytes(got, want, "rows of one access, %d rows" % rows)
