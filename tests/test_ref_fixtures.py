"""Replays the reference's own GPU example tests against their expected-output files
(tests/golden/ref/*.ref, copied from examples/python/gpu/tensors/): the inputs are the tensors the
files print, the expectations are the results they print. Each case runs twice: on the CPU oracle
(always) and on the device library (marked gpu). Cases: tensor_add_02, ocean_min_01,
ocean_and_01 / or_01 / xor_01, ocean_logical_01, ocean_bitshift_01, ocean_sign_01, ocean_fabs_01,
ocean_axis_reduce_04, ocean_sum_02, ocean_sumabs_01, ocean_all_01, ocean_maximumabs_02,
ocean_gemm_01."""
import os

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh
import ref_format as RF

orc = H.orc
REFDIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref")


def load(name):
    return RF.parse_ref(open(os.path.join(REFDIR, name + ".ref")).read())


def tensors(items, device="gpu0"):
    return [t for t in items if isinstance(t, RF.RefTensor)]


class Engine:
    """One operation on strided numpy storage arrays, executed by the oracle or by the device library."""

    def __init__(self, gpu, stream=None):
        self.gpu, self.stream = gpu, stream

    def _operand(self, arr, dtype, view=None):
        op = H.Operand(arr, arr if view is None else view, dtype)
        return op.upload(self.stream) if self.gpu else op

    def _ptr(self, op, parent=None):
        return op.dptr() if self.gpu else op.hptr(parent)

    def _result(self, op, parent):
        if self.gpu:
            out = op.download(); op.free(); return out
        return parent

    def binary(self, name, dtype, x, y):
        op = oh.B[name]
        shape = np.broadcast_shapes(x.shape, y.shape)
        rd = oh.lib.och_binary_result_dtype(op, dtype)
        z = np.asfortranarray(np.zeros(shape, H.storage(rd)))
        a = self._operand(x, dtype, np.broadcast_to(x, shape)); b = self._operand(y, oh.lib.och_binary_operand2_dtype(op, dtype), np.broadcast_to(y, shape))
        c = self._operand(z, rd)
        if self.gpu:
            H.gpu_binary(self.stream, op, dtype, a, b, c)
        else:
            H.cpu_binary(op, dtype, a, b, c, z)
        if self.gpu:
            a.free(); b.free()
        return rd, self._result(c, z)

    def unary(self, name, dtype, x):
        op = oh.U[name]
        rd = oh.lib.och_unary_result_dtype(op, dtype)
        z = np.asfortranarray(np.zeros(x.shape, H.storage(rd)))
        a, c = self._operand(x, dtype), self._operand(z, rd)
        if self.gpu:
            H.gpu_unary(self.stream, op, dtype, a, c); a.free()
        else:
            H.cpu_unary(op, dtype, a, c, z)
        return rd, self._result(c, z)

    def cast(self, ts, td, x):
        z = np.asfortranarray(np.zeros(x.shape, H.storage(td)))
        a, c = self._operand(x, ts), self._operand(z, td)
        nd = x.ndim
        args = (ts, td, nd, oh.sizes(a.shape), oh.strides(a.strides), self._ptr(a), nd, oh.sizes(c.shape), oh.strides(c.strides), self._ptr(c, z))
        if self.gpu:
            oh.check(oh.lib.och_copy(*args, self.stream.handle)); a.free()
        else:
            assert orc.lib.oracle_copy(*args, 1) == 0
        return self._result(c, z)

    def swap_cast(self, ts, td, x):
        """converting copy that reverses the bytes of every element (real part) on the way: byte-swapped source or destination"""
        z = np.asfortranarray(np.zeros(x.shape, H.storage(td)))
        a, c = self._operand(x, ts), self._operand(z, td)
        nd = x.ndim
        args = (ts, td, nd, oh.sizes(a.shape), oh.strides(a.strides), self._ptr(a), nd, oh.sizes(c.shape), oh.strides(c.strides), self._ptr(c, z))
        if self.gpu:
            oh.check(oh.lib.och_byteswap_copy(*args, self.stream.handle)); a.free()
        else:
            assert orc.lib.oracle_byteswap_copy(*args, 1) == 0
        return self._result(c, z)

    def reshape_copy(self, ts, td, parent, view, dst_shape, swap=False):
        """copy a (strided / broadcast) view into a dense tensor of another shape with the same number of elements, converting
        (and reversing the bytes of every element when swap is set); elements are taken in Ocean's order, first index fastest"""
        z = np.asfortranarray(np.zeros(dst_shape, H.storage(td)))
        a = H.Operand(parent, view, ts); c = self._operand(z, td)
        if self.gpu:
            a.upload(self.stream)
        args = (ts, td, view.ndim, oh.sizes(a.shape), oh.strides(a.strides), self._ptr(a), z.ndim, oh.sizes(c.shape), oh.strides(c.strides), self._ptr(c, z))
        fn = (oh.lib.och_byteswap_copy if swap else oh.lib.och_copy) if self.gpu else (orc.lib.oracle_byteswap_copy if swap else orc.lib.oracle_copy)
        if self.gpu:
            oh.check(fn(*args, self.stream.handle)); a.free()
        else:
            assert fn(*args, 1) == 0
        return self._result(c, z)

    def strided_copy(self, ts, td, src_parent, src_view, dst_parent, dst_view):
        """dst_view <- src_view, converting; both are views (any strides: zero, negative) into their parent arrays. Returns
        the destination parent afterwards."""
        z = dst_parent.copy(order="K")
        zview = np.ndarray(shape=dst_view.shape, dtype=z.dtype, buffer=z, strides=dst_view.strides,
                           offset=dst_view.__array_interface__["data"][0] - dst_parent.__array_interface__["data"][0]) if dst_view.size else z
        a = H.Operand(src_parent, src_view, ts); c = H.Operand(z, zview, td)
        if self.gpu:
            a.upload(self.stream); c.upload(self.stream)
        args = (ts, td, src_view.ndim, oh.sizes(a.shape), oh.strides(a.strides), self._ptr(a), dst_view.ndim, oh.sizes(c.shape), oh.strides(c.strides), self._ptr(c, z))
        if self.gpu:
            oh.check(oh.lib.och_copy(*args, self.stream.handle)); a.free()
        else:
            assert orc.lib.oracle_copy(*args, 1) == 0
        return self._result(c, z)

    def byteswap(self, dtype, x):
        """reverse the bytes of every element in place (a byte-swapped destination of another type is written in native order
        first and swapped afterwards, tensor_copy_cpu.c:140-156)"""
        z = x.copy(order="F")
        c = self._operand(z, dtype)
        args = (dtype, z.ndim, oh.sizes(z.shape), oh.strides(z.strides), self._ptr(c, z))
        if self.gpu:
            oh.check(oh.lib.och_byteswap(*args, self.stream.handle))
        else:
            assert orc.lib.oracle_byteswap(*args, 1) == 0
        return self._result(c, z)

    def binary_inplace(self, name, dtype, parent, view, y):
        """view (op)= y on a strided view of `parent`; returns the parent afterwards"""
        op = oh.B[name]
        work = parent.copy()
        v = np.lib.stride_tricks.as_strided(work, shape=view.shape, strides=view.strides)
        a = H.Operand(work, v, dtype); b = self._operand(y, dtype, np.broadcast_to(y, view.shape))
        if self.gpu:
            a.upload(self.stream)
            H.gpu_binary(self.stream, op, dtype, a, b, a)
            out = a.download(); a.free(); b.free()
            return out
        H.cpu_binary(op, dtype, a, b, a, work)
        return work

    def fill(self, dtype, n, value):
        z = np.zeros(n, H.storage(dtype))
        c = self._operand(z, dtype)
        sc = H.raw_scalar(RF.to_storage(dtype, np.array([value])))
        args = (dtype, 1, oh.sizes([n]), oh.strides(z.strides), self._ptr(c, z), sc)
        if self.gpu:
            oh.check(oh.lib.och_fill(*args, self.stream.handle))
        else:
            assert orc.lib.oracle_fill(*args, 1) == 0
        return self._result(c, z)

    def fill_nan(self, dtype, x, value):
        z = x.copy()
        c = self._operand(z, dtype)
        sc = H.raw_scalar(RF.to_storage(dtype, np.array([value])))
        args = (dtype, z.ndim, oh.sizes(z.shape), oh.strides(z.strides), self._ptr(c, z), sc)
        if self.gpu:
            oh.check(oh.lib.och_fill_nan(*args, self.stream.handle))
        else:
            assert orc.lib.oracle_fill_nan(*args, 1) == 0
        return self._result(c, z)

    def steps_complex(self, dtype, n, offset, step):
        z = np.zeros(n, H.storage(dtype))
        c = self._operand(z, dtype)
        args = (dtype, 1, oh.sizes([n]), oh.strides(z.strides), self._ptr(c, z), oh.CDouble(offset.real, offset.imag), oh.CDouble(step.real, step.imag))
        if self.gpu:
            oh.check(oh.lib.och_steps_cdouble(*args, self.stream.handle))
        else:
            assert orc.lib.oracle_steps_cdouble(*args, 1) == 0
        return self._result(c, z)

    def gemm_raw(self, dtype, m, n, k, a, b, c0=None):
        """C (m x n, column-major, dense) <- A (m x k) * B (k x n); empty operands allowed"""
        c = np.zeros(m * n, H.storage(dtype)) if c0 is None else c0.copy()
        al = RF.to_storage(dtype, np.array([1])); be = RF.to_storage(dtype, np.array([0]))
        lda, ldb, ldc = max(m, 1), max(k, 1), max(m, 1)
        if self.gpu:
            da, db, dc = oh.to_device(a, self.stream), oh.to_device(b, self.stream), oh.to_device(c, self.stream)
            oh.check(oh.lib.och_gemm(dtype, b"N", b"N", m, n, k, orc.ptr(al), da.ptr, lda, db.ptr, ldb, orc.ptr(be), dc.ptr, ldc, 1, self.stream.handle))
            out = dc.download(c.dtype, m * n)
            for t in (da, db, dc):
                t.free()
            return out
        keep = np.zeros(1, c.dtype)                      # valid addresses for empty operands
        assert orc.lib.oracle_gemm(dtype, b"N", b"N", m, n, k, orc.ptr(al), orc.ptr(a if a.size else keep), lda, orc.ptr(b if b.size else keep), ldb,
                                   orc.ptr(be), orc.ptr(c if c.size else keep), ldc, 1) == 0
        return c

    def reduce(self, name, dtype, x, p=0.0):
        op = oh.R[name]
        rd = oh.lib.och_reduce_result_dtype(op, dtype)
        out = np.zeros(1, H.storage(rd))
        a = self._operand(x, dtype)
        if self.gpu:
            oh.check(oh.lib.och_reduce_all(op, dtype, x.ndim, oh.sizes(a.shape), oh.strides(a.strides), a.dptr(), None, None, p, orc.ptr(out), None, self.stream.handle))
            a.free()
        else:
            assert orc.lib.oracle_reduce_all(op, dtype, x.ndim, oh.sizes(a.shape), oh.strides(a.strides), a.hptr(), None, None, p, orc.ptr(out), 1) == 0
        return rd, out

    def axis(self, name, dtype, parent, view, axes, keepdims=False, p=0.0):
        op = oh.R[name]
        rd = oh.lib.och_reduce_result_dtype(op, dtype)
        kept = [view.shape[d] for d in range(view.ndim) if d not in axes]
        z = np.asfortranarray(np.zeros(kept if kept else [1], H.storage(rd)))
        a = H.Operand(parent, view, dtype); c = H.Operand(z, z if kept else z.reshape(()), rd)
        if self.gpu:
            a.upload(self.stream); c.upload(self.stream)
        cfg = H.axis_config(a, c, axes, self.stream, device=self.gpu)
        if self.gpu:
            oh.check(oh.lib.och_reduce_axis(op, dtype, cfg, p)); a.free()
        else:
            assert orc.lib.oracle_reduce_axis(op, dtype, cfg, p) == 0
        out = self._result(c, z)
        if keepdims:
            out = out.reshape([1 if d in axes else view.shape[d] for d in range(view.ndim)], order="F")
        return rd, out

    def gemm(self, dtype, alpha, a, b):
        m, k = a.shape; n = b.shape[1]
        c = np.asfortranarray(np.zeros((m, n), H.storage(dtype)))
        al = RF.to_storage(dtype, np.array([alpha])); be = RF.to_storage(dtype, np.array([0]))
        if self.gpu:
            da, db, dc = oh.to_device(a.reshape(-1, order="F"), self.stream), oh.to_device(b.reshape(-1, order="F"), self.stream), oh.to_device(c.reshape(-1, order="F"), self.stream)
            oh.check(oh.lib.och_gemm(dtype, b"N", b"N", m, n, k, orc.ptr(al), da.ptr, m, db.ptr, k, orc.ptr(be), dc.ptr, m, 1, self.stream.handle))
            out = dc.download(c.dtype, m * n).reshape((m, n), order="F")
            for t in (da, db, dc):
                t.free()
            return out
        assert orc.lib.oracle_gemm(dtype, b"N", b"N", m, n, k, orc.ptr(al), orc.ptr(a), m, orc.ptr(b), k, orc.ptr(be), orc.ptr(c), m, 1) == 0
        return c


@pytest.fixture(params=["oracle", pytest.param("device", marks=pytest.mark.gpu)])
def engine(request):
    if request.param == "oracle":
        return Engine(False)
    request.getfixturevalue("hip")
    return Engine(True, request.getfixturevalue("stream"))


def store(t):
    return RF.to_storage(t.dtype, t.values)


def test_parser_reads_every_fixture():
    for f in sorted(os.listdir(REFDIR)):
        items = RF.parse_ref(open(os.path.join(REFDIR, f)).read())
        assert items, f
    ts = tensors(load("ocean_axis_reduce_04"))
    assert ts[0].shape == [2, 3, 4] and ts[0].values[1, 2, 3] == 23 and ts[0].values[1, 0, 0] == 1 and ts[0].values[0, 1, 0] == 2
    assert ts[3].shape == [2, 3, 1]


def test_tensor_add_02(engine):
    ts = [t for t in tensors(load("tensor_add_02")) if t.device == "gpu0"]
    # per type: a, +a, a + s, a (after a += s), with s = True / 3 / 3.0
    for g, s in zip(range(0, 12, 4), (1, 3, 3)):
        a = ts[g]
        y = RF.to_storage(a.dtype, np.array([s]))
        rd, got = engine.binary("add", a.dtype, store(a), y)
        RF.assert_matches(rd, got, ts[g + 2], "a + s"); RF.assert_matches(rd, got, ts[g + 3], "a += s")
        RF.assert_matches(a.dtype, store(a), ts[g + 1], "+a")


def test_ocean_min_01(engine):
    ts = tensors(load("ocean_min_01"))
    assert len(ts) == 50
    for g in range(0, 50, 10):
        a1, a2 = ts[g], ts[g + 1]
        x, y = store(a1), store(a2)
        for k, (name, p, q) in enumerate([("min", x, y), ("min", y, x), ("max", x, y), ("fmin", x, y), ("fmin", y, x), ("fmax", x, y)]):
            rd, got = engine.binary(name, a1.dtype, p, q)
            RF.assert_matches(rd, got, ts[g + 2 + k], "%s %s #%d" % (name, H.NAMES[a1.dtype], k))
        rd, got = engine.binary("fmin", a1.dtype, x, y)
        RF.assert_matches(rd, got, ts[g + 8], "fmin into r1")
        RF.assert_matches(H.CFLOAT, engine.cast(rd, H.CFLOAT, got), ts[g + 9], "fmin into a complex-float destination")


@pytest.mark.parametrize("name,op", [("ocean_and_01", "bitwise_and"), ("ocean_or_01", "bitwise_or"), ("ocean_xor_01", "bitwise_xor")])
def test_bitwise_broadcast(engine, name, op):
    ts = tensors(load(name))
    assert len(ts) == 20
    for g in range(0, 20, 5):
        a1, a2 = ts[g], ts[g + 1]                       # 1 x 5 row and 6 x 1 column
        rd, got = engine.binary(op, a1.dtype, store(a1), store(a2))
        for k in (2, 3, 4):
            RF.assert_matches(rd, got, ts[g + k], "%s %s" % (op, H.NAMES[a1.dtype]))


def test_ocean_logical_01(engine):
    ts = tensors(load("ocean_logical_01"))
    assert len(ts) == 55
    for g in range(0, 55, 11):
        a1, a2 = ts[g], ts[g + 1]
        # the interface converts the operands to bool first
        x = engine.cast(a1.dtype, H.BOOL, store(a1)); y = engine.cast(a2.dtype, H.BOOL, store(a2))
        for k, op in enumerate(("logical_and", "logical_or", "logical_xor")):
            rd, got = engine.binary(op, H.BOOL, x, y)
            RF.assert_matches(H.BOOL, got, ts[g + 2 + 3 * k], op); RF.assert_matches(H.BOOL, got, ts[g + 3 + 3 * k], op)
            r2 = ts[g + 4 + 3 * k]
            assert r2.byteswapped and r2.dtype == H.INT16
            RF.assert_matches(H.INT16, engine.cast(H.BOOL, H.INT16, got), r2, op + " into int16")


def test_ocean_bitshift_01(engine):
    ts = tensors(load("ocean_bitshift_01"))
    assert len(ts) == 20
    for g in range(0, 20, 5):
        a, b = ts[g], ts[g + 1]                         # 1 x 4 row, 6 shift counts (uint8)
        counts = RF.to_storage(H.INT8, b.values.reshape(6, 1))
        rd, got = engine.binary("bitshift_left", a.dtype, store(a), counts)
        RF.assert_matches(rd, got, ts[g + 2], "a << b"); RF.assert_matches(rd, got, ts[g + 3], "bitshiftLeft(a, b, r)")
        rd, got = engine.binary("bitshift_left", a.dtype, store(a), RF.to_storage(H.INT8, np.array([[1]])))
        RF.assert_matches(rd, got, ts[g + 4], "a <<= 1")


def test_ocean_sign_01(engine):
    ts = tensors(load("ocean_sign_01"))
    assert len(ts) == 18
    for g in range(0, 18, 3):
        a = ts[g]
        rd, got = engine.unary("sign", a.dtype, store(a))
        RF.assert_matches(rd, got, ts[g + 1], "sign %s" % H.NAMES[a.dtype])
        RF.assert_matches(H.INT8, engine.cast(rd, H.INT8, got), ts[g + 2], "sign into int8")


def test_ocean_fabs_01(engine):
    ts = tensors(load("ocean_fabs_01"))
    assert len(ts) == 10
    inputs = [H.INT8, H.INT16, H.FLOAT, H.CHALF, H.CDOUBLE]
    for k, dt in enumerate(inputs):                     # fabs keeps the type; absolute of a complex number is real
        x = RF.to_storage(dt, np.array([-3 - 4j]))
        rd, got = engine.unary("fabs", dt, x)
        assert rd == ts[k].dtype
        RF.assert_matches(rd, got, ts[k], "fabs %s" % H.NAMES[dt])
        rd, got = engine.unary("absolute", dt, x)
        assert rd == ts[5 + k].dtype
        RF.assert_matches(rd, got, ts[5 + k], "absolute %s" % H.NAMES[dt])


def test_ocean_axis_reduce_04(engine):
    ts = tensors(load("ocean_axis_reduce_04"))
    A = store(ts[0])                                    # 2 x 3 x 4 float
    rd, got = engine.axis("norm2", H.FLOAT, A, A, [0, 1])
    RF.assert_matches(rd, got, ts[1], "norm2 over [0,1]")
    flipped = A[:, ::-1, :]                             # fliplr: dimension 1 reversed (a view with a negative stride)
    rd, got = engine.axis("minimum", H.FLOAT, A, flipped, [0])
    RF.assert_matches(rd, got, ts[2], "minimum over 0")
    rd, got = engine.axis("maximum", H.FLOAT, A, flipped, [2], keepdims=True)
    RF.assert_matches(rd, got, ts[3], "maximum over 2, keepdims")
    rd, got = engine.axis("norm", H.FLOAT, A, flipped, [0, 1], p=3.0)
    RF.assert_matches(rd, got, ts[5], "3-norm over [0,1]")
    half = engine.cast(rd, H.HALF, got)
    w = np.asarray(ts[4].values)
    assert np.abs(RF.from_storage(H.HALF, half) - w).max() <= 2 ** -5      # one half ulp at 32..64 (the reference stores the half result directly)


def scalars(items):
    return [v for it in items if isinstance(it, tuple) and it[0] == "scalars" for v in it[1]]


def test_scalar_reductions(engine):
    vals = scalars(load("ocean_sum_02"))                # int64 [1,2,3]; bool [T,F,T]; then [1,2,5] as int8, int16, half, chalf, cdouble
    cases = [(H.INT64, [1, 2, 3]), (H.BOOL, [1, 0, 1])] + [(d, [1, 2, 5]) for d in (H.INT8, H.INT16, H.HALF, H.CHALF, H.CDOUBLE)]
    assert len(vals) == len(cases)
    for (dt, data), want in zip(cases, vals):
        rd, got = engine.reduce("sum", dt, RF.to_storage(dt, np.array(data)))
        RF.assert_matches(rd, got, np.array([want]), "sum %s" % H.NAMES[dt])
    vals = scalars(load("ocean_sumabs_01"))
    cases = [(H.INT64, [1, -2, 3])] + [(d, [1, -2, 5]) for d in (H.INT8, H.INT16, H.HALF, H.CHALF, H.CDOUBLE)]
    assert len(vals) == len(cases)
    for (dt, data), want in zip(cases, vals):
        rd, got = engine.reduce("sum_abs", dt, RF.to_storage(dt, np.array(data)))
        RF.assert_matches(rd, got, np.array([want]), "sumAbs %s" % H.NAMES[dt])
    assert scalars(load("ocean_all_01")) == [False]
    rd, got = engine.reduce("all", H.INT64, RF.to_storage(H.INT64, np.array([1, 1, 1, 1, 0, 1])))
    assert rd == H.BOOL and got[0] == 0


def test_ocean_maximumabs_02(engine):
    items = load("ocean_maximumabs_02")
    rows = [it[1] for it in items if isinstance(it, tuple) and it[0] == "scalars"]
    dtypes = [H.BOOL, H.INT8, H.UINT8, H.INT32, H.HALF, H.FLOAT, H.CHALF, H.DOUBLE]
    assert len(rows) == len(dtypes)
    for dt, row in zip(dtypes, rows):
        a = RF.to_storage(dt, np.array([1, -3, 2]) if dt != H.UINT8 else np.array([1, 253, 2]))
        rd, got = engine.reduce("maximum_abs", dt, a)
        RF.assert_matches(rd, got, np.array([row[0]]), "maximumAbs %s" % H.NAMES[dt])
        both = np.asfortranarray(np.stack([a, a], axis=1))
        rd, got = engine.reduce("maximum_abs", dt, both)
        RF.assert_matches(rd, got, np.array([row[2]]), "maximumAbs of [A, B]")
        b = RF.to_storage(dt, np.array([-1, -3, 2]) if dt != H.UINT8 else np.array([255, 253, 2]))
        rd, got = engine.reduce("minimum_abs", dt, b)
        RF.assert_matches(rd, got, np.array([row[3]]), "minimumAbs %s" % H.NAMES[dt])


def test_ocean_gemm_01(engine):
    ts = tensors(load("ocean_gemm_01"))
    a = store(ts[0])                                    # 3 x 3 complex-float, column-major
    alphas = ts[1].values.reshape(-1)                   # 1 x 1 x 3 complex-half, one factor per slice of the result
    want = ts[2]
    for k in range(3):
        got = engine.gemm(H.CFLOAT, complex(alphas[k]), a, a)
        RF.assert_matches(H.CFLOAT, got, want.values[:, :, k], "gemm slice %d" % k)
