"""The paths that tensors above the 32-bit launch counts take, exercised on small tensors by lowering the limits.

The reference switches its kernels to 64-bit indices for large extents (solid/src/core/gpu/op/apply_elemwise.c:66-99);
this library keeps 32-bit index arithmetic inside a launch and cuts the work on the host instead:
  * elementwise engine (binary, unary, cast / byteswap copy, fill, masked fill, steps): runs along the outermost
    dimension, launched one after the other (och_elemwise_set_launch_limit);
  * copy between different shapes: runs along the flat index both sides share, 64-bit decomposition in the kernel;
  * index_to_offset: runs of the index count; gather / scatter / fill: 64-bit decomposition of the work-item number;
  * axis reductions with a reduced range above the limit: pieces of the range, each a launch that leaves raw
    accumulators in the stream's workspace, folded by one finish kernel (och_reduce_axis_set_range_limit).
Every cut result is compared bit for bit with the uncut call and with the CPU oracle (floating sums: with the
float64 evaluation, to the tolerance of the other reduction tests).
"""
import ctypes as C

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh
from test_reduce_axis_gpu import run_case, to_f64

pytestmark = pytest.mark.gpu
orc = H.orc

LIMITS = (64, 200, 1000, 4096)


@pytest.fixture
def limits():
    """Restores every limit when the test ends, whatever happened."""
    yield
    oh.lib.och_elemwise_set_launch_limit(0)
    oh.lib.och_reduce_axis_set_range_limit(0)


def launches(elemsizes, shape, strides_list):
    return oh.elemwise_analyze(elemsizes, shape, strides_list, [4096] * len(elemsizes)).launches


def views(dtype, rng, layout):
    """(x parent, x view, y parent, y view, z parent, z view) in Ocean order (numpy views transposed so that
    dimension 0 is the fastest where the layout says so)."""
    def data(n, kind="general"):
        return H.random_data(dtype, n, rng, kind)
    if layout == "one_dim":
        n = 5003
        x, y, z = data(n), data(n), data(n)
        return x, x, y, y, z, z
    if layout == "one_dim_strided":
        n = 3001
        x, y, z = data(2 * n), data(3 * n), data(n)
        return x, x[::2], y, y[::-3], z, z
    if layout == "two_dims_strided":
        x, y, z = data(45 * 120).reshape(45, 120), data(45 * 120).reshape(45, 120), data(45 * 60).reshape(45, 60)
        return x, x[:, ::2].T, y, y[:, 1::2].T, z, z.T                  # shape (60, 45)
    if layout == "broadcast_row":
        x, y, z = data(70 * 96).reshape(70, 96), data(96).reshape(1, 96), data(70 * 96).reshape(70, 96)
        return x, x.T, y, np.broadcast_to(y, (70, 96)).T, z, z.T        # shape (96, 70), y broadcast along dim 1
    if layout == "transposed":
        x, y, z = data(130 * 150).reshape(130, 150), data(130 * 150).reshape(150, 130), data(130 * 150).reshape(150, 130)
        return x, x, y, y.T, z, z.T                                     # shape (130, 150): x is the transposed operand
    if layout == "odd_rows":
        x, y, z = data(40 * 133).reshape(40, 133), data(40 * 140).reshape(40, 140), data(40 * 131).reshape(40, 131)
        return x, x[:, 1:132].T, y, y[:, 3:134].T, z, z.T               # shape (131, 40): rows that are not whole vectors
    if layout == "three_dims":
        x, y, z = data(9 * 14 * 48).reshape(9, 14, 48), data(9 * 14 * 48).reshape(9, 14, 48), data(9 * 7 * 48).reshape(9, 7, 48)
        return x, x[:, ::2, :].T, y, y[:, 1::2, :].T, z, z.T            # shape (48, 7, 9)
    raise ValueError(layout)


LAYOUTS = ["one_dim", "one_dim_strided", "two_dims_strided", "broadcast_row", "transposed", "odd_rows", "three_dims"]
EW_TYPES = [H.BOOL, H.INT8, H.INT16, H.INT32, H.INT64, H.HALF, H.FLOAT, H.DOUBLE, H.CFLOAT, H.CDOUBLE]


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("dtype", EW_TYPES, ids=lambda d: H.NAMES[d])
def test_binary_and_unary_cut_into_runs(hip, stream, limits, dtype, layout):
    rng = np.random.default_rng(7000 + 31 * dtype + LAYOUTS.index(layout))
    xp, xv, yp, yv, zp, zv = views(dtype, rng, layout)
    x = H.Operand(xp, xv, dtype).upload(stream); y = H.Operand(yp, yv, dtype).upload(stream)
    es = H.storage(dtype).itemsize
    for opname in ("add", "multiply"):
        op = oh.B[opname]
        if not oh.lib.och_binary_supported(op, dtype):
            continue
        z = H.Operand(zp, zv, dtype).upload(stream)
        H.gpu_binary(stream, op, dtype, x, y, z)
        whole = z.download()
        want = zp.copy()
        H.cpu_binary(op, dtype, x, y, z, want)
        H.assert_same_bytes(whole.view(np.uint8), want.view(np.uint8), "uncut %s %s %s" % (opname, H.NAMES[dtype], layout))
        z.free()
        for limit in LIMITS:
            assert oh.lib.och_elemwise_set_launch_limit(limit) == 0
            assert launches([es, es, es], z.shape, [x.strides, y.strides, z.strides]) >= -(-zv.size // limit)
            z = H.Operand(zp, zv, dtype).upload(stream)
            H.gpu_binary(stream, op, dtype, x, y, z)
            got = z.download()
            z.free()
            oh.lib.och_elemwise_set_launch_limit(0)
            H.assert_same_bytes(got.view(np.uint8), whole.view(np.uint8),
                                "%s %s %s with at most %d elements per launch" % (opname, H.NAMES[dtype], layout, limit))
    uop = oh.U["negative"] if oh.lib.och_unary_supported(oh.U["negative"], dtype) else oh.U["bitwise_not"]
    if oh.lib.och_unary_supported(uop, dtype):
        z = H.Operand(zp, zv, dtype).upload(stream)
        H.gpu_unary(stream, uop, dtype, x, z)
        whole = z.download(); z.free()
        want = zp.copy()
        H.cpu_unary(uop, dtype, x, z, want)
        H.assert_same_bytes(whole.view(np.uint8), want.view(np.uint8), "uncut unary %s %s" % (H.NAMES[dtype], layout))
        for limit in LIMITS:
            assert oh.lib.och_elemwise_set_launch_limit(limit) == 0
            z = H.Operand(zp, zv, dtype).upload(stream)
            H.gpu_unary(stream, uop, dtype, x, z)
            got = z.download(); z.free()
            oh.lib.och_elemwise_set_launch_limit(0)
            H.assert_same_bytes(got.view(np.uint8), whole.view(np.uint8), "unary %s %s limit %d" % (H.NAMES[dtype], layout, limit))
    x.free(); y.free()


CAST_PAIRS = [(H.INT16, H.FLOAT, 1), (H.FLOAT, H.DOUBLE, 0), (H.DOUBLE, H.HALF, 0), (H.CFLOAT, H.CDOUBLE, 0), (H.INT64, H.INT8, 1),
              (H.HALF, H.FLOAT, 1), (H.UINT8, H.BOOL, 0), (H.CDOUBLE, H.FLOAT, 1)]


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("src,dst,swap", CAST_PAIRS, ids=["%s-%s%s" % (H.NAMES[a], H.NAMES[b], "-swapped" if s else "") for a, b, s in CAST_PAIRS])
def test_cast_copy_cut_into_runs(hip, stream, limits, src, dst, swap, layout):
    rng = np.random.default_rng(7300 + 17 * src + dst + LAYOUTS.index(layout))
    xp, xv, _, _, _, _ = views(src, rng, layout)
    _, _, _, _, zp, zv = views(dst, rng, layout)
    x = H.Operand(xp, xv, src).upload(stream)
    gfn = oh.lib.och_byteswap_copy if swap else oh.lib.och_copy
    cfn = orc.lib.oracle_byteswap_copy if swap else orc.lib.oracle_copy
    nd = len(zv.shape)

    def run():
        z = H.Operand(zp, zv, dst).upload(stream)
        oh.check(gfn(src, dst, nd, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), nd, oh.sizes(z.shape), oh.strides(z.strides), z.dptr(), stream.handle))
        out = z.download(); z.free()
        return z, out
    z, whole = run()
    want = zp.copy()
    assert cfn(src, dst, nd, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(), nd, oh.sizes(z.shape), oh.strides(z.strides), z.hptr(want), 1) == 0
    H.assert_same_bytes(whole.view(np.uint8), want.view(np.uint8), "uncut cast %s" % layout)
    for limit in LIMITS:
        assert oh.lib.och_elemwise_set_launch_limit(limit) == 0
        _, got = run()
        oh.lib.och_elemwise_set_launch_limit(0)
        H.assert_same_bytes(got.view(np.uint8), whole.view(np.uint8), "cast %s limit %d" % (layout, limit))
    x.free()


@pytest.mark.parametrize("dtype", [H.BOOL, H.UINT8, H.INT16, H.INT32, H.HALF, H.FLOAT, H.DOUBLE, H.CHALF, H.CDOUBLE], ids=lambda d: H.NAMES[d])
def test_fill_family_and_steps_cut_into_runs(hip, stream, limits, dtype):
    """fill, fill_nan, masked_fill, byteswap and the three steps builders; steps depends on the flat index of every
    element, which each run must continue where the one before it ended."""
    rng = np.random.default_rng(7600 + dtype)
    value = H.raw_scalar(H.random_data(dtype, 1, rng, "general"))
    for layout in ("one_dim", "two_dims_strided", "odd_rows", "three_dims"):
        _, _, _, _, zp, zv = views(dtype, rng, layout)
        if dtype >= H.HALF:
            flat = zp.reshape(-1)
            flat[::7] = H.random_data(dtype, flat[::7].size, rng, "special")
        mp = rng.integers(0, 2, zp.shape).astype(np.uint8)
        mv = np.ndarray(shape=zv.shape, dtype=np.uint8, buffer=mp, strides=[s // zp.dtype.itemsize for s in zv.strides],
                        offset=(zv.__array_interface__["data"][0] - zp.__array_interface__["data"][0]) // zp.dtype.itemsize)
        m = H.Operand(mp, mv, H.BOOL).upload(stream)
        nd = len(zv.shape)

        def calls(z):
            sz, st = oh.sizes(z.shape), oh.strides(z.strides)
            out = [("fill", lambda p: oh.lib.och_fill(dtype, nd, sz, st, p, value, stream.handle),
                    lambda p: orc.lib.oracle_fill(dtype, nd, sz, st, p, value, 1)),
                   ("masked_fill", lambda p: oh.lib.och_masked_fill(dtype, nd, sz, st, p, oh.strides(m.strides), m.dptr(), value, stream.handle),
                    lambda p: orc.lib.oracle_masked_fill(dtype, nd, sz, st, p, oh.strides(m.strides), m.hptr(), value, 1)),
                   ("byteswap", lambda p: oh.lib.och_byteswap(dtype, nd, sz, st, p, stream.handle),
                    lambda p: orc.lib.oracle_byteswap(dtype, nd, sz, st, p, 1)),
                   ("steps_int64", lambda p: oh.lib.och_steps_int64(dtype, nd, sz, st, p, 0 if dtype == H.BOOL else -3, 1, stream.handle),
                    lambda p: orc.lib.oracle_steps_int64(dtype, nd, sz, st, p, 0 if dtype == H.BOOL else -3, 1, 1)),
                   ("steps_double", lambda p: oh.lib.och_steps_double(dtype, nd, sz, st, p, 0.5, 1.0 / 64, stream.handle),
                    lambda p: orc.lib.oracle_steps_double(dtype, nd, sz, st, p, 0.5, 1.0 / 64, 1)),
                   ("steps_cdouble", lambda p: oh.lib.och_steps_cdouble(dtype, nd, sz, st, p, oh.CDouble(1.0, 2.0), oh.CDouble(1.0 / 32, 1.0 / 128), stream.handle),
                    lambda p: orc.lib.oracle_steps_cdouble(dtype, nd, sz, st, p, oh.CDouble(1.0, 2.0), oh.CDouble(1.0 / 32, 1.0 / 128), 1))]
            if dtype >= H.HALF:
                out.append(("fill_nan", lambda p: oh.lib.och_fill_nan(dtype, nd, sz, st, p, value, stream.handle),
                            lambda p: orc.lib.oracle_fill_nan(dtype, nd, sz, st, p, value, 1)))
            return out
        probe = H.Operand(zp, zv, dtype)
        for index, (name, _, _) in enumerate(calls(probe)):
            results = []
            for limit in (0,) + LIMITS:
                assert oh.lib.och_elemwise_set_launch_limit(limit) == 0
                z = H.Operand(zp, zv, dtype).upload(stream)
                _, gpu_call, cpu_call = calls(z)[index]
                oh.check(gpu_call(z.dptr()))
                results.append(z.download()); z.free()
                oh.lib.och_elemwise_set_launch_limit(0)
                if limit == 0:
                    want = zp.copy()
                    assert cpu_call(z.hptr(want)) == 0
                    H.assert_same_bytes(results[0].view(np.uint8), want.view(np.uint8), "uncut %s %s %s" % (name, H.NAMES[dtype], layout))
                else:
                    H.assert_same_bytes(results[-1].view(np.uint8), results[0].view(np.uint8),
                                        "%s %s %s with at most %d elements per launch" % (name, H.NAMES[dtype], layout, limit))
        m.free()


@pytest.mark.parametrize("dtype", [H.INT8, H.INT16, H.FLOAT, H.DOUBLE, H.CDOUBLE], ids=lambda d: H.NAMES[d])
def test_copy_between_different_shapes_cut_along_the_flat_index(hip, stream, limits, dtype):
    """Reshape copy (solid/src/core/gpu/template_copy.cu:35-51): the flat index runs over each side in its own dimension
    order; above the limit the kernel decomposes a 64-bit flat index and the launches cover runs of it."""
    rng = np.random.default_rng(7900 + dtype)
    src_parent = H.random_data(dtype, 24 * 100, rng, "general").reshape(24, 100)
    src_view = src_parent[:, ::2].T                                          # Ocean shape (50, 24), strided
    dst_parent = H.random_data(dtype, 30 * 45, rng, "general").reshape(30, 45)
    dst_view = dst_parent[:, 2:42].T                                          # Ocean shape (40, 30): same 1200 elements
    x = H.Operand(src_parent, src_view, dtype).upload(stream)
    for dst_type in (dtype, H.DOUBLE if dtype != H.DOUBLE else H.FLOAT):
        dp = dst_parent if dst_type == dtype else H.random_data(dst_type, 30 * 45, rng, "general").reshape(30, 45)
        dv = dp[:, 2:42].T
        results = []
        for limit in (0,) + LIMITS:
            assert oh.lib.och_elemwise_set_launch_limit(limit) == 0
            z = H.Operand(dp, dv, dst_type).upload(stream)
            oh.check(oh.lib.och_copy(dtype, dst_type, 2, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(),
                                     2, oh.sizes(z.shape), oh.strides(z.strides), z.dptr(), stream.handle))
            results.append(z.download()); z.free()
            oh.lib.och_elemwise_set_launch_limit(0)
        want = dp.copy()
        assert orc.lib.oracle_copy(dtype, dst_type, 2, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(),
                                   2, oh.sizes(z.shape), oh.strides(z.strides), z.hptr(want), 1) == 0
        for limit, got in zip((0,) + LIMITS, results):
            H.assert_same_bytes(got.view(np.uint8), want.view(np.uint8), "reshape copy %s -> %s limit %d" % (H.NAMES[dtype], H.NAMES[dst_type], limit))
    x.free()


def test_index_operations_above_the_launch_limit(hip, stream, limits):
    """index_to_offset in runs; gather / scatter / fill with the 64-bit decomposition of the work-item number."""
    rng = np.random.default_rng(8100)
    n, dims = 3000, (40, 25, 30)
    idx = np.stack([rng.integers(0, d, n) for d in dims]).astype(np.int64)            # (3, n): Ocean shape (n, 3)
    strides = np.array([8, 8 * 40, 8 * 40 * 25], np.int64)
    didx = oh.to_device(idx, stream)
    want = (idx * strides[:, None]).sum(axis=0)
    src = rng.standard_normal(dims[::-1])
    dsrc = oh.to_device(src, stream)
    # per-dimension offset tables for a gather of a (17, 11, 13) block
    picks = [rng.integers(0, d, k).astype(np.int64) for d, k in zip(dims, (17, 11, 13))]
    tables = [oh.to_device(p * s, stream) for p, s in zip(picks, strides)]
    table_ptrs = (C.POINTER(C.c_int64) * 3)(*[C.cast(t.ptr, C.POINTER(C.c_int64)) for t in tables])
    block = src[np.ix_(picks[2], picks[1], picks[0])]
    for limit in (0, 64, 1000):
        assert oh.lib.och_elemwise_set_launch_limit(limit) == 0
        dout = oh.DeviceBuffer(8 * n, stream)
        oh.check(oh.lib.och_index_to_offset(H.INT64, 3, strides.ctypes.data_as(C.POINTER(C.c_int64)), 8 * n, n, 8, didx.ptr, 8, dout.ptr, stream.handle))
        assert np.array_equal(dout.download(np.int64), want), "index_to_offset limit %d" % limit
        dout.free()
        got = oh.DeviceBuffer(block.nbytes, stream)
        oh.check(oh.lib.och_get_index(H.DOUBLE, 3, oh.sizes([17, 11, 13]), table_ptrs, oh.strides([0, 0, 0]), dsrc.ptr,
                                      oh.strides([8, 8 * 17, 8 * 17 * 11]), got.ptr, stream.handle))
        assert np.array_equal(got.download(np.float64).reshape(13, 11, 17), block), "gather limit %d" % limit
        target = oh.to_device(np.zeros(dims[::-1]), stream)
        oh.check(oh.lib.och_set_index(H.DOUBLE, 3, oh.sizes([17, 11, 13]), table_ptrs, oh.strides([0, 0, 0]), target.ptr,
                                      oh.strides([8, 8 * 17, 8 * 17 * 11]), got.ptr, stream.handle))
        expect = np.zeros(dims[::-1]); expect[np.ix_(picks[2], picks[1], picks[0])] = block
        assert np.array_equal(target.download(np.float64).reshape(dims[::-1]), expect), "scatter limit %d" % limit
        oh.check(oh.lib.och_fill_index(H.DOUBLE, 3, oh.sizes([17, 11, 13]), table_ptrs, oh.strides([0, 0, 0]), target.ptr,
                                       H.raw_scalar(np.array([2.5])), stream.handle))
        expect[np.ix_(picks[2], picks[1], picks[0])] = 2.5
        assert np.array_equal(target.download(np.float64).reshape(dims[::-1]), expect), "fill limit %d" % limit
        got.free(); target.free()
        oh.lib.och_elemwise_set_launch_limit(0)
    for t in tables:
        t.free()
    didx.free(); dsrc.free()


def test_launch_limit_rejects_values_out_of_range(hip, limits):
    assert oh.lib.och_elemwise_set_launch_limit(63) == -1 and b"between 64" in oh.lib.och_last_error()
    assert oh.lib.och_elemwise_set_launch_limit(1 << 33) == -1
    assert oh.lib.och_elemwise_set_launch_limit(64) == 0 and oh.lib.och_elemwise_set_launch_limit(0) == 0


RANGE_CASES = [((3, 5000), [1]), ((5000, 3), [0]), ((7, 40, 50), [1, 2]), ((40, 7, 50), [0, 2]), ((2000,), [0]), ((33, 9, 31), [0, 1, 2]),
               ((600, 40), [0]), ((40, 600), [1])]


@pytest.mark.parametrize("dtype", [H.INT8, H.INT32, H.FLOAT, H.DOUBLE, H.CFLOAT], ids=lambda d: H.NAMES[d])
def test_axis_reduction_with_a_reduced_range_above_the_limit(hip, stream, limits, dtype):
    """A reduced range longer than one launch counts is cut into pieces along its outermost reduced dimension (index by
    index and further inside when one index is still too long); every piece leaves raw accumulators in the workspace
    and one finish kernel folds them in the order of the reduced index. Integer sums, counts and extremes are bit for
    bit those of the uncut call and the oracle; floating sums agree with the float64 evaluation."""
    rng = np.random.default_rng(8300 + dtype)
    for shape, axes in RANGE_CASES:
        parent = H.random_data(dtype, int(np.prod(shape)), rng, "general").reshape(shape[::-1])
        view = parent.T
        v = to_f64(dtype, view)
        for name in ("sum", "maximum", "nnz", "norm2", "any"):
            if not oh.lib.och_reduce_supported(oh.R[name], dtype):
                continue
            oh.lib.och_reduce_axis_set_range_limit(0)
            rd, whole, want = run_case(stream, name, dtype, parent, view, axes)
            exact = (dtype in (H.INT8, H.INT32) and name != "norm2") or name in ("maximum", "nnz", "any")
            if exact:
                H.assert_same_bytes(whole, want, "uncut %s %s %s" % (name, H.NAMES[dtype], shape))
            for limit in (4096, 1000, 97, 8):
                oh.lib.och_reduce_axis_set_range_limit(limit)
                rd, got, _ = run_case(stream, name, dtype, parent, view, axes)
                oh.lib.och_reduce_axis_set_range_limit(0)
                what = "%s %s %s axes=%s with at most %d reduced elements per launch" % (name, H.NAMES[dtype], shape, axes, limit)
                if exact:
                    H.assert_same_bytes(got, whole, what)
                    continue
                g = to_f64(rd, got)
                ax = tuple(axes)
                truth = {"sum": v.sum(axis=ax), "norm2": np.sqrt((np.abs(v) ** 2).sum(axis=ax))}[name].T
                scale = np.abs(v).sum(axis=ax).T if name == "sum" else np.abs(truth)
                tol = 1e-12 if dtype == H.DOUBLE else 1e-5
                assert np.all(np.abs(g - truth) <= tol * np.maximum(np.asarray(scale), 1e-6)), what


def test_axis_range_pieces_are_folded_in_a_fixed_order(hip, stream, limits):
    """The same cut gives the same bits on every run (the fold order depends on the cut alone), for a floating sum whose
    value depends on the order of its additions."""
    rng = np.random.default_rng(8400)
    parent = (rng.standard_normal((5, 30000)) * 10.0 ** rng.integers(-6, 6, (5, 30000))).astype(np.float32)
    oh.lib.och_reduce_axis_set_range_limit(1000)
    first = None
    for _ in range(5):
        rd, got, _ = run_case(stream, "sum", H.FLOAT, parent, parent.T, [0])
        if first is None:
            first = got.copy()
        assert got.tobytes() == first.tobytes()
    oh.lib.och_reduce_axis_set_range_limit(0)
