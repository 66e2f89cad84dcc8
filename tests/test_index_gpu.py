"""Parity of the device index operations (och_add_if_negative, och_index_to_offset, och_get_index,
och_set_index, och_fill_index) with the oracle; bit-exact. Mirrors what
examples/python/gpu/index/*.py exercise through OcTensor indexing (index lists and ranges per
dimension, scalar fill, tensor assignment)."""
import numpy as np
import pytest

import helpers as H
import index_cases as IC
import ocean_hip as oh

orc = H.orc
pytestmark = pytest.mark.gpu
TYPES = [H.BOOL, H.INT8, H.UINT16, H.INT32, H.HALF, H.FLOAT, H.DOUBLE, H.INT64, H.CHALF, H.CFLOAT, H.CDOUBLE]


@pytest.mark.parametrize("dtype", TYPES, ids=[H.NAMES[d] for d in TYPES])
def test_gather_scatter_fill(hip, stream, dtype):
    rng = np.random.default_rng(140 + dtype)
    for shape, tables in (((7, 5, 6), (True, False, True)), ((33, 20, 17), (False, True, False)), ((64, 3, 50), (True, True, True)),
                          ((9, 11, 13), (False, False, False))):
        case = IC.build_case(dtype, rng, shape=shape, tables=tables)
        parent = case["parent"]
        sizes, strides, offs = IC.lib_order(case)
        htab = IC.pointer_table(offs, lambda t: t.ctypes.data)
        dev_tables = [oh.to_device(t, stream) if t is not None else None for t in offs]
        dtab = IC.pointer_table(dev_tables, lambda b: b.address)
        dst_strides = IC.dense_strides(sizes, parent.itemsize)
        nd = len(sizes)
        # gather
        dparent = oh.to_device(parent, stream)
        out = np.zeros(case["sizes"], parent.dtype)
        dout = oh.to_device(out, stream)
        oh.check(oh.lib.och_get_index(dtype, nd, oh.sizes(sizes), dtab, oh.strides(strides), dparent.ptr, oh.strides(dst_strides), dout.ptr, stream.handle))
        assert orc.lib.oracle_get_index(dtype, nd, oh.sizes(sizes), htab, oh.strides(strides), orc.ptr(parent), oh.strides(dst_strides), orc.ptr(out)) == 0
        H.assert_same_bytes(dout.download(parent.dtype, out.size).reshape(out.shape), out, "gather %s" % (shape,))
        # scatter
        src = H.random_data(dtype, out.size, rng).reshape(out.shape)
        dsrc = oh.to_device(src, stream)
        oh.check(oh.lib.och_set_index(dtype, nd, oh.sizes(sizes), dtab, oh.strides(strides), dparent.ptr, oh.strides(dst_strides), dsrc.ptr, stream.handle))
        want = parent.copy()
        assert orc.lib.oracle_set_index(dtype, nd, oh.sizes(sizes), htab, oh.strides(strides), orc.ptr(want), oh.strides(dst_strides), orc.ptr(src)) == 0
        H.assert_same_bytes(dparent.download(parent.dtype, parent.size).reshape(parent.shape), want, "scatter %s" % (shape,))
        # fill
        val = H.random_data(dtype, 1, rng)
        oh.check(oh.lib.och_fill_index(dtype, nd, oh.sizes(sizes), dtab, oh.strides(strides), dparent.ptr, H.raw_scalar(val), stream.handle))
        assert orc.lib.oracle_fill_index(dtype, nd, oh.sizes(sizes), htab, oh.strides(strides), orc.ptr(want), H.raw_scalar(val)) == 0
        H.assert_same_bytes(dparent.download(parent.dtype, parent.size).reshape(parent.shape), want, "fill %s" % (shape,))
        for b in [dparent, dout, dsrc] + [t for t in dev_tables if t is not None]:
            b.free()


def test_gather_large_and_empty(hip, stream):
    rng = np.random.default_rng(3)
    n, m = 4096, 513
    parent = rng.standard_normal((m, n)).astype(np.float32)
    rows = rng.integers(0, m, size=1000).astype(np.int64)
    offs = rows * parent.strides[0]
    dtab_buf = oh.to_device(offs, stream)
    dtab = IC.pointer_table([None, dtab_buf], lambda b: b.address)
    dparent = oh.to_device(parent, stream)
    dout = oh.DeviceBuffer(4 * n * rows.size, stream)
    oh.check(oh.lib.och_get_index(H.FLOAT, 2, oh.sizes([n, rows.size]), dtab, oh.strides([4, 0]), dparent.ptr, oh.strides([4, 4 * n]), dout.ptr, stream.handle))
    H.assert_same_bytes(dout.download(np.float32, n * rows.size).reshape(rows.size, n), parent[rows], "row gather")
    # empty selection: nothing happens
    assert oh.lib.och_get_index(H.FLOAT, 2, oh.sizes([n, 0]), dtab, oh.strides([4, 0]), dparent.ptr, oh.strides([4, 4 * n]), dout.ptr, stream.handle) == 0
    for b in (dtab_buf, dparent, dout):
        b.free()


@pytest.mark.parametrize("dtype", [H.INT8, H.HALF, H.FLOAT, H.DOUBLE, H.CDOUBLE], ids=lambda d: H.NAMES[d])
@pytest.mark.parametrize("shift", [0, 1])
def test_row_gather_scatter_fill(hip, stream, dtype, shift):
    """Whole rows through an offset table on the slow dimension (rows move as 16-byte runs where both ends are aligned);
    `shift` elements into the allocations makes the rows unaligned for element sizes below 16. Against numpy indexing."""
    rng = np.random.default_rng(7 + dtype + shift)
    n, m, k = 352, 130, 77
    flat = H.random_data(dtype, m * n + shift, rng)
    es = flat.itemsize
    parent = flat[shift:].reshape(m, n)
    rows = rng.permutation(m)[:k].astype(np.int64)
    dtab_buf = oh.to_device(rows * (n * es), stream)
    dtab = IC.pointer_table([None, dtab_buf], lambda b: b.address)
    dflat = oh.to_device(flat, stream)
    dout = oh.to_device(np.zeros(k * n + shift, flat.dtype), stream)
    import ctypes as C
    pp, po = C.c_void_p(dflat.address + shift * es), C.c_void_p(dout.address + shift * es)
    sz = oh.sizes([n, k])
    oh.check(oh.lib.och_get_index(dtype, 2, sz, dtab, oh.strides([es, 0]), pp, oh.strides([es, es * n]), po, stream.handle))
    H.assert_same_bytes(dout.download(flat.dtype, k * n + shift)[shift:].reshape(k, n), parent[rows], "row gather")
    src = H.random_data(dtype, k * n + shift, rng)
    dsrc = oh.to_device(src, stream)
    ps = C.c_void_p(dsrc.address + shift * es)
    oh.check(oh.lib.och_set_index(dtype, 2, sz, dtab, oh.strides([es, 0]), pp, oh.strides([es, es * n]), ps, stream.handle))
    want = parent.copy(); want[rows] = src[shift:].reshape(k, n)
    H.assert_same_bytes(dflat.download(flat.dtype, m * n + shift)[shift:].reshape(m, n), want, "row scatter")
    val = H.random_data(dtype, 1, rng)
    half = rows[: k // 2]
    dtab2_buf = oh.to_device(half * (n * es), stream)
    dtab2 = IC.pointer_table([None, dtab2_buf], lambda b: b.address)
    oh.check(oh.lib.och_fill_index(dtype, 2, oh.sizes([n, half.size]), dtab2, oh.strides([es, 0]), pp, H.raw_scalar(val), stream.handle))
    want[half] = val[0]
    got = dflat.download(flat.dtype, m * n + shift)
    H.assert_same_bytes(got[shift:].reshape(m, n), want, "row fill")
    H.assert_same_bytes(got[:shift], flat[:shift], "bytes before the parent")
    for b in (dtab_buf, dtab2_buf, dflat, dout, dsrc):
        b.free()


@pytest.mark.parametrize("dtype", [H.INT8, H.INT16, H.INT32, H.INT64], ids=lambda d: H.NAMES[d])
def test_add_if_negative(hip, stream, dtype):
    rng = np.random.default_rng(dtype)
    x = H.random_data(dtype, 64 * 331, rng).reshape(64, 331)
    v = x[:, ::2]
    op = H.Operand(x, v, dtype).upload(stream)
    val = H.raw_scalar(np.array([57], x.dtype))
    oh.check(oh.lib.och_add_if_negative(dtype, 2, oh.sizes(v.shape[::-1]), oh.strides(v.strides[::-1]), op.dptr(), val, stream.handle))
    want = x.copy()
    assert orc.lib.oracle_add_if_negative(dtype, 2, oh.sizes(v.shape[::-1]), oh.strides(v.strides[::-1]), orc.ptr(want), val) == 0
    H.assert_same_bytes(op.download(), want, "add_if_negative")
    op.free()
    assert oh.lib.och_add_if_negative(H.FLOAT, 1, oh.sizes([4]), oh.strides([4]), None, val, stream.handle) != 0


@pytest.mark.parametrize("dtype", [H.UINT8, H.UINT16, H.UINT32, H.UINT64, H.INT8, H.INT16, H.INT32, H.INT64], ids=lambda d: H.NAMES[d])
def test_index_to_offset(hip, stream, dtype):
    rng = np.random.default_rng(20 + dtype)
    nd, n = 4, 10007
    idx = rng.integers(0, 100, size=(n, nd)).astype(H.storage(dtype))
    strides = np.array([8, 800, -24, 1 << 33], np.int64)
    es = idx.itemsize
    didx = oh.to_device(idx, stream)
    dout = oh.DeviceBuffer(8 * n, stream)
    oh.check(oh.lib.och_index_to_offset(dtype, nd, strides.ctypes.data_as(IC.P64), es, n, nd * es, didx.ptr, 8, dout.ptr, stream.handle))
    want = np.zeros(n, np.int64)
    assert orc.lib.oracle_index_to_offset(dtype, nd, strides.ctypes.data_as(IC.P64), es, n, nd * es, orc.ptr(idx), 8, orc.ptr(want)) == 0
    assert np.array_equal(dout.download(np.int64, n), want)
    didx.free(); dout.free()


@pytest.mark.parametrize("shape,density", [((7,), 0.5), ((5, 9), 0.3), ((17, 33, 64), 0.1), ((515, 2048), 0.5), ((3, 4, 5, 6, 7), 0.9),
                                           ((100000,), 0.0), ((100000,), 1.0), ((4, 0), 0.5), ((3000, 3001), 0.02)])
def test_find_and_mask_to_offset(hip, stream, shape, density):
    """och_find_count / och_find_apply against the oracle, on a dense mask and on a strided view (every second
    element, reversed) of a larger one. Dimensions go to the library fastest first (reversed numpy order)."""
    import ctypes as C
    rng = np.random.default_rng(len(shape) * 31 + int(density * 10))
    nd = len(shape)
    big = (rng.random(tuple(2 * s + 1 for s in shape)) < density).astype(np.uint8)
    dbig = oh.to_device(big, stream)
    dense = tuple(slice(0, s) for s in shape)
    strided = tuple(slice(2 * s - 1, None, -2) if s else slice(0, 0) for s in shape)
    for sel in (dense, strided):
        view = big[sel]
        assert view.shape == shape
        sz, st = oh.sizes(shape[::-1]), oh.strides(view.strides[::-1])
        off = view.ctypes.data - big.ctypes.data if view.size else 0
        hptr, dptr = C.c_void_p(big.ctypes.data + off), C.c_void_p(dbig.address + off)
        work = oh.DeviceBuffer(oh.lib.och_find_workspace_size(view.size), stream)
        nnz = C.c_size_t(12345)
        oh.check(oh.lib.och_find_count(nd, sz, st, dptr, work.ptr, C.byref(nnz), stream.handle))
        want_n = orc.lib.oracle_find(nd, sz, st, hptr, None, None)
        assert nnz.value == want_n == int(view.sum())
        out = oh.DeviceBuffer(8 * max(1, want_n * nd), stream)
        oh.check(oh.lib.och_find_apply(nd, sz, st, dptr, work.ptr, None, out.ptr, stream.handle))
        want = np.zeros(want_n * nd, np.int64)
        orc.lib.oracle_find(nd, sz, st, hptr, None, want.ctypes.data_as(IC.P64))
        assert np.array_equal(out.download(np.int64, want_n * nd), want)
        mult = np.array([8, -800, 12345, 7, 1 << 33][:nd], np.int64)
        oh.check(oh.lib.och_find_apply(nd, sz, st, dptr, work.ptr, mult.ctypes.data_as(IC.P64), out.ptr, stream.handle))
        want = np.zeros(want_n, np.int64)
        orc.lib.oracle_find(nd, sz, st, hptr, mult.ctypes.data_as(IC.P64), want.ctypes.data_as(IC.P64))
        assert np.array_equal(out.download(np.int64, want_n), want)
        work.free(); out.free()
    dbig.free()


@pytest.mark.parametrize("shape,shift", [((1 << 20,), 0), ((1 << 20,), 16), ((1 << 20,), 3), ((37, 4096), 0), ((5, 7, 48), 0),
                                         ((5, 7, 48), 32), ((33, 40), 0), ((3, 16), 0)])
def test_find_contiguous_mask(hip, stream, shape, shift):
    """Dense masks whose fastest dimension is a multiple of 16 (the 16-byte load path when the base is aligned too; `shift`
    bytes into the allocation) against numpy.nonzero and numpy.ravel_multi_index."""
    import ctypes as C
    rng = np.random.default_rng(sum(shape) + shift)
    mask = (rng.random(shape) < 0.3).astype(np.uint8) * rng.integers(1, 255, shape).astype(np.uint8)
    n, nd = mask.size, len(shape)
    raw = np.zeros(n + 64, np.uint8); raw[shift:shift + n] = mask.ravel()
    draw = oh.to_device(raw, stream)
    sz, st = oh.sizes(shape[::-1]), oh.strides(mask.strides[::-1])
    work = oh.DeviceBuffer(oh.lib.och_find_workspace_size(n), stream)
    nnz = C.c_size_t(0)
    dptr = C.c_void_p(draw.address + shift)
    oh.check(oh.lib.och_find_count(nd, sz, st, dptr, work.ptr, C.byref(nnz), stream.handle))
    hits = np.nonzero(mask)
    assert nnz.value == len(hits[0])
    out = oh.DeviceBuffer(8 * max(1, nnz.value * nd), stream)
    oh.check(oh.lib.och_find_apply(nd, sz, st, dptr, work.ptr, None, out.ptr, stream.handle))
    # numpy order (last numpy axis fastest) is the library's order (its dimension 0 fastest); indices come fastest first
    want = np.stack(hits[::-1], axis=1).astype(np.int64)
    assert np.array_equal(out.download(np.int64, nnz.value * nd).reshape(-1, nd), want)
    mult = np.array([3, -1000, 1 << 35][:nd], np.int64)
    oh.check(oh.lib.och_find_apply(nd, sz, st, dptr, work.ptr, mult.ctypes.data_as(IC.P64), out.ptr, stream.handle))
    assert np.array_equal(out.download(np.int64, nnz.value), want @ mult)
    draw.free(); work.free(); out.free()
