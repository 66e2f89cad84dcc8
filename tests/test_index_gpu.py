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
