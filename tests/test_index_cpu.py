"""Pins the oracle's index operations (oracle/oracle_index.c) against numpy's integer-array
indexing, which fixes the expected result independently: gather = parent[np.ix_(...)],
scatter / fill = assignment through the same index, add_if_negative = np.where, and
index_to_offset = an integer dot product. The reference ships no golden file for these
(they sit behind OcTensor indexing, examples/python/cpu/index/*.py print whole tensors)."""
import numpy as np
import pytest

import helpers as H
import index_cases as IC
import ocean_hip as oh

orc = H.orc
TYPES = [H.BOOL, H.INT8, H.UINT16, H.INT32, H.HALF, H.FLOAT, H.DOUBLE, H.INT64, H.CHALF, H.CFLOAT, H.CDOUBLE]


@pytest.mark.parametrize("dtype", TYPES, ids=[H.NAMES[d] for d in TYPES])
@pytest.mark.parametrize("tables", [(True, False, True), (False, False, False), (True, True, True), (False, True, False)])
def test_oracle_gather_scatter_fill(dtype, tables):
    rng = np.random.default_rng(40 + dtype)
    case = IC.build_case(dtype, rng, tables=tables)
    parent = case["parent"]
    sizes, strides, offs = IC.lib_order(case)
    tab = IC.pointer_table(offs, lambda t: t.ctypes.data)
    view = parent[np.ix_(*case["idx"])]
    # gather
    out = np.zeros(case["sizes"], parent.dtype)
    assert orc.lib.oracle_get_index(dtype, 3, oh.sizes(sizes), tab, oh.strides(strides), orc.ptr(parent),
                                    oh.strides(IC.dense_strides(sizes, parent.itemsize)), orc.ptr(out)) == 0
    H.assert_same_bytes(out, view, "gather")
    # scatter (distinct indices: the result does not depend on the order)
    src = H.random_data(dtype, out.size, rng).reshape(out.shape)
    want = parent.copy(); want[np.ix_(*case["idx"])] = src
    got = parent.copy()
    assert orc.lib.oracle_set_index(dtype, 3, oh.sizes(sizes), tab, oh.strides(strides), orc.ptr(got),
                                    oh.strides(IC.dense_strides(sizes, parent.itemsize)), orc.ptr(src)) == 0
    H.assert_same_bytes(got, want, "scatter")
    # fill
    val = H.random_data(dtype, 1, rng)
    want = parent.copy(); want[np.ix_(*case["idx"])] = val[0]
    got = parent.copy()
    assert orc.lib.oracle_fill_index(dtype, 3, oh.sizes(sizes), tab, oh.strides(strides), orc.ptr(got), H.raw_scalar(val)) == 0
    H.assert_same_bytes(got, want, "fill")


def test_oracle_gather_with_repeats():
    rng = np.random.default_rng(5)
    case = IC.build_case(H.DOUBLE, rng, tables=(True, True, False), repeat=True)
    parent = case["parent"]
    sizes, strides, offs = IC.lib_order(case)
    tab = IC.pointer_table(offs, lambda t: t.ctypes.data)
    out = np.zeros(case["sizes"], parent.dtype)
    assert orc.lib.oracle_get_index(H.DOUBLE, 3, oh.sizes(sizes), tab, oh.strides(strides), orc.ptr(parent),
                                    oh.strides(IC.dense_strides(sizes, 8)), orc.ptr(out)) == 0
    H.assert_same_bytes(out, parent[np.ix_(*case["idx"])], "gather with repeated indices")


@pytest.mark.parametrize("dtype", [H.INT8, H.INT16, H.INT32, H.INT64], ids=lambda d: H.NAMES[d])
def test_oracle_add_if_negative(dtype):
    rng = np.random.default_rng(dtype)
    x = H.random_data(dtype, 6 * 35, rng).reshape(6, 35)
    v = x[:, ::2]
    want = x.copy(); w = want[:, ::2]; w[w < 0] += 29
    assert orc.lib.oracle_add_if_negative(dtype, 2, oh.sizes(v.shape[::-1]), oh.strides(v.strides[::-1]), orc.ptr(x),
                                          H.raw_scalar(np.array([29], x.dtype))) == 0
    H.assert_same_bytes(x, want, "add_if_negative")


@pytest.mark.parametrize("dtype", [H.UINT8, H.INT16, H.UINT32, H.INT64], ids=lambda d: H.NAMES[d])
def test_oracle_index_to_offset(dtype):
    rng = np.random.default_rng(dtype)
    nd, n = 3, 41
    idx = rng.integers(0, 50, size=(n, nd)).astype(H.storage(dtype))       # row j holds the nd indices of element j
    strides = np.array([8, 800, -24], np.int64)
    out = np.zeros(n, np.int64)
    es = idx.itemsize
    assert orc.lib.oracle_index_to_offset(dtype, nd, strides.ctypes.data_as(IC.P64), es, n, nd * es, orc.ptr(idx), 8, orc.ptr(out)) == 0
    assert np.array_equal(out, idx.astype(np.int64) @ strides)


@pytest.mark.parametrize("shape", [(7,), (5, 9), (4, 3, 6), (2, 3, 2, 5)])
def test_oracle_find(shape):
    """Non-zero positions in element order with the first dimension fastest: numpy's nonzero on the
    transposed (C-ordered) view gives exactly that order."""
    rng = np.random.default_rng(len(shape))
    mask = np.asfortranarray(rng.integers(0, 3, shape) == 0).astype(np.uint8)      # Ocean order: mask[i0, i1, ...]
    nd = len(shape)
    want = np.stack(np.nonzero(mask.T)[::-1], axis=1)            # rows sorted with the LAST numpy axis of mask.T ... i.e. i0 fastest
    n = orc.lib.oracle_find(nd, oh.sizes(shape), oh.strides(mask.strides), orc.ptr(mask), None, None)
    assert n == int(mask.sum())
    out = np.zeros((n, nd), np.int64)
    assert orc.lib.oracle_find(nd, oh.sizes(shape), oh.strides(mask.strides), orc.ptr(mask), None, out.ctypes.data_as(IC.P64)) == n
    assert np.array_equal(out, want)
    mult = np.array([3, 100, -7, 1000][:nd], np.int64)
    off = np.zeros(n, np.int64)
    assert orc.lib.oracle_find(nd, oh.sizes(shape), oh.strides(mask.strides), orc.ptr(mask), mult.ctypes.data_as(IC.P64), off.ctypes.data_as(IC.P64)) == n
    assert np.array_equal(off, want @ mult)
