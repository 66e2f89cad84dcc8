"""Index operations replayed against the reference's expected-output files: examples/python/gpu/index/index_008
(gathers through index lists, coordinate lists and boolean masks on a GPU tensor) and the CPU examples ocean_find_01 /
tensor_find_01 (find is absent from the reference's GPU module; its CPU output defines the order of the result).
Ocean's interface turns an indexing expression into per-dimension byte-offset tables (index lists), offsets from
coordinates (indexToOffset) or from a mask (find / maskToOffset) and then calls getIndex; the replay does the same with
the oracle (always) and with the device library (gpu marker)."""
import ctypes as C

import numpy as np
import pytest

import helpers as H
import index_cases as IC
import ocean_hip as oh
import ref_format as RF
from test_ref_fixtures import load, tensors

orc = H.orc


class IndexEngine:
    def __init__(self, gpu, stream=None):
        self.gpu, self.stream = gpu, stream
        self.keep = []

    def _dev(self, a):
        b = oh.to_device(a, self.stream); self.keep.append(b); return b

    def close(self):
        for b in self.keep:
            b.free()
        self.keep = []

    def gather(self, dtype, parent, lists):
        """parent: Fortran-ordered array (Ocean order); lists[d]: index list for dimension d or None for the full range"""
        es = parent.itemsize
        sizes = [len(l) if l is not None else parent.shape[d] for d, l in enumerate(lists)]
        tables = [(np.asarray(l, np.int64) * parent.strides[d]) if l is not None else None for d, l in enumerate(lists)]
        out = np.zeros(sizes, parent.dtype, order="F")
        nd = len(sizes)
        if self.gpu:
            dt = [self._dev(t) if t is not None else None for t in tables]
            tab = IC.pointer_table(dt, lambda b: b.address)
            dp, do = self._dev(parent.reshape(-1, order="F")), self._dev(out.reshape(-1, order="F"))
            oh.check(oh.lib.och_get_index(dtype, nd, oh.sizes(sizes), tab, oh.strides(parent.strides), dp.ptr, oh.strides(out.strides), do.ptr, self.stream.handle))
            return do.download(parent.dtype, out.size).reshape(sizes, order="F")
        tab = IC.pointer_table(tables, lambda t: t.ctypes.data)
        assert orc.lib.oracle_get_index(dtype, nd, oh.sizes(sizes), tab, oh.strides(parent.strides), orc.ptr(parent), oh.strides(out.strides), orc.ptr(out)) == 0
        return out

    def gather_offsets(self, dtype, parent, offsets):
        """elements of parent at the given byte offsets"""
        n = len(offsets)
        out = np.zeros(n, parent.dtype)
        offs = np.ascontiguousarray(offsets, np.int64)
        if self.gpu:
            dt, dp, do = self._dev(offs), self._dev(parent.reshape(-1, order="F")), self._dev(out)
            tab = IC.pointer_table([dt], lambda b: b.address)
            oh.check(oh.lib.och_get_index(dtype, 1, oh.sizes([n]), tab, oh.strides([0]), dp.ptr, oh.strides([parent.itemsize]), do.ptr, self.stream.handle))
            return do.download(parent.dtype, n)
        tab = IC.pointer_table([offs], lambda t: t.ctypes.data)
        assert orc.lib.oracle_get_index(dtype, 1, oh.sizes([n]), tab, oh.strides([0]), orc.ptr(parent), oh.strides([parent.itemsize]), orc.ptr(out)) == 0
        return out

    def index_to_offset(self, coords, strides):
        """coords: nd x n int64 (Fortran order: one coordinate tuple per column); result: n byte offsets"""
        nd, n = coords.shape
        st = np.asarray(strides, np.int64)
        out = np.zeros(n, np.int64)
        flat = np.ascontiguousarray(coords.reshape(-1, order="F"))
        if self.gpu:
            dc, do = self._dev(flat), self._dev(out)
            oh.check(oh.lib.och_index_to_offset(H.INT64, nd, st.ctypes.data_as(IC.P64), 8, n, 8 * nd, dc.ptr, 8, do.ptr, self.stream.handle))
            return do.download(np.int64, n)
        assert orc.lib.oracle_index_to_offset(H.INT64, nd, st.ctypes.data_as(IC.P64), 8, n, 8 * nd, orc.ptr(flat), 8, orc.ptr(out)) == 0
        return out

    def find(self, mask, multiplier=None):
        """mask: Fortran-ordered uint8; result: nd x nnz indices (Fortran order), or nnz offsets when a multiplier is given"""
        nd = mask.ndim
        mult = np.asarray(multiplier, np.int64) if multiplier is not None else None
        pm = mult.ctypes.data_as(IC.P64) if mult is not None else None
        if self.gpu:
            dm = self._dev(mask.reshape(-1, order="F"))
            work = oh.DeviceBuffer(oh.lib.och_find_workspace_size(mask.size), self.stream); self.keep.append(work)
            nnz = C.c_size_t()
            oh.check(oh.lib.och_find_count(nd, oh.sizes(mask.shape), oh.strides(mask.strides), dm.ptr, work.ptr, C.byref(nnz), self.stream.handle))
            n = nnz.value
            do = oh.DeviceBuffer(8 * max(1, n * nd), self.stream); self.keep.append(do)
            oh.check(oh.lib.och_find_apply(nd, oh.sizes(mask.shape), oh.strides(mask.strides), dm.ptr, work.ptr, pm, do.ptr, self.stream.handle))
            flat = do.download(np.int64, n if mult is not None else n * nd)
        else:
            n = orc.lib.oracle_find(nd, oh.sizes(mask.shape), oh.strides(mask.strides), orc.ptr(mask), None, None)
            flat = np.zeros(n if mult is not None else n * nd, np.int64)
            orc.lib.oracle_find(nd, oh.sizes(mask.shape), oh.strides(mask.strides), orc.ptr(mask), pm, flat.ctypes.data_as(IC.P64))
        return flat if mult is not None else flat.reshape((nd, n), order="F")


@pytest.fixture(params=["oracle", pytest.param("device", marks=pytest.mark.gpu)])
def engine(request):
    if request.param == "oracle":
        e = IndexEngine(False)
    else:
        request.getfixturevalue("hip")
        e = IndexEngine(True, request.getfixturevalue("stream"))
    yield e
    e.close()


def test_index_008(engine):
    ts = tensors(load("index_008"))
    assert len(ts) == 12
    a = np.asfortranarray(np.arange(25, dtype=np.int64).reshape((5, 5), order="F"))      # arange(25).reshape(5, 5)
    RF.assert_matches(H.INT64, a, ts[0], "a")
    for k, lists in ((1, [[1, 2, 1], None]), (2, [None, [0, 2, 1]]), (3, [[2, 1], None]), (4, [None, [1, 2]])):
        RF.assert_matches(H.INT64, engine.gather(H.INT64, a, lists), ts[k], "index lists %s" % (lists,))
    got = engine.gather(H.INT64, a, [[2, 1], [1, 2, 2, 2]])
    RF.assert_matches(H.INT64, got.reshape((2, 4, 1), order="F"), ts[5], "a[[2,1],[1,2,2,2],None]")
    # a[[[1,2],[2,3],[3,4]]]: a list of coordinates -> offsets -> gather
    coords = np.asfortranarray(np.array([[1, 2, 3], [2, 3, 4]], np.int64))
    offs = engine.index_to_offset(coords, a.strides)
    assert list(offs) == [8 * 11, 8 * 17, 8 * 23]
    RF.assert_matches(H.INT64, engine.gather_offsets(H.INT64, a, offs), ts[6], "coordinate list")
    # b = (a <= a.T), f = find(b), a[None, b], a[None, f]
    b = ts[7]
    assert b.dtype == H.BOOL and np.array_equal(b.values, a <= a.T)
    mask = np.asfortranarray(b.values.astype(np.uint8))
    f = engine.find(mask)
    RF.assert_matches(H.INT64, f, ts[8], "find(b)")
    by_mask = engine.gather_offsets(H.INT64, a, engine.find(mask, a.strides))             # maskToOffset, then gather
    RF.assert_matches(H.INT64, by_mask.reshape((1, 15)), ts[9], "a[None, b]")
    by_coords = engine.gather_offsets(H.INT64, a, engine.index_to_offset(f, a.strides))
    RF.assert_matches(H.INT64, by_coords.reshape((1, 15)), ts[10], "a[None, f]")
    # one boolean list per dimension: each becomes an index list
    rows = engine.find(np.array([1, 0, 1, 0, 1], np.uint8)).reshape(-1); cols = engine.find(np.array([1, 1, 0, 0, 1], np.uint8)).reshape(-1)
    RF.assert_matches(H.INT64, engine.gather(H.INT64, a, [list(rows), list(cols)]), ts[11], "boolean lists")


def test_find_examples(engine):
    ts = tensors(load("ocean_find_01_cpu"))
    a = ts[0]                                           # 2 x 3 x 2 bool
    RF.assert_matches(H.INT64, engine.find(np.asfortranarray(a.values.astype(np.uint8))), ts[1], "find of a 2 x 3 x 2 mask")
    ts = tensors(load("tensor_find_01_cpu"))
    a = ts[0]                                           # 2 x 5 int64: the interface converts to bool first
    RF.assert_matches(H.INT64, engine.find(np.asfortranarray((a.values != 0).astype(np.uint8))), ts[1], "find of the non-zero elements")
