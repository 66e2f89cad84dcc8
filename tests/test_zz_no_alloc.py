"""och_reduce_all_device_noalloc: the full reduction for callers that cannot allocate.

Its scratch (partial slots + ticket counter) is a fixed array inside the library's device code; every call on a device
shares it and it keeps what the last call left. The entry point is compared with och_reduce_all_device (library-owned
scratch) on the same inputs, bit for bit (both run the same kernels with the same launch geometry, so even floating
sums must agree exactly), on two calls in a row of which the second is smaller, for several operations and layouts.
"""
import ctypes as C

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

orc = H.orc

CASES = [  # (operation, dtype, numpy dtype)
    ("sum", H.DOUBLE, np.float64), ("sum", H.FLOAT, np.float32), ("norm2", H.FLOAT, np.float32),
    ("maximum", H.DOUBLE, np.float64), ("sum", H.INT16, np.int16), ("nnz", H.INT8, np.int8), ("any", H.BOOL, np.bool_),
    ("sum", H.CFLOAT, np.complex64),
]


def _both(stream, op, dtype, dev, shape, strides, offset):
    """Result bytes of the existing entry point and of the one that allocates nothing, same operand."""
    rd = oh.lib.och_reduce_result_dtype(op, dtype)
    nbytes = np.dtype(H.storage(rd)).itemsize
    outs = []
    for noalloc in (False, True):
        res = oh.DeviceBuffer(64, stream)
        oh.check(oh.lib.och_memset_async(res.ptr, 0xEE, 64, stream.handle))
        ptr = C.c_void_p(dev.address + offset)
        if noalloc:
            oh.check(oh.lib.och_reduce_all_device_noalloc(op, dtype, len(shape), oh.sizes(shape), oh.strides(strides), ptr,
                                                          None, None, 0.0, res.ptr, stream.handle))
        else:
            oh.check(oh.lib.och_reduce_all_device(op, dtype, len(shape), oh.sizes(shape), oh.strides(strides), ptr,
                                                  None, None, 0.0, res.ptr, None, stream.handle))
        outs.append(res.download(np.uint8, 64)[:nbytes].tobytes())
        res.free()
    return rd, outs


@pytest.mark.gpu
@pytest.mark.parametrize("name,dtype,npt", CASES, ids=lambda v: v if isinstance(v, str) else None)
def test_noalloc_matches_existing_entry_point(hip, stream, name, dtype, npt):
    rng = np.random.default_rng(4100 + dtype)
    op = oh.R[name]
    n_big, n_small = (1 << 22) + 13, 1000 + 7          # the big call fills all partial slots, the small one uses one block
    if npt == np.bool_:
        host = rng.integers(0, 2, n_big).astype(np.bool_)
    elif np.issubdtype(npt, np.integer):
        info = np.iinfo(npt)
        host = rng.integers(info.min, info.max, n_big, dtype=npt, endpoint=True)
    elif np.issubdtype(npt, np.complexfloating):
        host = (rng.standard_normal(n_big) + 1j * rng.standard_normal(n_big)).astype(npt)
    else:
        host = rng.standard_normal(n_big).astype(npt)
    es = host.itemsize
    dev = oh.to_device(host, stream)
    # call 1: everything; call 2 (smaller): a prefix; call 3: a strided 2-D view (every second element of 300 rows of 1000)
    plans = [((n_big,), (es,), 0, host), ((n_small,), (es,), 0, host[:n_small]),
             ((500, 300), (2 * es, 1000 * es), 3 * es, host[3:3 + 300 * 1000].reshape(300, 1000)[:, ::2].T)]
    for shape, strides, offset, view in plans:
        rd, (want, got) = _both(stream, op, dtype, dev, shape, strides, offset)
        assert got == want, (name, shape)
        # and against the CPU oracle / exact arithmetic for the operations whose bits are fixed
        if name in ("maximum", "nnz", "any") or (name == "sum" and np.issubdtype(npt, np.integer)):
            val = np.frombuffer(got, H.storage(rd))[0]
            ref = {"maximum": lambda v: v.max(), "nnz": lambda v: np.count_nonzero(v), "any": lambda v: v.any(),
                   "sum": lambda v: v.astype(np.int64).sum()}[name](view)
            assert val == ref, (name, shape, val, ref)
    dev.free()


@pytest.mark.gpu
def test_noalloc_after_library_scratch_was_used_on_another_stream(hip, stream):
    """The fixed array is separate from the per-stream scratch: alternating the two entry points on two streams (each
    stream synchronised before the other is used, as the contract asks for the shared array) keeps both right."""
    rng = np.random.default_rng(4242)
    other = oh.Stream()
    x = rng.integers(-1000, 1000, 1 << 20).astype(np.int64)
    dx = oh.to_device(x, stream)
    stream.synchronize()
    res = oh.DeviceBuffer(16, stream)
    for r, s in enumerate([stream, other, stream, other]):
        n = x.size - 1000 * r
        oh.check(oh.lib.och_reduce_all_device_noalloc(oh.R["sum"], H.INT64, 1, oh.sizes([n]), oh.strides([8]), dx.ptr, None, None, 0.0,
                                                      res.ptr, s.handle))
        s.synchronize()
        assert res.download(np.int64, 1)[0] == x[:n].sum()
    dx.free(); res.free()
    other.synchronize(); other.destroy()


def test_noalloc_rejects_sizes_beyond_the_maximum():
    """Checked before the device is touched, so it runs without a GPU."""
    limit = oh.lib.och_reduce_all_noalloc_max_elements()
    assert limit == 1 << 40
    dummy = C.c_void_p(256)
    rc = oh.lib.och_reduce_all_device_noalloc(oh.R["sum"], H.INT8, 2, oh.sizes([1 << 21, 1 << 20]), oh.strides([1, 1 << 21]), dummy,
                                              None, None, 0.0, dummy, None)
    assert rc == -1 and b"elements" in oh.lib.och_last_error()
