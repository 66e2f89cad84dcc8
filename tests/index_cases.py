"""Shared case builder for the index-operation tests (gather / scatter / fill through offset tables)."""
import ctypes as C

import numpy as np

import helpers as H

P64 = C.POINTER(C.c_int64)


def build_case(dtype, rng, shape=(7, 5, 6), tables=(True, False, True), repeat=False):
    """A source parent of `shape` (numpy order, last index fastest), and per dimension either an
    index list (turned into a byte-offset table) or a plain stride walk over a prefix.
    Returns dict with the parent, the per-dim index arrays, byte-offset tables and view sizes.
    Dimensions are passed to the library fastest first (reversed numpy order)."""
    parent = H.random_data(dtype, int(np.prod(shape)), rng).reshape(shape)
    idx, offs, sizes, strides = [], [], [], []
    for d, n in enumerate(shape):
        st = parent.strides[d]
        if tables[d]:
            k = n + 2 if repeat else max(1, n - 2)
            ind = rng.integers(0, n, size=k) if repeat else rng.permutation(n)[:k]
            idx.append(ind.astype(np.int64)); offs.append((ind * st).astype(np.int64)); sizes.append(k)
        else:
            k = max(1, n - 1)
            idx.append(np.arange(k, dtype=np.int64)); offs.append(None); sizes.append(k)
        strides.append(st)
    return dict(parent=parent, idx=idx, offs=offs, sizes=sizes, strides=strides)


def lib_order(case):
    """(sizes, strides, offset tables) fastest dimension first."""
    return case["sizes"][::-1], case["strides"][::-1], case["offs"][::-1]


def pointer_table(tables, address_of):
    """int64** for the library: address_of(table) gives the address of a table (host or device)."""
    arr = (P64 * len(tables))()
    for i, t in enumerate(tables):
        arr[i] = C.cast(C.c_void_p(address_of(t)), P64) if t is not None else P64()
    return arr


def dense_strides(sizes, itemsize):
    st, acc = [], itemsize
    for s in sizes:
        st.append(acc); acc *= s
    return st
