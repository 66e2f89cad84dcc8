"""Matrix products replayed against the expected-output files of the reference's CPU example tests (the GPU examples hold
three products only): ocean_gemm_02 / 03 / 07 / 08a (real and complex operands, 'T' and 'C' modes, vectors),
ocean_gemm_09a-d (all nine mode pairs for float, double, complex-float, complex-double), ocean_multiply_01 (int16) and
ocean_multiply_02 (bool: OR of ANDs). Inputs are the matrices the scripts build; all values are small integers, so the
printed results are exact for any summation order. Runs on the oracle (always) and on the device library (gpu)."""
import re

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh
import ref_format as RF
from test_ref_fixtures import load, tensors

orc = H.orc


class GemmEngine:
    def __init__(self, gpu, stream=None):
        self.gpu, self.stream = gpu, stream

    def product(self, dtype, ta, a, tb, b, alpha=1):
        """op(a) * op(b) for Fortran-ordered numpy matrices of storage type; returns the dense column-major result"""
        a, b = np.asfortranarray(a), np.asfortranarray(b)
        m, k = (a.shape if ta == "N" else a.shape[::-1])
        k2, n = (b.shape if tb == "N" else b.shape[::-1])
        assert k == k2
        c = np.zeros((m, n), a.dtype, order="F")
        al, be = RF.to_storage(dtype, np.array([alpha])), RF.to_storage(dtype, np.array([0]))
        if self.gpu:
            da, db, dc = [oh.to_device(x.reshape(-1, order="F"), self.stream) for x in (a, b, c)]
            oh.check(oh.lib.och_gemm(dtype, ta.encode(), tb.encode(), m, n, k, orc.ptr(al), da.ptr, a.shape[0], db.ptr, b.shape[0],
                                     orc.ptr(be), dc.ptr, m, 1, self.stream.handle))
            out = dc.download(c.dtype, m * n).reshape((m, n), order="F")
            for t in (da, db, dc):
                t.free()
            return out
        assert orc.lib.oracle_gemm(dtype, ta.encode(), tb.encode(), m, n, k, orc.ptr(al), orc.ptr(a), a.shape[0], orc.ptr(b), b.shape[0],
                                   orc.ptr(be), orc.ptr(c), m, 1) == 0
        return c


@pytest.fixture(params=["oracle", pytest.param("device", marks=pytest.mark.gpu)])
def engine(request):
    if request.param == "oracle":
        return GemmEngine(False)
    request.getfixturevalue("hip")
    return GemmEngine(True, request.getfixturevalue("stream"))


def mat(dtype, rows):
    """matrix given row by row (Ocean's 'r' order)"""
    return RF.to_storage(dtype, np.array(rows))


def test_small_products(engine):
    ts = tensors(load("ocean_gemm_02_cpu"))             # complex-float 2 x 2 times a vector
    a, b = mat(H.CFLOAT, [[1 + 2j, 2 + 1j], [3 + 0j, 4 + 2j]]), mat(H.CFLOAT, [[1 + 1j], [2 - 3j]])
    RF.assert_matches(H.CFLOAT, engine.product(H.CFLOAT, "N", a, "N", b).reshape(-1), ts[0], "gemm_02")
    ts = tensors(load("ocean_gemm_03_cpu"))
    a = mat(H.FLOAT, [[1, 2], [3, 4]]); b = RF.to_storage(H.FLOAT, np.arange(6.0).reshape((2, 3), order="F"))
    RF.assert_matches(H.FLOAT, a, ts[0], "a"); RF.assert_matches(H.FLOAT, b, ts[1], "b")
    RF.assert_matches(H.FLOAT, engine.product(H.FLOAT, "T", a, "N", b), ts[2], "a.T * b")
    RF.assert_matches(H.FLOAT, engine.product(H.FLOAT, "N", a, "N", b), ts[3], "a * b")
    ts = tensors(load("ocean_gemm_07_cpu"))             # a is given column by column here: asTensor([[0,1,2.],[3,4,5]]) is 3 x 2
    a = RF.to_storage(H.DOUBLE, np.array([[0, 3], [1, 4], [2, 5.]])); b = RF.to_storage(H.DOUBLE, np.arange(12.0).reshape((3, 4), order="F"))
    RF.assert_matches(H.DOUBLE, a.T, ts[0], "a.T"); RF.assert_matches(H.DOUBLE, b, ts[1], "b")
    RF.assert_matches(H.DOUBLE, engine.product(H.DOUBLE, "T", a, "N", b), ts[2], "gemm(1, a, 'T', b)")
    RF.assert_matches(H.DOUBLE, engine.product(H.DOUBLE, "N", a, "T", a), ts[3], "gemm(1, a, a, 'T')")


def test_conjugate_modes(engine):
    ts = tensors(load("ocean_gemm_08a_cpu"))
    a, b = mat(H.CFLOAT, [[1 + 2j, 2 + 3j]]), mat(H.CFLOAT, [[1], [2 + 1j]])             # 1 x 2 row, 2-vector
    RF.assert_matches(H.CFLOAT, a, ts[0], "a"); RF.assert_matches(H.CFLOAT, b.reshape(-1), ts[2], "b")
    at, bt = np.asfortranarray(a.T), np.asfortranarray(b.T)                               # a.T is 2 x 1, b.T is 1 x 2
    RF.assert_matches(H.CFLOAT, engine.product(H.CFLOAT, "N", a, "N", b).reshape(-1), ts[3], "a * b")
    RF.assert_matches(H.CFLOAT, engine.product(H.CFLOAT, "C", at, "N", b).reshape(-1), ts[4], "a.T^H * b")
    RF.assert_matches(H.CFLOAT, engine.product(H.CFLOAT, "C", at, "C", bt), ts[5], "a.T^H * b.T^H")
    RF.assert_matches(H.CFLOAT, engine.product(H.CFLOAT, "N", a, "C", bt), ts[6], "a * b.T^H")


@pytest.mark.parametrize("name,dtype", [("ocean_gemm_09a_cpu", H.FLOAT), ("ocean_gemm_09b_cpu", H.DOUBLE), ("ocean_gemm_09c_cpu", H.CFLOAT), ("ocean_gemm_09d_cpu", H.CDOUBLE)])
def test_all_mode_pairs(engine, name, dtype):
    """A is 2 x 3 ('N') or 3 x 2, B is 3 x 4 ('N') or 4 x 3, filled with 0, 1, 2, ... in memory order (complex types:
    real and imaginary parts interleaved); the file prints the 2 x 4 product for every mode pair (8 layouts each)."""
    items = load(name)
    seen = 0
    cplx = dtype in (H.CFLOAT, H.CDOUBLE)

    def filled(shape):
        n = shape[0] * shape[1]
        v = (np.arange(0, 2 * n, 2) + 1j * np.arange(1, 2 * n, 2)) if cplx else np.arange(n)
        return RF.to_storage(dtype, v.reshape(shape, order="F"))
    cache = {}
    for pos, it in enumerate(items):
        if not (isinstance(it, tuple) and it[0] == "text" and it[1].startswith("Setting:")):
            continue
        ta, tb = re.search(r"transA='(\w)', transB='(\w)'", it[1]).groups()
        want = next(x for x in items[pos + 1:] if isinstance(x, RF.RefTensor))
        assert want.shape == [2, 4]
        if (ta, tb) not in cache:
            cache[(ta, tb)] = engine.product(dtype, ta, filled((2, 3) if ta == "N" else (3, 2)), tb, filled((3, 4) if tb == "N" else (4, 3)))
        RF.assert_matches(dtype, cache[(ta, tb)], want, "%s: transA=%s transB=%s" % (name, ta, tb))
        seen += 1
    assert seen == 72 and len(cache) == 9


def test_integer_and_bool_products(engine):
    ts = tensors(load("ocean_multiply_01_cpu"))
    a = mat(H.INT16, [[1, 2], [3, 4]])
    for k, (ta, tb) in enumerate((("N", "N"), ("T", "N"), ("N", "T"), ("T", "T"))):
        RF.assert_matches(H.INT16, engine.product(H.INT16, ta, a, tb, a), ts[2 + k], "int16 %s%s" % (ta, tb))
    ts = tensors(load("ocean_multiply_02_cpu"))
    A = mat(H.BOOL, [[0, 0, 1], [0, 1, 1], [1, 0, 0]])
    RF.assert_matches(H.BOOL, A, ts[0], "A"); RF.assert_matches(H.BOOL, A.T, ts[1], "A'")
    for k, (ta, tb) in enumerate((("N", "N"), ("N", "T"), ("T", "N"), ("T", "T"))):
        RF.assert_matches(H.BOOL, engine.product(H.BOOL, ta, A, tb, A), ts[2 + k], "bool %s%s" % (ta, tb))
