"""och_mgs_project (one launch) against the sequence it replaces: per column one dot product and one rank-1 update
through gemm, run on the oracle, and against the same recurrence in extended precision.

Bar: normwise, ||v_gpu - v_ref|| <= tol * (||v_0|| + sum_i |r_i| ||q_i||) and |r_gpu - r_ref| <= tol * ||q_i|| ||v||,
tol = 1e-5 (float, cfloat) / 1e-13 (double, cdouble): the summation order of the dot products differs."""
import ctypes as C

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

orc = H.orc
pytestmark = pytest.mark.gpu
TYPES = [H.FLOAT, H.DOUBLE, H.CFLOAT, H.CDOUBLE]
TOL = {H.FLOAT: 1e-5, H.CFLOAT: 1e-5, H.DOUBLE: 1e-13, H.CDOUBLE: 1e-13}


def make(dtype, n, k, ldq, rng):
    st = H.storage(dtype)
    def rnd(m):
        a = rng.uniform(-1, 1, m)
        if dtype in H.COMPLEX_TYPES:
            a = a + 1j * rng.uniform(-1, 1, m)
        return a.astype(st)
    Q = (rnd(ldq * k) / np.sqrt(max(n, 1))).astype(st)
    return Q, rnd(n)


def reference(Q, v, n, k, ldq):
    wide = np.clongdouble if np.iscomplexobj(v) else np.longdouble
    x = v.astype(wide); r = np.zeros(k, wide); scale = float(np.linalg.norm(v))
    for i in range(k):
        q = Q[i * ldq:i * ldq + n].astype(wide)
        r[i] = np.vdot(q, x).astype(v.dtype)            # the coefficient is rounded to the element type before use
        x = x - r[i] * q
        scale += float(abs(r[i])) * float(np.linalg.norm(q.astype(np.complex128 if np.iscomplexobj(v) else np.float64)))
    return x, r, scale


@pytest.mark.parametrize("dtype", TYPES, ids=[H.NAMES[d] for d in TYPES])
@pytest.mark.parametrize("n,k,pad", [(1, 1, 0), (100, 7, 3), (1024, 1, 0), (4096, 33, 0), (5000, 5, 8), (16384, 3, 0), (20000, 4, 1)])
def test_mgs_project(hip, stream, dtype, n, k, pad):
    rng = np.random.default_rng(n + 31 * k + dtype)
    ldq = n + pad
    Q, v = make(dtype, n, k, ldq, rng)
    dQ, dv = oh.to_device(Q, stream), oh.to_device(v, stream)
    dr = oh.to_device(np.zeros(k, v.dtype), stream)
    oh.check(oh.lib.och_mgs_project(dtype, n, k, dQ.ptr, ldq, dv.ptr, dr.ptr, stream.handle))
    got_v, got_r = dv.download(v.dtype, n), dr.download(v.dtype, k)
    want_v, want_r, scale = reference(Q, v, n, k, ldq)
    assert np.linalg.norm((got_v - want_v).astype(np.complex128)) <= TOL[dtype] * scale
    assert np.abs((got_r - want_r).astype(np.complex128)).max() <= TOL[dtype] * scale
    # Q is not written
    assert np.array_equal(dQ.download(Q.dtype, Q.size), Q)
    # without the coefficient array (short vectors only)
    if n <= 16384:
        dv2 = oh.to_device(v, stream)
        oh.check(oh.lib.och_mgs_project(dtype, n, k, dQ.ptr, ldq, dv2.ptr, None, stream.handle))
        assert np.array_equal(dv2.download(v.dtype, n).view(np.uint8), got_v.view(np.uint8))
        dv2.free()
    for b in (dQ, dv, dr):
        b.free()


@pytest.mark.parametrize("dtype", [H.DOUBLE, H.CFLOAT], ids=lambda d: H.NAMES[d])
def test_mgs_project_matches_gemm_sequence(hip, stream, dtype):
    """The unfused sequence on the oracle: r_i = q_i^H v by gemm('C', 'N', 1, 1, n), v <- v - q_i r_i by gemm('N', 'N', n, 1, 1)."""
    rng = np.random.default_rng(77 + dtype)
    n, k, ldq = 777, 9, 800
    Q, v = make(dtype, n, k, ldq, rng)
    one, zero, minus = [np.array([c]).astype(v.dtype) for c in (1, 0, -1)]
    want = v.copy(); coeff = np.zeros(k, v.dtype)
    for i in range(k):
        qi = Q[i * ldq:]
        assert orc.lib.oracle_gemm(dtype, b"C", b"N", 1, 1, n, orc.ptr(one), orc.ptr(qi), ldq, orc.ptr(want), n, orc.ptr(zero), orc.ptr(coeff[i:]), 1, 1) == 0
        assert orc.lib.oracle_gemm(dtype, b"N", b"N", n, 1, 1, orc.ptr(minus), orc.ptr(qi), ldq, orc.ptr(coeff[i:]), 1, orc.ptr(one), orc.ptr(want), n, 1) == 0
    dQ, dv, dr = oh.to_device(Q, stream), oh.to_device(v, stream), oh.to_device(np.zeros(k, v.dtype), stream)
    oh.check(oh.lib.och_mgs_project(dtype, n, k, dQ.ptr, ldq, dv.ptr, dr.ptr, stream.handle))
    scale = float(np.linalg.norm(v)) + float(np.abs(coeff).sum())
    assert np.linalg.norm(dv.download(v.dtype, n) - want) <= TOL[dtype] * scale
    assert np.abs(dr.download(v.dtype, k) - coeff).max() <= TOL[dtype] * scale
    for b in (dQ, dv, dr):
        b.free()


def test_mgs_project_errors(hip, stream):
    buf = oh.DeviceBuffer(1024, stream)
    assert oh.lib.och_mgs_project(H.INT32, 4, 1, buf.ptr, 4, buf.ptr, None, stream.handle) != 0
    assert oh.lib.och_mgs_project(H.DOUBLE, 8, 2, buf.ptr, 4, buf.ptr, None, stream.handle) != 0        # ldq < n
    assert oh.lib.och_mgs_project(H.DOUBLE, 8, 2, None, 8, buf.ptr, None, stream.handle) != 0
    assert oh.lib.och_mgs_project(H.DOUBLE, 0, 2, None, 8, None, None, stream.handle) == 0              # nothing to do
    buf.free()
