"""Parity of the unary elementwise kernels (och_unary) with the CPU oracle.

Reference tests of the same kind: examples/python/gpu/tensors/ocean_unary_01.py,
ocean_fabs_01/02.py, ocean_sign_01.py, ocean_not_01.py, ocean_logical_01.py (same call on
ocean.cpu and ocean.gpu[0], printed side by side).

Bit-exact: every operation made of IEEE basic operations or integer arithmetic (negative,
conj, bitwise/logical not, reciprocal, square, sqrt of real types, fabs, sign, ceil, floor,
trunc, round, the is* queries, complex negative / conj / reciprocal / square / sign / rounding).
Transcendental functions call the device math library, which is not bit-identical to the
host libm: real types within 8 ulp (half: 1 code), integers (computed through double and
truncated) within 1, complex within 2e-5 (cfloat, chalf) / 1e-12 (cdouble) relative to the
magnitude of the result.
"""
import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

pytestmark = pytest.mark.gpu
N = 2051

EXACT = {"negative", "bitwise_not", "logical_not", "conj", "reciprocal", "square", "sign", "ceil", "floor",
         "trunc", "round", "isinf", "isnan", "isfinite", "isposinf", "isneginf"}
EXACT_REAL_ONLY = {"sqrt", "absolute", "fabs"}       # complex versions use hypot


def input_data(name, dtype, rng):
    if dtype in (H.INT8, H.INT16, H.UINT8, H.UINT16) and name in EXACT:
        return H.random_data(dtype, N, rng, "full")
    if dtype in H.INT_TYPES:
        kind = "small" if name in ("exp", "exp2", "exp10", "expm1", "sinh", "cosh", "square") else "general"
        d = H.random_data(dtype, N, rng, kind)
        if name in ("exp10",):
            d = np.clip(d, -3, 3).astype(d.dtype)
        return d
    if dtype == H.BOOL:
        return H.random_data(dtype, N, rng)
    if name in EXACT or name in EXACT_REAL_ONLY:
        d = H.random_data(dtype, N, rng, "special")
        if name in EXACT_REAL_ONLY and dtype in H.COMPLEX_TYPES:
            d = H.random_data(dtype, N, rng, "general")
        return d
    small = {"arcsin", "arccos", "arctanh"}
    if name in small:
        v = rng.uniform(-0.95, 0.95, N)
    elif name == "arccosh":
        v = rng.uniform(1.05, 9.0, N)
    elif name in ("log", "log2", "log10", "cbrt"):
        v = rng.uniform(0.05, 9.0, N)
    elif name == "log1p":
        v = rng.uniform(-0.9, 9.0, N)
    elif name in ("exp10",):
        v = rng.uniform(-3, 3, N)
    else:
        v = rng.uniform(-4, 4, N)
    w = rng.uniform(-2, 2, N)
    if dtype == H.HALF:
        return H.f32_to_half_bits(v.astype(np.float32))
    if dtype == H.FLOAT:
        return v.astype(np.float32)
    if dtype == H.DOUBLE:
        return v
    if name in small:
        w = rng.uniform(-0.5, 0.5, N)
    if dtype == H.CHALF:
        out = np.empty(N, dtype=H.storage(dtype))
        out["real"] = H.f32_to_half_bits(v.astype(np.float32))
        out["imag"] = H.f32_to_half_bits(w.astype(np.float32))
        return out
    return (v + 1j * w).astype(H.storage(dtype))


def half_to_f32(bits):
    return np.array([H.orc.lib.oracle_half_to_float(int(b)) for b in bits.reshape(-1)], dtype=np.float32).reshape(bits.shape)


def compare(name, dtype, rdtype, got, want):
    exact = name in EXACT or (name in EXACT_REAL_ONLY and dtype not in H.COMPLEX_TYPES)
    if exact:
        H.assert_same_bytes(got, want, "%s %s" % (name, H.NAMES[dtype]))
    elif rdtype in H.INT_TYPES:
        d = np.abs(got.astype(np.int64) - want.astype(np.int64))
        assert d.max() <= 1, "%s %s: integer result differs by %d" % (name, H.NAMES[dtype], d.max())
    elif rdtype == H.HALF:
        d = np.abs(got.astype(np.int32) - want.astype(np.int32))
        assert d.max() <= 1
    elif rdtype in (H.FLOAT, H.DOUBLE):
        assert H.max_ulp_diff(got, want) <= 8, "%s %s: %d ulp" % (name, H.NAMES[dtype], H.max_ulp_diff(got, want))
    elif rdtype == H.CHALF:
        g = half_to_f32(got["real"]) + 1j * half_to_f32(got["imag"])
        w = half_to_f32(want["real"]) + 1j * half_to_f32(want["imag"])
        assert np.all(np.abs(g - w) <= 4e-3 * np.maximum(np.abs(w), 1e-2))
    else:
        tol = 2e-5 if rdtype == H.CFLOAT else 1e-12
        if name == "cbrt":
            tol = 2e-5          # the CPU table evaluates pow in single precision for every type
        assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-3)), "%s %s" % (name, H.NAMES[dtype])


CASES = [(op, dt) for op in range(len(oh.UNARY_OPS)) for dt in H.ALL_TYPES]


@pytest.mark.parametrize("op,dtype", CASES, ids=["%s-%s" % (oh.UNARY_OPS[o], H.NAMES[d]) for o, d in CASES])
def test_unary(hip, stream, op, dtype):
    name = oh.UNARY_OPS[op]
    sup = bool(oh.lib.och_unary_supported(op, dtype))
    assert sup == bool(H.orc.lib.oracle_unary_supported(op, dtype)), "support tables disagree"
    if not sup:
        assert oh.lib.och_unary(op, dtype, 1, oh.sizes([1]), oh.strides([0]), None, oh.strides([0]), None, stream.handle) == -1
        return
    rng = np.random.default_rng(4000 + op * 16 + dtype)
    rdtype = oh.lib.och_unary_result_dtype(op, dtype)
    x = H.Operand.contiguous(input_data(name, dtype, rng), dtype).upload(stream)
    # complex arctanh: the CPU macro never writes the real part; start both sides from zeros
    y = H.Operand.contiguous(np.zeros(N, dtype=H.storage(rdtype)), rdtype).upload(stream)
    H.gpu_unary(stream, op, dtype, x, y)
    want = y.parent.copy()
    H.cpu_unary(op, dtype, x, y, want)
    got = y.download()
    x.free(); y.free()
    if name == "arctanh" and dtype in H.COMPLEX_TYPES:
        # reference quirk (unary_ops.h:467-475): both terms go to .imag, .real is never assigned.
        # The kernel stores the logarithm term in .real; the CPU's .imag holds that same term.
        if dtype == H.CHALF:
            assert np.abs(got["real"].astype(np.int32) - want["imag"].astype(np.int32)).max() <= 1
        else:
            tol = 2e-5 if dtype == H.CFLOAT else 1e-12
            assert np.all(np.abs(got.real - want.imag) <= tol * np.maximum(np.abs(want.imag), 1e-3))
            xin = x.parent
            assert np.allclose(got.imag, np.arctanh(xin.astype(np.complex128)).imag, rtol=1e-4, atol=1e-5)
        return
    compare(name, dtype, rdtype, got, want)


@pytest.mark.parametrize("dtype", [H.INT16, H.FLOAT, H.DOUBLE, H.CFLOAT], ids=lambda d: H.NAMES[d])
def test_unary_layouts_and_in_place(hip, stream, dtype):
    rng = np.random.default_rng(31 + dtype)
    op = oh.U["square"]
    A = H.random_data(dtype, 40 * 30, rng).reshape(40, 30)
    Z = np.zeros((30, 40), dtype=A.dtype)
    x = H.Operand(A, A.T[::-1, ::2], dtype).upload(stream)
    z = H.Operand(Z, Z[:, ::2], dtype).upload(stream)
    H.gpu_unary(stream, op, dtype, x, z)
    want = Z.copy()
    H.cpu_unary(op, dtype, x, z, want, nthreads=3)
    H.assert_same_bytes(z.download(), want, "strided square")
    # in place on a strided view
    oh.check(oh.lib.och_unary(op, dtype, 2, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), None, None, stream.handle))
    want = A.copy()
    assert H.orc.lib.oracle_unary(op, dtype, 2, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(want), None, None, 1) == 0
    H.assert_same_bytes(x.download(), want, "in-place square")
    x.free(); z.free()
