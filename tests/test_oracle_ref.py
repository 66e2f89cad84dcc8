"""Pins the CPU oracle (oracle/liboracle.so) against the reference's own arithmetic.

oracle/_ref/libocean_ref.so is built from the reference sources where they lie (operation
macros binary_ops.h / unary_ops.h / reduce_ops.h, conversion macros dtype_assign.h, half.c)
by oracle/Makefile; these tests run every (operation, type) pair of both libraries on the
same inputs -- exhaustive for 8-bit operands and all 65536 half patterns, seeded random plus
edge values otherwise -- and require identical bytes: both sides are compiled by the same
compiler against the same libm, so even the transcendental functions must agree exactly.

What stays unpinned (inputs excluded here, undefined behaviour in the reference itself):
int32/int64 division-family operations whose sign test `x*y < 0` overflows, most-negative
/ -1, shift counts >= the promoted width, float -> integer casts of out-of-range values.
"""
import ctypes as C

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

orc = H.orc
pytestmark = pytest.mark.skipif(not orc.ref_built(), reason="oracle/_ref was not built (reference tree absent)")

REF_BIN = ["add", "subtract", "multiply", "divide", "true_divide", "floor_divide", "power", "mod", "fmod",
           "min", "max", "fmin", "fmax", "lt", "le", "eq", "ne", "ge", "gt",
           "bitwise_and", "bitwise_or", "bitwise_xor", "logical_and", "logical_or", "logical_xor",
           "bitshift_left", "bitshift_right"]
assert REF_BIN == oh.BINARY_OPS


def call_ref(fnptr, proto, *args):
    return proto(fnptr)(*args)


BIN_PROTO = C.CFUNCTYPE(None, C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p)
UN_PROTO = C.CFUNCTYPE(None, C.c_size_t, C.c_void_p, C.c_void_p)
RED_PROTO = C.CFUNCTYPE(None, C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p)


def edge_values(dtype, rng, n):
    """Test inputs: random values plus the type's edge cases."""
    st = H.storage(dtype)
    if dtype == H.BOOL:
        return rng.integers(0, 2, n).astype(np.uint8)
    if dtype in H.INT_TYPES:
        info = np.iinfo(st)
        small = st.itemsize <= 2
        v = rng.integers(info.min, info.max, n, dtype=st, endpoint=True) if small else \
            rng.integers(max(info.min, -30000), min(info.max, 30000), n, endpoint=True).astype(st)
        edges = np.array([0, 1, 2, 3, info.max if small else 12345] + ([-1, -2, -3, info.min if small else -12345] if info.min < 0 else []), dtype=st)
        v[:edges.size] = edges
        return v
    vals = rng.uniform(-8, 8, n)
    specials = [0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.0, np.inf, -np.inf, np.nan, 1e-3, -1e-3, 6.5e4, 3.0, -3.0, 1e-7]
    vals[:len(specials)] = specials
    rng.shuffle(vals)
    if dtype in (H.HALF, H.FLOAT, H.DOUBLE):
        if dtype == H.HALF:
            bits = H.f32_to_half_bits(vals.astype(np.float32))
            bits[: 64] = rng.integers(0, 0x10000, 64).astype(np.uint16)      # raw patterns incl. subnormals / NaN payloads
            return bits
        return vals.astype(st)
    im = rng.uniform(-8, 8, n)
    im[:len(specials)] = specials[::-1]
    rng.shuffle(im)
    if dtype == H.CHALF:
        out = np.empty(n, st)
        out["real"] = H.f32_to_half_bits(vals.astype(np.float32))
        out["imag"] = H.f32_to_half_bits(im.astype(np.float32))
        return out
    return (vals + 1j * im).astype(st)


def second_operand(op, dtype, rng, n, x):
    name = oh.BINARY_OPS[op]
    if name in ("bitshift_left", "bitshift_right"):
        lim = 63 if oh.TYPE_SIZE[dtype] == 8 else 31
        return H.INT8, rng.integers(-lim, lim, n, endpoint=True).astype(np.int8)
    if name == "power" and dtype <= H.INT64:
        return H.INT16, rng.integers(-3, 9, n, endpoint=True).astype(np.int16)
    y = edge_values(dtype, rng, n)
    rng.shuffle(y)
    if dtype in (H.INT32, H.INT64, H.UINT32, H.UINT64) and name in ("divide", "floor_divide", "mod"):
        y[::5] = 0
    return dtype, y


PAIRS = [(op, dt) for op in range(len(oh.BINARY_OPS)) for dt in H.ALL_TYPES]


@pytest.mark.parametrize("op,dtype", PAIRS, ids=["%s-%s" % (oh.BINARY_OPS[o], H.NAMES[d]) for o, d in PAIRS])
def test_binary_matches_reference(op, dtype):
    fn = orc.load_ref().ref_binary(op, dtype)
    sup = bool(orc.lib.oracle_binary_supported(op, dtype))
    name = oh.BINARY_OPS[op]
    if not fn:
        # aliases of template_binary.c that the driver does not instantiate (same code under another name)
        alias_ok = (dtype == H.BOOL and name in ("min", "max", "fmin", "fmax")) or \
                   (name in ("bitwise_and", "bitwise_or", "bitwise_xor") and False)
        assert (not sup) or alias_ok, "oracle defines %s for %s but the reference does not" % (name, H.NAMES[dtype])
        return
    assert sup, "reference defines %s for %s but the oracle does not" % (name, H.NAMES[dtype])
    rng = np.random.default_rng(op * 31 + dtype)
    if dtype in (H.INT8, H.UINT8, H.BOOL) and name not in ("bitshift_left", "bitshift_right", "power"):
        vals = np.arange(256, dtype=np.uint8).view(H.storage(dtype)) if dtype != H.BOOL else np.array([0, 1], np.uint8)
        x = np.repeat(vals, vals.size)
        y = np.tile(vals, vals.size)
        dt2 = dtype
    else:
        n = 6000
        x = edge_values(dtype, rng, n)
        dt2, y = second_operand(op, dtype, rng, n, x)
    rdtype = H.BOOL if name in ("lt", "le", "eq", "ne", "ge", "gt") else dtype
    n = x.size
    z_ref = np.zeros(n, H.storage(rdtype))
    z_orc = np.zeros(n, H.storage(rdtype))
    call_ref(fn, BIN_PROTO, n, orc.ptr(x), orc.ptr(y), orc.ptr(z_ref))
    es1, es2, es3 = oh.TYPE_SIZE[dtype], oh.TYPE_SIZE[dt2], oh.TYPE_SIZE[rdtype]
    assert orc.lib.oracle_binary(op, dtype, 1, oh.sizes([n]), oh.strides([es1]), orc.ptr(x), oh.strides([es2]), orc.ptr(y),
                                 oh.strides([es3]), orc.ptr(z_orc)) == 0
    H.assert_same_bytes(z_orc, z_ref, "%s %s" % (name, H.NAMES[dtype]))


UPAIRS = [(op, dt) for op in range(len(oh.UNARY_OPS)) for dt in H.ALL_TYPES]


@pytest.mark.parametrize("op,dtype", UPAIRS, ids=["%s-%s" % (oh.UNARY_OPS[o], H.NAMES[d]) for o, d in UPAIRS])
def test_unary_matches_reference(op, dtype):
    fn = orc.load_ref().ref_unary(op, dtype)
    name = oh.UNARY_OPS[op]
    sup = bool(orc.lib.oracle_unary_supported(op, dtype))
    assert sup == bool(fn), "support differs for %s %s" % (name, H.NAMES[dtype])
    if not fn:
        return
    rng = np.random.default_rng(7000 + op * 31 + dtype)
    if dtype in (H.INT8, H.UINT8):
        x = np.arange(256, dtype=np.uint8).view(H.storage(dtype)).copy()
    elif dtype == H.HALF:
        x = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    else:
        x = edge_values(dtype, rng, 5000)
    if dtype in H.INT_TYPES and name not in ("negative", "bitwise_not", "reciprocal", "square", "fabs", "sign", "absolute",
                                              "isinf", "isnan", "isfinite", "isposinf", "isneginf"):
        # results go through double and a cast back: keep them inside the type's range
        lim = {"exp": 4, "exp2": 6, "exp10": 2, "expm1": 4, "sinh": 4, "cosh": 4}.get(name, 100)
        x = np.clip(x.astype(np.int64), -lim if np.iinfo(x.dtype).min < 0 else 0, lim).astype(x.dtype)
        if name in ("arccosh",):
            x = np.maximum(x, 1).astype(x.dtype)
        if name in ("arcsin", "arccos", "arctanh"):
            x = np.clip(x, -1 if np.iinfo(x.dtype).min < 0 else 0, 1).astype(x.dtype)
            if name == "arctanh":
                x[:] = 0
        if name in ("log", "log2", "log10") and np.iinfo(x.dtype).min >= 0:
            x = np.maximum(x, 1).astype(x.dtype)
        if name == "log1p" and np.iinfo(x.dtype).min < 0:
            x = np.maximum(x, 0).astype(x.dtype)
    rdtype = H.BOOL if name.startswith("is") else (dtype - 3 if (name == "absolute" and dtype >= H.CHALF) else dtype)
    n = x.size
    y_ref = np.zeros(n, H.storage(rdtype))
    y_orc = np.zeros(n, H.storage(rdtype))
    call_ref(fn, UN_PROTO, n, orc.ptr(x), orc.ptr(y_ref))
    assert orc.lib.oracle_unary(op, dtype, 1, oh.sizes([n]), oh.strides([oh.TYPE_SIZE[dtype]]), orc.ptr(x),
                                oh.strides([oh.TYPE_SIZE[rdtype]]), orc.ptr(y_orc), 1) == 0
    H.assert_same_bytes(y_orc, y_ref, "%s %s" % (name, H.NAMES[dtype]))


def test_half_conversion_exhaustive():
    """All 65536 half patterns to float, and a float sweep (every exponent, ties, boundaries) to half."""
    for h in range(0x10000):
        a = orc.lib.oracle_half_to_float(h)
        b = orc.load_ref().ref_half_to_float(h)
        assert np.float32(a).view(np.uint32) == np.float32(b).view(np.uint32) or (a != a and b != b), hex(h)
    rng = np.random.default_rng(3)
    bits = np.concatenate([
        rng.integers(0, 1 << 32, 200000, dtype=np.uint64).astype(np.uint32),
        (np.arange(0, 256, dtype=np.uint32) << 23),                             # every exponent, zero mantissa
        (np.arange(100, 150, dtype=np.uint32)[:, None] << 23 | np.array([0x1000, 0x0FFF, 0x1001, 0x3000, 0x7FFFFF, 0x7FE000, 0x7FF000], np.uint32)[None, :]).reshape(-1),
    ])
    bits = np.concatenate([bits, bits | np.uint32(0x80000000)])
    floats = bits.view(np.float32)
    for f in floats[:: 7]:
        assert orc.lib.oracle_float_to_half(float(f)) == orc.load_ref().ref_float_to_half(float(f)), float(f)


CPAIRS = [(s, d) for s in H.ALL_TYPES for d in H.ALL_TYPES]


@pytest.mark.parametrize("ts,td", CPAIRS, ids=["%s-%s" % (H.NAMES[s], H.NAMES[d]) for s, d in CPAIRS])
def test_conversions_match_reference(ts, td):
    """SOLID_ASSIGN and SOLID_BYTESWAP_ASSIGN for all 225 type pairs (values representable in the target)."""
    rng = np.random.default_rng(900 + ts * 15 + td)
    n = 3000
    x = edge_values(ts, rng, n)
    if ts in H.FLOAT_TYPES + H.COMPLEX_TYPES and td in H.INT_TYPES:
        # float -> integer is only defined for values inside the target range
        hi = min(120, int(np.iinfo(H.storage(td)).max))
        lo = -hi if np.iinfo(H.storage(td)).min < 0 else 0
        v = rng.uniform(lo, hi, n)
        if ts == H.HALF:
            x = H.f32_to_half_bits(v.astype(np.float32))
        elif ts == H.CHALF:
            x["real"] = H.f32_to_half_bits(v.astype(np.float32))
        elif ts in H.COMPLEX_TYPES:
            x = np.empty(n, x.dtype)
            x.real, x.imag = v, rng.uniform(-5, 5, n)
        else:
            x = v.astype(x.dtype)
    for swap, getter, orfn in ((0, orc.load_ref().ref_assign, orc.lib.oracle_copy), (1, orc.load_ref().ref_swap_assign, orc.lib.oracle_byteswap_copy)):
        fn = getter(ts, td)
        assert fn
        src = x.copy()
        if swap:      # store the source byte-reversed so that the swapped read sees the same values
            assert orc.lib.oracle_byteswap(ts, 1, oh.sizes([n]), oh.strides([oh.TYPE_SIZE[ts]]), orc.ptr(src), 1) == 0
        y_ref = np.zeros(n, H.storage(td))
        y_orc = np.zeros(n, H.storage(td))
        call_ref(fn, UN_PROTO, n, orc.ptr(src), orc.ptr(y_ref))
        assert orfn(ts, td, 1, oh.sizes([n]), oh.strides([oh.TYPE_SIZE[ts]]), orc.ptr(src),
                    1, oh.sizes([n]), oh.strides([oh.TYPE_SIZE[td]]), orc.ptr(y_orc), 2) == 0
        H.assert_same_bytes(y_orc, y_ref, "%s -> %s swap=%d" % (H.NAMES[ts], H.NAMES[td], swap))


def work_bytes(dtype, value_array):
    """Bytes of one value converted to the reference's work type (half -> float, chalf -> cfloat)."""
    if dtype == H.HALF:
        return np.array([orc.lib.oracle_half_to_float(int(value_array[0]))], np.float32).tobytes()
    if dtype == H.CHALF:
        return np.array([orc.lib.oracle_half_to_float(int(value_array["real"][0])),
                         orc.lib.oracle_half_to_float(int(value_array["imag"][0]))], np.float32).tobytes()
    return value_array[:1].tobytes()


RPAIRS = [(op, dt) for op in range(len(oh.REDUCE_OPS)) for dt in H.ALL_TYPES]


@pytest.mark.parametrize("op,dtype", RPAIRS, ids=["%s-%s" % (oh.REDUCE_OPS[o], H.NAMES[d]) for o, d in RPAIRS])
def test_reductions_match_reference(op, dtype):
    """Serial fold of a contiguous vector: init / accumulate / finalize code of reduce_ops.h."""
    name = oh.REDUCE_OPS[op]
    fn = orc.load_ref().ref_reduce(op, dtype)
    sup = bool(orc.lib.oracle_reduce_supported(op, dtype))
    if not fn:
        # *_nan variants of integer types forward to the plain operation in the CPU sources
        assert (not sup) or (name.endswith("_nan") and dtype <= H.INT64)
        return
    assert sup
    rng = np.random.default_rng(12000 + op * 31 + dtype)
    n = 777
    if dtype in H.INT_TYPES or dtype == H.BOOL:
        x = H.random_data(dtype, n, rng, "small" if name.startswith("prod") else "general")
        if name.startswith("prod"):
            x = x[:12]
    else:
        x = H.random_data(dtype, n, rng, "small" if name.startswith("prod") else "general")
        if name.startswith("prod"):
            x = x[:40]
        if name.endswith("_nan") or name in ("any_nan", "all_finite", "any_inf", "maximum", "minimum"):
            y = x.view(np.uint8).copy().view(x.dtype)
            nanv = H.random_data(dtype, 16, rng, "special")
            y[5:21] = nanv
            x = y
    n = x.size
    bounds = H.random_data(dtype, 2, rng, "general")
    lo, hi = bounds[0:1].copy(), bounds[1:2].copy()
    p = 3.0
    b1, b2 = oh.Scalar(), oh.Scalar()
    C.memmove(C.byref(b1), lo.ctypes.data, lo.dtype.itemsize)
    C.memmove(C.byref(b2), hi.ctypes.data, hi.dtype.itemsize)
    # parameter block of the reference function
    if name in ("all_lt", "all_le", "all_gt", "all_ge"):
        prm = work_bytes(dtype, lo)
    elif name.startswith("all_g") and len(name) == 8:
        prm = work_bytes(dtype, lo) + work_bytes(dtype, hi)
    elif name in ("norm", "norm_nan"):
        if dtype <= H.INT64:
            prm = np.array([p / 2, 1 / p], np.float64).tobytes()
        else:
            wt = np.float64 if dtype in (H.DOUBLE, H.CDOUBLE) else np.float32
            prm = np.array([p / 2, 1 / p], wt).tobytes()
    else:
        prm = b"\0" * 16
    prm_buf = C.create_string_buffer(prm, max(len(prm), 16))
    rdtype = orc.lib.oracle_reduce_result_dtype(op, dtype)
    r_ref = np.zeros(1, H.storage(rdtype))
    r_orc = np.zeros(1, H.storage(rdtype))
    call_ref(fn, RED_PROTO, n, orc.ptr(x), C.cast(prm_buf, C.c_void_p), orc.ptr(r_ref))
    assert orc.lib.oracle_reduce_all(op, dtype, 1, oh.sizes([n]), oh.strides([oh.TYPE_SIZE[dtype]]), orc.ptr(x),
                                     C.byref(b1), C.byref(b2), p, orc.ptr(r_orc), 1) == 0
    if name in ("norm", "norm_nan") and H.INT8 <= dtype <= H.INT64:
        # the reference converts the two double parameters of signed-integer norms through an
        # integer-typed copy routine (template_reduce_all.c:356-361); its result is not meaningful
        return
    H.assert_same_bytes(r_orc, r_ref, "%s %s" % (name, H.NAMES[dtype]))
