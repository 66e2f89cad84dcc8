"""Pins, without a GPU, the oracle functions for which the reference holds no fixture: masked fill and the
two real-valued `steps` builders. What fixes their bits is the mathematics:

 * masked fill (solid/src/core/cpu/template_fill.c, solid/include/solid/core/generic/unary_ops.h `fill`):
   result = value where the boolean mask is non-zero, the old element elsewhere -- numpy.where;
 * steps (solid/src/core/cpu/template_steps.c:31-100): element i of the flat index, first dimension fastest, is
   offset + i * step evaluated in the parameter's arithmetic (int64 parameters meet the size_t index, so the
   sum is an unsigned 64-bit value that wraps), converted to the work type with C's conversion rules and then
   to the element type; complex types take the value as real part with a zero imaginary part.

The expected values are computed here with numpy integer / float64 arithmetic and numpy's casts (which follow
C for in-range values); half results go through the half converter, which is pinned exhaustively against the
reference's half.c elsewhere (tests/test_oracle_ref.py)."""
import ctypes as C

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh
import oracle_lib as orc

IDS = [H.NAMES[d] for d in H.ALL_TYPES]


def scalar_from(dtype, element):
    s = oh.Scalar()
    C.memset(C.byref(s), 0, C.sizeof(s))
    C.memmove(C.byref(s), element.ctypes.data, element.dtype.itemsize)
    return s


# ---------------------------------------------------------------------------------------------- masked fill
MASK_LAYOUTS = ["contiguous", "strided_view_transposed_mask", "broadcast_mask_row", "negative_stride", "three_dims"]


def masked_fill_case(layout, dtype, rng):
    """Returns (parent, view_of, mask_parent, mask_view): view_of(array shaped like parent) is the filled view,
    mask_view has the same shape."""
    kind = "special" if dtype >= H.HALF else "full" if dtype in H.INT_TYPES else "general"
    if layout == "contiguous":
        parent = H.random_data(dtype, 1000, rng, kind)
        mask = rng.integers(0, 2, 1000).astype(np.uint8)
        return parent, (lambda p: p), mask, mask
    if layout == "strided_view_transposed_mask":
        parent = H.random_data(dtype, 50 * 31, rng, kind).reshape(31, 50)
        mask = rng.integers(0, 2, (50, 31)).astype(np.uint8)
        return parent, (lambda p: p[1::2, ::3]), mask, mask.T[1::2, ::3]
    if layout == "broadcast_mask_row":
        parent = H.random_data(dtype, 40 * 17, rng, kind).reshape(40, 17)
        mask = rng.integers(0, 2, (1, 17)).astype(np.uint8)
        return parent, (lambda p: p), mask, np.broadcast_to(mask, (40, 17))
    if layout == "negative_stride":
        parent = H.random_data(dtype, 24 * 30, rng, kind).reshape(24, 30)
        mask = rng.integers(0, 2, (24, 30)).astype(np.uint8)
        return parent, (lambda p: p[::-1, ::2]), mask, mask[:, ::-2]
    parent = H.random_data(dtype, 6 * 7 * 8, rng, kind).reshape(6, 7, 8)
    mask = rng.integers(0, 2, (8, 6, 7)).astype(np.uint8)
    return parent, (lambda p: p[:, ::2, 1:7]), mask, mask.transpose(1, 2, 0)[:, ::2, 1:7]


@pytest.mark.parametrize("layout", MASK_LAYOUTS)
@pytest.mark.parametrize("dtype", H.ALL_TYPES, ids=IDS)
def test_masked_fill_is_numpy_where(dtype, layout):
    rng = np.random.default_rng(1000 + 17 * dtype + MASK_LAYOUTS.index(layout))
    parent, view_of, mask_parent, mask_view = masked_fill_case(layout, dtype, rng)
    # any non-zero mask byte counts as set (the mask is read as a boolean)
    mask_parent[mask_parent != 0] = rng.integers(1, 256, int((mask_parent != 0).sum())).astype(np.uint8)
    value = H.random_data(dtype, 1, rng, "general")
    view = view_of(parent)
    x = H.Operand(parent, view, dtype)
    m = H.Operand(mask_parent, mask_view, H.BOOL)
    assert (mask_view != 0).any() and (mask_view == 0).any()
    for nthreads in (1, 3):
        got = parent.copy()
        assert orc.lib.oracle_masked_fill(dtype, view.ndim, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(got),
                                          oh.strides(m.strides), m.hptr(), scalar_from(dtype, value), nthreads) == 0
        want = parent.copy()
        want_view = view_of(want)
        assert want_view.strides == view.strides
        want_view[...] = np.where(mask_view != 0, value[0], want_view)
        # whole parents are compared: elements outside the view must keep their bytes
        H.assert_same_bytes(got.view(np.uint8), want.view(np.uint8), "masked fill %s %s" % (H.NAMES[dtype], layout))


def test_masked_fill_rejects_unknown_type():
    one = np.zeros(1, np.uint8)
    assert orc.lib.oracle_masked_fill(15, 1, oh.sizes([1]), oh.strides([1]), orc.ptr(one), oh.strides([1]), orc.ptr(one),
                                      oh.Scalar(), 1) == -1


# ---------------------------------------------------------------------------------------------------- steps
def flat_index(shape):
    """Flat index of every element, first dimension fastest (Ocean's order), as an array of that shape."""
    return np.arange(int(np.prod(shape)), dtype=np.uint64).reshape(shape[::-1]).transpose()


def store_expected(dtype, want_view, real_values, kind):
    """Writes `real_values` (uint64 for the int64 builder, float64 for the double builder) into the view with
    the conversion C applies: integer truncation modulo 2^bits, round-to-nearest to float, the library's own
    float -> half."""
    st = H.storage(dtype)
    if dtype == H.BOOL:
        want_view[...] = real_values.astype(np.uint8)           # the work type of bool is its 8-bit storage
    elif dtype in H.INT_TYPES:
        if kind == "int64":
            want_view[...] = real_values.astype(st)             # uint64 -> narrower integer: keeps the low bits
        else:
            want_view[...] = np.trunc(real_values).astype(np.int64).astype(st)
    elif dtype == H.HALF:
        want_view[...] = H.f32_to_half_bits(real_values.astype(np.float32))
    elif dtype in (H.FLOAT, H.DOUBLE):
        want_view[...] = real_values.astype(st)
    elif dtype == H.CHALF:
        want_view["real"] = H.f32_to_half_bits(real_values.astype(np.float32))
        want_view["imag"] = 0
    else:
        want_view[...] = real_values.astype(np.float32 if dtype == H.CFLOAT else np.float64).astype(st)


STEP_LAYOUTS = ["one_dim", "strided_first_dim", "three_dims_permuted"]


def steps_view(layout, dtype):
    st = H.storage(dtype)
    if layout == "one_dim":
        parent = np.zeros(700, st)
        return parent, parent[3:700:2]
    if layout == "strided_first_dim":
        parent = np.zeros((9, 74), st)
        return parent, parent[:, ::2].T                          # shape (37, 9), first dimension strided
    parent = np.zeros((5, 6, 14), st)
    return parent, parent.transpose(1, 2, 0)[:, 1:14:3, :]       # shape (6, 5, 5)


INT64_PARAMS = [(0, 1), (3, 2), (-5, 3), (250, 1), (1 << 40, -(1 << 33)), (-1, -1), (7, 0)]


@pytest.mark.parametrize("layout", STEP_LAYOUTS)
@pytest.mark.parametrize("dtype", H.ALL_TYPES, ids=IDS)
def test_steps_int64_is_offset_plus_index_times_step(dtype, layout):
    for offset, step in INT64_PARAMS:
        parent, view = steps_view(layout, dtype)
        parent[...] = H.random_data(dtype, parent.size, np.random.default_rng(5), "general").reshape(parent.shape)
        x = H.Operand(parent, view, dtype)
        index = flat_index(view.shape)
        with np.errstate(over="ignore"):
            values = np.uint64(offset % (1 << 64)) + index * np.uint64(step % (1 << 64))     # wraps modulo 2^64
        # the unsigned sum is what gets converted: a negative result reads as a value near 2^64 for floating types
        # (and is out of the half range: it becomes infinity there)
        for nthreads in (1, 4):
            got = parent.copy()
            assert orc.lib.oracle_steps_int64(dtype, view.ndim, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(got),
                                              offset, step, nthreads) == 0
            want = parent.copy()
            want_view = np.ndarray(shape=view.shape, dtype=parent.dtype, buffer=want, offset=x.offset, strides=view.strides)
            store_expected(dtype, want_view, values, "int64")
            H.assert_same_bytes(got.view(np.uint8), want.view(np.uint8),
                                "steps_int64 %s %s (%d, %d)" % (H.NAMES[dtype], layout, offset, step))


def test_steps_int64_known_values():
    """Hand-computed anchors, independent of the helper above."""
    out = np.zeros(6, np.uint8)
    assert orc.lib.oracle_steps_int64(H.UINT8, 1, oh.sizes([6]), oh.strides([1]), orc.ptr(out), 250, 3, 1) == 0
    assert out.tolist() == [250, 253, 0, 3, 6, 9]                               # wraps modulo 256
    out = np.zeros(4, np.int8)
    assert orc.lib.oracle_steps_int64(H.INT8, 1, oh.sizes([4]), oh.strides([1]), orc.ptr(out), 126, 1, 1) == 0
    assert out.tolist() == [126, 127, -128, -127]
    out = np.zeros(5, np.uint8)
    assert orc.lib.oracle_steps_int64(H.BOOL, 1, oh.sizes([5]), oh.strides([1]), orc.ptr(out), 254, 1, 1) == 0
    assert out.tolist() == [254, 255, 0, 1, 2]                                  # bool keeps the low byte as it is
    out = np.zeros((3, 2), np.float32)                                          # C order (3, 2) = Ocean shape (2, 3)
    assert orc.lib.oracle_steps_int64(H.FLOAT, 2, oh.sizes([2, 3]), oh.strides([4, 8]), orc.ptr(out), 10, 5, 1) == 0
    assert out.tolist() == [[10, 15], [20, 25], [30, 35]]
    out = np.zeros(3, np.float64)
    assert orc.lib.oracle_steps_int64(H.DOUBLE, 1, oh.sizes([3]), oh.strides([8]), orc.ptr(out), -1, 1, 1) == 0
    assert out.tolist() == [float(2 ** 64), 0.0, 1.0]                           # -1 as an unsigned 64-bit sum
    out = np.zeros(3, np.complex64)
    assert orc.lib.oracle_steps_int64(H.CFLOAT, 1, oh.sizes([3]), oh.strides([8]), orc.ptr(out), 2, 3, 1) == 0
    assert out.tolist() == [2 + 0j, 5 + 0j, 8 + 0j]
    out = np.zeros(4, np.uint16)
    assert orc.lib.oracle_steps_int64(H.HALF, 1, oh.sizes([4]), oh.strides([2]), orc.ptr(out), 0, 1024, 1) == 0
    assert out.view(np.float16).tolist() == [0.0, 1024.0, 2048.0, 3072.0]


def double_params(dtype):
    """(offset, step) pairs whose values stay inside the element type's range (a float -> integer conversion of an
    out-of-range value is undefined in C, so neither the reference nor the oracle defines it)."""
    if dtype in (H.BOOL, H.UINT8, H.INT8):
        return [(0.0, 0.25), (1.5, 0.125), (100.9, 0.0)]
    if dtype in (H.UINT16, H.UINT32, H.UINT64):
        return [(0.25, 0.5), (7.0, 1.75), (3.999, 1e-3)]
    if dtype in (H.INT16, H.INT32, H.INT64):
        return [(0.25, 0.5), (-7.5, 1.75), (3.999, -1e-3), (-0.999, 0.0)]
    return [(0.25, 0.5), (-7.5, 1.75), (1e-3, 1 / 3), (0.1, -0.7), (65000.0, 100.0), (1e-7, 1e-8)]


@pytest.mark.parametrize("layout", STEP_LAYOUTS)
@pytest.mark.parametrize("dtype", H.ALL_TYPES, ids=IDS)
def test_steps_double_is_offset_plus_index_times_step(dtype, layout):
    for offset, step in double_params(dtype):
        parent, view = steps_view(layout, dtype)
        parent[...] = H.random_data(dtype, parent.size, np.random.default_rng(6), "general").reshape(parent.shape)
        x = H.Operand(parent, view, dtype)
        values = offset + flat_index(view.shape).astype(np.float64) * step      # one multiply, one add, unfused
        for nthreads in (1, 4):
            got = parent.copy()
            assert orc.lib.oracle_steps_double(dtype, view.ndim, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(got),
                                               offset, step, nthreads) == 0
            want = parent.copy()
            want_view = np.ndarray(shape=view.shape, dtype=parent.dtype, buffer=want, offset=x.offset, strides=view.strides)
            store_expected(dtype, want_view, values, "double")
            H.assert_same_bytes(got.view(np.uint8), want.view(np.uint8),
                                "steps_double %s %s (%r, %r)" % (H.NAMES[dtype], layout, offset, step))


def test_steps_double_known_values():
    out = np.zeros(5, np.int32)
    assert orc.lib.oracle_steps_double(H.INT32, 1, oh.sizes([5]), oh.strides([4]), orc.ptr(out), -1.5, 0.75, 1) == 0
    assert out.tolist() == [-1, 0, 0, 0, 1]                                     # -1.5 -0.75 0 0.75 1.5, truncated toward zero
    out = np.zeros(5, np.uint8)
    assert orc.lib.oracle_steps_double(H.BOOL, 1, oh.sizes([5]), oh.strides([1]), orc.ptr(out), 0.0, 0.5, 1) == 0
    assert out.tolist() == [0, 0, 1, 1, 2]
    out = np.zeros(4, np.float32)
    assert orc.lib.oracle_steps_double(H.FLOAT, 1, oh.sizes([4]), oh.strides([4]), orc.ptr(out), 0.1, 0.1, 1) == 0
    assert out.tolist() == [float(np.float32(0.1 + i * 0.1)) for i in range(4)]
    out = np.zeros(3, np.complex128)
    assert orc.lib.oracle_steps_double(H.CDOUBLE, 1, oh.sizes([3]), oh.strides([16]), orc.ptr(out), 1.0, -0.5, 1) == 0
    assert out.tolist() == [1 + 0j, 0.5 + 0j, 0j]
    out = np.zeros(3, np.uint16)
    assert orc.lib.oracle_steps_double(H.HALF, 1, oh.sizes([3]), oh.strides([2]), orc.ptr(out), 0.5, 0.25, 1) == 0
    assert out.view(np.float16).tolist() == [0.5, 0.75, 1.0]


def test_steps_cdouble_parts_follow_the_double_builder():
    """The complex builder is the double builder applied to each part (real types keep the real part only)."""
    for dtype in H.ALL_TYPES:
        off, stp = (oh.CDouble(0.5, 2.0), oh.CDouble(0.25, 0.125))
        n = 40
        got = np.zeros(n, H.storage(dtype))
        es = got.dtype.itemsize
        assert orc.lib.oracle_steps_cdouble(dtype, 1, oh.sizes([n]), oh.strides([es]), orc.ptr(got), off, stp, 2) == 0
        re = np.zeros(n, H.storage(dtype)); im = np.zeros(n, H.storage(dtype))
        assert orc.lib.oracle_steps_double(dtype, 1, oh.sizes([n]), oh.strides([es]), orc.ptr(re), 0.5, 0.25, 1) == 0
        assert orc.lib.oracle_steps_double(dtype, 1, oh.sizes([n]), oh.strides([es]), orc.ptr(im), 2.0, 0.125, 1) == 0
        if dtype in H.COMPLEX_TYPES:
            if dtype == H.CHALF:
                assert (got["real"] == re["real"]).all() and (got["imag"] == im["real"]).all()
            else:
                assert (got.real == re.real).all() and (got.imag == im.real).all()
        else:
            assert got.tobytes() == re.tobytes()
