"""More of the reference's GPU example tests replayed against their expected-output files (tests/golden/ref/):
ocean_bitshift_02, ocean_not_01, ocean_fabs_02, ocean_power_01 / 02 / 03, ocean_unary_01, ocean_cast_01,
tensor_dtype_cast_01, tensor_copy_03 / 04 / 06 / 07, tensor_add_01, tensor_subtract_01, tensor_multiply_01, tensor_divide_01,
tensor_fill_01, tensor_fillnan_01 (CPU twin, see below), ocean_linspace_03, ocean_sum_01, ocean_maximumabs_01,
tensor_axis_norm2_01, ocean_gemm_10 / 11. The inputs are the values the example scripts build (they are listed
with each test); the expectations are the printed results. Where Ocean's interface converts operands before it
calls the device module (result type of `int8 ** 0.5` is half, of `2 ** int8` int64, ...), the replay converts
them to the type the file shows for the result and runs the operation in that type, as the interface does.
Every case runs on the CPU oracle (always) and on the device library (gpu marker)."""
import ctypes as C
import os

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh
import ref_format as RF
from test_ref_fixtures import Engine, load, tensors, store, scalars

orc = H.orc


@pytest.fixture(params=["oracle", pytest.param("device", marks=pytest.mark.gpu)])
def engine(request):
    if request.param == "oracle":
        return Engine(False)
    request.getfixturevalue("hip")
    return Engine(True, request.getfixturevalue("stream"))


def col(dtype, values):
    """n x 1 storage array; row(): 1 x n"""
    return RF.to_storage(dtype, np.asarray(values).reshape(-1, 1))


def row(dtype, values):
    return RF.to_storage(dtype, np.asarray(values).reshape(1, -1))


def test_ocean_bitshift_02(engine):
    ts = tensors(load("ocean_bitshift_02"))
    assert len(ts) == 20
    for g in range(0, 20, 5):
        a, b = ts[g], ts[g + 1]                         # 1 x 4 row [0,1,2,9], shift counts [0,1,2,4,6,8]
        counts = RF.to_storage(H.INT8, b.values.reshape(6, 1))
        rd, got = engine.binary("bitshift_right", a.dtype, store(a), counts)
        RF.assert_matches(rd, got, ts[g + 2], "a >> b"); RF.assert_matches(rd, got, ts[g + 3], "bitshiftRight(a, b, r)")
        rd, got = engine.binary("bitshift_right", a.dtype, store(a), RF.to_storage(H.INT8, np.array([[1]])))
        RF.assert_matches(rd, got, ts[g + 4], "a >>= 1")


def test_ocean_not_01(engine):
    ts = tensors(load("ocean_not_01"))
    assert len(ts) == 18
    for g in range(0, 18, 6):
        a = ts[g]                                       # [0, 1, -1] in bool, int8, uint8
        x = store(a)
        rd, got = engine.unary("bitwise_not", a.dtype, x)
        for k in (1, 2, 4):
            RF.assert_matches(rd, got, ts[g + k], "bitwiseNot %s" % H.NAMES[a.dtype])
        rd, got = engine.unary("logical_not", H.BOOL, engine.cast(a.dtype, H.BOOL, x))      # the interface converts to bool first
        assert rd == H.BOOL
        RF.assert_matches(rd, got, ts[g + 3], "logicalNot")
        RF.assert_matches(a.dtype, engine.cast(H.BOOL, a.dtype, got), ts[g + 5], "logicalNot into the operand's type")


def test_ocean_fabs_02(engine):
    ts = tensors(load("ocean_fabs_02"))
    assert len(ts) == 10
    dtypes = [H.INT8, H.INT16, H.FLOAT, H.CHALF, H.CDOUBLE]
    for k, dt in enumerate(dtypes):                     # the result is converted into a destination of another type
        x = RF.to_storage(dt, np.array([-3 - 4j]))
        for base, name in ((0, "fabs"), (5, "absolute")):
            rd, got = engine.unary(name, dt, x)
            want = ts[base + k]
            RF.assert_matches(want.dtype, engine.cast(rd, want.dtype, got), want, "%s %s into %s" % (name, H.NAMES[dt], H.NAMES[want.dtype]))


def power(engine, dtype, base, base_dtype, exponent, exponent_dtype):
    """base ** exponent in `dtype`: the interface converts the base to the result type and the exponent to the type the
    operation takes there (int16 for integer results, the result type otherwise)"""
    et = oh.lib.och_binary_operand2_dtype(oh.B["power"], dtype)
    return engine.binary("power", dtype, engine.cast(base_dtype, dtype, base), engine.cast(exponent_dtype, et, exponent))


def test_ocean_power_01(engine):
    ts = tensors(load("ocean_power_01"))
    assert len(ts) == 16
    for g, dt in zip(range(0, 16, 4), (H.INT8, H.INT32, H.FLOAT, H.CFLOAT)):
        a = RF.to_storage(dt, np.array([1, 2, 3, 4]))
        for k, (swap, s) in enumerate(((False, 2), (True, 2), (False, 0.5), (True, 2.0))):
            want = ts[g + k]
            y = RF.to_storage(H.DOUBLE, np.array([s]))
            rd, got = power(engine, want.dtype, y, H.DOUBLE, a, dt) if swap else power(engine, want.dtype, a, dt, y, H.DOUBLE)
            RF.assert_matches(rd, got, want, "power_01 %s case %d" % (H.NAMES[dt], k))


def test_ocean_power_02(engine):
    ts = tensors(load("ocean_power_02"))
    assert len(ts) == 16
    for g, dt in zip(range(0, 16, 4), (H.INT8, H.INT32, H.FLOAT, H.CFLOAT)):
        a = row(dt, [1, 2, 3, 4])
        for k, (swap, other) in enumerate(((False, [0, 1, 2]), (True, [1, 2, 3]), (False, [0, 0.5, 1]), (True, [1.0, 2.0, 3.0]))):
            want = ts[g + k]
            y = col(H.DOUBLE, other)
            rd, got = power(engine, want.dtype, y, H.DOUBLE, a, dt) if swap else power(engine, want.dtype, a, dt, y, H.DOUBLE)
            RF.assert_matches(rd, got, want, "power_02 %s case %d" % (H.NAMES[dt], k))


def test_ocean_power_03(engine):
    ts = tensors(load("ocean_power_03"))
    assert len(ts) == 7
    a, b = row(H.FLOAT, [1, 2, 3, 4]), col(H.FLOAT, [0, 0.5, 1, 2])
    rd, got = engine.binary("power", H.FLOAT, a, b)
    for k in range(4):
        RF.assert_matches(rd, got, ts[k], "a ** b")
    RF.assert_matches(H.CDOUBLE, engine.cast(rd, H.CDOUBLE, got), ts[4], "power into complex-double")
    RF.assert_matches(H.INT16, engine.cast(rd, H.INT16, got), ts[5], "power into int16")
    rd, got = engine.binary("power", H.FLOAT, a, row(H.FLOAT, [1, 1, 1, 0.5]))
    RF.assert_matches(rd, got, ts[6], "a **= [1, 1, 1, 0.5]")


def test_ocean_unary_01(engine):
    ts = tensors(load("ocean_unary_01"))
    assert len(ts) == 4
    a = RF.to_storage(H.INT8, np.array([1, 2, 3]))
    # square(a, b) with b of type int16: computed in int8, stored as int16; then from a byte-swapped source
    # (one-byte elements: the swap is the identity) and into a byte-swapped int16 destination
    rd, sq = engine.unary("square", H.INT8, a)
    got = engine.cast(rd, H.INT16, sq)
    for k in range(3):
        RF.assert_matches(H.INT16, got, ts[k], "square into int16 #%d" % k)
    assert ts[3].byteswapped
    swapped = engine.swap_cast(H.INT16, H.INT16, got)              # what lands in the byte-swapped destination
    assert np.array_equal(swapped.view(np.uint8).reshape(-1, 2)[:, ::-1].reshape(-1).view(np.int16), got.reshape(-1))
    RF.assert_matches(H.INT16, swapped.byteswap(), ts[3], "square into a byte-swapped int16 tensor")


def test_casts(engine):
    ts = tensors(load("ocean_cast_01"))                 # A = [1, 2, 3] (int64) moved / converted: int64, float, half, int64, int8, int64 (storages), scalars
    a = RF.to_storage(H.INT64, np.array([1, 2, 3]))
    for want in ts[:6]:
        RF.assert_matches(want.dtype, engine.cast(H.INT64, want.dtype, a), want, "cast to %s" % H.NAMES[want.dtype])
    c = RF.to_storage(H.INT8, np.array([10]))
    RF.assert_matches(H.INT8, c.reshape(()), ts[6], "int8 scalar"); RF.assert_matches(H.INT16, engine.cast(H.INT8, H.INT16, c).reshape(()), ts[7], "int16 scalar")
    ts = tensors(load("tensor_dtype_cast_01"))          # float [1,2,3] -> int8, complex-double; [[1,2,3],[4,5,6.]] -> half
    f = RF.to_storage(H.FLOAT, np.array([1, 2, 3]))
    RF.assert_matches(H.INT8, engine.cast(H.FLOAT, H.INT8, f), ts[0], "int8(A)")
    RF.assert_matches(H.CDOUBLE, engine.cast(H.FLOAT, H.CDOUBLE, f), ts[1], "cdouble(A.storage)")
    d = RF.to_storage(H.DOUBLE, np.array([[1, 4], [2, 5], [3, 6.]]))
    RF.assert_matches(H.HALF, engine.cast(H.DOUBLE, H.HALF, d), ts[2], "half([[1,2,3],[4,5,6.]])")


def test_tensor_copy_03(engine):
    ts = tensors(load("tensor_copy_03"))
    a = ts[0]                                           # arange(18) as 3 x 6 int64, stored byte-swapped on the host
    assert a.byteswapped and a.dtype == H.INT64
    native = store(a)
    raw = np.asfortranarray(native.byteswap())          # the bytes as they sit in memory
    for k, td in ((4, H.FLOAT), (5, H.FLOAT), (6, H.DOUBLE), (7, H.INT64)):
        got = engine.swap_cast(H.INT64, td, raw)        # byte-swapped source, native destination
        RF.assert_matches(td, got, ts[k], "copy of a byte-swapped int64 tensor into %s" % H.NAMES[td])


def test_tensor_copy_04(engine):
    """A broadcast device tensor (arange(4) shown as 4 x 3, stride zero along dimension 1) copied into flat host tensors of
    other types, two of them byte-swapped; the flat result is then shown under several shapes."""
    ts = tensors(load("tensor_copy_04"))
    base = np.arange(4, dtype=np.float32)
    view = np.lib.stride_tricks.as_strided(base, shape=(4, 3), strides=(4, 0))
    RF.assert_matches(H.FLOAT, view, ts[0], "a")
    for k, (td, swapped) in enumerate(((H.HALF, True), (H.DOUBLE, True), (H.INT8, False), (H.DOUBLE, False))):
        native = engine.reshape_copy(H.FLOAT, td, base, view, (12,))
        if swapped:                                     # what the byte-swapped destination holds, read back in its own byte order
            stored = engine.byteswap(td, native)
            assert stored.tobytes() == native.byteswap().tobytes()
        assert ts[1 + k].byteswapped == swapped
        RF.assert_matches(td, native.reshape((4, 3), order="F"), ts[1 + k], "copy into %s%s" % (H.NAMES[td], " (byte-swapped)" if swapped else ""))
    for want, shape in zip(ts[5:], ((3, 4), (2, 6), (6, 2))):
        RF.assert_matches(H.DOUBLE, native.reshape(shape, order="F"), want, "reshape %s" % (shape,))


def test_tensor_copy_06(engine):
    ts = tensors(load("tensor_copy_06"))
    c = ts[0]                                           # arange(18) as 3 x 6 float, byte-swapped on the host
    raw = np.asfortranarray(store(c).byteswap())
    got = engine.reshape_copy(H.FLOAT, H.DOUBLE, raw, raw, (18,), swap=True)
    RF.assert_matches(H.DOUBLE, got, ts[3], "storage after the copy"); RF.assert_matches(H.DOUBLE, got, ts[4], "d after the copy")


def test_tensor_copy_07(engine):
    ts = tensors(load("tensor_copy_07"))
    A = np.asfortranarray(np.arange(15, dtype=np.float32).reshape((3, 5), order="F"))
    RF.assert_matches(H.FLOAT, A, ts[0], "A"); RF.assert_matches(H.FLOAT, A.T, ts[1], "A.T")
    assert A.T.strides == (12, 4)                        # the strides the file prints for A.T
    # cpu(A.T): same strides on the other device; flipAxis(0) and swapAxes are views
    RF.assert_matches(H.FLOAT, A[::-1, :], ts[3], "A.flipAxis(0)"); RF.assert_matches(H.FLOAT, A[::-1, :].T, ts[4], "its transpose")
    # C = zeros(B.size) is dense (strides 4, 20); C.copy(B) gathers the transposed view
    got = engine.reshape_copy(H.FLOAT, H.FLOAT, A, A.T, (5, 3))
    assert got.strides == (4, 20)
    RF.assert_matches(H.FLOAT, got, ts[8], "C after C.copy(B)"); RF.assert_matches(H.FLOAT, got.T, ts[9], "C.T")
    flipped = engine.reshape_copy(H.FLOAT, H.FLOAT, A, A[::-1, :], (3, 5))
    RF.assert_matches(H.FLOAT, flipped, ts[3], "dense copy of the flipped view")


def test_tensor_add_01(engine):
    ts = tensors(load("tensor_add_01"))
    A = np.zeros(100, np.float32); A[:15] = np.arange(15)
    RF.assert_matches(H.FLOAT, A, ts[0], "A"); RF.assert_matches(H.FLOAT, A[:15], ts[1], "B")
    # C views the first 15 elements as 5 x 3 with strides (3, 1) elements: C += 100 in place
    view = np.lib.stride_tricks.as_strided(A, shape=(5, 3), strides=(12, 4))
    RF.assert_matches(H.FLOAT, view, ts[2], "C")
    got = engine.binary_inplace("add", H.FLOAT, A, view, RF.to_storage(H.FLOAT, np.array([100])))
    RF.assert_matches(H.FLOAT, np.lib.stride_tricks.as_strided(got, shape=(5, 3), strides=(12, 4)), ts[3], "C += 100")
    RF.assert_matches(H.FLOAT, got, ts[4], "A afterwards: only the 15 viewed elements changed")


@pytest.mark.parametrize("name,op,groups", [
    ("tensor_subtract_01", "subtract", [(H.BOOL, 1, 4), (H.INT8, 3, 4), (H.FLOAT, 3, 4)]),
    ("tensor_multiply_01", "multiply", [(H.BOOL, 1, 4), (H.INT8, 3, 3), (H.FLOAT, 3, 3)]),
    ("tensor_divide_01", "divide", [(H.BOOL, 1, 3), (H.INT8, 3, 3), (H.FLOAT, 3, 3)])])
def test_arithmetic_with_scalars(engine, name, op, groups):
    """a (op) s and a (op)= s for bool, int8 and float; subtract also prints -a, multiply and divide on bool also
    combine with the tensor [True, False, True]."""
    ts = [t for t in tensors(load(name)) if t.device == "gpu0"]
    assert len(ts) == sum(g[2] for g in groups)
    pos = 0
    for dt, s, count in groups:
        a = ts[pos]; x = store(a); y = RF.to_storage(dt, np.array([s]))
        k = pos + 1
        if op == "subtract":
            rd, neg = engine.unary("negative", dt, x)
            RF.assert_matches(rd, neg, ts[k], "-a"); k += 1
        rd, got = engine.binary(op, dt, x, y)
        RF.assert_matches(rd, got, ts[k], "a %s s (%s)" % (op, H.NAMES[dt])); k += 1
        if dt == H.BOOL and op in ("multiply", "divide"):
            mask = RF.to_storage(H.BOOL, np.array([1, 0, 1]))
            rd, got = engine.binary(op, dt, x, mask)
            while k < pos + count:
                RF.assert_matches(rd, got, ts[k], "a %s [True, False, True]" % op); k += 1
        else:
            RF.assert_matches(rd, got, ts[k], "a %s= s" % op); k += 1
        assert k == pos + count
        pos += count


def test_fill_and_fillnan(engine):
    ts = tensors(load("tensor_fill_01"))
    assert len(ts) == 6
    for g, dt in zip(range(0, 6, 2), (H.INT16, H.FLOAT, H.CHALF)):
        for k, v in enumerate((24, 36)):
            got = engine.fill(dt, 1, v)
            RF.assert_matches(dt, got.reshape(()), ts[g + k], "fill %s with %d" % (H.NAMES[dt], v))
    # the GPU file of this example shows every element replaced: the reference's GPU function launches its plain fill
    # kernel (solid/src/core/gpu/template_fill.cu:72-79). The defined behaviour -- only NaN is replaced,
    # unary_ops.h:332-334 -- is what the CPU twin of the example prints, and what is built here.
    want = tensors(load("tensor_fillnan_01_cpu"))[0]
    got = engine.fill_nan(H.FLOAT, RF.to_storage(H.FLOAT, np.array([np.nan, 3, 4, np.nan])), np.inf)
    RF.assert_matches(H.FLOAT, got, want, "fillNaN(inf)")


def test_ocean_linspace_03(engine):
    ts = tensors(load("ocean_linspace_03"))
    want = ts[2]                                        # linspace(1+2j, 2+1j, 5) as complex-half on the device
    assert want.dtype == H.CHALF and want.device == "gpu0"
    got = engine.steps_complex(H.CHALF, 5, 1 + 2j, (1 - 1j) / 4)
    RF.assert_matches(H.CHALF, got, want, "linspace complex-half")


def test_scalar_reductions_more(engine):
    assert scalars(load("ocean_sum_01")) == [0.0]       # sum of an empty tensor
    rd, got = engine.reduce("sum", H.DOUBLE, np.zeros(0))
    assert got[0] == 0
    items = load("ocean_maximumabs_01")
    A = items[0]                                        # 2 x 2 complex-double
    rd, got = engine.reduce("maximum_abs", H.CDOUBLE, store(A))
    assert rd == H.DOUBLE and abs(got[0] - scalars(items)[0]) <= 6e-6 * got[0] and abs(got[0] - np.sqrt(10)) < 1e-14


def test_tensor_axis_norm2_01(engine):
    ts = tensors(load("tensor_axis_norm2_01"))
    assert ts[0].values is None and ts[0].shape == [65, 64]              # printed in part
    parent = np.arange(64 * 65, dtype=np.float64).reshape(64, 65, order="F")     # arange(64*65).reshape(64, 65)
    a = parent.T                                                        # .T: a 65 x 64 view whose rows are contiguous
    rd, got = engine.axis("norm2", H.DOUBLE, parent, a, [0])
    RF.assert_matches(rd, got, ts[1], "norm(a, 2, 0)"); RF.assert_matches(rd, got, ts[2], "numpy.linalg.norm of the columns")
    rd, got = engine.axis("norm2", H.DOUBLE, parent, a, [1])
    RF.assert_matches(rd, got, ts[3], "norm(a, 2, 1)"); RF.assert_matches(rd, got, ts[4], "numpy.linalg.norm of the rows")
    rd, got = engine.axis("norm2", H.DOUBLE, parent, a, [0, 1])
    assert abs(got.reshape(-1)[0] - 154882.040792) <= 1e-6 and abs(float(ts[5].values) - got.reshape(-1)[0]) <= 1.0


def test_gemm_with_empty_operands(engine):
    ts = tensors(load("ocean_gemm_10"))                 # (0 x 5) * (5) -> empty
    assert ts[0].shape == [0]
    assert engine.gemm_raw(H.FLOAT, 0, 1, 5, np.zeros(0, np.float32), np.ones(5, np.float32)).size == 0
    want = tensors(load("ocean_gemm_11"))[0]            # (5 x 0) * (0 x 5) -> 5 x 5 zeros, whatever C held before
    got = engine.gemm_raw(H.FLOAT, 5, 5, 0, np.zeros(0, np.float32), np.zeros(0, np.float32), c0=np.full(25, 7, np.float32))
    RF.assert_matches(H.FLOAT, got.reshape((5, 5), order="F"), want, "product over an empty inner dimension")


PAIRS = [(4, 3), (4, -3), (-4, 3), (-4, -3), (-2, -3), (2, -3), (10, 5), (10, -5)]


@pytest.mark.parametrize("name,op", [("ocean_divide_01_cpu", "divide"), ("ocean_floordivide_01_cpu", "floor_divide"), ("ocean_truedivide_01_cpu", "true_divide")])
def test_division_of_either_sign(engine, name, op):
    """a (op) b for the eight sign combinations the CPU example prints, in int8, half, float and double: integer `divide`
    and `floorDivide` round towards minus infinity, integer `trueDivide` truncates (binary_ops.h:154-235)."""
    ts = tensors(load(name))
    assert len(ts) == 32
    for g, (a, b) in enumerate(PAIRS):
        for k, dt in enumerate((H.INT8, H.HALF, H.FLOAT, H.DOUBLE)):
            rd, got = engine.binary(op, dt, RF.to_storage(dt, np.array([a])), RF.to_storage(dt, np.array([b])))
            RF.assert_matches(rd, got, ts[4 * g + k], "%d %s %d (%s)" % (a, op, b, H.NAMES[dt]))


def test_mod_and_fmod(engine):
    ts = tensors(load("ocean_fmod_01_cpu"))
    a, b = [-20, 20, -20, 20], [3, 3, -3, -3]
    for base, op in ((0, "mod"), (4, "fmod")):           # mod takes the sign of the divisor, fmod that of the dividend
        for k, dt in enumerate((H.INT64, H.FLOAT, H.DOUBLE)):
            rd, got = engine.binary(op, dt, RF.to_storage(dt, np.array(a)), RF.to_storage(dt, np.array(b)))
            RF.assert_matches(rd, got, ts[base + k], "%s %s" % (op, H.NAMES[dt]))
            RF.assert_matches(rd, got, ts[base + 3].values, "%s: the values the example expects" % op)


def test_sqrt_and_negative_over_types(engine):
    ts = tensors(load("tensor_sqrt_01_cpu"))
    assert len(ts) == 6
    # sqrt of an integer tensor is computed in double (the interface converts first); negative reals give NaN, complex
    # numbers their principal root; the last case stores the int8 -> double result into uint8 (NaN and fractions truncate)
    u8 = RF.to_storage(H.UINT8, np.arange(5))
    RF.assert_matches(H.DOUBLE, engine.unary("sqrt", H.DOUBLE, engine.cast(H.UINT8, H.DOUBLE, u8))[1], ts[0], "sqrt(uint8)")
    lin = np.linspace(-5, 5, 11)
    RF.assert_matches(H.DOUBLE, engine.unary("sqrt", H.DOUBLE, RF.to_storage(H.DOUBLE, lin))[1], ts[1], "sqrt(int16) in double")
    for want, dt in zip(ts[2:5], (H.HALF, H.FLOAT, H.CDOUBLE)):
        rd, got = engine.unary("sqrt", dt, RF.to_storage(dt, lin))
        RF.assert_matches(rd, got, want, "sqrt %s" % H.NAMES[dt])
    ts2 = tensors(load("ocean_sqrt_cpu"))               # arange(10) double, byte-swapped source and destination: values as above
    rd, got = engine.unary("sqrt", H.DOUBLE, RF.to_storage(H.DOUBLE, np.arange(10.0)))
    RF.assert_matches(rd, got, ts2[1], "sqrt(arange(10))"); RF.assert_matches(rd, got, ts2[2], "in place")
    ts = tensors(load("tensor_negative_01_cpu"))
    assert len(ts) == 6
    RF.assert_matches(H.BOOL, engine.unary("negative", H.BOOL, RF.to_storage(H.BOOL, np.array([1, 0, 0])))[1], ts[0], "-bool")
    # -uint8 is computed in int16 (the interface converts to the signed type that holds the range)
    RF.assert_matches(H.INT16, engine.unary("negative", H.INT16, RF.to_storage(H.INT16, np.arange(5)))[1], ts[1], "-uint8 as int16")
    for want, dt in zip(ts[2:], (H.INT16, H.HALF, H.FLOAT, H.CDOUBLE)):
        rd, got = engine.unary("negative", dt, RF.to_storage(dt, lin))
        RF.assert_matches(rd, got, want, "negative %s" % H.NAMES[dt])
    want = tensors(load("tensor_negative_02_cpu"))[0]   # -(-128) wraps to -128 in int8
    RF.assert_matches(H.INT8, engine.unary("negative", H.INT8, RF.to_storage(H.INT8, np.array([-128, -1, 0, 1, 127])))[1], want, "negative int8 extremes")
    want = tensors(load("ocean_power_04_cpu"))[0]       # integer power with a negative exponent is 0 (binary_ops.h:238-248)
    rd, got = power(engine, H.INT64, RF.to_storage(H.INT64, np.array([2, 3, 4])), H.INT64, RF.to_storage(H.INT64, np.array([-1])), H.INT64)
    RF.assert_matches(rd, got, want, "[2, 3, 4] ** -1")
