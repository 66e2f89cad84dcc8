"""Reductions replayed against the expected-output files of the reference's CPU example tests: ocean_axis_reduce_01 / 02
(axis sums of int8 into int64, keepdims, converted destinations; the three threading regimes), ocean_axis_sum_01 (sum,
sumAbs, prod and their NaN-skipping variants on complex data), ocean_axis_all_01, ocean_axis_nnz_01, ocean_norm_01 / 02
(p-norms; the interface maps p = 0, 1, inf to nnz, sumAbs, maximumAbs, tensor_itf.c:5405-5446). Runs on the oracle
(always) and on the device library (gpu marker)."""
import numpy as np
import pytest

import helpers as H
import ocean_hip as oh
import ref_format as RF
from test_ref_fixtures import Engine, load, tensors, scalars

orc = H.orc


@pytest.fixture(params=["oracle", pytest.param("device", marks=pytest.mark.gpu)])
def engine(request):
    if request.param == "oracle":
        return Engine(False)
    request.getfixturevalue("hip")
    return Engine(True, request.getfixturevalue("stream"))


def F(dtype, values):
    return RF.to_storage(dtype, np.asarray(values))


def test_axis_reduce_01(engine):
    ts = tensors(load("ocean_axis_reduce_01_cpu"))
    a = F(H.INT8, np.arange(60).reshape((3, 4, 5), order="F"))
    rd, got = engine.axis("sum", H.INT8, a, a, [2])
    assert rd == H.INT64
    RF.assert_matches(rd, got, ts[0], "sum(a, 2)")
    rd, kept = engine.axis("sum", H.INT8, a, a, [2], keepdims=True)
    RF.assert_matches(rd, kept, ts[1], "sum(a, 2, True)"); RF.assert_matches(rd, kept, ts[3], "into an int64 3 x 4 x 1 destination")
    assert ts[2].byteswapped and ts[2].dtype == H.DOUBLE                # computed as int64, converted, stored byte-swapped
    RF.assert_matches(H.DOUBLE, engine.cast(rd, H.DOUBLE, got), ts[2], "into a byte-swapped double destination")


def test_axis_reduce_02(engine):
    ts = tensors(load("ocean_axis_reduce_02_cpu"))
    for want, shape, axis in zip(ts, ((10, 10), (100, 50), (3, 10000)), (0, 0, 1)):
        a = np.ones(shape, np.float64, order="F")
        rd, got = engine.axis("sum", H.DOUBLE, a, a, [axis])
        RF.assert_matches(rd, got, want, "sum of ones %s over %d" % (shape, axis))


def test_axis_sum_01(engine):
    ts = tensors(load("ocean_axis_sum_01_cpu"))
    a = ts[0]                                           # 3 x 2 complex-double with one NaN
    x = RF.to_storage(H.CDOUBLE, a.values)
    for k, op in enumerate(("sum", "sum_nan", "sum_abs", "sum_abs_nan", "prod", "prod_nan")):
        rd, got = engine.axis(op, H.CDOUBLE, x, x, [0])
        assert rd == ts[1 + k].dtype
        RF.assert_matches(rd, got, ts[1 + k], op)


def test_axis_all_01(engine):
    ts = tensors(load("ocean_axis_all_01_cpu"))
    a = RF.to_storage(H.INT64, ts[0].values)            # 2 x 4 int64
    rd, got = engine.axis("all", H.INT64, a, a, [0])
    RF.assert_matches(rd, got, ts[1], "all(a, 0)")
    rd, got = engine.axis("any", H.INT64, a, a, [0], keepdims=True)
    RF.assert_matches(rd, got, ts[2], "any(a, 0, True)")
    # integers are always finite: the interface answers allFinite / anyInf without the device (ts[3], ts[4])
    assert ts[3].values.all() and not ts[4].values.any()


def test_axis_nnz_01(engine):
    items = load("ocean_axis_nnz_01_cpu")
    ts = tensors(items)
    a = RF.to_storage(H.INT8, ts[0].values)             # arange(45) % 12 as 3 x 5 x 3
    assert np.array_equal(ts[0].values, (np.arange(45) % 12).reshape((3, 5, 3), order="F"))
    rd, got = engine.reduce("nnz", H.INT8, a)
    assert rd == H.UINT64 and got[0] == scalars(items)[0] == 41
    for want, axes in zip(ts[1:], ([0], [1], [2], [0, 1])):
        rd, got = engine.axis("nnz", H.INT8, a, a, axes, keepdims=True)
        RF.assert_matches(rd, got, want, "nnz over %s" % axes)


def test_norm_01(engine):
    """norm(m, p) of the six values [[1+2j, 1+3j, 2], [2+1j, -3-4j, 0]] stored as int8, half, double (real parts) and
    complex-half, complex-float. Column 1 of the file is Ocean's result. For signed integers and p = 3 the reference
    returns 1: it writes the exponents p/2 and 1/p into double fields through an integer conversion
    (template_reduce_all.c:349-360); that case is left out, the defined value is checked instead."""
    items = load("ocean_norm_01_cpu")
    rows = [it[1] for it in items if isinstance(it, tuple) and it[0] == "scalars"]
    assert len(rows) == 25
    vals = np.array([[1 + 2j, 1 + 3j, 2 + 0j], [2 + 1j, -3 - 4j, 0 + 0j]])
    for g, dt in enumerate((H.INT8, H.HALF, H.DOUBLE, H.CHALF, H.CFLOAT)):
        x = F(dt, vals)
        for row, (p, op) in zip(rows[5 * g:5 * g + 5], ((0, "nnz"), (1, "sum_abs"), (2, "norm2"), (3, "norm"), (np.inf, "maximum_abs"))):
            want = row[1] if len(row) == 3 else row[0]          # "inf" in the first column does not parse as a row of three for p = inf
            if dt == H.INT8 and p == 3:
                rd, got = engine.reduce("norm", dt, x, p=3.0)
                assert abs(float(RF.from_storage(rd, got)[0]) - (1 + 1 + 8 + 8 + 27) ** (1 / 3)) < 1e-6     # the CPU path's pow is powf (unary_ops_cpu.h:87)
                continue
            rd, got = engine.reduce(op, dt, x, p=float(p) if op == "norm" else 0.0)
            g_val = float(np.real(RF.from_storage(rd, got)[0]))
            # printed with 7 decimals; results of type float may differ by one unit in the last place of a float between
            # a float accumulation (the reference) and a double accumulation rounded once (the device), half likewise
            tol = {H.HALF: 1e-3, H.CHALF: 1e-3, H.CFLOAT: 2.4e-7}.get(dt, 6e-8)
            assert abs(g_val - want) <= tol * max(1.0, abs(want)), "%s p=%s: got %.8f, file %.8f" % (H.NAMES[dt], p, g_val, want)


def test_norm_02(engine):
    items = load("ocean_norm_02_cpu")
    ts = tensors(items)
    a = RF.to_storage(H.DOUBLE, ts[0].values)           # [[1, 2, nan], [3, 4, -5]] as 2 x 3
    glob = scalars(items)[:5]                           # normNaN(a, p) for p = 0, 1, 2, 3, inf
    for want, op, p in zip(glob, ("nnz_nan", "sum_abs_nan", "norm2_nan", "norm_nan", "maximum_abs"), (0, 0, 0, 3.0, 0)):
        rd, got = engine.reduce(op, H.DOUBLE, a, p=p)
        assert abs(float(RF.from_storage(rd, got)[0]) - want) <= 6e-5 * want, op
    for base, suffix in ((1, ""), (6, "_nan")):         # norm(a, p, [0]) and normNaN(a, p, [0])
        for k, (op, p) in enumerate((("nnz", 0), ("sum_abs", 0), ("norm2", 0), ("norm", 3.0), ("maximum_abs", 0))):
            name = op + suffix if op != "maximum_abs" else op
            rd, got = engine.axis(name, H.DOUBLE, a, a, [0], p=p)
            assert rd == ts[base + k].dtype
            RF.assert_matches(rd, got, ts[base + k], "%s over axis 0" % name)
    tail = scalars(items)[5:]
    assert tail == [5.0, 5.0] or len(tail) == 2
    rd, got = engine.reduce("nnz", H.DOUBLE, a); assert got[0] == tail[0]
    rd, got = engine.reduce("nnz_nan", H.DOUBLE, a); assert got[0] == tail[1]


NAN = float("nan")


@pytest.mark.parametrize("name,op,y,cases", [
    ("ocean_maximum_01_cpu", "maximum", complex(3, NAN),
     [[NAN, 2], [1, NAN, 2], [2, NAN, 1], ["x", 2 + 1j], ["y", 1 + 2j], ["y", 1 + 3j], ["y", 1 + 4j], ["x", "y"], ["y", "x"],
      [1 + 1j, 2 + 0j], [1 + 1j, 2 + 1j], [1 + 1j, 2 + 2j], [1 + 1j, 1 + 0j], [1 + 2j, 1 + 2j], [1 + 2j, 1 + 3j]]),
    ("ocean_minimum_01_cpu", "minimum", complex(1, NAN),
     [[NAN, 2], [1, NAN, 2], [2, NAN, 1], ["x", 2 + 1j], ["y", 0 + 2j], ["y", 1 + 3j], ["y", 2 + 4j], ["x", "y"], ["y", "x"],
      [2 + 1j, 1 + 0j], [2 + 1j, 1 + 1j], [2 + 1j, 1 + 2j], [1 + 1j, 1 + 2j], [1 + 2j, 1 + 2j], [1 + 4j, 1 + 3j]]),
    ("ocean_maximum_abs_01_cpu", "maximum_abs", complex(1, NAN),
     [[NAN, 2], [1, NAN, 2], [-2, NAN, 1], ["x", 3 + 4j], ["y", 0 + 2j], ["x", "y"], [3 + 4j, 1 + 0j], [1 + 0j, 3 + 4j]]),
    ("ocean_minimum_abs_01_cpu", "minimum_abs", complex(1, NAN),
     [[NAN, 2], [1, NAN, 2], [-2, NAN, 1], ["x", 3 + 4j], ["y", 0 + 2j], ["x", "y"], [3 + 4j, 1 + 0j], [1 + 0j, 3 + 4j]])])
def test_extremes_with_nan_and_complex_order(engine, name, op, y, cases):
    """maximum / minimum (and of absolute values) over half vectors with NaN (NaN is skipped) and over complex-half vectors
    (ordered by real part, then imaginary part; an element with a NaN part never wins unless nothing else is there).
    x = NaN + 1j, y as given; the first three cases of each file are real (half), the others complex-half."""
    vals = scalars(load(name))
    assert len(vals) == len(cases)
    x = complex(NAN, 1)
    for k, (case, want) in enumerate(zip(cases, vals)):
        dt = H.HALF if k < 3 else H.CHALF
        data = np.array([x if v == "x" else y if v == "y" else v for v in case], dtype=np.complex128)
        rd, got = engine.reduce(op, dt, RF.to_storage(dt, data))
        RF.assert_matches(rd, got, np.array([want]), "%s %s" % (op, case))
