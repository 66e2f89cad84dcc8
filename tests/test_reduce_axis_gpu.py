"""Parity of the axis reductions (och_reduce_axis) with the CPU oracle.

Reference tests of the same kind: examples/python/gpu/tensors/ocean_axis_reduce_04.py,
tensor_axis_norm2_01.py (against numpy.linalg.norm), examples/python/cpu/tensors/
axis_reduce_01..04.py (int8 -> int64 sums, several axes), axis_sum_01.py (NaN variants).
Exact for logical / counting / integer / extrema operations; floating sums and norms within
1e-5 (half 2e-3, double 1e-12) of a float64 evaluation, relative to the sum of magnitudes.
"""
import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

pytestmark = pytest.mark.gpu
orc = H.orc

AXIS_OPS = ["any", "all", "all_finite", "any_inf", "any_nan", "nnz", "nnz_nan", "sum", "sum_nan", "prod", "prod_nan",
            "sum_abs", "sum_abs_nan", "maximum", "minimum", "maximum_abs", "minimum_abs", "norm", "norm_nan", "norm2", "norm2_nan"]
EXACT = {"any", "all", "all_finite", "any_inf", "any_nan", "nnz", "nnz_nan", "maximum", "minimum"}


def to_f64(dtype, a):
    if dtype == H.HALF:
        return np.array([orc.lib.oracle_half_to_float(int(b)) for b in a.reshape(-1)], np.float64).reshape(a.shape)
    if dtype == H.CHALF:
        out = np.empty(a.shape, np.complex128)
        out.real, out.imag = to_f64(H.HALF, a["real"]), to_f64(H.HALF, a["imag"])
        return out
    return a.astype(np.complex128 if dtype >= H.CFLOAT else np.float64)


def run_case(stream, name, dtype, parent, view, axes, p=3.0, shift=0):
    """shift: the destination starts that many elements into its allocation (not 16-byte aligned any more)."""
    op = oh.R[name]
    rd = oh.lib.och_reduce_result_dtype(op, dtype)
    kept_shape = [n for d, n in enumerate(view.shape) if d not in axes]
    if shift:
        flat = np.zeros(int(np.prod(kept_shape)) + shift, H.storage(rd))
        out_parent, out_view = flat, flat[shift:].reshape(kept_shape[::-1]).T
        src = H.Operand(parent, view, dtype).upload(stream)
        dst = H.Operand(out_parent, out_view, rd).upload(stream)
        cfg = H.axis_config(src, dst, axes, stream)
        oh.check(oh.lib.och_reduce_axis(op, dtype, cfg, p))
        got = dst.download()
        want = out_parent.copy()
        dsth = H.Operand(want, want[shift:].reshape(kept_shape[::-1]).T, rd)
        assert orc.lib.oracle_reduce_axis(op, dtype, H.axis_config(src, dsth, axes, device=False), p) == 0
        src.free(); dst.free()
        return rd, got, want
    out_parent = np.zeros(kept_shape[::-1] if kept_shape else (1,), H.storage(rd))     # column-major destination
    out_view = out_parent.T if kept_shape else out_parent.reshape(())
    src = H.Operand(parent, view, dtype).upload(stream)
    dst = H.Operand(out_parent, out_view, rd).upload(stream)
    cfg = H.axis_config(src, dst, axes, stream)
    oh.check(oh.lib.och_reduce_axis(op, dtype, cfg, p))
    got = dst.download()
    want = out_parent.copy()
    dsth = H.Operand(want, want.T if kept_shape else want.reshape(()), rd)
    cfgh = H.axis_config(src, dsth, axes, device=False)
    assert orc.lib.oracle_reduce_axis(op, dtype, cfgh, p) == 0
    src.free(); dst.free()
    return rd, got, want


CASES = [(n, d) for n in AXIS_OPS for d in H.ALL_TYPES]


@pytest.mark.parametrize("name,dtype", CASES, ids=["%s-%s" % (n, H.NAMES[d]) for n, d in CASES])
def test_axis_all_ops(hip, stream, name, dtype):
    op = oh.R[name]
    if not oh.lib.och_reduce_supported(op, dtype):
        cfg = oh.ReduceAxisConfig()
        assert oh.lib.och_reduce_axis(op, dtype, cfg, 0.0) == -1
        return
    rng = np.random.default_rng(500 + op * 16 + dtype)
    small = name.startswith("prod") or dtype in (H.HALF, H.CHALF)
    shape = (6, 5, 7) if name.startswith("prod") else (37, 20, 11)
    parent = H.random_data(dtype, int(np.prod(shape)), rng, "small" if small else "general").reshape(shape[::-1])
    view = parent.T                                  # Ocean order: dimension 0 fastest
    if dtype >= H.HALF and name in ("any_nan", "any_inf", "all_finite", "maximum", "minimum", "nnz", "nnz_nan"):
        flat = parent.reshape(-1)
        flat[3:19] = H.random_data(dtype, 16, rng, "special")
    for axes in ([0], [1], [2], [0, 2], [0, 1, 2]):
        rd, got, want = run_case(stream, name, dtype, parent, view, axes)
        what = "%s %s axes=%s" % (name, H.NAMES[dtype], axes)
        isint = dtype <= H.INT64
        if name in EXACT or (isint and not name.startswith("norm")):
            if name == "nnz_nan" and dtype == H.CHALF:
                continue                              # CPU macro quirk, see test_reduce_gpu.py
            H.assert_same_bytes(got, want, what)
            continue
        if name == "prod_nan" and dtype >= H.CHALF:
            continue                                  # CPU accumulate step has a sign slip (reduce_ops.h:784)
        g, w = to_f64(rd, got), to_f64(rd, want)
        tol = 1e-12 if dtype in (H.DOUBLE, H.CDOUBLE) else (4e-3 if dtype in (H.HALF, H.CHALF) else 1e-5)
        if name in ("norm", "norm_nan"):
            tol = max(tol, 1e-5)                      # CPU pow is single precision
        v = to_f64(dtype, view)
        scale = np.abs(v).sum(axis=tuple(axes)).T if name.startswith("sum") else np.abs(w)
        if name.startswith("prod"):
            tol *= 50
        with np.errstate(invalid="ignore"):
            ok = (g == w) | (np.abs(g - w) <= tol * np.maximum(np.abs(np.asarray(scale)), 1e-6))
        assert np.all(ok), what


def test_axis_layouts(hip, stream):
    """Non-contiguous sources: sliced / transposed views, reduction along the fast and the slow axis,
    single-output and no-reduction corner cases."""
    rng = np.random.default_rng(2)
    parent = rng.integers(-99, 99, size=(24, 40, 64), dtype=np.int32)
    view = parent[::2, 1::3, ::-2].transpose(2, 0, 1)          # shape (32, 12, 13), mixed strides
    for axes in ([0], [1], [2], [1, 2], [0, 1], [0, 1, 2], []):
        for name in ("sum", "maximum", "nnz"):
            rd, got, want = run_case(stream, name, H.INT32, parent, view, axes)
            H.assert_same_bytes(got, want, "%s axes=%s" % (name, axes))
    # long reduction, few outputs (block-per-output path) and many outputs, short reduction
    big = rng.integers(-9, 9, size=(3, 50000), dtype=np.int16)
    rd, got, want = run_case(stream, "sum", H.INT16, big, big.T, [0])
    H.assert_same_bytes(got, want, "long reduction")
    wide = rng.integers(-9, 9, size=(5, 70000), dtype=np.int8)
    rd, got, want = run_case(stream, "sum", H.INT8, wide, wide.T, [1])
    H.assert_same_bytes(got, want, "many outputs")
    assert rd == H.INT64


@pytest.mark.parametrize("dtype", [H.FLOAT, H.DOUBLE], ids=lambda d: H.NAMES[d])
def test_config3_axis_reductions(hip, stream, dtype):
    """benchmark configuration 3, axis part: sum and min along axis 0 and axis 1 of a 3-D 512 x 512 x 256
    non-contiguous view (cut from a larger parent so that no two dimensions merge), N(0,1) data.
    min is exact; sum within 1e-5 / 1e-12 of the float64 result relative to the sum of magnitudes."""
    rng = np.random.default_rng(303)
    st = H.storage(dtype)
    parent = rng.standard_normal((258, 514, 516)).astype(st)
    view = parent[1:257, 1:513, 2:514].transpose(2, 1, 0)       # (512, 512, 256): dim 0 unit stride, padded pitches
    assert view.shape == (512, 512, 256)
    v64 = view.astype(np.float64)
    tol = 1e-5 if dtype == H.FLOAT else 1e-12
    for axis in (0, 1):
        rd, got, want = run_case(stream, "sum", dtype, parent, view, [axis])
        ref = v64.sum(axis=axis).T
        scale = np.abs(v64).sum(axis=axis).T
        assert np.all(np.abs(got.astype(np.float64) - ref) <= tol * scale), "axis %d sum" % axis
        rd, got, want = run_case(stream, "minimum", dtype, parent, view, [axis])
        H.assert_same_bytes(got, want, "axis %d min" % axis)
        H.assert_same_bytes(got, view.min(axis=axis).T.copy(), "axis %d min vs numpy" % axis)


SLICED = [  # Ocean shape (dimension 0 fastest), reduced axes: few outputs (or output groups) and a long reduced range
    ((1024, 3000), [1]),          # row sums of a column-major matrix: per-thread kernel, pieces along the reduced dimension
    ((200, 300, 64), [1, 2]),     # per-thread kernel, pieces of whole rows of the reduced range
    ((200, 300, 64), [0, 1]),     # a block per output, two reduced dimensions
    ((300000, 8), [0]),           # eight outputs, each a long contiguous row
    ((8, 300000), [1]),           # eight outputs, reduced dimension strided
    ((64, 5, 4000), [0, 2]),
    ((70001,), [0]),
]


@pytest.mark.parametrize("dtype", [H.INT32, H.FLOAT, H.DOUBLE, H.CFLOAT], ids=lambda d: H.NAMES[d])
def test_axis_reductions_cut_into_pieces(hip, stream, dtype):
    """Too few outputs to occupy the device: the reduced range is cut into pieces (grid y), every piece leaves its
    accumulator in the stream's workspace and a second kernel folds the pieces in a fixed order. Integers and extremes are exact,
    floating sums / norms within the usual bounds of the float64 result."""
    rng = np.random.default_rng(900 + dtype)
    for shape, axes in SLICED:
        parent = H.random_data(dtype, int(np.prod(shape)), rng, "general").reshape(shape[::-1])
        view = parent.T
        v = to_f64(dtype, view)
        for name in ("sum", "maximum", "nnz", "norm2", "sum_abs"):
            if not oh.lib.och_reduce_supported(oh.R[name], dtype):
                continue
            rd, got, want = run_case(stream, name, dtype, parent, view, axes)
            what = "%s %s %s axes=%s" % (name, H.NAMES[dtype], shape, axes)
            if dtype == H.INT32 and name != "norm2" or name in ("maximum", "nnz"):
                H.assert_same_bytes(got, want, what)
                continue
            # floating sums: against the float64 evaluation (the oracle adds in the element type, serially, and is the
            # less accurate side on ranges this long)
            g = to_f64(rd, got)
            ax = tuple(axes)
            truth = {"sum": v.sum(axis=ax), "sum_abs": np.abs(v).sum(axis=ax), "norm2": np.sqrt((np.abs(v) ** 2).sum(axis=ax))}[name].T
            scale = np.abs(v).sum(axis=ax).T if name == "sum" else np.abs(truth)
            tol = 1e-12 if dtype == H.DOUBLE else 1e-5
            assert np.all(np.abs(g - truth) <= tol * np.maximum(np.asarray(scale), 1e-6)), what


VECTOR_STORES = [(H.BOOL, "any"), (H.BOOL, "sum"), (H.INT8, "sum"), (H.UINT8, "maximum"), (H.INT16, "sum"), (H.INT16, "nnz"),
                 (H.INT32, "minimum"), (H.HALF, "maximum"), (H.FLOAT, "any"), (H.FLOAT, "maximum"), (H.FLOAT, "nnz"),
                 (H.DOUBLE, "all"), (H.DOUBLE, "minimum"), (H.CFLOAT, "nnz"), (H.CFLOAT, "any")]


@pytest.mark.parametrize("dtype,name", VECTOR_STORES, ids=["%s-%s" % (H.NAMES[d], n) for d, n in VECTOR_STORES])
def test_axis_results_stored_as_vectors(hip, stream, dtype, name):
    """Neighbouring threads own neighbouring outputs and a thread's results (16 bytes of input wide: 2 to 16 of them) are
    neighbours in the destination: they leave in stores of up to 16 bytes -- 1-byte logical results, 2- and 4-byte
    extremes, 8-byte sums and counts in several stores per thread. Every result is exact. The same reduction into a
    destination that starts one element into its allocation takes the element-wise stores and gives the same values,
    and nothing is written in front of it."""
    rng = np.random.default_rng(1200 + 16 * dtype + len(name))
    for shape, axes in (((192, 37), [1]), ((64, 9, 5), [1]), ((4096, 3), [1])):
        parent = H.random_data(dtype, int(np.prod(shape)), rng, "general").reshape(shape[::-1])
        rd, got, want = run_case(stream, name, dtype, parent, parent.T, axes)
        H.assert_same_bytes(got, want, "%s %s %s aligned" % (name, H.NAMES[dtype], shape))
        rd, got1, want1 = run_case(stream, name, dtype, parent, parent.T, axes, shift=1)
        H.assert_same_bytes(got1, want1, "%s %s %s shifted by one element" % (name, H.NAMES[dtype], shape))


ROW_MODE_TYPES = [H.BOOL, H.INT8, H.INT16, H.HALF, H.INT32, H.FLOAT, H.CFLOAT]


@pytest.mark.parametrize("dtype", ROW_MODE_TYPES, ids=lambda d: H.NAMES[d])
def test_axis_rows_that_are_not_whole_vectors(hip, stream, dtype):
    """Reductions along a contiguous dimension whose rows are not whole aligned 16-byte groups (odd width, odd pitch, a
    view that starts inside a 16-byte unit): the rows are read in aligned 16-byte chunks and the elements of the first
    and last chunk outside the row are left out. A block per output, a few lanes per output, two reduced dimensions and
    a reduced range cut into pieces; what lies next to the rows in the parent would change every result if counted."""
    rng = np.random.default_rng(4100 + dtype)
    layouts = [((37, 1024), lambda p: p[:, 3:1003].T, [0]),                      # 37 outputs, a block each
               ((1500, 70), lambda p: p[:, 1:70].T, [0]),                        # 1500 outputs, a few lanes each
               ((29, 1001), lambda p: p[:, 0:999].T, [0]),                       # every row placed differently
               ((6, 40, 130), lambda p: p[:, :, 1:101].transpose(2, 1, 0), [0, 2]),
               ((3, 300001), lambda p: p[:, 1:300000].T, [0]),                   # three outputs, rows cut into pieces
               # the kept dimension is the contiguous one: a thread owns an aligned chunk of neighbouring outputs
               ((37, 1024), lambda p: p[:, 3:1003].T, [1]),
               ((9, 50, 48), lambda p: p[:, :, 1:44].transpose(2, 1, 0), [1]),
               ((9, 50, 48), lambda p: p[:, :, 1:44].transpose(2, 1, 0), [1, 2]),
               ((300000, 48), lambda p: p[:, 1:40].T, [1])]                      # 39 outputs, a long range cut into pieces
    for shape, build, axes in layouts:
        n = int(np.prod(shape))
        parent = H.random_data(dtype, n, rng, "small" if dtype == H.HALF else "general").reshape(shape)
        inside = np.zeros(shape, bool); build(inside)[...] = True
        poison = H.random_data(dtype, n, rng, "positive" if dtype != H.BOOL else "general")
        flat, mask = parent.reshape(-1), ~inside.reshape(-1)
        flat[mask] = poison[mask]
        view = build(parent)
        v = to_f64(dtype, view)
        for name in ("sum", "maximum", "nnz"):
            if not oh.lib.och_reduce_supported(oh.R[name], dtype):
                continue
            rd, got, want = run_case(stream, name, dtype, parent, view, axes)
            what = "%s %s parent %s" % (name, H.NAMES[dtype], shape)
            if name != "sum" or dtype <= H.INT64:
                H.assert_same_bytes(got, want, what)
                continue
            g, ax = to_f64(rd, got), tuple(axes)
            truth, scale = v.sum(axis=ax).T, np.abs(v).sum(axis=ax).T
            tol = 4e-3 if dtype == H.HALF else 1e-5
            assert np.all(np.abs(g - truth) <= tol * np.maximum(np.asarray(scale), 1e-6)), what


def test_axis_reductions_with_more_outputs_than_a_launch_counts(hip, stream):
    """A reduction with more outputs than one launch counts is cut along its outermost kept dimension into reductions of
    their own (runs of that dimension, or single indices when one index is still too much). The limit is lowered so
    that small tensors are cut; integer results are bit for bit those of the uncut call and of the oracle."""
    rng = np.random.default_rng(41)
    parent = rng.integers(-99, 99, size=(11, 30, 26, 40), dtype=np.int32)
    view = parent[::2, 1::3, :, ::-2].transpose(3, 1, 2, 0)          # shape (20, 10, 26, 6), mixed strides
    try:
        for axes in ([0], [1], [3], [1, 2], [0, 3]):
            for name in ("sum", "maximum", "nnz"):
                oh.lib.och_reduce_axis_set_output_limit(0)
                rd, whole, want = run_case(stream, name, H.INT32, parent, view, axes)
                H.assert_same_bytes(whole, want, "uncut %s axes=%s" % (name, axes))
                for limit in (1000, 250, 37, 5, 1):
                    oh.lib.och_reduce_axis_set_output_limit(limit)
                    rd, got, _ = run_case(stream, name, H.INT32, parent, view, axes)
                    H.assert_same_bytes(got, whole, "%s axes=%s with at most %d outputs per launch" % (name, axes, limit))
    finally:
        oh.lib.och_reduce_axis_set_output_limit(0)


SHORT_ROWS = [(H.FLOAT, 8, 5000), (H.FLOAT, 4, 4099), (H.INT32, 16, 3001), (H.DOUBLE, 64, 1100), (H.DOUBLE, 2, 70001), (H.INT8, 256, 1030), (H.INT8, 16, 9000),
              (H.HALF, 32, 2050), (H.CFLOAT, 8, 2049), (H.INT16, 512, 1025), (H.INT64, 128, 1024)]


@pytest.mark.parametrize("dtype,row,nrows", SHORT_ROWS, ids=["%s-%dx%d" % (H.NAMES[d], r, n) for d, r, n in SHORT_ROWS])
def test_axis_short_contiguous_rows(hip, stream, dtype, row, nrows):
    """Many outputs, each the reduction of one short contiguous row of 1 ... 64 aligned 16-byte groups: the lanes that
    share an output load one group each and every lane group takes four outputs, so the last wave has outputs that do
    not exist. Counts, extremes and integer sums are exact; floating sums within the usual bound."""
    rng = np.random.default_rng(5200 + dtype + row)
    parent = H.random_data(dtype, row * nrows, rng, "general").reshape(nrows, row)
    view = parent.T                                                          # Ocean shape (row, nrows): the row is dimension 0
    v = to_f64(dtype, view)
    for name in ("sum", "maximum", "nnz", "any", "norm2", "minimum_abs"):
        if not oh.lib.och_reduce_supported(oh.R[name], dtype):
            continue
        rd, got, want = run_case(stream, name, dtype, parent, view, [0])
        what = "%s %s rows of %d x %d" % (name, H.NAMES[dtype], row, nrows)
        if (dtype <= H.INT64 and name != "norm2") or name in ("maximum", "nnz", "any") or (name == "minimum_abs" and dtype < H.CHALF):
            H.assert_same_bytes(got, want, what)
            continue
        g = to_f64(rd, got)
        truth = {"sum": v.sum(axis=0), "norm2": np.sqrt((np.abs(v) ** 2).sum(axis=0)), "minimum_abs": np.abs(v).min(axis=0)}[name]
        scale = np.abs(v).sum(axis=0) if name == "sum" else np.abs(truth)
        tol = 1e-12 if dtype == H.DOUBLE else (4e-3 if dtype == H.HALF else 1e-5)
        assert np.all(np.abs(g - truth) <= tol * np.maximum(np.asarray(scale), 1e-6)), what
