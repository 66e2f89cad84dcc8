"""Parity of the full reductions (och_reduce_all) with the CPU oracle and with exact arithmetic.

Reference tests of the same kind: examples/python/gpu/tensors/ocean_sum_01/02.py, ocean_sumabs_01.py,
ocean_maximumabs_01/02.py, ocean_min_01.py, ocean_all_01.py (CPU and GPU printed side by side),
examples/python/cpu/tensors/ocean_norm_01/02.py, axis_sum_01.py (NaN variants).

Exact (bit-for-bit against the oracle): any/all/all_finite/any_inf/any_nan, nnz, the range checks,
integer and bool sums / products / extrema / abs-extrema, float maximum / minimum (NaNs ignored).
Tolerance: floating sums, products and norms. The GPU accumulates in double as a tree; Ocean's CPU
path folds serially in the input precision per thread, so its own result moves with the thread
count. The GPU result is therefore gated against an exact (math.fsum / float64) evaluation of the
same inputs: relative 1e-5 for half/float inputs, 1e-12 for double, measured against sum|x| for
sums (the sum itself can cancel) and against the value for norms and products; the distance to the
literal CPU fold is reported with looser bounds.
"""
import ctypes as C
import math

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

pytestmark = pytest.mark.gpu
orc = H.orc

EXACT_OPS = {"any", "all", "all_finite", "any_inf", "any_nan", "nnz", "nnz_nan", "all_lt", "all_le", "all_gt", "all_ge",
             "all_gtlt", "all_gtle", "all_gelt", "all_gele", "maximum", "minimum"}


def to_float64(dtype, a):
    """Values of a storage array as float64 / complex128."""
    if dtype == H.HALF:
        return np.array([orc.lib.oracle_half_to_float(int(b)) for b in a.reshape(-1)], np.float64).reshape(a.shape)
    if dtype == H.CHALF:
        out = np.empty(a.shape, np.complex128)
        out.real, out.imag = to_float64(H.HALF, a["real"]), to_float64(H.HALF, a["imag"])
        return out
    if dtype == H.BOOL:
        return a.astype(np.float64)
    return a.astype(np.complex128 if dtype >= H.CFLOAT else np.float64)


def gpu_reduce(stream, op, dtype, x, b1=None, b2=None, p=0.0):
    rd = oh.lib.och_reduce_result_dtype(op, dtype)
    out = np.zeros(1, H.storage(rd))
    oh.check(oh.lib.och_reduce_all(op, dtype, len(x.shape), oh.sizes(x.shape), oh.strides(x.strides), x.dptr(),
                                   b1, b2, p, orc.ptr(out), None, stream.handle))
    return rd, out


def cpu_reduce(op, dtype, x, b1=None, b2=None, p=0.0, nthreads=1):
    rd = orc.lib.oracle_reduce_result_dtype(op, dtype)
    out = np.zeros(1, H.storage(rd))
    assert orc.lib.oracle_reduce_all(op, dtype, len(x.shape), oh.sizes(x.shape), oh.strides(x.strides), x.hptr(),
                                     b1, b2, p, orc.ptr(out), nthreads) == 0
    return rd, out


def check_against_truth(name, dtype, rd, got, xd):
    """Tolerance checks for floating sums / products / norms against float64 evaluation."""
    v = to_float64(dtype, xd).reshape(-1)
    g = to_float64(rd, got)[0]
    tol = 1e-12 if dtype in (H.DOUBLE, H.CDOUBLE) else (2e-3 if dtype in (H.HALF, H.CHALF) else 1e-5)
    skipnan = name.endswith("_nan")
    if skipnan:
        bad = np.isnan(v.real) | np.isnan(v.imag) if np.iscomplexobj(v) else np.isnan(v)
        v = v[~bad]
    if name in ("sum", "sum_nan"):
        if np.iscomplexobj(v):
            ref = complex(math.fsum(v.real), math.fsum(v.imag)); scale = math.fsum(np.abs(v.real)) + math.fsum(np.abs(v.imag))
        else:
            ref = math.fsum(v); scale = math.fsum(np.abs(v))
        assert abs(g - ref) <= tol * max(scale, 1e-30), (name, g, ref)
    elif name in ("sum_abs", "sum_abs_nan"):
        ref = math.fsum(np.abs(v)); assert abs(g - ref) <= tol * ref
    elif name in ("prod", "prod_nan"):
        ref = np.prod(v.astype(np.complex128 if np.iscomplexobj(v) else np.longdouble))
        assert abs(g - complex(ref) if np.iscomplexobj(v) else g - float(ref)) <= 20 * tol * abs(complex(ref))
    elif name in ("norm2", "norm2_nan"):
        ref = math.sqrt(math.fsum(np.abs(v) ** 2)); assert abs(g - ref) <= tol * ref
    elif name in ("norm", "norm_nan"):
        ref = math.fsum(np.abs(v) ** 3.0) ** (1 / 3.0); assert abs(g - ref) <= max(tol, 1e-6) * ref
    elif name in ("maximum_abs", "minimum_abs"):
        a = np.abs(v); a = a[~np.isnan(a)]
        ref = a.max() if name == "maximum_abs" else a.min()
        assert abs(g - ref) <= tol * max(ref, 1e-30)
    else:
        raise AssertionError("unhandled " + name)


PAIRS = [(op, dt) for op in range(len(oh.REDUCE_OPS)) for dt in H.ALL_TYPES]


@pytest.mark.parametrize("op,dtype", PAIRS, ids=["%s-%s" % (oh.REDUCE_OPS[o], H.NAMES[d]) for o, d in PAIRS])
def test_reduce_all(hip, stream, op, dtype):
    name = oh.REDUCE_OPS[op]
    sup = bool(oh.lib.och_reduce_supported(op, dtype))
    assert sup == bool(orc.lib.oracle_reduce_supported(op, dtype))
    if not sup:
        return
    assert oh.lib.och_reduce_result_dtype(op, dtype) == orc.lib.oracle_reduce_result_dtype(op, dtype)
    rng = np.random.default_rng(2000 + op * 16 + dtype)
    n = 70001 if not name.startswith("prod") else 23
    if dtype in (H.HALF, H.CHALF) and not (name in EXACT_OPS):
        n = min(n, 3001)                          # keeps half-precision sums inside the half range
    kind = "small" if (name.startswith("prod") or dtype in (H.HALF, H.CHALF)) else "general"
    if name in ("all", "all_finite") or name.startswith("all_"):
        kind = "positive"
    xd = H.random_data(dtype, n, rng, kind)
    if dtype >= H.HALF and name in ("any_nan", "any_inf", "all_finite", "maximum", "minimum", "nnz", "nnz_nan"):
        sp = H.random_data(dtype, 64, rng, "special")
        xd[100:164] = sp
        xd[0] = sp[0]                             # a special value may lead the tensor (a leading NaN must not stick to max/min)
    elif dtype >= H.HALF and name.endswith("_nan"):
        # NaN entries (no infinities: they would make the exact value infinite) that the operation must skip
        idx = rng.choice(n, size=max(2, n // 10), replace=False)
        nan_elem = H.random_data(dtype, 1, rng, "general")
        raw = nan_elem.view(np.uint16 if dtype in (H.HALF, H.CHALF) else (np.float32 if dtype in (H.FLOAT, H.CFLOAT) else np.float64))
        raw[0] = 0x7F00 if dtype in (H.HALF, H.CHALF) else np.nan
        xd[idx] = nan_elem[0]
        xd[0] = nan_elem[0]
    bounds = H.random_data(dtype, 2, rng, "general")
    b1, b2 = oh.Scalar(), oh.Scalar()
    C.memmove(C.byref(b1), bounds[0:1].ctypes.data, bounds.dtype.itemsize)
    C.memmove(C.byref(b2), bounds[1:2].ctypes.data, bounds.dtype.itemsize)
    p = 3.0
    x = H.Operand.contiguous(xd, dtype).upload(stream)
    rd, got = gpu_reduce(stream, op, dtype, x, C.byref(b1), C.byref(b2), p)
    _, want = cpu_reduce(op, dtype, x, C.byref(b1), C.byref(b2), p, nthreads=4)
    x.free()
    isint = dtype <= H.INT64
    if name in EXACT_OPS or (isint and not name.startswith("norm")):
        if name == "nnz_nan" and dtype == H.CHALF:
            # the CPU macro re-converts the float parts through the half type (reduce_ops.h:329-330) and so
            # treats |x| < 1 as zero; the kernel counts true non-zeros
            v = to_float64(dtype, xd)
            want = np.array([np.count_nonzero(~np.isnan(v.real) & ~np.isnan(v.imag) & (v != 0))], np.uint64)
        H.assert_same_bytes(got, want, "%s %s" % (name, H.NAMES[dtype]))
        return
    if isint:       # integer norms: double results
        v = to_float64(dtype, xd)
        ref = math.sqrt(math.fsum(v * v)) if name.startswith("norm2") else math.fsum(np.abs(v) ** 3.0) ** (1 / 3.0)
        assert abs(got[0] - ref) <= (1e-12 if name.startswith("norm2") else 1e-6) * ref
        return
    check_against_truth(name, dtype, rd, got, xd)
    if name == "prod_nan" and dtype >= H.CHALF:
        return                                   # CPU accumulate step has a sign slip (reduce_ops.h:784)
    # distance to the literal CPU fold (4 threads): informative bound, an order looser
    g, w = to_float64(rd, got)[0], to_float64(rd, want)[0]
    loose = 1e-10 if dtype in (H.DOUBLE, H.CDOUBLE) else (2e-2 if dtype in (H.HALF, H.CHALF) else 1e-3)
    if name in ("norm", "norm_nan"):
        loose = max(loose, 1e-5)                  # the CPU evaluates pow in single precision for every type
    if not (np.isnan(g) and np.isnan(w)):
        assert abs(g - w) <= loose * max(abs(w), 1.0), (name, g, w)


def test_reduce_strided_and_empty(hip, stream):
    rng = np.random.default_rng(9)
    parent = rng.integers(-50, 50, size=(33, 50, 20), dtype=np.int32)
    view = parent[::2, 1::3, ::-1].transpose(2, 0, 1)
    x = H.Operand(parent, view, H.INT32).upload(stream)
    for name in ("sum", "maximum", "minimum", "nnz", "sum_abs", "any", "all"):
        _, got = gpu_reduce(stream, oh.R[name], H.INT32, x)
        _, want = cpu_reduce(oh.R[name], H.INT32, x)
        H.assert_same_bytes(got, want, "strided " + name)
    assert got is not None
    x.free()
    # empty tensor: sum is 0, maximum is an error
    e = H.Operand.contiguous(np.zeros(4, np.float32), H.FLOAT).upload(stream)
    out = np.ones(1, np.float32)
    oh.check(oh.lib.och_reduce_all(oh.R["sum"], H.FLOAT, 1, oh.sizes([0]), oh.strides([4]), e.dptr(), None, None, 0.0, orc.ptr(out), None, stream.handle))
    assert out[0] == 0
    assert oh.lib.och_reduce_all(oh.R["maximum"], H.FLOAT, 1, oh.sizes([0]), oh.strides([4]), e.dptr(), None, None, 0.0, orc.ptr(out), None, stream.handle) == -1
    e.free()


@pytest.mark.parametrize("dtype", [H.FLOAT, H.DOUBLE], ids=lambda d: H.NAMES[d])
def test_config3_full_reductions(hip, stream, dtype):
    """benchmark configuration 3, full reductions: sum, 2-norm and max of an 8192 x 8192 N(0,1) tensor.
    max is exact; sum within 1e-5 (float) / 1e-12 (double) of the exact sum relative to sum|x|, and also
    relative to |sum| itself thanks to double accumulation; norm2 within the same relative tolerance."""
    n = 8192 * 8192
    rng = np.random.default_rng(33)
    xd = rng.standard_normal(n).astype(H.storage(dtype))
    x = H.Operand.contiguous(xd, dtype).upload(stream)
    tol = 1e-5 if dtype == H.FLOAT else 1e-12
    _, s = gpu_reduce(stream, oh.R["sum"], dtype, x)
    _, nrm = gpu_reduce(stream, oh.R["norm2"], dtype, x)
    _, mx = gpu_reduce(stream, oh.R["maximum"], dtype, x)
    x.free()
    v = xd.astype(np.float64)
    exact_sum = math.fsum(v)
    assert abs(float(s[0]) - exact_sum) <= tol * abs(exact_sum)
    exact_norm = math.sqrt(math.fsum(v * v))
    assert abs(float(nrm[0]) - exact_norm) <= tol * exact_norm
    assert mx[0] == xd.max()
    # determinism: a second launch gives the same bits
    x = H.Operand.contiguous(xd, dtype).upload(stream)
    _, s2 = gpu_reduce(stream, oh.R["sum"], dtype, x)
    x.free()
    H.assert_same_bytes(s, s2, "repeatability")


@pytest.mark.parametrize("dtype", [H.CFLOAT, H.CDOUBLE, H.CHALF], ids=lambda d: H.NAMES[d])
def test_complex_extremes_when_every_element_has_a_nan_part(hip, stream, dtype):
    """The reference starts from the first element and lets only NaN-free elements replace it (reduce_ops.h:912-968):
    when every element has a NaN part the result is the first element, whatever the size and the layout of the
    reduction (many blocks, axis reductions of both kinds); one NaN-free element anywhere wins."""
    rng = np.random.default_rng(5 + dtype)
    n = 300001
    re, im = rng.uniform(-5, 5, n), rng.uniform(-5, 5, n)
    pick = rng.random(n) < 0.5
    re[pick] = np.nan; im[~pick] = np.nan
    def as_storage(re, im):
        if dtype == H.CHALF:
            out = np.empty(n, H.storage(dtype)); out["real"] = H.f32_to_half_bits(re.astype(np.float32)); out["imag"] = H.f32_to_half_bits(im.astype(np.float32))
            return out
        out = np.empty(n, H.storage(dtype)); out.real, out.imag = re, im
        return out
    for clean_at in (None, 123457):
        r2, i2 = re.copy(), im.copy()
        if clean_at is not None:
            r2[clean_at], i2[clean_at] = -4.0, 2.0
        data = as_storage(r2, i2)
        x = H.Operand.contiguous(data, dtype).upload(stream)
        for name in ("maximum", "minimum"):
            _, got = gpu_reduce(stream, oh.R[name], dtype, x)
            _, want = cpu_reduce(oh.R[name], dtype, x)
            assert got.tobytes() == want.tobytes() == data[0 if clean_at is None else clean_at].tobytes(), (name, clean_at)
        x.free()
        # the same through the axis kernels: 3 rows of 100000 (cooperative kernel), 100000 columns of 3 (per-thread kernel)
        mat = data[:300000].reshape(3, 100000)
        for view, axes in ((mat, [1]), (mat.T, [0])):
            src = H.Operand(mat, view, dtype).upload(stream)
            kept = [view.shape[d] for d in range(view.ndim) if d not in axes]
            z = np.zeros(kept, data.dtype)
            dst = H.Operand(z, z, dtype).upload(stream)
            zc = z.copy(); cdst = H.Operand(zc, zc, dtype)
            for name in ("maximum", "minimum"):
                oh.check(oh.lib.och_reduce_axis(oh.R[name], dtype, H.axis_config(src, dst, axes, stream), 0.0))
                assert orc.lib.oracle_reduce_axis(oh.R[name], dtype, H.axis_config(src, cdst, axes, device=False), 0.0) == 0
                assert dst.download().tobytes() == zc.tobytes(), (name, axes, clean_at)
            src.free(); dst.free()


def test_reductions_on_two_streams_do_not_share_scratch(hip, stream):
    """Ocean gives every storage its own stream, so full reductions of different tensors run concurrently; the partial
    results and the ticket counter they use belong to the stream. Two streams reduce different data back to back, many
    times, without synchronisation in between; every result must equal the one computed alone."""
    rng = np.random.default_rng(77)
    other = oh.Stream()
    n = 1 << 21
    xs = [rng.integers(-1000, 1000, n).astype(np.int64), rng.integers(-1000, 1000, n).astype(np.int64)]
    streams = [stream, other]
    bufs = [oh.to_device(x, s) for x, s in zip(xs, streams)]
    reps = 40
    outs = [oh.DeviceBuffer(8 * reps, s) for s in streams]
    for s in streams:
        s.synchronize()
    for r in range(reps):
        for k in (0, 1):
            oh.check(oh.lib.och_reduce_all_device(oh.R["sum"], H.INT64, 1, oh.sizes([n - r]), oh.strides([8]), bufs[k].ptr, None, None, 0.0,
                                                  C.c_void_p(outs[k].address + 8 * r), None, streams[k].handle))
    for k in (0, 1):
        got = outs[k].download(np.int64, reps)
        want = np.array([xs[k][:n - r].sum() for r in range(reps)])
        assert np.array_equal(got, want), "stream %d" % k
    for b in bufs + outs:
        b.free()
    other.synchronize(); other.destroy()


def test_cross_block_hand_over_of_full_reductions_under_load(hip, stream):
    """The blocks of a full reduction hand their partial results to the block that draws the last ticket through device
    memory, with relaxed device-scope atomics and a wait for the writer's stores in front of the ticket. A partial that
    the last block read before it had arrived would give a wrong sum. Six streams run long series of full reductions at
    once -- large sources (one block per compute unit, all their partials in flight) and small ones (few blocks, the last
    block arrives almost at once), interleaved -- on integer data whose sums are known exactly; every result is compared,
    and the first mismatch stops the test with its position."""
    rng = np.random.default_rng(78)
    nstreams, reps = 6, 150
    streams = [stream] + [oh.Stream() for _ in range(nstreams - 1)]
    big, small = 1 << 23, 1 << 14
    data = [rng.integers(-1000, 1000, big).astype(np.int32) for _ in range(nstreams)]
    prefix = [np.concatenate([[0], np.cumsum(d.astype(np.int64))]) for d in data]
    bufs = [oh.to_device(d, s) for d, s in zip(data, streams)]
    outs = [oh.DeviceBuffer(8 * reps, s) for s in streams]
    lengths = [[(big - 17 * r - k) if (r + k) % 3 else (small + 5 * r + k) for r in range(reps)] for k in range(nstreams)]
    for s in streams:
        s.synchronize()
    for r in range(reps):
        for k in range(nstreams):
            oh.check(oh.lib.och_reduce_all_device(oh.R["sum"], H.INT32, 1, oh.sizes([lengths[k][r]]), oh.strides([4]), bufs[k].ptr, None, None, 0.0,
                                                  C.c_void_p(outs[k].address + 8 * r), None, streams[k].handle))
    for k in range(nstreams):
        got = outs[k].download(np.int64, reps)
        want = np.array([prefix[k][lengths[k][r]] for r in range(reps)])
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "stream %d, reduction %d of %d elements: got %d, want %d" % (k, bad[0], lengths[k][bad[0]], got[bad[0]], want[bad[0]])
    for b in bufs + outs:
        b.free()
    for s in streams[1:]:
        s.synchronize(); s.destroy()


ROW_TYPES = [H.BOOL, H.INT8, H.UINT8, H.INT16, H.UINT16, H.HALF, H.INT32, H.FLOAT, H.INT64, H.DOUBLE, H.CHALF, H.CFLOAT]


@pytest.mark.parametrize("dtype", ROW_TYPES, ids=lambda d: H.NAMES[d])
def test_reduce_rows_that_are_not_whole_vectors(hip, stream, dtype):
    """Contiguous rows that the 16-byte path cannot take as they are -- a width that is not a multiple of the vector
    length, a row pitch that is not a multiple of 16 bytes, a view that starts inside a 16-byte unit, a single misaligned
    run -- are read in aligned 16-byte chunks whose elements outside the row are left out. The elements next to every
    row (the rest of the parent) hold values that would change every result if one of them were counted. Counts,
    extremes and integer sums are exact; floating sums are within the usual bound of the float64 value."""
    rng = np.random.default_rng(3100 + dtype)
    es = np.dtype(H.storage(dtype)).itemsize
    layouts = []            # (parent shape, view builder)
    layouts.append(((37, 1024), lambda p: p[:, 3:1003].T))                 # 1000 wide, starts 3 elements in, aligned pitch
    layouts.append(((29, 1001), lambda p: p[:, 0:999].T))                  # odd width, odd pitch: every row placed differently
    layouts.append(((5000,), lambda p: p[1:4998]))                         # one run that starts one element in
    layouts.append(((5, 7, 130), lambda p: p[:, :, 1:101].transpose(2, 1, 0)))
    layouts.append(((300, 70), lambda p: p[:, 1:70].T))                    # rows a little over 64 bytes for 1-byte types
    layouts.append(((400, 33), lambda p: p[:, 1:32].T))                    # 31 elements: two or three chunks per row of bytes
    for shape, build in layouts:
        n = int(np.prod(shape))
        kind = "small" if dtype in (H.HALF, H.CHALF) else "general"
        parent = H.random_data(dtype, n, rng, kind).reshape(shape)
        view = build(parent)
        inside = np.zeros(shape, bool); build(inside)[...] = True
        # poison what lies outside the view: large values (and a non-zero count) that no result may reflect
        flat = parent.reshape(-1); mask = ~inside.reshape(-1)
        poison = H.random_data(dtype, n, rng, "positive" if dtype != H.BOOL else "general")
        flat[mask] = poison[mask]
        x = H.Operand(parent, view, dtype).upload(stream)
        for name in ("sum", "maximum", "minimum", "nnz", "any", "all"):
            op = oh.R[name]
            if not oh.lib.och_reduce_supported(op, dtype):
                continue
            rd, got = gpu_reduce(stream, op, dtype, x)
            _, want = cpu_reduce(op, dtype, x)
            what = "%s %s parent %s" % (name, H.NAMES[dtype], shape)
            if name != "sum" or dtype <= H.INT64:
                H.assert_same_bytes(got, want, what)
            else:
                check_against_truth(name, dtype, rd, got, np.ascontiguousarray(view))
        x.free()


def test_strided_reductions_in_several_launches(hip, stream):
    """A layout of several dimensions with more elements than one launch indexes is cut along its outer dimensions; the
    launches share the partial slots and the ticket counter. The limit is lowered so that small tensors take this path:
    integer results must equal the one-launch results bit for bit, the float64 sum is within the usual bound, and the
    counter is left at zero (the ordinary reduction that follows is right)."""
    rng = np.random.default_rng(77)
    parent = rng.integers(-100, 100, size=(9, 14, 40, 66), dtype=np.int32)
    views = [parent[:, 1:13, ::2, 1:65].transpose(3, 2, 1, 0),         # every dimension strided: 64 x 20 x 12 x 9 in Ocean order
             parent[::2, :, 3:39, 2:50],                               # numpy order: the last axis is Ocean's first dimension
             parent[3, 2:9, :, 1:64]]
    try:
        for view in views:
            x = H.Operand(parent, view, H.INT32).upload(stream)
            want = {}
            for name in ("sum", "maximum", "minimum", "nnz", "sum_abs"):
                oh.lib.och_reduce_set_part_limit(0)
                _, want[name] = gpu_reduce(stream, oh.R[name], H.INT32, x)
                _, cpu = cpu_reduce(oh.R[name], H.INT32, x)
                H.assert_same_bytes(want[name], cpu, "one launch " + name)
            # every limit keeps the number of launches within the 512 that share the slots
            for limit in (view.size // 2 + 1, 5000, 997) + ((200, 64) if view.ndim == 3 else ()):
                oh.lib.och_reduce_set_part_limit(limit)
                for name in want:
                    _, got = gpu_reduce(stream, oh.R[name], H.INT32, x)
                    H.assert_same_bytes(got, want[name], "%s with at most %d elements per launch, view %s" % (name, limit, view.shape))
            x.free()
        # floating point: order of the fold differs between the cuts, the bound does not
        pf = rng.standard_normal((40, 50, 30))
        vf = pf[1:39, ::2, 2:29].transpose(1, 2, 0)
        x = H.Operand(pf, vf, H.DOUBLE).upload(stream)
        for limit in (0, 4096, 333):
            oh.lib.och_reduce_set_part_limit(limit)
            for name in ("sum", "norm2"):
                rd, got = gpu_reduce(stream, oh.R[name], H.DOUBLE, x)
                check_against_truth(name, H.DOUBLE, rd, got, np.ascontiguousarray(vf))
        # a first dimension that alone exceeds the limit is refused, and the refusal leaves the counter usable
        oh.lib.och_reduce_set_part_limit(8)
        out = np.zeros(1, np.float64)
        assert oh.lib.och_reduce_all(oh.R["sum"], H.DOUBLE, len(x.shape), oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), None, None, 0.0,
                                     orc.ptr(out), None, stream.handle) == -1
        assert "first dimension" in oh.lib.och_last_error().decode()
        oh.lib.och_reduce_set_part_limit(0)
        rd, got = gpu_reduce(stream, oh.R["sum"], H.DOUBLE, x)
        check_against_truth("sum", H.DOUBLE, rd, got, np.ascontiguousarray(vf))
        x.free()
    finally:
        oh.lib.och_reduce_set_part_limit(0)
