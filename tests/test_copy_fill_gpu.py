"""Parity of copy / cast / byteswap / fill / steps kernels with the CPU oracle (bit-exact).

Reference tests of the same kind: examples/python/gpu/tensors/tensor_copy_01..09.py (zero
stride broadcast copies, byteswapped sources, cross-dtype), tensor_dtype_cast_01.py,
ocean_cast_01.py, tensor_fill_01.py, tensor_fillnan_01.py, ocean_linspace_03.py.
Float -> integer conversions use in-range values only (out-of-range is undefined in the
reference, dtype_assign.h:109).
"""
import ctypes as C

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

pytestmark = pytest.mark.gpu
orc = H.orc


def source_values(ts, td, n, rng):
    x = H.random_data(ts, n, rng, "full" if ts in H.INT_TYPES and oh.TYPE_SIZE[ts] <= 2 else "general")
    if ts in H.FLOAT_TYPES + H.COMPLEX_TYPES and td in H.INT_TYPES:
        hi = min(120, int(np.iinfo(H.storage(td)).max))
        lo = -hi if np.iinfo(H.storage(td)).min < 0 else 0
        v = rng.uniform(lo, hi, n)
        if ts == H.HALF:
            x = H.f32_to_half_bits(v.astype(np.float32))
        elif ts == H.CHALF:
            x["real"] = H.f32_to_half_bits(v.astype(np.float32))
        elif ts in H.COMPLEX_TYPES:
            x = np.empty(n, H.storage(ts)); x.real, x.imag = v, rng.uniform(-5, 5, n)
        else:
            x = v.astype(H.storage(ts))
    elif ts in H.FLOAT_TYPES + H.COMPLEX_TYPES:
        x = H.random_data(ts, n, rng, "special")
    return x


PAIRS = [(s, d) for s in H.ALL_TYPES for d in H.ALL_TYPES]


@pytest.mark.parametrize("ts,td", PAIRS, ids=["%s-%s" % (H.NAMES[s], H.NAMES[d]) for s, d in PAIRS])
def test_cast_copy_all_pairs(hip, stream, ts, td):
    """och_copy and och_byteswap_copy for all 15 x 15 type pairs, contiguous and step-2 source."""
    rng = np.random.default_rng(300 + ts * 15 + td)
    n = 1030
    for swap in (0, 1):
        for step in (1, 2):
            xd = source_values(ts, td, n * step, rng)
            if swap:
                assert orc.lib.oracle_byteswap(ts, 1, oh.sizes([n * step]), oh.strides([oh.TYPE_SIZE[ts]]), orc.ptr(xd), 1) == 0
            x = H.Operand(xd, xd[::step], ts).upload(stream)
            y = H.Operand.contiguous(np.zeros(n, H.storage(td)), td).upload(stream)
            gfn = oh.lib.och_byteswap_copy if swap else oh.lib.och_copy
            cfn = orc.lib.oracle_byteswap_copy if swap else orc.lib.oracle_copy
            oh.check(gfn(ts, td, 1, oh.sizes([n]), oh.strides(x.strides), x.dptr(), 1, oh.sizes([n]), oh.strides(y.strides), y.dptr(), stream.handle))
            want = y.parent.copy()
            assert cfn(ts, td, 1, oh.sizes([n]), oh.strides(x.strides), x.hptr(), 1, oh.sizes([n]), oh.strides(y.strides), y.hptr(want), 2) == 0
            got = y.download()
            x.free(); y.free()
            H.assert_same_bytes(got, want, "%s -> %s swap=%d step=%d" % (H.NAMES[ts], H.NAMES[td], swap, step))


@pytest.mark.parametrize("ts,td", [(H.FLOAT, H.FLOAT), (H.INT16, H.FLOAT), (H.CFLOAT, H.CDOUBLE), (H.DOUBLE, H.INT32), (H.UINT8, H.BOOL)],
                         ids=lambda v: H.NAMES[v] if isinstance(v, int) else None)
def test_reshape_and_strided_copy(hip, stream, ts, td):
    """Different shapes with equal element count (reshape copy), transposed and broadcast sources."""
    rng = np.random.default_rng(17 + ts)
    # reshape: source 12 x 10 view (step 2 rows) -> destination 8 x 15, both column-major walks
    src_parent = source_values(ts, td, 24 * 10, rng).reshape(10, 24)       # numpy (10,24): fastest index last
    sv = src_parent.T[::2, :]                                              # shape (12,10), strides (2*es, 24*es)
    dst_parent = np.zeros((15, 8), H.storage(td))
    dv = dst_parent.T                                                      # shape (8,15) column-major
    x = H.Operand(src_parent, sv, ts).upload(stream)
    y = H.Operand(dst_parent, dv, td).upload(stream)
    oh.check(oh.lib.och_copy(ts, td, 2, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), 2, oh.sizes(y.shape), oh.strides(y.strides), y.dptr(), stream.handle))
    want = dst_parent.copy()
    assert orc.lib.oracle_copy(ts, td, 2, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(), 2, oh.sizes(y.shape), oh.strides(y.strides), y.hptr(want), 1) == 0
    H.assert_same_bytes(y.download(), want, "reshape copy")
    x.free(); y.free()
    # broadcast source (zero stride) into a transposed destination
    row = source_values(ts, td, 33, rng).reshape(1, 33)
    bv = np.broadcast_to(row, (21, 33))
    dst_parent = np.zeros((33, 21), H.storage(td))
    x = H.Operand(row, bv, ts).upload(stream)
    y = H.Operand(dst_parent, dst_parent.T, td).upload(stream)
    oh.check(oh.lib.och_copy(ts, td, 2, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), 2, oh.sizes(y.shape), oh.strides(y.strides), y.dptr(), stream.handle))
    want = dst_parent.copy()
    assert orc.lib.oracle_copy(ts, td, 2, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(), 2, oh.sizes(y.shape), oh.strides(y.strides), y.hptr(want), 1) == 0
    H.assert_same_bytes(y.download(), want, "broadcast copy")
    x.free(); y.free()


@pytest.mark.parametrize("dtype", H.ALL_TYPES, ids=[H.NAMES[d] for d in H.ALL_TYPES])
def test_byteswap_in_place(hip, stream, dtype):
    rng = np.random.default_rng(5 + dtype)
    parent = H.random_data(dtype, 40 * 23, rng).reshape(23, 40)
    x = H.Operand(parent, parent[::2, 1::3], dtype).upload(stream)
    oh.check(oh.lib.och_byteswap(dtype, 2, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), stream.handle))
    want = parent.copy()
    assert orc.lib.oracle_byteswap(dtype, 2, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(want), 1) == 0
    got = x.download()
    H.assert_same_bytes(got.view(np.uint8), want.view(np.uint8), "byteswap %s" % H.NAMES[dtype])
    # swapping twice restores the original bytes
    oh.check(oh.lib.och_byteswap(dtype, 2, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), stream.handle))
    H.assert_same_bytes(x.download().view(np.uint8), parent.view(np.uint8), "double byteswap")
    x.free()


def scalar_for(dtype, rng):
    v = H.random_data(dtype, 1, rng, "general")
    s = oh.Scalar()
    C.memset(C.byref(s), 0, C.sizeof(s))
    C.memmove(C.byref(s), v.ctypes.data, v.dtype.itemsize)
    return s


@pytest.mark.parametrize("dtype", H.ALL_TYPES, ids=[H.NAMES[d] for d in H.ALL_TYPES])
def test_fill_family(hip, stream, dtype):
    rng = np.random.default_rng(60 + dtype)
    value = scalar_for(dtype, rng)
    parent = H.random_data(dtype, 50 * 31, rng, "special" if dtype >= H.HALF else "general").reshape(31, 50)
    view = parent[1::2, ::3]
    mask_parent = rng.integers(0, 2, size=(50, 31)).astype(np.uint8)
    mview = mask_parent.T[1::2, ::3]
    for what in ("fill", "fill_nan", "masked_fill"):
        if what == "fill_nan" and dtype < H.HALF:
            assert oh.lib.och_fill_nan(dtype, 1, oh.sizes([1]), oh.strides([1]), None, value, stream.handle) == -1
            continue
        x = H.Operand(parent, view, dtype).upload(stream)
        want = parent.copy()
        if what == "masked_fill":
            m = H.Operand(mask_parent, mview, H.BOOL).upload(stream)
            oh.check(oh.lib.och_masked_fill(dtype, 2, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), oh.strides(m.strides), m.dptr(), value, stream.handle))
            assert orc.lib.oracle_masked_fill(dtype, 2, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(want), oh.strides(m.strides), m.hptr(), value, 2) == 0
            m.free()
        else:
            gfn = getattr(oh.lib, "och_" + what); cfn = getattr(orc.lib, "oracle_" + what)
            oh.check(gfn(dtype, 2, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), value, stream.handle))
            assert cfn(dtype, 2, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(want), value, 2) == 0
        got = x.download()
        x.free()
        H.assert_same_bytes(got.view(np.uint8), want.view(np.uint8), "%s %s" % (what, H.NAMES[dtype]))


@pytest.mark.parametrize("dtype", H.ALL_TYPES, ids=[H.NAMES[d] for d in H.ALL_TYPES])
def test_steps(hip, stream, dtype):
    """arange / linspace building blocks: value = offset + index * step with the flat index taken in
    the caller's dimension order."""
    n0, n1 = 37, 9
    parent = np.zeros((n1, 2 * n0), H.storage(dtype))
    view = parent[:, ::2].T                                               # shape (n0, n1), dim 0 strided
    cases = [("int64", (3, 2)), ("double", (0.25, 0.5)), ("cdouble", (oh.CDouble(1.0, -2.0), oh.CDouble(0.5, 0.25)))]
    if dtype in (H.BOOL, H.UINT8, H.INT8):
        cases[0] = ("int64", (0, 1) if dtype != H.BOOL else (0, 0))
        cases[1] = ("double", (0.0, 0.25))
        cases[2] = ("cdouble", (oh.CDouble(0.0, 0.0), oh.CDouble(0.25, 0.125)))
    # integer parameters wrap as an unsigned 64-bit sum before the conversion (template_steps.c:31-40): negative
    # values, wrap-around of the narrow types and a sum that passes 2^64 must all come out as on the CPU
    cases += [("int64", (-5, 3)), ("int64", (250, 1)), ("int64", (1 << 40, -(1 << 33))), ("int64", (-1, -1))]
    if dtype >= H.HALF or dtype in (H.INT16, H.INT32, H.INT64):
        cases += [("double", (-7.5, 1.75)), ("double", (1e-3, 1.0 / 3))]
    for kind, (a, b) in cases:
        x = H.Operand(parent, view, dtype).upload(stream)
        want = parent.copy()
        gfn = getattr(oh.lib, "och_steps_" + kind); cfn = getattr(orc.lib, "oracle_steps_" + kind)
        oh.check(gfn(dtype, 2, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), a, b, stream.handle))
        assert cfn(dtype, 2, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(want), a, b, 2) == 0
        got = x.download()
        x.free()
        H.assert_same_bytes(got.view(np.uint8), want.view(np.uint8), "steps_%s %s" % (kind, H.NAMES[dtype]))


def test_config4_cast_byteswap(hip, stream):
    """benchmark configuration 4 at reduced size (the full size is test_config4_full_size):
    int16 3-D tensor (full int16 range, stored byteswapped, step-2 slice) -> contiguous float32, and
    complex64 -> complex128."""
    rng = np.random.default_rng(4)
    d0, d1, d2 = 256, 64, 16
    parent = rng.integers(-32768, 32767, size=(d2, d1, 2 * d0), dtype=np.int16, endpoint=True)
    swapped = parent.byteswap()                       # bytes as a big-endian producer would have written them
    view = swapped.transpose(2, 1, 0)[::2]            # Ocean order: dim 0 fastest, step 2 along it
    assert view.shape == (d0, d1, d2)
    x = H.Operand(swapped, view, H.INT16).upload(stream)
    out = np.zeros((d2, d1, d0), np.float32)
    y = H.Operand(out, out.transpose(2, 1, 0), H.FLOAT).upload(stream)
    oh.check(oh.lib.och_byteswap_copy(H.INT16, H.FLOAT, 3, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(),
                                      3, oh.sizes(y.shape), oh.strides(y.strides), y.dptr(), stream.handle))
    want = out.copy()
    assert orc.lib.oracle_byteswap_copy(H.INT16, H.FLOAT, 3, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(),
                                        3, oh.sizes(y.shape), oh.strides(y.strides), y.hptr(want), 4) == 0
    got = y.download()
    x.free(); y.free()
    H.assert_same_bytes(got, want, "config 4a")
    H.assert_same_bytes(got, parent[:, :, ::2].astype(np.float32), "config 4a vs numpy")     # closed form: exact conversion
    n = 1 << 20
    z = (rng.uniform(-1, 1, n) + 1j * rng.uniform(-1, 1, n)).astype(np.complex64)
    x = H.Operand.contiguous(z, H.CFLOAT).upload(stream)
    y = H.Operand.contiguous(np.zeros(n, np.complex128), H.CDOUBLE).upload(stream)
    oh.check(oh.lib.och_copy(H.CFLOAT, H.CDOUBLE, 1, oh.sizes([n]), oh.strides([8]), x.dptr(), 1, oh.sizes([n]), oh.strides([16]), y.dptr(), stream.handle))
    got = y.download()
    x.free(); y.free()
    H.assert_same_bytes(got, z.astype(np.complex128), "config 4b")


def test_config4_full_size(hip, stream):
    """benchmark configuration 4 at its full size, bit for bit against the closed form (every int16 is exactly
    representable in float32 and every float32 in float64, so numpy's astype is the exact answer) and against the
    oracle: int16 1024 x 1024 x 64, uniform over the whole range, stored byte-swapped, every second element of the
    first dimension -> contiguous float32; complex64 -> complex128, 2^26 elements with parts from U(-1, 1)."""
    rng = np.random.default_rng(404)
    d0, d1, d2 = 1024, 1024, 64
    parent = rng.integers(-32768, 32767, size=(d2, d1, 2 * d0), dtype=np.int16, endpoint=True)
    swapped = parent.byteswap()
    view = swapped.transpose(2, 1, 0)[::2]
    assert view.shape == (d0, d1, d2)
    x = H.Operand(swapped, view, H.INT16).upload(stream)
    out = np.zeros((d2, d1, d0), np.float32)
    y = H.Operand(out, out.transpose(2, 1, 0), H.FLOAT).upload(stream)
    oh.check(oh.lib.och_byteswap_copy(H.INT16, H.FLOAT, 3, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(),
                                      3, oh.sizes(y.shape), oh.strides(y.strides), y.dptr(), stream.handle))
    got = y.download()
    want = out
    assert orc.lib.oracle_byteswap_copy(H.INT16, H.FLOAT, 3, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(),
                                        3, oh.sizes(y.shape), oh.strides(y.strides), y.hptr(want), 16) == 0
    x.free(); y.free()
    assert got.tobytes() == want.tobytes(), "config 4a, full size, against the oracle"
    assert np.array_equal(got, parent[:, :, ::2].astype(np.float32)), "config 4a, full size, against the closed form"
    del parent, swapped, got, want, out
    n = 1 << 26
    z = np.empty(n, np.complex64)
    z.real = rng.uniform(-1, 1, n).astype(np.float32); z.imag = rng.uniform(-1, 1, n).astype(np.float32)
    x = H.Operand.contiguous(z, H.CFLOAT).upload(stream)
    dst = oh.DeviceBuffer(16 * n, stream)
    oh.check(oh.lib.och_copy(H.CFLOAT, H.CDOUBLE, 1, oh.sizes([n]), oh.strides([8]), x.dptr(), 1, oh.sizes([n]), oh.strides([16]), dst.ptr, stream.handle))
    got = dst.download(np.complex128, n)
    x.free(); dst.free()
    want = np.empty(n, np.complex128)
    assert orc.lib.oracle_copy(H.CFLOAT, H.CDOUBLE, 1, oh.sizes([n]), oh.strides([8]), orc.ptr(z), 1, oh.sizes([n]), oh.strides([16]), orc.ptr(want), 16) == 0
    assert got.tobytes() == want.tobytes(), "config 4b, full size, against the oracle"
    assert np.array_equal(got, z.astype(np.complex128)), "config 4b, full size, against the closed form"


STEP2_TYPES = [H.BOOL, H.INT8, H.UINT8, H.INT16, H.HALF, H.INT32, H.FLOAT, H.INT64, H.DOUBLE, H.CFLOAT]


@pytest.mark.parametrize("dtype", STEP2_TYPES, ids=lambda d: H.NAMES[d])
def test_step2_sources(hip, stream, dtype):
    """Sources that are every second element of their first dimension (x[::2]) are read in wide loads of which the odd
    elements are dropped, when alignment allows, and element by element otherwise; both must give the oracle's bytes.
    Cases: aligned and misaligned starts, lengths that are and are not multiples of the vector length, a second
    dimension with an aligned and with an odd pitch, the last element of the view being the last of its buffer (the
    dropped element behind it would lie outside), same-type copies and widening casts, with and without byte swap."""
    rng = np.random.default_rng(900 + dtype)
    dst_types = [dtype, H.FLOAT if dtype not in (H.FLOAT, H.CFLOAT) else H.DOUBLE]
    if dtype == H.CFLOAT:
        dst_types = [H.CFLOAT, H.CDOUBLE]
    cases = []      # (parent elements, start, count, rows, pitch in elements)
    for start in (0, 1, 2, 8):
        for count in (1, 5, 64, 257, 1024):
            cases.append((start, count, 1, 0))
    cases += [(0, 128, 7, 256), (0, 128, 7, 258), (4, 100, 5, 301), (0, 64, 3, 128)]
    for start, count, rows, pitch in cases:
        nparent = start + 2 * count - 1 if rows == 1 else start + (rows - 1) * pitch + 2 * count - 1
        parent = H.random_data(dtype, nparent, rng, "full")
        if rows == 1:
            view = parent[start:start + 2 * count - 1:2]
        else:
            view = np.lib.stride_tricks.as_strided(parent[start:], shape=(rows, count), strides=(pitch * parent.itemsize, 2 * parent.itemsize)).T
        for dt2 in dst_types:
            for swap in (0, 1):
                if swap and dtype in (H.BOOL, H.INT8, H.UINT8):
                    continue
                x = H.Operand(parent, view, dtype).upload(stream)
                out = np.zeros(view.size + 3, H.storage(dt2))
                o = 1 if (start + count) % 2 else 0                    # destinations that wide stores can and cannot take
                oview = out[o:o + view.size] if rows == 1 else out[o:o + view.size].reshape(rows, count).T
                y = H.Operand(out, oview, dt2).upload(stream)
                gfn, cfn = (oh.lib.och_byteswap_copy, orc.lib.oracle_byteswap_copy) if swap else (oh.lib.och_copy, orc.lib.oracle_copy)
                nd = len(x.shape)
                oh.check(gfn(dtype, dt2, nd, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), nd, oh.sizes(y.shape), oh.strides(y.strides), y.dptr(), stream.handle))
                want = out.copy()
                assert cfn(dtype, dt2, nd, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(), nd, oh.sizes(y.shape), oh.strides(y.strides), y.hptr(want), 1) == 0
                got = y.download()
                x.free(); y.free()
                H.assert_same_bytes(got.view(np.uint8), want.view(np.uint8), "step-2 %s -> %s swap %d case %s" % (H.NAMES[dtype], H.NAMES[dt2], swap, (start, count, rows, pitch)))


def test_memset_is_exact_at_any_alignment_and_size(hip, stream):
    """och_memset_async (Buffer_zero, storage_gpu.c:283-302) fills by a kernel: unaligned head and tail bytes, the
    16-byte body and a large buffer, with the neighbouring bytes untouched."""
    rng = np.random.default_rng(77)
    base = rng.integers(0, 256, 1 << 16, dtype=np.uint8)
    for off, n, val in ((0, 0, 1), (0, 1, 7), (3, 5, 0), (1, 15, 255), (5, 16, 9), (13, 100, 0x81), (16, 4096, 0), (7, 40001, 3), (0, 1 << 16, 0)):
        d = oh.to_device(base, stream)
        oh.check(oh.lib.och_memset_async(C.c_void_p(d.address + off), val, n, stream.handle))
        want = base.copy(); want[off:off + n] = val & 0xFF
        assert np.array_equal(d.download(np.uint8), want), (off, n, val)
        d.free()
    big = oh.DeviceBuffer((64 << 20) + 3, stream)
    oh.check(oh.lib.och_memset_async(big.ptr, 0x5A, big.nbytes, stream.handle))
    got = big.download(np.uint8)
    assert got.min() == 0x5A and got.max() == 0x5A
    big.free()


def half_conversion_floats():
    """float32 bit patterns that reach every branch of the float -> half rule (half.c:101-149) on both sides of each
    boundary: every exponent with mantissas just below, at and above the rounding tie, with the kept bits all clear, all
    set (the carry runs into the exponent) and mixed; both signs; zeros, subnormals, infinities and NaNs."""
    low = np.array([0x0000, 0x0001, 0x0FFF, 0x1000, 0x1001, 0x1FFF], np.uint32)                  # the 13 bits that are dropped
    kept = np.array([0x000, 0x001, 0x155, 0x2AA, 0x3FE, 0x3FF], np.uint32) << 13              # the 10 bits that are kept
    mant = (kept[:, None] | low[None, :]).reshape(-1)
    ex = np.arange(256, dtype=np.uint32) << 23
    bits = (ex[:, None] | mant[None, :]).reshape(-1)
    bits = np.concatenate([bits, bits | np.uint32(0x80000000)])
    rng = np.random.default_rng(99)
    extra = rng.integers(0, 1 << 32, 200000, dtype=np.uint64).astype(np.uint32)
    near = (rng.integers(100, 150, 200000).astype(np.uint32) << 23) | rng.integers(0, 1 << 23, 200000).astype(np.uint32) | (rng.integers(0, 2, 200000).astype(np.uint32) << 31)
    return np.concatenate([bits, extra, near]).view(np.float32)


def test_half_conversions_cover_every_rule(hip, stream):
    """All 65536 half patterns to float and double, and a set of floats built to hit every branch of the float -> half
    rule (ties, the carry into the exponent, the flush below 2^-15, the exponents 2^-15 and 2^16 that the CPU routine
    encodes in its own way, overflow, NaN), bit for bit against the oracle, whose converter is pinned exhaustively
    against the reference's half.c. Lanes that take the integer routine sit next to lanes that do not."""
    halfs = np.arange(65536, dtype=np.uint16)
    rng = np.random.default_rng(7)
    halfs = np.concatenate([halfs, rng.permutation(halfs)])                  # special values scattered among ordinary ones
    n = halfs.size
    src = oh.to_device(halfs, stream)
    for dst_type, npt in ((H.FLOAT, np.float32), (H.DOUBLE, np.float64)):
        es = np.dtype(npt).itemsize
        dst = oh.DeviceBuffer(es * n, stream)
        oh.check(oh.lib.och_copy(H.HALF, dst_type, 1, oh.sizes([n]), oh.strides([2]), src.ptr, 1, oh.sizes([n]), oh.strides([es]), dst.ptr, stream.handle))
        got = dst.download(npt)
        want = np.empty(n, npt)
        assert orc.lib.oracle_copy(H.HALF, dst_type, 1, oh.sizes([n]), oh.strides([2]), orc.ptr(halfs), 1, oh.sizes([n]), oh.strides([es]), orc.ptr(want), 4) == 0
        assert got.tobytes() == want.tobytes(), "half -> %s" % H.NAMES[dst_type]
        dst.free()
    src.free()
    floats = half_conversion_floats()
    n = floats.size
    src = oh.to_device(floats, stream)
    dst = oh.DeviceBuffer(2 * n, stream)
    oh.check(oh.lib.och_copy(H.FLOAT, H.HALF, 1, oh.sizes([n]), oh.strides([4]), src.ptr, 1, oh.sizes([n]), oh.strides([2]), dst.ptr, stream.handle))
    got = dst.download(np.uint16)
    want = np.empty(n, np.uint16)
    assert orc.lib.oracle_copy(H.FLOAT, H.HALF, 1, oh.sizes([n]), oh.strides([4]), orc.ptr(floats), 1, oh.sizes([n]), oh.strides([2]), orc.ptr(want), 4) == 0
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, "float -> half: %d differ, first %r -> got %#06x want %#06x" % (bad.size, floats[bad[0]], got[bad[0]], want[bad[0]])
    src.free(); dst.free()
    # arithmetic on the half types goes through both converters: x + y, x * y and x / y on every pairing of a few hundred
    # patterns that include both zeros, subnormals, the largest finite value, infinities and NaNs
    pats = np.concatenate([np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x7BFF, 0xFBFF, 0x7C00, 0xFC00, 0x7C01, 0x7E00, 0xFE01, 0x3C00, 0xBC00,
                                     0x0200, 0x8200, 0x3555, 0x7800, 0xF800], np.uint16),
                           rng.integers(0, 65536, 236).astype(np.uint16)])
    x = np.repeat(pats, pats.size); y = np.tile(pats, pats.size)
    n = x.size
    dx, dy, dz = oh.to_device(x, stream), oh.to_device(y, stream), oh.DeviceBuffer(2 * n, stream)
    sz, st = oh.sizes([n]), oh.strides([2])
    for opname in ("add", "multiply", "divide", "subtract"):
        oh.check(oh.lib.och_binary(oh.B[opname], H.HALF, 1, sz, st, dx.ptr, st, dy.ptr, st, dz.ptr, stream.handle))
        got = dz.download(np.uint16)
        want = np.empty(n, np.uint16)
        assert orc.lib.oracle_binary(oh.B[opname], H.HALF, 1, sz, st, orc.ptr(x), st, orc.ptr(y), st, orc.ptr(want)) == 0
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "half %s: %d differ, first %#06x, %#06x -> got %#06x want %#06x" % (opname, bad.size, x[bad[0]], y[bad[0]], got[bad[0]], want[bad[0]])
    for b in (dx, dy, dz):
        b.free()
