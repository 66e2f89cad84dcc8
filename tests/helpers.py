"""Shared helpers of the parity tests: seeded test data for every element type, strided
views, and paired execution of one operation on the GPU (through the C ABI) and in the
CPU oracle on identical inputs."""
import ctypes as C

import numpy as np

import ocean_hip as oh
import oracle_lib as orc

orc.setup(oh)

(BOOL, UINT8, UINT16, UINT32, UINT64, INT8, INT16, INT32, INT64,
 HALF, FLOAT, DOUBLE, CHALF, CFLOAT, CDOUBLE) = range(15)
ALL_TYPES = list(range(15))
INT_TYPES = [UINT8, UINT16, UINT32, UINT64, INT8, INT16, INT32, INT64]
SIGNED_TYPES = [INT8, INT16, INT32, INT64]
FLOAT_TYPES = [HALF, FLOAT, DOUBLE]
COMPLEX_TYPES = [CHALF, CFLOAT, CDOUBLE]
NAMES = oh.DTYPE_NAMES


def storage(dtype):
    return np.dtype(oh.NP_STORAGE[dtype])


def f32_to_half_bits(a):
    """float32 array -> Ocean half bit patterns, through the oracle's software converter."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    flat_in, flat_out = a.reshape(-1), out.reshape(-1)
    if flat_in.size >= 64:
        # the same converter, applied by the oracle's converting copy instead of one call per element
        n = flat_in.size
        assert orc.lib.oracle_copy(FLOAT, HALF, 1, oh.sizes([n]), oh.strides([4]), orc.ptr(flat_in), 1, oh.sizes([n]), oh.strides([2]), orc.ptr(flat_out), 8) == 0
        return out
    for i in range(flat_in.size):
        flat_out[i] = orc.lib.oracle_float_to_half(float(flat_in[i]))
    return out


def random_half_bits(rng, n, special=True):
    """Random half bit patterns covering normals, subnormals, zeros, infinities and NaNs."""
    bits = rng.integers(0, 0x10000, size=n, dtype=np.uint32).astype(np.uint16)
    if not special:
        bits &= np.uint16(0xBBFF)          # clears the top exponent bit: finite, |x| < 2
    return bits


def random_data(dtype, n, rng, kind="general"):
    """n elements of `dtype` in its numpy storage type.
    kind: 'general' (values near zero, mixed signs), 'small' (small magnitudes, safe for products and powers),
          'positive', 'special' (adds inf / nan / zeros for floating types), 'full' (whole integer range)."""
    st = storage(dtype)
    if dtype == BOOL:
        return rng.integers(0, 2, size=n).astype(np.uint8)
    if dtype in INT_TYPES:
        info = np.iinfo(st)
        if kind == "full":
            return rng.integers(info.min, info.max, size=n, dtype=st, endpoint=True)
        lo, hi = (-100, 100) if info.min < 0 else (0, 200)
        if kind == "small":
            lo, hi = (-6, 6) if info.min < 0 else (0, 12)
        if kind == "positive":
            lo, hi = 1, 100
        return rng.integers(lo, hi, size=n, endpoint=True).astype(st)
    scale = {"general": 10.0, "small": 2.0, "positive": 10.0, "special": 10.0, "full": 10.0}[kind]

    def reals(m):
        v = rng.uniform(-scale, scale, size=m)
        if kind == "positive":
            v = np.abs(v) + 0.25
        if kind == "special" and m >= 16:
            idx = rng.choice(m, size=max(4, m // 8), replace=False)
            v[idx] = rng.choice([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 0.5, 65504.0, 1e-8, -1e-8], size=idx.size)
        return v
    if dtype == HALF:
        return f32_to_half_bits(reals(n).astype(np.float32))
    if dtype == FLOAT:
        return reals(n).astype(np.float32)
    if dtype == DOUBLE:
        return reals(n)
    if dtype == CHALF:
        out = np.empty(n, dtype=st)
        out["real"] = f32_to_half_bits(reals(n).astype(np.float32))
        out["imag"] = f32_to_half_bits(reals(n).astype(np.float32))
        return out
    if dtype == CFLOAT:
        return (reals(n) + 1j * reals(n)).astype(np.complex64)
    return reals(n) + 1j * reals(n)


class Operand:
    """A strided view into a parent host buffer, mirrored by a device buffer of the same bytes."""

    def __init__(self, parent, view, dtype):
        self.parent, self.view, self.dtype = parent, view, dtype
        self.offset = view.__array_interface__["data"][0] - parent.__array_interface__["data"][0]
        self.shape = list(view.shape)
        self.strides = list(view.strides)
        self.dev = None

    @staticmethod
    def contiguous(data, dtype, shape=None):
        parent = np.ascontiguousarray(data)
        view = parent if shape is None else np.ndarray(shape=shape, dtype=parent.dtype, buffer=parent,
                                                       strides=fortran_strides(shape, parent.dtype.itemsize))
        return Operand(parent, view, dtype)

    def upload(self, stream):
        # bytes in memory order (the parent is C- or Fortran-contiguous)
        self.dev = oh.to_device(self.parent.ravel(order="K").view(np.uint8), stream)
        return self

    def dptr(self):
        return C.c_void_p(self.dev.address + self.offset)

    def hptr(self, parent=None):
        base = self.parent if parent is None else parent
        return C.c_void_p(base.__array_interface__["data"][0] + self.offset)

    def download(self):
        raw = self.dev.download(np.uint8, self.parent.nbytes)
        return np.ndarray(shape=self.parent.shape, dtype=self.parent.dtype, buffer=raw, strides=self.parent.strides)

    def free(self):
        if self.dev is not None:
            self.dev.free()
            self.dev = None


def fortran_strides(shape, itemsize):
    st, acc = [], itemsize
    for s in shape:
        st.append(acc)
        acc *= s
    return st


def _canonical_nans(a):
    """Copy of a float / complex array with every NaN replaced by one fixed NaN pattern."""
    a = np.array(a, copy=True)
    if a.dtype.kind == "c":
        parts = a.view(a.real.dtype)
    else:
        parts = a
    parts[np.isnan(parts)] = np.nan
    return a


def assert_same_bytes(got, want, what=""):
    """Bit-for-bit equality. For float32/float64/complex data a NaN matches any NaN: an invalid
    operation yields the default NaN of the executing hardware, whose sign bit differs between
    the x86 host (set) and the GPU (clear); no value information is lost by ignoring it."""
    got, want = np.ascontiguousarray(got), np.ascontiguousarray(want)
    if got.dtype == want.dtype and got.dtype.kind in "fc":
        got, want = _canonical_nans(got), _canonical_nans(want)
    g = got.view(np.uint8).reshape(-1)
    w = want.view(np.uint8).reshape(-1)
    if g.size != w.size or not np.array_equal(g, w):
        bad = np.nonzero(g != w)[0] if g.size == w.size else []
        first = int(bad[0]) if len(bad) else -1
        isz = got.dtype.itemsize
        detail = ""
        if first >= 0:
            e = first // isz
            detail = " element %d: got %r want %r" % (e, got.reshape(-1)[e], want.reshape(-1)[e])
        raise AssertionError("%s: %d of %d bytes differ (first at byte %d)%s" % (what, len(bad), g.size, first, detail))


def max_ulp_diff(got, want):
    """Largest distance in units in the last place between two float arrays of equal dtype (NaN == NaN)."""
    got, want = np.asarray(got), np.asarray(want)
    if got.dtype.kind == "c":
        return max(max_ulp_diff(got.real, want.real), max_ulp_diff(got.imag, want.imag))
    it = {4: np.int32, 8: np.int64}[got.dtype.itemsize]
    gi, wi = got.view(it).astype(np.int64), want.view(it).astype(np.int64)
    sign = np.int64(1) << (got.dtype.itemsize * 8 - 1)
    gi = np.where(gi < 0, -(gi & (sign - 1)), gi)
    wi = np.where(wi < 0, -(wi & (sign - 1)), wi)
    both_nan = np.isnan(got) & np.isnan(want)
    d = np.abs(gi - wi)
    d[both_nan] = 0
    return int(d.max()) if d.size else 0


def gpu_binary(stream, op, dtype, a, b, z):
    oh.check(oh.lib.och_binary(op, dtype, len(z.shape), oh.sizes(z.shape), oh.strides(a.strides), a.dptr(),
                               oh.strides(b.strides), b.dptr(), oh.strides(z.strides), z.dptr(), stream.handle))


def cpu_binary(op, dtype, a, b, z, zparent):
    st = orc.lib.oracle_binary(op, dtype, len(z.shape), oh.sizes(z.shape), oh.strides(a.strides), a.hptr(),
                               oh.strides(b.strides), b.hptr(), oh.strides(z.strides), z.hptr(zparent))
    assert st == 0


def gpu_unary(stream, op, dtype, a, z):
    oh.check(oh.lib.och_unary(op, dtype, len(z.shape), oh.sizes(z.shape), oh.strides(a.strides), a.dptr(),
                              oh.strides(z.strides), z.dptr(), stream.handle))


def cpu_unary(op, dtype, a, z, zparent, nthreads=1):
    st = orc.lib.oracle_unary(op, dtype, len(z.shape), oh.sizes(z.shape), oh.strides(a.strides), a.hptr(),
                              oh.strides(z.strides), z.hptr(zparent), nthreads)
    assert st == 0


def axis_config(src, dst, axes, stream=None, device=True):
    """och_reduce_axis_config for reducing `axes` of Operand src into Operand dst (dst has the kept
    dimensions only), prepared the way OcSolid_analyzeReduceAxis does: kept dimensions sorted by
    destination stride, reduced dimensions by source stride, unit dimensions dropped."""
    cfg = oh.ReduceAxisConfig()
    kept = [d for d in range(len(src.shape)) if d not in axes]
    outer = [(src.shape[d], src.strides[d], dst.strides[i]) for i, d in enumerate(kept) if src.shape[d] != 1]
    outer.sort(key=lambda t: abs(t[2]))
    inner = sorted([(src.shape[d], src.strides[d]) for d in axes if src.shape[d] != 1], key=lambda t: abs(t[1]))
    cfg.ndims = len(outer)
    for i, (n, s1, s2) in enumerate(outer):
        cfg.size[i], cfg.strides1[i], cfg.strides2[i] = n, s1, s2
    cfg.rdims = len(inner)
    for i, (n, s) in enumerate(inner):
        cfg.rsize[i], cfg.rstrides[i] = n, s
    if device:
        cfg.ptr1, cfg.ptr2 = src.dptr().value, dst.dptr().value
        cfg.stream = stream.handle if stream is not None else None
    else:
        cfg.ptr1, cfg.ptr2 = src.hptr().value, dst.hptr().value
    return cfg


def raw_scalar(element):
    """och_scalar holding the bytes of one stored element (numpy array of size 1, any storage type)."""
    a = np.ascontiguousarray(element).reshape(-1)[:1]
    s = oh.Scalar()
    C.memset(C.byref(s), 0, C.sizeof(s))
    C.memmove(C.byref(s), a.ctypes.data, a.itemsize)
    return s
