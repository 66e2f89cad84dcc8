"""Reader for the expected-output files (.ref) of the reference's example tests: Ocean's printed
tensors ("(:,:,k)" slices, rows = dimension 0, columns = dimension 1, closing line
"<tensor.TYPE of size AxB on DEVICE>") and bare scalar lines; plus conversion between parsed
values and the storage representation used by the parity tests."""
import re

import numpy as np

import helpers as H

TYPE_NAMES = {"bool": H.BOOL, "uint8": H.UINT8, "uint16": H.UINT16, "uint32": H.UINT32, "uint64": H.UINT64,
              "int8": H.INT8, "int16": H.INT16, "int32": H.INT32, "int64": H.INT64, "half": H.HALF, "float": H.FLOAT,
              "double": H.DOUBLE, "complex-half": H.CHALF, "complex-float": H.CFLOAT, "complex-double": H.CDOUBLE}
_NUM = r"(?:-?\d+(?:\.\d+)?(?:e[+-]?\d+)?|-?nan|-?inf)"
_TOKEN = re.compile(r"(True|False)|(%s)\s*([+-])\s*(%s)j|(%s)" % (_NUM, _NUM, _NUM))
_TENSOR = re.compile(r"^<(?:empty )?(?:tensor|storage)\.([\w-]+) of size ([\dx]+) on (\w+)( \(byteswapped\))?>$")
_SCALAR = re.compile(r"^<scalar\.([\w-]+) on (\w+)>$")


def parse_values(line):
    out = []
    for m in _TOKEN.finditer(line):
        if m.group(1):
            out.append(m.group(1) == "True")
        elif m.group(2):
            im = float(m.group(4)) * (-1 if m.group(3) == "-" else 1)
            out.append(complex(float(m.group(2)), im))
        else:
            out.append(float(m.group(5)))
    return out


class RefTensor:
    def __init__(self, dtype, shape, values, device, byteswapped):
        self.dtype, self.shape, self.device, self.byteswapped = dtype, shape, device, byteswapped
        self.values = values            # numpy complex128 / float64 / bool array in Ocean index order A[i0, i1, ...]; None: printed in part only

    def __repr__(self):
        return "RefTensor(%s, %s, %s)" % (H.NAMES[self.dtype], self.shape, self.device)


def parse_ref(text):
    """List of items in file order: RefTensor objects (tensors, storages printed as one-dimensional tensors, and
    "<scalar...>" zero-dimensional tensors with shape []), ('scalars', [values]) for lines made of values only, and
    ('text', line) for headings."""
    items, rows = [], []
    in_slices = False
    for line in text.splitlines():
        s = line.strip()
        if not s:
            continue
        m = _SCALAR.match(s)
        if m:                                                        # a zero-dimensional tensor: one value, then this line
            flat = [v for r in rows for v in r]
            assert len(flat) == 1, "scalar printed with %d values" % len(flat)
            items.append(RefTensor(TYPE_NAMES[m.group(1)], [], np.array(flat[0]), m.group(2), False))
            rows = []
            continue
        m = _TENSOR.match(s)
        if m:
            dtype = TYPE_NAMES[m.group(1)]
            shape = [int(x) for x in m.group(2).split("x")]
            flat = [v for r in rows for v in r]
            n = int(np.prod(shape))
            if len(flat) != n:                                    # large tensors are printed with rows left out
                items.append(RefTensor(dtype, shape, None, m.group(3), bool(m.group(4))))
                rows = []
                in_slices = False
                continue
            if n == 0:
                arr = np.zeros(shape)
            elif len(shape) == 1:
                arr = np.array(flat)
            else:
                # slices follow in order of the higher dimensions (first of them fastest); each slice lists rows of dimension 0
                d0, d1 = shape[0], shape[1]
                nsl = n // (d0 * d1)
                a = np.array(flat).reshape(nsl, d0, d1)          # [slice, i0, i1]
                arr = np.moveaxis(a, 0, 2).reshape([d0, d1] + shape[2:], order="F")
            items.append(RefTensor(dtype, shape, arr, m.group(3), bool(m.group(4))))
            rows = []
            in_slices = False
            continue
        if re.match(r"^\((:|\d+)(,(:|\d+))*\)$", s):
            if rows and not in_slices:                            # value lines before the first slice header: bare scalars
                for r in rows:
                    items.append(("scalars", r))
                rows = []
            in_slices = True
            continue
        vals = parse_values(s)
        rest = _TOKEN.sub("", s).replace(">", "").strip()
        if vals and not rest:
            rows.append(vals)
        else:
            if rows:                                              # value lines not closed by a tensor line: bare scalars
                for r in rows:
                    items.append(("scalars", r))
                rows = []
            if vals and s.startswith(">>>"):
                items.append(("scalars", vals))
            else:
                items.append(("text", s))
    for r in rows:
        items.append(("scalars", r))
    return items


def to_storage(dtype, values):
    """numpy storage array (Fortran order, same shape) for parsed values, converting as Ocean's asTensor does for these cases."""
    v = np.asarray(values)
    shape = v.shape
    st = H.storage(dtype)
    if dtype == H.BOOL:
        out = (v != 0).astype(np.uint8)
    elif dtype in H.INT_TYPES:
        out = np.asarray(np.real(v)).astype(np.float64).astype(np.int64).astype(st)
    elif dtype == H.HALF:
        out = H.f32_to_half_bits(np.real(v).astype(np.float32).reshape(-1)).reshape(shape)
    elif dtype in (H.FLOAT, H.DOUBLE):
        out = np.real(v).astype(st)
    elif dtype == H.CHALF:
        out = np.empty(shape, st)
        out["real"] = H.f32_to_half_bits(np.real(v).astype(np.float32).reshape(-1)).reshape(shape)
        out["imag"] = H.f32_to_half_bits(np.imag(v).astype(np.float32).reshape(-1)).reshape(shape)
    else:
        out = v.astype(st)
    return np.asfortranarray(out)


def half_bits_to_float(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float64)


def from_storage(dtype, arr):
    """float64 / complex128 / bool values of a storage array."""
    if dtype == H.BOOL:
        return arr != 0
    if dtype == H.HALF:
        return half_bits_to_float(arr)
    if dtype == H.CHALF:                                              # not real + 1j * imag: that turns a NaN imaginary part into NaN + NaNj
        out = np.empty(np.shape(arr), np.complex128)
        out.real, out.imag = half_bits_to_float(arr["real"]), half_bits_to_float(arr["imag"])
        return out
    if dtype in H.COMPLEX_TYPES:
        return arr.astype(np.complex128)
    return arr.astype(np.float64)


def assert_matches(dtype, got_storage, ref, what=""):
    """Stored result against printed values: exact for bool / integers, to the printed precision
    (5 decimals, relative for large magnitudes) for floating types; NaN matches NaN."""
    got = from_storage(dtype, got_storage)
    want = np.asarray(ref.values if isinstance(ref, RefTensor) else ref)
    assert list(got.shape) == list(want.shape), "%s: shape %s, expected %s" % (what, got.shape, want.shape)
    if dtype == H.BOOL:
        assert np.array_equal(got, want.astype(bool)), what
        return
    if dtype in H.INT_TYPES:
        assert np.array_equal(got, np.real(want)), "%s: got %s want %s" % (what, got, want)
        return
    g, w = got.astype(np.complex128), want.astype(np.complex128)
    for gp, wp in ((g.real, w.real), (g.imag, w.imag)):
        nan = np.isnan(wp)
        assert np.array_equal(np.isnan(gp), nan), what
        inf = np.isinf(wp)
        assert np.array_equal(gp[inf], wp[inf]) and not np.isinf(gp[~inf & ~nan]).any(), what
        nan = nan | inf
        ok = np.abs(gp[~nan] - wp[~nan]) <= 6e-6 * np.maximum(1.0, np.abs(wp[~nan]))
        assert ok.all(), "%s: got %s want %s" % (what, gp, wp)
