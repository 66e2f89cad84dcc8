"""Elementwise operations on unit-stride rows that are not whole aligned 16-byte vectors: sub-matrices of odd width,
rows that start inside a 16-byte unit, pitches that are not multiples of 16 bytes, operands misaligned differently from
each other. These run on the row kernels (aligned units of the destination, one wide access per operand for units inside
a row, single elements at the two ends). Checked bit for bit against the oracle over the WHOLE parent buffers, whose bytes
outside the views hold values that must survive; the launch analysis confirms that the row kernels are what runs."""
import ctypes as C

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

pytestmark = pytest.mark.gpu
orc = H.orc

ROW_TYPES = [H.BOOL, H.INT8, H.UINT16, H.HALF, H.FLOAT, H.INT32, H.DOUBLE, H.CHALF, H.CFLOAT]


def plan_of(operands):
    es = [np.dtype(H.storage(o.dtype)).itemsize for o in operands]
    return oh.elemwise_analyze(es, operands[0].shape, [o.strides for o in operands], [o.dev.address + o.offset for o in operands])


def layouts(dtype, rdtype, rng):
    """(name, x parent, x view, y parent, y view, z parent, z view): every z parent is filled with values to be kept."""
    out = []
    keep = lambda shape: H.random_data(rdtype, int(np.prod(shape)), rng, "positive" if rdtype != H.BOOL else "general").reshape(shape)
    data = lambda shape: H.random_data(dtype, int(np.prod(shape)), rng).reshape(shape)
    # numpy order: the last axis is the row
    A, B, Z = data((37, 1024)), data((37, 1024)), keep((37, 1024))
    out.append(("odd width, same start", A, A[:, 3:1002], B, B[:, 3:1002], Z, Z[:, 3:1002]))
    A, B, Z = data((29, 1001)), data((31, 1003)), keep((29, 1007))
    out.append(("odd pitches, three different starts", A, A[:, 1:1000], B, B[2:31, 4:1003], Z, Z[:, 7:1006]))
    A, B, Z = data((5000,)), data((5003,)), keep((5001,))
    out.append(("one dimension, misaligned inputs", A, A[1:4998], B, B[5:5002], Z, Z[0:4997]))
    A, B, Z = data((5000,)), data((5000,)), keep((5002,))
    out.append(("one dimension, misaligned destination", A, A[0:4999], B, B[0:4999], Z, Z[3:5002]))
    A, Z = data((6, 7, 131)), keep((6, 7, 140))
    row = data((1, 1, 131))
    out.append(("three dimensions, row broadcast", A, A[:, :, 1:130], row, np.broadcast_to(row, (6, 7, 131))[:, :, 1:130], Z, Z[:, :, 9:138]))
    col = data((40, 1))
    A, Z = data((40, 75)), keep((40, 80))
    out.append(("column broadcast", A, A[:, 2:73], col, np.broadcast_to(col, (40, 71)), Z, Z[:, 5:76]))
    A, B, Z = data((33, 70)), data((33, 200)), keep((33, 70))
    out.append(("stepped second input", A, A[:, 1:70], B, B[:, 3:141:2], Z, Z[:, 1:70]))
    A, B, Z = data((300, 33)), data((300, 33)), keep((300, 35))
    out.append(("rows of 31 elements", A, A[:, 1:32], B, B[:, 2:33], Z, Z[:, 3:34]))
    return out


@pytest.mark.parametrize("opname", ["add", "lt", "multiply"])
@pytest.mark.parametrize("dtype", ROW_TYPES, ids=[H.NAMES[d] for d in ROW_TYPES])
def test_binary_rows(hip, stream, opname, dtype):
    op = oh.B[opname]
    if not oh.lib.och_binary_supported(op, dtype):
        pytest.skip("not defined for this type")
    rdtype = oh.lib.och_binary_result_dtype(op, dtype)
    rng = np.random.default_rng(500 + dtype)
    seen_rows = 0
    for name, xp, xv, yp, yv, zp, zv in layouts(dtype, rdtype, rng):
        x = H.Operand(xp, xv, dtype).upload(stream)
        y = H.Operand(yp, yv, dtype).upload(stream)
        z = H.Operand(zp, zv, rdtype).upload(stream)
        seen_rows += plan_of([x, y, z]).kernel == oh.KERNEL_ROWS
        H.gpu_binary(stream, op, dtype, x, y, z)
        want = zp.copy()
        H.cpu_binary(op, dtype, x, y, z, want)
        got = z.download()
        for t in (x, y, z):
            t.free()
        H.assert_same_bytes(got, want, "%s %s: %s" % (opname, H.NAMES[dtype], name))
    wide_enough = max(np.dtype(H.storage(dtype)).itemsize, np.dtype(H.storage(rdtype)).itemsize) < 16
    assert seen_rows >= (6 if wide_enough else 0), "the row kernels were chosen for %d layouts" % seen_rows


CAST_PAIRS = [(H.INT8, H.INT8), (H.INT8, H.FLOAT), (H.FLOAT, H.INT8), (H.HALF, H.FLOAT), (H.FLOAT, H.HALF), (H.HALF, H.HALF), (H.FLOAT, H.FLOAT),
              (H.UINT16, H.DOUBLE), (H.DOUBLE, H.FLOAT), (H.BOOL, H.UINT8), (H.CFLOAT, H.CHALF), (H.INT32, H.CFLOAT)]


@pytest.mark.parametrize("ts,td", CAST_PAIRS, ids=lambda v: H.NAMES[v] if isinstance(v, int) else None)
@pytest.mark.parametrize("swap", [0, 1])
def test_copy_and_cast_rows(hip, stream, ts, td, swap):
    rng = np.random.default_rng(900 + 16 * ts + td)
    kind = "small" if td in (H.INT8, H.UINT8, H.BOOL) or ts in (H.HALF, H.CHALF) else "general"
    src = lambda shape: H.random_data(ts, int(np.prod(shape)), rng, kind).reshape(shape)
    keep = lambda shape: H.random_data(td, int(np.prod(shape)), rng, "positive" if td != H.BOOL else "general").reshape(shape)
    cases = []
    A, Z = src((41, 520)), keep((41, 530))
    cases.append(("odd width", A, A[:, 1:516], Z, Z[:, 6:521]))
    A, Z = src((23, 1001)), keep((23, 999))
    cases.append(("odd pitches", A, A[:, 3:1000], Z, Z[:, 1:998]))
    A, Z = src((7001,)), keep((7003,))
    cases.append(("one dimension", A, A[2:6999], Z, Z[5:7002]))
    A, Z = src((4, 9, 67)), keep((4, 9, 70))
    cases.append(("three dimensions", A, A[:, :, 0:65], Z, Z[:, :, 3:68]))
    A, Z = src((50, 260)), keep((50, 131))
    cases.append(("stepped source", A, A[:, 1:259:2], Z, Z[:, 2:131]))
    fn_g = oh.lib.och_byteswap_copy if swap else oh.lib.och_copy
    fn_c = orc.lib.oracle_byteswap_copy if swap else orc.lib.oracle_copy
    seen_rows = 0
    for name, xp, xv, zp, zv in cases:
        x = H.Operand(xp, xv, ts).upload(stream)
        z = H.Operand(zp, zv, td).upload(stream)
        seen_rows += plan_of([x, z]).kernel == oh.KERNEL_ROWS
        nd = len(x.shape)
        oh.check(fn_g(ts, td, nd, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), nd, oh.sizes(z.shape), oh.strides(z.strides), z.dptr(), stream.handle))
        want = zp.copy()
        assert fn_c(ts, td, nd, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(), nd, oh.sizes(z.shape), oh.strides(z.strides), z.hptr(want), 1) == 0
        got = z.download()
        x.free(); z.free()
        H.assert_same_bytes(got, want, "%s -> %s swap=%d: %s" % (H.NAMES[ts], H.NAMES[td], swap, name))
    assert seen_rows >= 4


@pytest.mark.parametrize("dtype", [H.BOOL, H.INT8, H.HALF, H.FLOAT, H.INT64, H.CHALF], ids=lambda d: H.NAMES[d])
def test_fill_rows(hip, stream, dtype):
    rng = np.random.default_rng(300 + dtype)
    value = H.raw_scalar(H.random_data(dtype, 4, rng, "positive" if dtype != H.BOOL else "general")[1:2])
    for shape, build in (((37, 1024), lambda p: p[:, 3:1002]), ((29, 1001), lambda p: p[:, 1:1000]), ((5000,), lambda p: p[1:4998]), ((4, 9, 70), lambda p: p[:, :, 3:68])):
        parent = H.random_data(dtype, int(np.prod(shape)), rng).reshape(shape)
        view = build(parent)
        x = H.Operand(parent, view, dtype).upload(stream)
        if np.dtype(H.storage(dtype)).itemsize < 16:
            assert plan_of([x]).kernel == oh.KERNEL_ROWS
        nd = len(x.shape)
        oh.check(oh.lib.och_fill(dtype, nd, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(), value, stream.handle))
        want = parent.copy()
        assert orc.lib.oracle_fill(dtype, nd, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(want), value, 1) == 0
        got = x.download()
        x.free()
        H.assert_same_bytes(got.view(np.uint8), want.view(np.uint8), "fill %s parent %s" % (H.NAMES[dtype], shape))
