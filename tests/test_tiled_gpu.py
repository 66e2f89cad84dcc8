"""Parity of the LDS-tiled elementwise kernels with the CPU oracle.

The device library routes a call to its tiled kernels when an input is contiguous along a
dimension other than the destination's fastest one (a transposed view, the case of
examples/python/gpu/tensors/tensor_add_02.py and of the transposed-operand benchmark shape).
The cases below hit that path with whole tiles, ragged tile edges, outer dimensions, one or
both inputs transposed, broadcast partners, mixed element sizes (comparisons, casts) and
operands that just miss the alignment the tiled path needs (which must fall back silently).
Results are bit-identical to the oracle.
"""
import numpy as np
import pytest

import helpers as H
import ocean_hip as oh
orc = H.orc

pytestmark = pytest.mark.gpu

TYPES = [H.BOOL, H.INT8, H.INT16, H.INT32, H.UINT64, H.HALF, H.FLOAT, H.DOUBLE, H.CFLOAT, H.CDOUBLE]
SHAPES = [(64, 64), (192, 128), (80, 48), (272, 144), (1040, 16)]      # (m, n): m is the fastest output dimension


def run_binary(stream, opname, dtype, xp, xv, yp, yv, zp, zv, what):
    op = oh.B[opname]
    rdtype = oh.lib.och_binary_result_dtype(op, dtype)
    zp[...] = 0
    x = H.Operand(xp, xv, dtype).upload(stream)
    y = H.Operand(yp, yv, dtype).upload(stream)
    z = H.Operand(zp, zv, rdtype).upload(stream)
    H.gpu_binary(stream, op, dtype, x, y, z)
    want = zp.copy()
    H.cpu_binary(op, dtype, x, y, z, want)
    got = z.download()
    for t in (x, y, z):
        t.free()
    H.assert_same_bytes(got, want, "%s %s %s" % (opname, H.NAMES[dtype], what))


@pytest.mark.parametrize("opname", ["add", "lt"])
@pytest.mark.parametrize("dtype", TYPES, ids=[H.NAMES[d] for d in TYPES])
def test_binary_transposed_tiles(hip, stream, opname, dtype):
    rng = np.random.default_rng(900 + dtype)
    rdtype = oh.lib.och_binary_result_dtype(oh.B[opname], dtype)
    for m, n in SHAPES:
        A = H.random_data(dtype, m * n, rng).reshape(n, m)
        At = H.random_data(dtype, m * n, rng).reshape(m, n)
        Bt = H.random_data(dtype, m * n, rng).reshape(m, n)
        row = H.random_data(dtype, m, rng).reshape(1, m)
        col = H.random_data(dtype, n, rng).reshape(n, 1)
        Z = np.zeros((n, m), dtype=H.storage(rdtype))
        tag = "%dx%d " % (m, n)
        run_binary(stream, opname, dtype, A, A, Bt, Bt.T, Z, Z, tag + "second transposed")
        run_binary(stream, opname, dtype, At, At.T, A, A, Z, Z, tag + "first transposed")
        run_binary(stream, opname, dtype, At, At.T, Bt, Bt.T, Z, Z, tag + "both transposed")
        run_binary(stream, opname, dtype, At, At.T, row, np.broadcast_to(row, (n, m)), Z, Z, tag + "transposed + row")
        run_binary(stream, opname, dtype, col, np.broadcast_to(col, (n, m)), Bt, Bt.T, Z, Z, tag + "column + transposed")
        run_binary(stream, opname, dtype, At, At.T[::-1, :], A, A, Z, Z, tag + "transposed, reversed rows")
        # transposed slice of a wider parent (pitch larger than the extent)
        Wt = H.random_data(dtype, m * (n + 16), rng).reshape(m, n + 16)
        run_binary(stream, opname, dtype, Wt, Wt[:, 16:].T, A, A, Z, Z, tag + "transposed slice")
        # an offset of one element breaks the 16-byte alignment: the generic kernels take over
        run_binary(stream, opname, dtype, Wt, Wt[:, 1:n + 1].T, A, A, Z, Z, tag + "unaligned transposed slice")


@pytest.mark.parametrize("dtype", [H.INT8, H.FLOAT, H.DOUBLE, H.CDOUBLE], ids=lambda d: H.NAMES[d])
def test_binary_transposed_outer_dims(hip, stream, dtype):
    """3-D and 4-D operands: the tile spans dimensions (0, d1), the others form the grid's z index."""
    rng = np.random.default_rng(950 + dtype)
    b, n, m = 3, 48, 96
    P = H.random_data(dtype, b * n * m, rng).reshape(b, n, m)
    Q = H.random_data(dtype, b * n * m, rng).reshape(b, m, n)
    Z = np.zeros((b, n, m), dtype=H.storage(dtype))
    run_binary(stream, "add", dtype, P, P, Q, Q.transpose(0, 2, 1), Z, Z, "batched transpose")
    Q2 = H.random_data(dtype, b * n * m, rng).reshape(m, b, n)
    run_binary(stream, "multiply", dtype, P, P, Q2, Q2.transpose(1, 2, 0), Z, Z, "batch in the middle")
    c = 2
    P4 = H.random_data(dtype, c * b * n * m, rng).reshape(c, b, n, m)
    Q4 = H.random_data(dtype, c * b * n * m, rng).reshape(m, b, c, n)
    Z4 = np.zeros((c, b, n, m), dtype=H.storage(dtype))
    run_binary(stream, "subtract", dtype, P4, P4, Q4, Q4.transpose(2, 1, 3, 0), Z4, Z4, "4-d permuted")


CASTS = [(H.INT32, H.DOUBLE), (H.DOUBLE, H.INT8), (H.HALF, H.CDOUBLE), (H.FLOAT, H.FLOAT), (H.INT16, H.FLOAT),
         (H.CDOUBLE, H.CFLOAT), (H.UINT8, H.BOOL), (H.INT64, H.HALF)]


@pytest.mark.parametrize("ts,td", CASTS, ids=["%s-%s" % (H.NAMES[s], H.NAMES[d]) for s, d in CASTS])
def test_transposed_cast_copy(hip, stream, ts, td):
    rng = np.random.default_rng(970 + ts * 15 + td)
    for m, n in SHAPES:
        for swap in (0, 1):
            src = H.random_data(ts, m * n, rng, "small").reshape(m, n)
            dst = np.zeros((n, m), H.storage(td))
            x = H.Operand(src, src.T, ts).upload(stream)
            y = H.Operand(dst, dst, td).upload(stream)
            gfn = oh.lib.och_byteswap_copy if swap else oh.lib.och_copy
            cfn = orc.lib.oracle_byteswap_copy if swap else orc.lib.oracle_copy
            oh.check(gfn(ts, td, 2, oh.sizes(x.shape), oh.strides(x.strides), x.dptr(),
                         2, oh.sizes(y.shape), oh.strides(y.strides), y.dptr(), stream.handle))
            want = dst.copy()
            assert cfn(ts, td, 2, oh.sizes(x.shape), oh.strides(x.strides), x.hptr(),
                       2, oh.sizes(y.shape), oh.strides(y.strides), y.hptr(want), 1) == 0
            got = y.download()
            x.free(); y.free()
            H.assert_same_bytes(got, want, "%s -> %s %dx%d swap=%d" % (H.NAMES[ts], H.NAMES[td], m, n, swap))


@pytest.mark.parametrize("opname,dtype", [("negative", H.INT16), ("sqrt", H.FLOAT), ("negative", H.CDOUBLE), ("isnan", H.DOUBLE),
                                          ("conj", H.CFLOAT), ("ceil", H.HALF)],
                         ids=lambda v: v if isinstance(v, str) else H.NAMES[v])
def test_unary_transposed(hip, stream, opname, dtype):
    op = oh.U[opname]
    rdtype = oh.lib.och_unary_result_dtype(op, dtype)
    rng = np.random.default_rng(990 + dtype)
    for m, n in SHAPES:
        src = H.random_data(dtype, m * n, rng, "positive" if opname == "sqrt" else "general").reshape(m, n)
        dst = np.zeros((n, m), H.storage(rdtype))
        x = H.Operand(src, src.T, dtype).upload(stream)
        z = H.Operand(dst, dst, rdtype).upload(stream)
        H.gpu_unary(stream, op, dtype, x, z)
        want = dst.copy()
        H.cpu_unary(op, dtype, x, z, want)
        got = z.download()
        x.free(); z.free()
        if opname == "sqrt":
            assert H.max_ulp_diff(got, want) <= 1
        else:
            H.assert_same_bytes(got, want, "%s %s %dx%d" % (opname, H.NAMES[dtype], m, n))
