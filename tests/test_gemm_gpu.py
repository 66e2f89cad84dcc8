"""Parity of och_gemm with the CPU oracle (textbook triple loop, long-double accumulation).

Mirrors examples/python/cpu/tensors/ocean_gemm_01..11.py and examples/python/gpu/tensors/
ocean_gemm_01/10/11.py (modes N/T/C, vector shapes, empty operands, alpha/beta variants) and
ocean_multiply_02.py (bool GEMM = OR/AND), extended to every supported type.

Bars: bool and integers bit-exact (wrap-around arithmetic). Floating point: normwise
    ||C_gpu - C_oracle||_F <= tol * (|alpha| * || |A| |B| ||_F + |beta| * ||C_0||_F)
with tol = 1e-5 (float, cfloat), 1e-13 (double, cdouble) and 2e-3 (half: products and sums
are accumulated in float and rounded to half once).
The full-size products (8192^3 double/float, 4096^3 cfloat) are checked with random probe
vectors: C x must equal alpha * A (B x) + beta * C_0 x (Freivalds), to the same bars.
"""
import ctypes as C

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

orc = H.orc
pytestmark = pytest.mark.gpu

GEMM_TYPES = [d for d in H.ALL_TYPES if d != H.CHALF]
TOL = {H.HALF: 2e-3, H.FLOAT: 1e-5, H.CFLOAT: 1e-5, H.DOUBLE: 1e-13, H.CDOUBLE: 1e-13}


def as_float(dtype, a):
    """numpy float/complex view of stored data (half bits -> float32)."""
    if dtype == H.HALF:
        return a.view(np.float16).astype(np.float64)
    return a


def matrix(dtype, rows, cols, ld, rng, kind="small"):
    """Column-major rows x cols matrix inside an ld x cols parent; the padding rows hold junk
    that must never be read into the result."""
    flat = H.random_data(dtype, ld * max(cols, 1), rng, kind)
    # bool tensors hold 0 / 1 only (solid/src/core/cpu/template_blas.c:186); the 8-bit integer types use their whole range
    return flat


def scalar_of(dtype, value):
    st = H.storage(dtype)
    if dtype == H.HALF:
        return H.f32_to_half_bits(np.array([value], np.float32))
    if dtype == H.BOOL:
        return np.array([1 if value else 0], np.uint8)
    return np.array([value]).astype(st)


def run_case(stream, dtype, ta, tb, M, N, K, alpha, beta, rng, device_scalars=False, pad=3, kind="small"):
    rowsA, colsA = (M, K) if ta == "N" else (K, M)
    rowsB, colsB = (K, N) if tb == "N" else (N, K)
    ldA, ldB, ldC = max(rowsA, 1) + pad, max(rowsB, 1) + pad, max(M, 1) + pad
    A = matrix(dtype, rowsA, colsA, ldA, rng, kind)
    B = matrix(dtype, rowsB, colsB, ldB, rng, kind)
    C0 = matrix(dtype, M, N, ldC, rng, kind)
    al, be = scalar_of(dtype, alpha), scalar_of(dtype, beta)
    dA, dB, dC = oh.to_device(A, stream), oh.to_device(B, stream), oh.to_device(C0, stream)
    if device_scalars:
        dal, dbe = oh.to_device(al, stream), oh.to_device(be, stream)
        pal, pbe, mode = dal.ptr, dbe.ptr, 0
    else:
        pal, pbe, mode = orc.ptr(al), orc.ptr(be), 1
    oh.check(oh.lib.och_gemm(dtype, ta.encode(), tb.encode(), M, N, K, pal, dA.ptr, ldA, dB.ptr, ldB, pbe, dC.ptr, ldC, mode, stream.handle))
    got = dC.download(C0.dtype, C0.size)
    want = C0.copy()
    assert orc.lib.oracle_gemm(dtype, ta.encode(), tb.encode(), M, N, K, orc.ptr(al), orc.ptr(A), ldA, orc.ptr(B), ldB,
                               orc.ptr(be), orc.ptr(want), ldC, 4) == 0
    for b in (dA, dB, dC):
        b.free()
    what = "%s %s%s %dx%dx%d alpha=%r beta=%r" % (H.NAMES[dtype], ta, tb, M, N, K, alpha, beta)
    if dtype not in TOL:
        H.assert_same_bytes(got, want, what)
        return
    g, w = as_float(dtype, got).reshape(-1, ldC), as_float(dtype, want).reshape(-1, ldC)      # (cols, ld)
    # padding rows untouched
    H.assert_same_bytes(got.reshape(-1, ldC)[:, M:], C0.reshape(-1, ldC)[:, M:], what + " (padding)")
    a = np.abs(as_float(dtype, A).reshape(-1, ldA)[:colsA, :rowsA])
    b = np.abs(as_float(dtype, B).reshape(-1, ldB)[:colsB, :rowsB])
    opa = a.T if ta == "N" else a                 # (M, K) in row-major numpy terms
    opb = b.T if tb == "N" else b
    scale = abs(alpha) * np.linalg.norm(opa @ opb) + abs(beta) * np.linalg.norm(as_float(dtype, C0).reshape(-1, ldC)[:N, :M])
    err = np.linalg.norm((g - w)[:N, :M])
    assert np.isfinite(err) and err <= TOL[dtype] * max(scale, 1e-30), "%s: error %.3e, bound %.3e" % (what, err, TOL[dtype] * scale)


SHAPES = [(70, 50, 90), (128, 128, 64), (256, 128, 16), (130, 257, 33), (1, 1, 300), (1, 1, 4096), (3, 2, 1000),
          (200, 1, 64), (1, 200, 77), (64, 64, 1), (5, 3, 0), (17, 1, 1)]


@pytest.mark.parametrize("dtype", GEMM_TYPES, ids=[H.NAMES[d] for d in GEMM_TYPES])
def test_gemm_all_types(hip, stream, dtype):
    assert oh.lib.och_gemm_supported(dtype) == 1
    rng = np.random.default_rng(500 + dtype)
    modes = ["N", "T"] + (["C"] if dtype in H.COMPLEX_TYPES else [])
    cplx = dtype in H.COMPLEX_TYPES
    for (M, N, K) in SHAPES:
        for ta in modes:
            for tb in modes:
                alpha, beta = (1, 0)
                if (M + N + K + len(ta + tb)) % 2 == 0:
                    alpha, beta = ((2 - 1j, -1 + 0.5j) if cplx else (2, -1)) if dtype != H.BOOL else (1, 1)
                if dtype in (H.UINT8, H.UINT16, H.UINT32, H.UINT64) and beta == -1:
                    beta = 3
                run_case(stream, dtype, ta, tb, M, N, K, alpha, beta, rng)


@pytest.mark.parametrize("dtype", [H.INT32, H.HALF, H.FLOAT, H.DOUBLE, H.CFLOAT, H.CDOUBLE, H.BOOL], ids=lambda d: H.NAMES[d])
def test_gemm_scalars(hip, stream, dtype):
    """alpha / beta in device memory, zero alpha, beta = 0 with NaN in C (C must not be read)."""
    rng = np.random.default_rng(600 + dtype)
    run_case(stream, dtype, "N", "T", 96, 80, 40, 1, 1, rng, device_scalars=True)
    run_case(stream, dtype, "T", "N", 128, 128, 128, 1, 0, rng, device_scalars=True, pad=0)
    run_case(stream, dtype, "N", "N", 33, 65, 20, 0, 1, rng)
    run_case(stream, dtype, "N", "N", 1, 1, 512, 1, 1, rng, device_scalars=True)
    if dtype in (H.FLOAT, H.DOUBLE, H.CFLOAT, H.CDOUBLE):
        st = H.storage(dtype)
        M, N, K = 128, 128, 32
        A = H.random_data(dtype, M * K, rng, "small"); B = H.random_data(dtype, K * N, rng, "small")
        C0 = np.full(M * N, np.nan, st)
        dA, dB, dC = oh.to_device(A, stream), oh.to_device(B, stream), oh.to_device(C0, stream)
        one, zero = scalar_of(dtype, 1), scalar_of(dtype, 0)
        oh.check(oh.lib.och_gemm(dtype, b"N", b"N", M, N, K, orc.ptr(one), dA.ptr, M, dB.ptr, K, orc.ptr(zero), dC.ptr, M, 1, stream.handle))
        got = dC.download(st, M * N)
        assert np.isfinite(got.view(np.float32 if st in (np.float32, np.complex64) else np.float64)).all(), "beta = 0 must ignore C"
        for b in (dA, dB, dC):
            b.free()


@pytest.mark.parametrize("ta", ["N", "T"])
@pytest.mark.parametrize("tb", ["N", "T"])
def test_gemm_half_matrix_cores(hip, stream, ta, tb):
    """Half products large enough for the MFMA kernel: whole tiles with aligned operands (128-bit loads), ragged edges,
    leading dimensions that rule out wide loads, all three tile sizes, a long K, scalars in device memory."""
    rng = np.random.default_rng(900 + ord(ta) + 2 * ord(tb))
    for (M, N, K, pad, alpha, beta, dev) in [(128, 128, 64, 0, 1, 0, False), (256, 384, 96, 8, 2, -1, False), (200, 136, 100, 3, 1, 1, True),
                                              (64, 64, 32, 0, -1, 0.5, False), (96, 160, 2048, 0, 0.5, 0, True), (33, 47, 17, 5, 1, 0, False),
                                              (2560, 2304, 48, 0, 1, 1, False), (2500, 2300, 40, 4, 1, 0, False), (4096, 3072, 64, 0, 1, 0, False),
                                              (4000, 3100, 70, 0, -1, 1, True),
                                              # whole aligned 128 x 128 tiles, three and five slabs of K: the pipelined loop on the middle tile
                                              (2048, 2048, 192, 0, 2, -1, True), (2048, 2304, 320, 0, 1, 0, False),
                                              # results narrower than a tile, vectors, K below one MFMA step, K not a multiple of 8
                                              (2000, 1, 1000, 0, 1, 0, False), (1, 1500, 999, 0, 1, 1, False), (700, 9, 3, 1, 2, 0, False), (31, 31, 15, 0, 1, 0, False),
                                              # few tiles and a long K: cut along K, float partial sums added in order
                                              (128, 64, 8192, 0, 1, 0, False), (1, 1, 70000, 0, 1, -1, True), (100, 130, 5000, 4, -1, 1, False)]:
        run_case(stream, H.HALF, ta, tb, M, N, K, alpha, beta, rng, device_scalars=dev, pad=pad)


@pytest.mark.parametrize("dtype", [H.INT8, H.UINT8, H.BOOL], ids=lambda d: H.NAMES[d])
@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
def test_gemm_bytes_matrix_cores(hip, stream, dtype, ta, tb):
    """8-bit integer and bool products on the MFMA kernel (K >= 32), bit-exact against the oracle's wrap-around / OR-AND
    arithmetic: whole tiles with aligned operands, ragged edges, unaligned leading dimensions, all three tile sizes, a
    long K cut into slices, scalars in device memory, beta != 0."""
    rng = np.random.default_rng(950 + dtype + ord(ta) + 2 * ord(tb))
    neg = 3 if dtype == H.UINT8 else -1
    for (M, N, K, pad, alpha, beta, dev) in [(128, 128, 128, 0, 1, 0, False), (256, 384, 160, 16, 2, neg, False), (200, 136, 100, 3, 1, 1, True),
                                              (64, 64, 32, 0, neg, 1, False), (96, 160, 2048, 0, 3, 0, True), (33, 47, 37, 5, 1, 0, False),
                                              (2560, 2304, 256, 0, 1, 1, False), (2500, 2300, 130, 4, 1, 0, False), (4096, 3072, 128, 0, 1, 0, False),
                                              # whole aligned 128 x 128 tiles, three and five slabs of K: the pipelined loop on the middle tile
                                              (2048, 2048, 384, 0, 2, neg, True), (2048, 2304, 640, 0, 1, 0, False),
                                              (1, 1500, 999, 0, 1, 1, False), (128, 64, 8192, 0, 1, 0, False), (1, 1, 70000, 0, 1, neg, True)]:
        if dtype == H.BOOL:
            alpha, beta = (1 if alpha else 0), (1 if beta else 0)
        run_case(stream, dtype, ta, tb, M, N, K, alpha, beta, rng, device_scalars=dev, pad=pad, kind="full")


def check_large_product(stream, dtype, ta, tb, M, N, cases, rng, pad=0):
    """Large products checked without O(n^3) host work: eight complete rows and columns of C computed directly, and C
    times probe vectors against op(A) (op(B) x) -- in exact arithmetic modulo 256 for the 8-bit types, to the
    precision's bound for half and float. cases: (slabs of K, alpha, beta, scalars in device memory); pad: rows of
    junk between the columns of all three operands."""
    kt = {H.HALF: 64, H.FLOAT: 32, H.DOUBLE: 16, H.CFLOAT: 32, H.CDOUBLE: 16}.get(dtype, 128)
    exact = dtype not in (H.HALF, H.FLOAT, H.DOUBLE, H.CFLOAT, H.CDOUBLE)
    for slabs, alpha, beta, dev in cases:
        K = int(round(slabs * kt))
        rowsA, colsA = (M, K) if ta == "N" else (K, M)
        rowsB, colsB = (K, N) if tb == "N" else (N, K)
        ldA, ldB, ldC = rowsA + pad, rowsB + pad, M + pad
        A, B, C0 = matrix(dtype, rowsA, colsA, ldA, rng, "full" if exact else "small"), matrix(dtype, rowsB, colsB, ldB, rng, "full" if exact else "small"), \
            matrix(dtype, M, N, ldC, rng, "full" if exact else "small")
        al, be = scalar_of(dtype, alpha), scalar_of(dtype, beta)
        dA, dB, dC = oh.to_device(A, stream), oh.to_device(B, stream), oh.to_device(C0, stream)
        if dev:
            dal, dbe = oh.to_device(al, stream), oh.to_device(be, stream)
            pal, pbe, mode = dal.ptr, dbe.ptr, 0
        else:
            pal, pbe, mode = orc.ptr(al), orc.ptr(be), 1
        oh.check(oh.lib.och_gemm(dtype, ta.encode(), tb.encode(), M, N, K, pal, dA.ptr, ldA, dB.ptr, ldB, pbe, dC.ptr, ldC, mode, stream.handle))
        got = dC.download(C0.dtype, C0.size)
        for b in (dA, dB, dC):
            b.free()
        wide = np.int64 if exact else (np.complex128 if dtype in (H.CFLOAT, H.CDOUBLE) else np.float64)
        num = (lambda a: a.astype(np.int64)) if exact else (lambda a: as_float(dtype, a).astype(wide))
        mA, mB = num(A).reshape(colsA, ldA)[:, :rowsA].T, num(B).reshape(colsB, ldB)[:, :rowsB].T            # [row, col]
        op = {"N": lambda m: m, "T": lambda m: m.T, "C": lambda m: m.conj().T}
        opA, opB = op[ta](mA), op[tb](mB)
        c0, c = num(C0).reshape(N, ldC)[:, :M].T, num(got).reshape(N, ldC)[:, :M].T
        assert np.array_equal(got.reshape(N, ldC)[:, M:], C0.reshape(N, ldC)[:, M:]), "padding of C written"
        what = "%s %s%s %dx%dx%d alpha=%r beta=%r" % (H.NAMES[dtype], ta, tb, M, N, K, alpha, beta)

        def same(have, want, bound):
            if exact:
                assert np.array_equal(have % 256, want % 256), what
            else:
                assert (np.abs(have - want) <= TOL[dtype] * bound + 1e-30).all(), "%s: %.3e" % (what, np.abs(have - want).max())
        for i in list(rng.integers(0, M, 7)) + [M - 1]:
            row = alpha * (opA[i, :] @ opB) + beta * c0[i, :]
            same(c[i, :], row, abs(alpha) * (np.abs(opA[i, :]) @ np.abs(opB)) + abs(beta) * np.abs(c0[i, :]))
        for j in list(rng.integers(0, N, 7)) + [N - 1]:
            col = alpha * (opA @ opB[:, j]) + beta * c0[:, j]
            same(c[:, j], col, abs(alpha) * (np.abs(opA) @ np.abs(opB[:, j])) + abs(beta) * np.abs(c0[:, j]))
        X = rng.integers(-3, 4, (N, 6)).astype(wide)
        want = alpha * (opA @ (opB @ X)) + beta * (c0 @ X)
        have = c @ X
        if exact:
            assert np.array_equal(have % 256, want % 256), what + " (probe vectors)"
        else:
            bound = abs(alpha) * (np.abs(opA) @ (np.abs(opB) @ np.abs(X))) + abs(beta) * (np.abs(c0) @ np.abs(X))
            assert np.linalg.norm(have - want) <= TOL[dtype] * np.linalg.norm(bound), what + " (probe vectors)"


@pytest.mark.parametrize("choice", [1, 2, 3, 4], ids=["large_tile", "small_tile", "tiled_kernel", "smallest_tile"])
@pytest.mark.parametrize("dtype", [H.FLOAT, H.DOUBLE, H.CFLOAT, H.CDOUBLE], ids=lambda d: H.NAMES[d])
def test_gemm_pipelined_kernels_against_the_oracle(hip, stream, dtype, choice):
    """With the kernel choice fixed (och_gemm_set_kernel_choice) the pipelined kernels take every aligned product whose M and
    N are multiples of 4 (double, complex float: 2), however small: whole results against the oracle for single tiles, last
    tiles of a few rows and columns, one to nine slabs of K, a K with a remainder (host scalars: pipelined head + additive
    rest; device scalars: the tiled kernel), every transposition and conjugation. Choice 3 is the tiled kernel on the same
    shapes; choice 4 the 64 x 64 tiles of the float kernel (the other types have no such tile and take the one their model
    prefers)."""
    rng = np.random.default_rng(1600 + 10 * dtype + choice)
    slab = 16 if dtype in (H.DOUBLE, H.CDOUBLE) else 32
    cplx = dtype in (H.CFLOAT, H.CDOUBLE)
    modes = ["N", "T"] + (["C"] if cplx else [])
    shapes = [(128, 128, slab), (132, 260, 3 * slab), (388, 130 if dtype != H.FLOAT else 132, 2 * slab), (260, 516, 9 * slab + 8), (512, 256, 5 * slab),
              (256, 384, 4 * slab)]
    assert oh.lib.och_gemm_set_kernel_choice(7) != 0
    oh.check(oh.lib.och_gemm_set_kernel_choice(choice))
    try:
        for n, (M, N, K) in enumerate(shapes):
            for ta in modes:
                for tb in modes:
                    alpha, beta = ((2 - 1j, -1 + 0.5j) if cplx else (2, -1)) if (n + len(ta + tb) + ord(ta)) % 2 else (1, 0)
                    run_case(stream, dtype, ta, tb, M, N, K, alpha, beta, rng, device_scalars=(n % 3 == 2), pad=4)
    finally:
        oh.check(oh.lib.och_gemm_set_kernel_choice(0))


@pytest.mark.parametrize("choice,M,N", [(2, 2176, 2048), (2, 2180, 2052), (1, 4352, 4096), (2, 2560, 2048), (4, 1088, 1024), (4, 1092, 1028)],
                         ids=["small_tiles", "small_tiles_ragged", "large_tiles", "small_tiles_quarter_round", "smallest_tiles", "smallest_tiles_ragged"])
def test_gemm_float_last_round_cut_along_k(hip, stream, choice, M, N):
    """When the last round of the compute units is at most half full (here 16 tiles, or 17 x 17 - 256 = 33, on 256 units) its
    tiles are cut along K into shares of at least 8 slabs that fill the round; the shares are added in order by a second
    kernel. 64 slabs give 8 shares of 8 (7 of 10 where 33 tiles are cut, 4 of 16 where 64 are); 17 slabs give two shares of
    9 and 8 where 64 tiles are cut and none where 16 are (two shares would leave most compute units idle); with beta, scalars
    in host and device memory, a K with a remainder."""
    # (the sizes are chosen for 256 compute units; on another device the planner cuts differently or not at all, and the
    #  results are checked all the same)
    rng = np.random.default_rng(1900 + choice + M)
    oh.check(oh.lib.och_gemm_set_kernel_choice(choice))
    try:
        for ta, tb in (("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")):
            check_large_product(stream, H.FLOAT, ta, tb, M, N, ((64, 2, -1, ta == "T"), (17, 1, 0, False), (20.25, -0.5, 1, False)), rng)
    finally:
        oh.check(oh.lib.och_gemm_set_kernel_choice(0))


@pytest.mark.parametrize("choice,M,N", [(2, 2176, 2048), (2, 2178, 2050), (1, 4352, 2048), (2, 2560, 2048)],
                         ids=["small_tiles", "small_tiles_ragged", "large_tiles", "small_tiles_quarter_round"])
def test_gemm_double_last_round_cut_along_k(hip, stream, choice, M, N):
    """The same for double: 16 tiles (ragged sizes: 18 x 17 - 256 = 50) in the last round of 256 compute units, cut into 8
    (5) shares of the 64 slabs of 16 k, two shares of 17 slabs, a K with a remainder."""
    # (the sizes are chosen for 256 compute units; on another device the planner cuts differently or not at all, and the
    #  results are checked all the same)
    rng = np.random.default_rng(2000 + choice + M)
    oh.check(oh.lib.och_gemm_set_kernel_choice(choice))
    try:
        for ta, tb in (("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")):
            check_large_product(stream, H.DOUBLE, ta, tb, M, N, ((64, 2, -1, ta == "T"), (17, 1, 0, False), (20.3125, -0.5, 1, False)), rng)
    finally:
        oh.check(oh.lib.och_gemm_set_kernel_choice(0))


@pytest.mark.parametrize("dtype,M,N", [(H.CFLOAT, 2176, 2048), (H.CFLOAT, 2178, 2050), (H.CDOUBLE, 2176, 1024), (H.CDOUBLE, 2177, 1025)],
                         ids=["cfloat", "cfloat_ragged", "cdouble", "cdouble_ragged"])
def test_gemm_complex_last_round_cut_along_k(hip, stream, dtype, M, N):
    """The same for the complex types: the shares hold the complex sums before alpha (the four real accumulators already
    combined with the signs of the conjugations); complex alpha and beta are applied once, by the kernel that adds the shares."""
    # (the sizes are chosen for 256 compute units; on another device the planner cuts differently or not at all, and the
    #  results are checked all the same)
    rng = np.random.default_rng(2100 + dtype + M)
    oh.check(oh.lib.och_gemm_set_kernel_choice(1))
    try:
        for ta, tb in (("N", "N"), ("T", "N"), ("N", "C"), ("C", "T")):
            check_large_product(stream, dtype, ta, tb, M, N, ((64, 2 - 1j, -1 + 0.5j, ta == "T"), (17, 1, 0, False), (20.25, -0.5j, 1, False)), rng)
    finally:
        oh.check(oh.lib.och_gemm_set_kernel_choice(0))


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
def test_gemm_float_pipelined_whole_tiles(hip, stream, ta, tb):
    """float products of 256 whole aligned 256 x 256 tiles or more run on the hand-pipelined kernel: one slab of 32 k
    (start-up only), three and six slabs (clamped loads past the end, both LDS buffers reused), with and without beta,
    scalars in host and in device memory, columns with and without junk between them."""
    rng = np.random.default_rng(1300 + ord(ta) + 2 * ord(tb))
    check_large_product(stream, H.FLOAT, ta, tb, 4096, 4096, ((1, 1, 0, False), (3, 2, -1, True)), rng)
    check_large_product(stream, H.FLOAT, ta, tb, 4096, 4096, ((6, -1.5, 0.5, False),), rng, pad=12)
    # fewer than one 256 x 256 tile per compute unit: the same kernel on 128 x 128 tiles, two blocks per compute unit
    check_large_product(stream, H.FLOAT, ta, tb, 2048, 2048, ((1, 1, 0, False), (3, 2, -1, True), (6, -1.5, 0.5, False)), rng)
    check_large_product(stream, H.FLOAT, ta, tb, 2048 + 40, 2048 + 24, ((2, 0.5, 2, False),), rng, pad=4)
    # last tiles of four rows / four columns (the tile's loads are clamped to the rows that exist, the rest of the tile is not written)
    check_large_product(stream, H.FLOAT, ta, tb, 2564, 2560, ((2, 1, -1, False),), rng)
    check_large_product(stream, H.FLOAT, ta, tb, 2560, 2564, ((2, 1, 0, False),), rng, pad=8)
    # K that is not a whole number of slabs (scalars in host memory): the whole slabs pipelined, the rest added by a product of its own
    check_large_product(stream, H.FLOAT, ta, tb, 2048, 2048 + 24, ((9.25, 0.5, 2, False), (9.25, 0.5, 2, True)), rng)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T"), ("C", "N"), ("N", "C"), ("C", "C"), ("T", "C")])
def test_gemm_cfloat_pipelined_whole_tiles(hip, stream, ta, tb):
    """complex float products of 256 whole aligned 128 x 128 tiles or more run on the hand-pipelined kernel, which sums
    Ar Br, Ai Bi, Ar Bi and Ai Br apart and combines them with the signs the conjugations ask for: one, three and six
    slabs of 32 k, complex alpha and beta, scalars in host and in device memory, columns with and without junk between them."""
    rng = np.random.default_rng(1500 + ord(ta) + 2 * ord(tb))
    check_large_product(stream, H.CFLOAT, ta, tb, 2048, 2048, ((1, 1, 0, False), (3, 2 - 1j, -1 + 0.5j, True)), rng)
    check_large_product(stream, H.CFLOAT, ta, tb, 2048, 2048, ((6, -1.5j, 0.5, False),), rng, pad=6)
    check_large_product(stream, H.CFLOAT, ta, tb, 2048, 2048, ((8.125, 1 - 1j, 0.5j, False),), rng)            # a K of 8 slabs + 4
    check_large_product(stream, H.CFLOAT, ta, tb, 4098, 4098, ((2, 1, -1, False),), rng)                        # last tiles of two rows / columns


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "C"), ("C", "T")])
def test_gemm_cdouble_pipelined_tiles(hip, stream, ta, tb):
    """complex double products that fill the compute units with tiles of 128 x 64 run on the hand-pipelined kernel, whose
    three slab buffers rotate: one to four slabs of 16 k, a K with a remainder, odd M and N (last tiles of one row and one
    column), complex alpha and beta in host and in device memory."""
    rng = np.random.default_rng(1700 + ord(ta) + 2 * ord(tb))
    check_large_product(stream, H.CDOUBLE, ta, tb, 2048, 1024, ((1, 1, 0, False), (2, 2 - 1j, -1 + 0.5j, True), (3, -1j, 1, False), (4, 1, 0.5j, False)), rng)
    check_large_product(stream, H.CDOUBLE, ta, tb, 2049, 2049, ((9.3125, 1 - 1j, 0.5, False),), rng, pad=3)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
def test_gemm_double_pipelined_whole_tiles(hip, stream, ta, tb):
    """double products of 256 whole aligned 256 x 128 tiles or more run on the hand-pipelined kernel, whose three slab
    buffers rotate: one, two and three slabs of 16 k (start-up and each tail of the rotation), four and eight slabs (all
    buffers reused, clamped loads past the end), with and without beta, scalars in host and in device memory, columns with
    and without junk between them."""
    rng = np.random.default_rng(1400 + ord(ta) + 2 * ord(tb))
    check_large_product(stream, H.DOUBLE, ta, tb, 4096, 2048, ((1, 1, 0, False), (2, 2, -1, True), (3, -1, 1, False)), rng)
    check_large_product(stream, H.DOUBLE, ta, tb, 4096, 2048, ((4, 1.5, 0, True), (8, -1.5, 0.5, False)), rng, pad=6)
    check_large_product(stream, H.DOUBLE, ta, tb, 4096, 2048, ((9.3125, 2, -1, False),), rng)                    # a K of 9 slabs + 5
    check_large_product(stream, H.DOUBLE, ta, tb, 7938, 7938, ((2, 1, -1, False),), rng)                         # last tiles of two rows / columns


@pytest.mark.parametrize("dtype", [H.HALF, H.INT8, H.UINT8], ids=lambda d: H.NAMES[d])
@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
def test_gemm_pipelined_whole_tiles(hip, stream, dtype, ta, tb):
    """Products that the tile choice gives to the 256 x 256 tile (256 tiles or more) and that consist of whole aligned
    tiles run on the hand-pipelined loop: one slab (start-up only), three and five slabs (clamped loads past the end, both
    LDS buffers reused), with and without beta, scalars in host and in device memory."""
    rng = np.random.default_rng(1200 + dtype + ord(ta) + 2 * ord(tb))
    check_large_product(stream, dtype, ta, tb, 4096, 4096,
                        ((1, 1, 0, False), (3, 2, -1 if dtype != H.UINT8 else 3, True), (5, -1 if dtype != H.UINT8 else 5, 1, False)), rng)


@pytest.mark.parametrize("dtype", [H.HALF, H.INT8, H.FLOAT, H.DOUBLE, H.CFLOAT], ids=lambda d: H.NAMES[d])
@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
def test_gemm_whole_tiles_and_edge_strips(hip, stream, dtype, ta, tb):
    """A large aligned product whose sizes are not multiples of the tile: the whole tiles run on the pipelined loop, the
    columns to their right and the rows below them as products of their own; the last row and column are among those checked."""
    rng = np.random.default_rng(1300 + dtype + ord(ta) + 2 * ord(tb))
    check_large_product(stream, dtype, ta, tb, 8080, 8016, ((2, 2, -1, False),), rng)


def test_gemm_errors_and_empty(hip, stream):
    rng = np.random.default_rng(7)
    one = np.ones(1)
    buf = oh.to_device(rng.uniform(-1, 1, 64), stream)
    # empty result: no-op, returns success
    assert oh.lib.och_gemm(H.DOUBLE, b"N", b"N", 0, 5, 3, orc.ptr(one), buf.ptr, 1, buf.ptr, 3, orc.ptr(one), buf.ptr, 1, 1, stream.handle) == 0
    assert oh.lib.och_gemm(H.DOUBLE, b"N", b"N", 5, 0, 3, orc.ptr(one), buf.ptr, 5, buf.ptr, 3, orc.ptr(one), buf.ptr, 5, 1, stream.handle) == 0
    # chalf is not supported, as in the reference
    assert oh.lib.och_gemm_supported(H.CHALF) == 0
    assert oh.lib.och_gemm(H.CHALF, b"N", b"N", 2, 2, 2, orc.ptr(one), buf.ptr, 2, buf.ptr, 2, orc.ptr(one), buf.ptr, 2, 1, stream.handle) != 0
    assert b"not available" in oh.lib.och_last_error()
    assert oh.lib.och_gemm(H.DOUBLE, b"X", b"N", 2, 2, 2, orc.ptr(one), buf.ptr, 2, buf.ptr, 2, orc.ptr(one), buf.ptr, 2, 1, stream.handle) != 0
    assert oh.lib.och_gemm(H.DOUBLE, b"N", b"N", 4, 2, 2, orc.ptr(one), buf.ptr, 2, buf.ptr, 2, orc.ptr(one), buf.ptr, 4, 1, stream.handle) != 0
    assert b"leading dimension" in oh.lib.och_last_error()
    buf.free()


FULL = [(H.DOUBLE, 8192, "N", "N"), (H.DOUBLE, 8192, "T", "N"), (H.FLOAT, 8192, "N", "T"), (H.FLOAT, 8192, "N", "N"),
        (H.CFLOAT, 4096, "C", "N"), (H.CFLOAT, 4096, "N", "N"), (H.CDOUBLE, 2048, "N", "C")]


@pytest.mark.parametrize("dtype,n,ta,tb", FULL, ids=["%s-%d-%s%s" % (H.NAMES[d], n, a, b) for d, n, a, b in FULL])
def test_gemm_full_size_probe(hip, stream, dtype, n, ta, tb):
    """Benchmark-size products checked with probe vectors (no O(n^3) work on the host)."""
    rng = np.random.default_rng(800 + dtype + n)
    st = H.storage(dtype)
    cplx = dtype in H.COMPLEX_TYPES

    def rand():
        a = rng.uniform(-1, 1, n * n).astype(st if not cplx else (np.float32 if dtype == H.CFLOAT else np.float64))
        if cplx:
            a = (a + 1j * rng.uniform(-1, 1, n * n)).astype(st)
        return a.reshape(n, n)                           # numpy (col, row): column-major matrix
    A, B, C0 = rand(), rand(), rand()
    alpha, beta = ((0.5 - 0.25j, -1.5 + 1j) if cplx else (0.5, -1.5))
    al, be = scalar_of(dtype, alpha), scalar_of(dtype, beta)
    dA, dB, dC = oh.to_device(A, stream), oh.to_device(B, stream), oh.to_device(C0, stream)
    oh.check(oh.lib.och_gemm(dtype, ta.encode(), tb.encode(), n, n, n, orc.ptr(al), dA.ptr, n, dB.ptr, n, orc.ptr(be), dC.ptr, n, 1, stream.handle))
    got = dC.download(st, n * n).reshape(n, n)
    for b in (dA, dB, dC):
        b.free()
    wide = np.complex128 if cplx else np.float64

    def op(Mx, t):          # the mathematical matrix op(M) as a numpy array indexed [row, col]
        m = Mx.T            # column-major storage -> [row, col]
        return m if t == "N" else (m.T if t == "T" else m.conj().T)
    X = rng.uniform(-1, 1, (n, 4)).astype(wide)
    opA, opB = op(A, ta), op(B, tb)
    want = alpha * (opA.astype(wide) @ (opB.astype(wide) @ X)) + beta * (C0.T.astype(wide) @ X)
    have = got.T.astype(wide) @ X
    scale = abs(alpha) * np.linalg.norm(np.abs(opA).astype(np.float64) @ (np.abs(opB).astype(np.float64) @ np.abs(X))) \
        + abs(beta) * np.linalg.norm(np.abs(C0.T).astype(np.float64) @ np.abs(X))
    err = np.linalg.norm(have - want)
    assert err <= TOL[dtype] * scale, "probe error %.3e, bound %.3e" % (err, TOL[dtype] * scale)
    # and one directly computed row and column
    i = int(rng.integers(0, n))
    row = alpha * (opA[i, :].astype(wide) @ opB.astype(wide)) + beta * C0.T[i, :].astype(wide)
    assert np.linalg.norm(got.T[i, :] - row) <= TOL[dtype] * (np.linalg.norm(np.abs(opA[i, :]).astype(np.float64) @ np.abs(opB).astype(np.float64)) * abs(alpha)
                                                              + abs(beta) * np.linalg.norm(C0.T[i, :]))


def test_mgs_qr_pattern(hip, stream):
    """Modified Gram-Schmidt on a 512 x 48 double matrix driven the way the reference example does
    it: per pair one dot product (gemm with M = N = 1, result kept on the device), one rank-1 update
    (gemm with K = 1 reading that device scalar) and per column a norm and a scale."""
    rng = np.random.default_rng(11)
    m, n = 512, 48
    A = rng.uniform(-1, 1, (n, m))                       # column j = A[j, :]
    Q = oh.to_device(A, stream)
    R = oh.to_device(np.zeros((n, n)), stream)           # R[j, i] = r_ij (column-major n x n)
    one, zero, minus = np.ones(1), np.zeros(1), -np.ones(1)
    done, dzero, dminus = oh.to_device(one, stream), oh.to_device(zero, stream), oh.to_device(minus, stream)
    inv = oh.DeviceBuffer(8, stream)
    col = lambda j: C.c_void_p(Q.address + 8 * m * j)
    rij = lambda i, j: C.c_void_p(R.address + 8 * (i + n * j))
    nrm = np.zeros(1)
    ref = A.copy(); Rref = np.zeros((n, n))
    for j in range(n):
        for i in range(j):
            # r_ij = q_i' a_j  (device scalar), a_j -= q_i r_ij
            oh.check(oh.lib.och_gemm(H.DOUBLE, b"T", b"N", 1, 1, m, dminus.ptr, col(i), m, col(j), m, dzero.ptr, rij(i, j), 1, 0, stream.handle))
            oh.check(oh.lib.och_gemm(H.DOUBLE, b"N", b"N", m, 1, 1, done.ptr, col(i), m, rij(i, j), 1, done.ptr, col(j), m, 0, stream.handle))
            r = ref[i] @ ref[j]; Rref[j, i] = r; ref[j] -= r * ref[i]
        oh.check(oh.lib.och_reduce_all(oh.R["norm2"], H.DOUBLE, 1, oh.sizes([m]), oh.strides([8]), col(j), None, None, 0.0, orc.ptr(nrm), None, stream.handle))
        inv.upload(np.array([1.0 / nrm[0]]))
        oh.check(oh.lib.och_binary(oh.B["multiply"], H.DOUBLE, 1, oh.sizes([m]), oh.strides([8]), col(j), oh.strides([0]), inv.ptr,
                                   oh.strides([8]), col(j), stream.handle))
        nr = np.linalg.norm(ref[j]); Rref[j, j] = nr; ref[j] /= nr
    Qg = Q.download(np.float64, n * m).reshape(n, m)
    Rg = -R.download(np.float64, n * n).reshape(n, n)     # the dot products were stored negated (alpha = -1)
    assert np.abs(Qg @ Qg.T - np.eye(n)).max() < 1e-12
    assert np.abs(Qg - ref).max() < 1e-11
    off = ~np.eye(n, dtype=bool)
    assert np.abs(Rg[off] - Rref[off]).max() < 1e-11


def test_mgs_qr_window_on_the_4096_matrix(hip, stream):
    """The benchmark's modified Gram-Schmidt workload at its real shape: the first 64 columns of a 4096 x 4096 float64
    matrix with entries from U(-1, 1), per pair one dot product (gemm, M = N = 1, K = 4096, result kept on the device)
    and one rank-1 update (gemm, K = 1) reading that device scalar, per column a norm (full reduction into a device
    scalar) and a division by it -- 2016 pairs, 4160 launches, nothing read back in between. Run launch by launch
    and again recorded once and replayed as a graph, from the same start; both against the same recurrence evaluated
    in float64 on the host (dot products in extended precision). Bound: the GEMM bound of 1e-13 times the 64
    operations a column receives (columns have unit norm, so the bound is absolute)."""
    rng = np.random.default_rng(4096)
    m, ncol = 4096, 64
    A = rng.uniform(-1, 1, (m, m))                       # column j = A[j, :]
    pairs = [(i, j) for j in range(ncol) for i in range(j)]
    ref = A[:ncol].copy(); Rref = np.zeros((ncol, ncol))
    for j in range(ncol):
        for i in range(j):
            r = float(np.dot(ref[i].astype(np.longdouble), ref[j].astype(np.longdouble)))
            Rref[j, i] = r; ref[j] -= r * ref[i]
        nr = float(np.sqrt(np.dot(ref[j].astype(np.longdouble), ref[j].astype(np.longdouble))))
        Rref[j, j] = nr; ref[j] /= nr
    consts = oh.to_device(np.array([1.0, 0.0, -1.0]), stream)
    c_one, c_zero, c_minus = [C.c_void_p(consts.address + 8 * k) for k in range(3)]
    results = {}
    for mode in ("eager", "graph"):
        Q = oh.to_device(A, stream)
        R = oh.to_device(np.zeros((ncol, ncol)), stream)
        col = lambda j: C.c_void_p(Q.address + 8 * m * j)
        rij = lambda i, j: C.c_void_p(R.address + 8 * (i + ncol * j))

        def window():
            for j in range(ncol):
                for i in range(j):
                    oh.check(oh.lib.och_gemm(H.DOUBLE, b"T", b"N", 1, 1, m, c_minus, col(i), m, col(j), m, c_zero, rij(i, j), 1, 0, stream.handle))
                    oh.check(oh.lib.och_gemm(H.DOUBLE, b"N", b"N", m, 1, 1, c_one, col(i), m, rij(i, j), 1, c_one, col(j), m, 0, stream.handle))
                oh.check(oh.lib.och_reduce_all_device(oh.R["norm2"], H.DOUBLE, 1, oh.sizes([m]), oh.strides([8]), col(j), None, None, 0.0, rij(j, j), None, stream.handle))
                oh.check(oh.lib.och_binary(oh.B["divide"], H.DOUBLE, 1, oh.sizes([m]), oh.strides([8]), col(j), oh.strides([0]), rij(j, j), oh.strides([8]), col(j), stream.handle))
        if mode == "eager":
            window()
        else:
            oh.check(oh.lib.och_stream_begin_capture(stream.handle))
            window()
            graph = C.c_void_p()
            oh.check(oh.lib.och_stream_end_capture(stream.handle, C.byref(graph)))
            oh.check(oh.lib.och_graph_launch(graph, stream.handle))
            stream.synchronize()
            oh.check(oh.lib.och_graph_destroy(graph))
        Qg = Q.download(np.float64, ncol * m).reshape(ncol, m)
        Rg = R.download(np.float64, ncol * ncol).reshape(ncol, ncol)
        Rg[np.tril(np.ones((ncol, ncol), bool), -1)] *= -1                 # alpha = -1: the dot products are stored negated
        rest = Q.download(np.float64, m, offset=8 * m * ncol)
        Q.free(); R.free()
        assert np.array_equal(rest, A[ncol]), "a column outside the window was touched"
        assert np.abs(Qg @ Qg.T - np.eye(ncol)).max() < 1e-12, mode
        assert np.abs(Qg - ref).max() <= 1e-13 * ncol, (mode, np.abs(Qg - ref).max())
        low = np.tril(np.ones((ncol, ncol), bool))
        assert np.abs(Rg[low] - Rref[low]).max() <= 1e-13 * ncol * np.abs(Rref).max(), (mode, np.abs(Rg[low] - Rref[low]).max())
        results[mode] = (Qg, Rg)
    # the replayed graph runs the same kernels on the same data in the same order
    assert results["eager"][0].tobytes() == results["graph"][0].tobytes() and results["eager"][1].tobytes() == results["graph"][1].tobytes()
    consts.free()


BATCH_CASES = [  # dtype, ta, tb, M, N, K, batch sizes, B shared by the products, scalars on the device / varying per product
    (H.DOUBLE, "N", "N", 128, 128, 64, (3,), False, False),
    (H.DOUBLE, "T", "N", 70, 50, 90, (2, 3), True, True),
    (H.FLOAT, "N", "T", 130, 257, 33, (4,), False, True),
    (H.FLOAT, "T", "N", 1, 1, 700, (5, 2), False, True),            # dot products
    (H.CFLOAT, "C", "N", 65, 40, 50, (3,), True, False),
    (H.CDOUBLE, "N", "C", 33, 31, 17, (2, 2), False, True),
    (H.INT32, "N", "N", 70, 66, 40, (3,), False, True),
    (H.BOOL, "T", "T", 20, 30, 10, (2,), False, False),
    (H.HALF, "N", "N", 64, 64, 64, (3,), False, False),
    (H.INT8, "N", "T", 70, 66, 96, (3, 2), False, True),              # 8-bit MFMA kernel with batch offsets and per-product scalars
    (H.UINT8, "T", "N", 129, 64, 40, (2,), True, False),
    (H.BOOL, "N", "N", 64, 40, 64, (4,), False, True),
    (H.DOUBLE, "N", "N", 16, 16, 16, (1, 7, 1), False, "host"),       # host scalars that differ per product: one launch each
]


@pytest.mark.parametrize("case", BATCH_CASES, ids=lambda c: "%s-%s%s-%dx%dx%d-b%s" % (H.NAMES[c[0]], c[1], c[2], c[3], c[4], c[5], "x".join(map(str, c[6]))))
def test_gemm_batched_equals_loop(hip, stream, case):
    """och_gemm_batched (the reference's loop over the dimensions beyond the second, tensor_blas_gpu.c:171-252, as one
    launch) gives bit for bit what one och_gemm per product gives (those are held to the oracle above); integer
    results are also compared with the oracle directly."""
    run_batched(stream, case, (2, 1, 3))


PIPELINED_BATCH_CASES = [  # as above; aligned operands, sizes the pipelined kernels take when they are asked to
    (H.FLOAT, "N", "T", 260, 132, 96, (3,), False, True),
    (H.FLOAT, "T", "N", 128, 384, 64, (2, 2), True, False),
    (H.DOUBLE, "N", "N", 258, 130, 48, (3,), False, True),
    (H.DOUBLE, "T", "T", 384, 128, 32, (2,), False, "host"),
    (H.CFLOAT, "C", "N", 130, 258, 64, (3,), True, True),
    (H.CDOUBLE, "N", "C", 129, 67, 48, (2, 2), False, True),
]


@pytest.mark.parametrize("choice", [1, 2, 4], ids=["large_tile", "small_tile", "smallest_tile"])
@pytest.mark.parametrize("case", PIPELINED_BATCH_CASES, ids=lambda c: "%s-%s%s-%dx%dx%d-b%s" % (H.NAMES[c[0]], c[1], c[2], c[3], c[4], c[5], "x".join(map(str, c[6]))))
def test_gemm_batched_on_the_pipelined_kernels(hip, stream, case, choice):
    """The batch in grid z of the pipelined kernels (operand, scalar and result offsets per product; ragged last tiles):
    bit for bit what one product at a time gives with the same kernel, which is held to the oracle above."""
    oh.check(oh.lib.och_gemm_set_kernel_choice(choice))
    try:
        run_batched(stream, case, (4, 4, 4))
    finally:
        oh.check(oh.lib.och_gemm_set_kernel_choice(0))


def run_batched(stream, case, pads):
    dtype, ta, tb, M, N, K, bsize, share_b, scalars = case
    rng = np.random.default_rng(99 + dtype + M)
    rowsA, colsA = (M, K) if ta == "N" else (K, M)
    rowsB, colsB = (K, N) if tb == "N" else (N, K)
    ldA, ldB, ldC = rowsA + pads[0], rowsB + pads[1], M + pads[2]
    total = int(np.prod(bsize))
    item = np.dtype(H.storage(dtype)).itemsize
    A = H.random_data(dtype, ldA * colsA * total, rng, "small")
    B = H.random_data(dtype, ldB * colsB * (1 if share_b else total), rng, "small")
    C0 = H.random_data(dtype, ldC * N * total, rng, "small")
    vary = bool(scalars)
    als = np.concatenate([scalar_of(dtype, v) for v in (rng.integers(1, 3, total) if vary else [2] * total)])
    bes = np.concatenate([scalar_of(dtype, v) for v in (rng.integers(0, 2, total) if vary else [1] * total)])
    # byte strides per batch dimension, first dimension fastest
    mult = [int(np.prod(bsize[:d])) for d in range(len(bsize))]
    sA = [m * ldA * colsA * item for m in mult]
    sB = [0 if share_b else m * ldB * colsB * item for m in mult]
    sC = [m * ldC * N * item for m in mult]
    sS = [m * item if vary else 0 for m in mult]
    dA, dB = oh.to_device(A, stream), oh.to_device(B, stream)
    dC1, dC2 = oh.to_device(C0, stream), oh.to_device(C0, stream)
    on_host = scalars == "host" or scalars is False
    if on_host:
        pal, pbe = als.ctypes.data, bes.ctypes.data
    else:
        dal, dbe = oh.to_device(als, stream), oh.to_device(bes, stream)
        pal, pbe = dal.address, dbe.address
    oh.check(oh.lib.och_gemm_batched(dtype, ta.encode(), tb.encode(), M, N, K, pal, dA.ptr, ldA, dB.ptr, ldB, pbe, dC1.ptr, ldC,
                                     len(bsize), oh.sizes(bsize), oh.strides(sS), oh.strides(sA), oh.strides(sB), oh.strides(sS), oh.strides(sC),
                                     1 if on_host else 0, stream.handle))
    want = C0.copy()
    for z in range(total):
        idx = [(z // m) % n for m, n in zip(mult, bsize)]
        off = lambda st: sum(i * s for i, s in zip(idx, st))
        oh.check(oh.lib.och_gemm(dtype, ta.encode(), tb.encode(), M, N, K, pal + off(sS), dA.address + off(sA), ldA, dB.address + off(sB), ldB,
                                 pbe + off(sS), dC2.address + off(sC), ldC, 1 if on_host else 0, stream.handle))
        if dtype not in TOL:
            assert orc.lib.oracle_gemm(dtype, ta.encode(), tb.encode(), M, N, K, als.ctypes.data + off(sS), A.ctypes.data + off(sA), ldA,
                                       B.ctypes.data + off(sB), ldB, bes.ctypes.data + off(sS), want.ctypes.data + off(sC), ldC, 1) == 0
    got, loop = dC1.download(C0.dtype, C0.size), dC2.download(C0.dtype, C0.size)
    H.assert_same_bytes(got, loop, "batched vs loop")
    if dtype not in TOL:
        H.assert_same_bytes(got, want, "batched vs oracle")
    assert not np.array_equal(got, C0)
    for b in (dA, dB, dC1, dC2):
        b.free()


SKINNY = [(300, 1, 500), (1, 300, 500), (1000, 3, 70), (5, 2000, 33), (4100, 8, 129), (2050, 1, 4099), (8, 4097, 513), (66, 7, 5), (4096, 2, 64)]


@pytest.mark.parametrize("dtype", [H.FLOAT, H.DOUBLE, H.CFLOAT, H.CDOUBLE], ids=lambda d: H.NAMES[d])
def test_gemm_with_one_small_dimension(hip, stream, dtype):
    """Matrix x vector and matrix x few-columns products (and their transposes) take the streaming kernels: rows
    contiguous (split over K, partial results in the stream's workspace) or K contiguous (lanes share a row). Every mode
    pair, unaligned leading dimensions (pad = 3) and aligned ones, host and device scalars, beta != 0."""
    rng = np.random.default_rng(700 + dtype)
    cplx = dtype in H.COMPLEX_TYPES
    modes = ["N", "T"] + (["C"] if cplx else [])
    for (M, N, K) in SKINNY:
        for ta in modes:
            for tb in modes:
                alpha, beta = ((2 - 1j, -1 + 0.5j) if cplx else (2, -1)) if (M + K + len(ta)) % 2 else (1, 0)
                run_case(stream, dtype, ta, tb, M, N, K, alpha, beta, rng, device_scalars=(N % 2 == 0), pad=3 if (K % 2) else 0)


LONG_K = [(128, 128, 20000), (100, 70, 5003), (64, 200, 9000), (9, 9, 70000), (256, 130, 4096)]


@pytest.mark.parametrize("dtype", [H.FLOAT, H.DOUBLE, H.CFLOAT, H.CDOUBLE], ids=lambda d: H.NAMES[d])
def test_gemm_with_few_tiles_and_long_k(hip, stream, dtype):
    """Products with few output tiles and a long inner dimension are split over K: every slice leaves raw sums in the
    stream's workspace and a second kernel adds them in slice order and applies alpha / beta (beta != 0 included)."""
    rng = np.random.default_rng(800 + dtype)
    cplx = dtype in H.COMPLEX_TYPES
    for (M, N, K) in LONG_K:
        for ta, tb in (("N", "N"), ("T", "N"), ("N", "T"), ("C" if cplx else "T", "C" if cplx else "T")):
            alpha, beta = ((2 - 1j, -1 + 0.5j) if cplx else (2, -1)) if (M + len(ta)) % 2 else (1, 0)
            run_case(stream, dtype, ta, tb, M, N, K, alpha, beta, rng, device_scalars=(K % 2 == 0), pad=3 if (K % 2) else 0)


@pytest.mark.parametrize("dtype", [H.FLOAT, H.DOUBLE, H.CFLOAT, H.CDOUBLE], ids=lambda d: H.NAMES[d])
def test_gemm_seeded_shapes_under_the_automatic_choice(hip, stream, dtype):
    """Shapes drawn from a fixed seed, left to the library's own choice of kernel: M and N from 128 to 1500 (even, mostly
    multiples of 4, some odd), K from one slab to 6000 with and without a remainder, every mode pair, aligned and unaligned
    leading dimensions, alpha / beta trivial or not, scalars in host or device memory. Whatever the model picks -- large or
    small pipelined tile, last round cut along K, padded rest of K, tiled kernel -- the result is held to the same bound."""
    rng = np.random.default_rng(4200 + dtype)
    cplx = dtype in H.COMPLEX_TYPES
    slab = 16 if dtype in (H.DOUBLE, H.CDOUBLE) else 32
    modes = ["N", "T"] + (["C"] if cplx else [])
    for n in range(32):
        step = (4, 4, 2, 1)[n % 4]
        M, N = (int(rng.integers(128 // step, 1500 // step)) * step for _ in range(2))
        K = int(rng.integers(1, 6000 // slab)) * slab + (int(rng.integers(1, slab)) if n % 3 == 1 else 0)
        ta, tb = modes[int(rng.integers(len(modes)))], modes[int(rng.integers(len(modes)))]
        alpha, beta = ((2 - 1j, -1 + 0.5j) if cplx else (2, -1)) if n % 2 else (1, 0)
        check_large_product(stream, dtype, ta, tb, M, N, [(K / slab, alpha, beta, n % 5 == 4)], rng, pad=(0, 4, 0, 3)[(n // 4) % 4])


@pytest.mark.parametrize("dtype", [H.HALF, H.INT8, H.UINT8], ids=lambda d: H.NAMES[d])
def test_gemm_seeded_shapes_of_the_matrix_core_types(hip, stream, dtype):
    """The same for half (float accumulation, bound 2e-3) and the 8-bit integers (exact modulo 256): shapes from a fixed
    seed with M and N from 64 to 1500, whole tiles, edge strips and odd sizes, K with and without whole slabs, aligned and
    unaligned leading dimensions, both kinds of scalars."""
    rng = np.random.default_rng(4300 + dtype)
    slab = 64 if dtype == H.HALF else 128
    for n in range(24):
        step = (256, 128, 8, 1)[n % 4]
        M, N = (max(step, int(rng.integers(64, 1500)) // step * step) for _ in range(2))
        K = int(rng.integers(1, 4000 // slab)) * slab + (int(rng.integers(1, slab)) if n % 3 == 1 else 0)
        ta, tb = "NT"[int(rng.integers(2))], "NT"[int(rng.integers(2))]
        alpha, beta = (2, -1) if n % 2 else (1, 0)
        check_large_product(stream, dtype, ta, tb, M, N, [(K / slab, alpha, beta, n % 5 == 4)], rng, pad=(0, 8, 0, 3)[(n // 4) % 4])
