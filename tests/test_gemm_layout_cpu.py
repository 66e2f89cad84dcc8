"""The LDS layout of the four pipelined GEMM kernels (float, double, complex float, complex double), walked through on the host.

csrc/och_gemm_f32p_slab.h holds the index arithmetic of gemm_float_pipe_kernel (the counterpart of cublasSgemm in
src/core/gpu/op/tensor_blas_gpu.c:183-197): which 16 bytes every lane of every load instruction fetches and where in LDS
they land, where a lane reads its fragments, and which row and k a fragment value stands for. tests/gemm_slab_host.cpp
compiles that header for the host, builds a slab of a known matrix with the load functions and checks that every value an
MFMA would be given is the matrix element it has to be -- for both operand layouts, the three block tiles (256, 128, 64
rows) and last tiles of a matrix of which only a few rows exist."""
import ctypes as C
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLANG = "/opt/rocm/llvm/bin/clang++"


@pytest.fixture(scope="module")
def slab(tmp_path_factory):
    if not os.path.exists(CLANG):
        pytest.skip("ROCm's clang++ is not available (the header uses its vector types)")
    so = str(tmp_path_factory.mktemp("slab") / "gemm_slab_host.so")
    subprocess.run([CLANG, "-O1", "-std=c++17", "-shared", "-fPIC", "-I", os.path.join(ROOT, "ocean-tensor-package_amd", "csrc"),
                    os.path.join(ROOT, "tests", "gemm_slab_host.cpp"), "-o", so], check=True)
    lib = C.CDLL(so)
    lib.gemm_slab_check.restype = C.c_long
    lib.gemm_slab_check.argtypes = [C.c_int, C.c_int, C.c_uint, C.c_long, C.c_int]
    lib.gemm_slab_check_double.restype = C.c_long
    lib.gemm_slab_check_double.argtypes = [C.c_int, C.c_int, C.c_uint, C.c_long, C.c_int]
    lib.gemm_slab_check_cfloat.restype = C.c_long
    lib.gemm_slab_check_cfloat.argtypes = [C.c_int, C.c_uint, C.c_long, C.c_int]
    lib.gemm_slab_check_cdouble.restype = C.c_long
    lib.gemm_slab_check_cdouble.argtypes = [C.c_int, C.c_int, C.c_uint, C.c_long, C.c_int]
    return lib


@pytest.mark.parametrize("tile", [256, 128, 64])
@pytest.mark.parametrize("kc", [0, 1], ids=["contiguous_along_rows", "contiguous_along_k"])
def test_every_mfma_operand_is_the_matrix_element_it_has_to_be(slab, kc, tile):
    for rows in sorted({tile, tile - 4, tile // 2 + 4, tile // 2, 36, 8, 4}):
        if rows > tile:
            continue
        for ld in ((32, 36, 1000) if kc else (tile, tile + 8, 4 * tile + 4)):
            assert slab.gemm_slab_check(kc, tile, rows, ld, 1) == 0, (kc, tile, rows, ld)


@pytest.mark.parametrize("tile", [256, 128])
@pytest.mark.parametrize("kc", [0, 1], ids=["contiguous_along_rows", "contiguous_along_k"])
def test_every_double_mfma_operand_is_the_matrix_element_it_has_to_be(slab, kc, tile):
    """The same walk for gemm_double_pipe_kernel (csrc/och_gemm_f64p_slab.h): slabs of 16 k, operands of 256 rows (A of the
    large tile) and 128 rows, tiles of 16 rows, last tiles of which only a few rows exist (multiples of 2)."""
    for rows in sorted({tile, tile - 2, tile // 2 + 2, tile // 2, 34, 6, 2}):
        for ld in ((16, 18, 1000) if kc else (tile, tile + 6, 4 * tile + 2)):
            assert slab.gemm_slab_check_double(kc, tile, rows, ld, 1) == 0, (kc, tile, rows, ld)


@pytest.mark.parametrize("kc", [0, 1], ids=["contiguous_along_rows", "contiguous_along_k"])
def test_every_complex_mfma_operand_is_the_matrix_element_it_has_to_be(slab, kc):
    """gemm_cfloat_pipe_kernel (och_gemm_c32p_slab.h: 128 rows, 32 k) and gemm_cdouble_pipe_kernel (och_gemm_c64p_slab.h: 128
    and 64 rows, 16 k): real and imaginary part of every operand value, whole and ragged tiles."""
    for rows in (128, 126, 66, 64, 34, 2):
        for ld in ((32, 34, 1000) if kc else (128, 130, 517)):
            assert slab.gemm_slab_check_cfloat(kc, rows, ld, 1) == 0, (kc, rows, ld)
    for tile in (128, 64):
        for rows in sorted({tile, tile - 1, tile // 2 + 1, tile // 2, 17, 1}):
            for ld in ((16, 18, 1000) if kc else (tile, tile + 3, 4 * tile + 1)):
                assert slab.gemm_slab_check_cdouble(kc, tile, rows, ld, 1) == 0, (kc, tile, rows, ld)


def test_unknown_tile_is_refused(slab):
    assert slab.gemm_slab_check(0, 96, 96, 96, 0) == -1
    assert slab.gemm_slab_check_double(0, 64, 64, 64, 0) == -1
