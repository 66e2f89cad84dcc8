"""The micro-benchmarks that the measurements are set against (no counterpart in the reference): they run, their
arguments are checked, and their figures are those of a device of this kind (a loop of nothing but MFMAs cannot be slower
than the GEMM kernels; a streaming copy cannot be far below the kernels that copy)."""
import ctypes as C

import pytest

import ocean_hip as oh

pytestmark = pytest.mark.gpu


def mfma(stream, typ, kind, per, waves, iters=2000):
    ms, flop = C.c_float(), C.c_double()
    oh.check(oh.lib.och_mfmabench(typ, kind, per, waves, iters, 5, C.byref(ms), C.byref(flop), stream.handle))
    return ms.value, flop.value


def test_mfmabench_rates_and_instruction_costs(hip, stream):
    mfma(stream, 0, 0, 0, 4)                                             # clocks up
    floors = {0: 120e12, 1: 60e12, 2: 1000e12, 3: 2000e12}               # flop/s: well below what the GEMM kernels reach
    for typ, floor in floors.items():
        ms, flop = mfma(stream, typ, 0, 0, 4)
        assert flop / (ms * 1e-3) > floor, (typ, flop / ms / 1e9)
    base, flop = mfma(stream, 0, 0, 0, 4)
    assert flop == 2.0 * 32 * 32 * 2 * 16 * 2000 * 4 * hip.device_properties(0).multiprocessor_count
    valu, _ = mfma(stream, 0, 1, 4, 4)                                   # four v_mov after every MFMA: clearly slower
    salu, _ = mfma(stream, 0, 4, 4, 4)                                   # four scalar adds: free
    assert valu > 1.3 * base and salu < 1.15 * base, (base, valu, salu)
    two, _ = mfma(stream, 0, 0, 0, 8)                                    # two waves per SIMD: twice the work, twice the time
    assert 1.5 * base < two < 2.5 * base, (base, two)


def test_mfmabench_arguments(hip, stream):
    ms, flop = C.c_float(), C.c_double()
    for args in ((4, 0, 0, 4, 10, 1), (0, 8, 1, 4, 10, 1), (0, 1, 3, 4, 10, 1), (0, 0, 0, 5, 10, 1), (0, 0, 0, 4, 0, 1), (0, 0, 0, 4, 10, 0)):
        assert oh.lib.och_mfmabench(*args, C.byref(ms), C.byref(flop), stream.handle) != 0, args
        assert b"mfmabench" in oh.lib.och_last_error()


def test_membench_runs(hip, stream):
    med, best, moved = C.c_float(), C.c_float(), C.c_size_t()
    oh.check(oh.lib.och_membench(2, 2, 0, 0, 256, 0, 1 << 26, 3, 5, C.byref(med), C.byref(best), C.byref(moved), stream.handle))
    assert moved.value == 2 << 26 and best.value <= med.value
    assert moved.value / (med.value * 1e-3) > 3e12                        # a 67 MB copy streams at several TB/s
    assert oh.lib.och_membench(9, 2, 0, 0, 256, 0, 1 << 26, 3, 5, C.byref(med), C.byref(best), C.byref(moved), stream.handle) != 0
