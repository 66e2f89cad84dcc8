"""The micro-benchmarks that the measurements are set against (csrc/libocean_hip_bench.so, include/ocean_hip_bench.h; no
counterpart in the reference): they run, their arguments are checked, the work they report is the work they launch, and
their timings are sane. What the device sustains is a measurement (`bench.py --ceiling`), not an assertion: only bounds
loose enough for any device of this kind, at any clock, are tested here."""
import ctypes as C

import pytest

import ocean_hip as oh
import ocean_hip_bench as ohb

pytestmark = pytest.mark.gpu


def mfma(stream, typ, kind, per, waves, iters=2000):
    ms, flop = C.c_float(), C.c_double()
    oh.check(ohb.lib.och_mfmabench(typ, kind, per, waves, iters, 5, C.byref(ms), C.byref(flop), stream.handle))
    return ms.value, flop.value


def test_mfmabench_counts_its_work(hip, stream):
    units = hip.device_properties(0).multiprocessor_count
    per_mfma = {0: 2.0 * 32 * 32 * 2, 1: 2.0 * 16 * 16 * 4, 2: 2.0 * 32 * 32 * 16, 3: 2.0 * 32 * 32 * 32}
    for typ, ops in per_mfma.items():
        ms, flop = mfma(stream, typ, 0, 0, 4)
        assert flop == ops * 16 * 2000 * 4 * units and ms > 0
        assert flop / (ms * 1e-3) > 1e12                                  # matrix cores, not a scalar loop
    _, flop8 = mfma(stream, 0, 0, 0, 8)
    assert flop8 == 2 * per_mfma[0] * 16 * 2000 * 4 * units               # two waves per SIMD: twice the work
    base, _ = mfma(stream, 0, 0, 0, 4)
    valu, _ = mfma(stream, 0, 1, 4, 4)                                   # four vector moves after every MFMA cost time
    assert valu > base


def test_mfmabench_arguments(hip, stream):
    ms, flop = C.c_float(), C.c_double()
    for args in ((4, 0, 0, 4, 10, 1), (0, 8, 1, 4, 10, 1), (0, 1, 3, 4, 10, 1), (0, 0, 0, 5, 10, 1), (0, 0, 0, 4, 0, 1), (0, 0, 0, 4, 10, 0)):
        assert ohb.lib.och_mfmabench(*args, C.byref(ms), C.byref(flop), stream.handle) != 0, args
        assert b"mfmabench" in oh.lib.och_last_error()


def test_membench_runs(hip, stream):
    med, best, moved = C.c_float(), C.c_float(), C.c_size_t()
    oh.check(ohb.lib.och_membench(2, 2, 0, 0, 256, 0, 1 << 26, 3, 5, C.byref(med), C.byref(best), C.byref(moved), stream.handle))
    assert moved.value == 2 << 26 and 0 < best.value <= med.value
    assert moved.value / (med.value * 1e-3) > 1e11                        # device memory, not a host transfer
    assert ohb.lib.och_membench(9, 2, 0, 0, 256, 0, 1 << 26, 3, 5, C.byref(med), C.byref(best), C.byref(moved), stream.handle) != 0
    assert b"membench" in oh.lib.och_last_error()
