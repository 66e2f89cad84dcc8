"""The elementary functions the device library evaluates itself (csrc/och_math.h: powf, tanh on double, sinh, cosh, log1p
and the inverse hyperbolic functions in both precisions) against the host's libm, the functions the reference's CPU module calls (solid/include/solid/core/cpu/unary_ops_cpu.h:24-140; powf
for the power of float and double alike, binary_ops.h). The header uses IEEE basic operations only, so its host build
(tests/math_host.cpp, compiled here with g++) computes bit for bit what the kernels compute; what is established here on
millions of arguments holds on the device."""
import ctypes as C
import os
import shutil
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def mathlib(tmp_path_factory):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("g++ is not available")
    so = str(tmp_path_factory.mktemp("math") / "math_host.so")
    subprocess.run([gxx, "-O2", "-ffp-contract=off", "-shared", "-fPIC", "-I", os.path.join(ROOT, "ocean-tensor-package_amd", "csrc"),
                    os.path.join(ROOT, "tests", "math_host.cpp"), "-o", so], check=True)
    return C.CDLL(so)


def call2(lib, name, x, y):
    out = np.empty_like(x)
    getattr(lib, name)(C.c_size_t(x.size), x.ctypes.data_as(C.c_void_p), y.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
    return out


def call1(lib, name, x):
    out = np.empty_like(x)
    getattr(lib, name)(C.c_size_t(x.size), x.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
    return out


def ulps(got, want):
    """distance in units in the last place, element by element (NaN against NaN: 0; NaN against a number: huge)"""
    it = {4: np.int32, 8: np.int64}[got.dtype.itemsize]
    magnitude = np.int64({4: 0x7FFFFFFF, 8: 0x7FFFFFFFFFFFFFFF}[got.dtype.itemsize])
    gi, wi = got.view(it).astype(np.int64), want.view(it).astype(np.int64)
    gi = np.where(gi < 0, -(gi & magnitude), gi)
    wi = np.where(wi < 0, -(wi & magnitude), wi)
    d = np.abs(gi - wi)
    d[np.isnan(got) & np.isnan(want)] = 0
    d[np.isnan(got) != np.isnan(want)] = 1 << 40
    return d


def random_floats(rng, n):
    return rng.integers(0, 2 ** 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32)


N = 1_000_000

POWF_RANGES = {
    "moderate": lambda rng: (rng.uniform(0, 10, N).astype(np.float32), rng.uniform(-10, 10, N).astype(np.float32)),
    "wide_bases": lambda rng: (np.exp(rng.uniform(-87, 88, N)).astype(np.float32), rng.uniform(-3, 3, N).astype(np.float32)),
    "bases_near_one_large_exponents": lambda rng: (rng.uniform(0.9, 1.1, N).astype(np.float32), rng.uniform(-1000, 1000, N).astype(np.float32)),
    "subnormal_bases": lambda rng: (rng.integers(1, 1 << 23, N).astype(np.uint32).view(np.float32), rng.uniform(-1.2, 1.2, N).astype(np.float32)),
    "results_around_the_smallest_and_largest_floats": lambda rng: (rng.uniform(1.5, 2.5, N).astype(np.float32), rng.choice([-1.0, 1.0], N).astype(np.float32) * rng.uniform(90, 160, N).astype(np.float32)),
    "negative_bases_integer_exponents": lambda rng: (rng.uniform(-10, 10, N).astype(np.float32), rng.integers(-12, 12, N).astype(np.float32)),
    "negative_bases_any_exponent": lambda rng: (rng.uniform(-10, 10, N).astype(np.float32), rng.uniform(-4, 4, N).astype(np.float32)),
    "random_bits": lambda rng: (random_floats(rng, N), random_floats(rng, N)),
    "random_bit_bases_small_exponents": lambda rng: (random_floats(rng, N), rng.uniform(-2, 2, N).astype(np.float32)),
}


@pytest.mark.parametrize("name", list(POWF_RANGES))
def test_powf_is_within_one_unit_of_the_host_and_is_the_rounded_power(mathlib, name):
    """Never more than one unit in the last place from the host's powf, NaN exactly where the host gives NaN; and where the
    two differ it is this routine that agrees with the power computed in double precision and rounded to float (the
    host's powf is documented to be off by one unit now and then; this one in a few cases per million)."""
    rng = np.random.default_rng(sum(map(ord, name)))
    x, y = POWF_RANGES[name](rng)
    got, want = call2(mathlib, "host_och_powf", x, y), call2(mathlib, "host_libm_powf", x, y)
    d = ulps(got, want)
    worst = int(np.argmax(d))
    assert d[worst] <= 1, "powf(%r, %r) = %r, host %r" % (x[worst], y[worst], got[worst], want[worst])
    exact = (d == 0) & ~np.isnan(want)
    assert np.array_equal(np.signbit(got[exact]), np.signbit(want[exact]))          # zeros of the right sign
    with np.errstate(all="ignore"):
        rounded = np.power(x.astype(np.float64), y.astype(np.float64)).astype(np.float32)
    ordinary = np.isfinite(rounded) & (rounded != 0) & ~np.isnan(want)
    mine, host = int((ulps(got, rounded)[ordinary] != 0).sum()), int((ulps(want, rounded)[ordinary] != 0).sum())
    assert mine <= 20 and mine <= host + 5, (mine, host)


def test_powf_special_values_follow_the_host_bit_for_bit(mathlib):
    """zeros, ones, infinities, NaN, the largest and smallest floats, odd and even and fractional exponents, exponents from
    2^24 on (all even integers), either sign of everything: C99 F.10.4.4 as the host implements it."""
    sp = np.array([0.0, -0.0, 1.0, -1.0, 2.0, -2.0, 0.5, -0.5, np.inf, -np.inf, np.nan, 3.0, -3.0, 2.5, -2.5, 1e-45, -1e-45, 3.4e38,
                   -3.4e38, 1e-38, -1e-38, 16777215.0, 16777216.0, 16777218.0, 33554432.0, 1e10, -1e10, 0.99999994, 1.0000001,
                   -0.99999994, -1.0000001, 127.0, 128.0, -149.0, -150.0, 1 / 3, -1 / 3, 1e-30, -1e-30], dtype=np.float32)
    X, Y = np.meshgrid(sp, sp)
    x, y = X.ravel().copy(), Y.ravel().copy()
    got, want = call2(mathlib, "host_och_powf", x, y), call2(mathlib, "host_libm_powf", x, y)
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    bad = np.nonzero(~same)[0]
    assert bad.size == 0, [(x[i], y[i], got[i], want[i]) for i in bad[:10]]


@pytest.mark.parametrize("lo,hi", [(-1, 1), (-0.6, 0.6), (0, 1e-3), (-25, 25), (0.1, 0.4), (15, 25), (-1e-300, 1e-300)])
def test_tanh_is_within_three_units_of_the_host(mathlib, lo, hi):
    rng = np.random.default_rng(int(abs(lo) * 1000 + abs(hi) * 10))
    x = rng.uniform(lo, hi, N)
    got, want = call1(mathlib, "host_och_tanh", x), call1(mathlib, "host_libm_tanh", x)
    d = ulps(got, want)
    worst = int(np.argmax(d))
    assert d[worst] <= 3, "tanh(%r) = %r, host %r" % (x[worst], got[worst], want[worst])
    assert d.mean() < 0.7
    assert np.all(np.abs(got) <= 1.0) and np.array_equal(np.signbit(got), np.signbit(x))


def test_tanh_special_values_and_monotone_ends(mathlib):
    x = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-310, -1e-310, 5e-324, 19.0, 19.9, 20.0, 20.1, 400.0, -400.0, 1e300, -1e300,
                  np.log(2) / 2, np.log(2), 0.1732867951399863, 0.17328679513998635])
    got, want = call1(mathlib, "host_och_tanh", x), call1(mathlib, "host_libm_tanh", x)
    assert np.isnan(got[4]) and ulps(got, want).max() <= 3
    assert np.array_equal(got[:4].view(np.uint64), want[:4].view(np.uint64))            # signed zeros, +-1 at the infinities
    assert np.array_equal(got[5:8], x[5:8])                                              # tanh x = x for subnormal x
    assert np.all(got[9:13] == 1.0) and got[13] == -1.0 and got[14] == 1.0 and got[15] == -1.0


ONE_ARGUMENT = {
    # name: (ranges in double, ranges in float)
    "sinh": [(-1, 1), (0, 1e-3), (0.9, 1.1), (-22, 22), (-709, 709), (709, 712)],
    "cosh": [(-1, 1), (0, 1e-3), (0.9, 1.1), (-22, 22), (-709, 709), (709, 712)],
    "log1p": [(-0.999, 1), (-1e-3, 1e-3), (-0.5, 0.5), (0, 100), (1e10, 1e300), (-1, -0.99)],
    "atanh": [(-0.999, 0.999), (-1e-3, 1e-3), (0.4, 0.6), (0.99, 1.0)],
    "asinh": [(-1, 1), (-1e-3, 1e-3), (1.9, 2.1), (-100, 100), (1e8, 1e9), (1e100, 1e300)],
    "acosh": [(1, 1.001), (1, 2), (1.9, 2.1), (2, 100), (1e8, 1e9), (1e100, 1e300)],
}
SPECIAL = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-300, -1e-300, 1e-40, -1.0, 1.0, -2.0, 0.5, -0.5, 2.0, 2.0 ** 28, 2.0 ** 28 + 1, 1e-20, -1e-20, 3e38,
           -3e38, 710.4, 710.5, 89.4, 89.5, 88.7, 1.0 - 2.0 ** -53, -1.0 + 2.0 ** -53, 1.0 + 2.0 ** -52]


@pytest.mark.parametrize("single", [False, True], ids=["double", "float"])
@pytest.mark.parametrize("name", list(ONE_ARGUMENT))
def test_hyperbolic_and_log1p_routines_stay_within_three_units_of_the_host(mathlib, name, single):
    """double: within 3 units in the last place of the host's function; float (evaluated in double precision and rounded
    once): within 2 of the host's float function and within 1 of the host's double function rounded to float. NaN, the
    infinities and signed zeros exactly as the host gives them."""
    dt = np.float32 if single else np.float64
    fn = name + ("f" if single else "")
    rng = np.random.default_rng(sum(map(ord, fn)))
    for lo, hi in ONE_ARGUMENT[name]:
        if single:
            if lo >= 1e100:
                lo, hi = 1e30, 3e38
            elif abs(hi) >= 700:
                lo, hi = (lo / 709 * 88, hi / 709 * 88) if hi <= 709 else (88, 91)
        x = rng.uniform(lo, hi, N // 2).astype(dt)
        got, want = call1(mathlib, "host_och_" + fn, x), call1(mathlib, "host_libm_" + fn, x)
        d = ulps(got, want)
        worst = int(np.argmax(d))
        assert d[worst] <= (2 if single else 3), "%s(%r) = %r, host %r" % (fn, x[worst], got[worst], want[worst])
        if single:
            with np.errstate(all="ignore"):
                rounded = call1(mathlib, "host_libm_" + name, x.astype(np.float64)).astype(np.float32)
            assert ulps(got, rounded).max() <= 1
            assert (ulps(got, rounded) != 0).mean() < 1e-4          # the correctly rounded value but for a few cases
    x = np.array(SPECIAL, dtype=dt)
    got, want = call1(mathlib, "host_och_" + fn, x), call1(mathlib, "host_libm_" + fn, x)
    d = ulps(got, want)
    assert d.max() <= 3, [(a, b, c) for a, b, c in zip(x, got, want) if not (a == a and b == c)][:5]
    unusual = ~np.isfinite(want) | (want == 0)
    assert np.array_equal(got[unusual & ~np.isnan(want)].view(np.uint32 if single else np.uint64),
                          want[unusual & ~np.isnan(want)].view(np.uint32 if single else np.uint64))
