"""The Python surface of the GPU module (ocean_gpu.py) against what `import pyOcean_gpu` provides in the reference:
the module-level names (pyOcean_device_gpu.c:128-158) and the property list of the device type
(pyOcean_device_gpu.c:65-94)."""
import numpy as np
import pytest

import ocean_host as host

# PY_GET_ENTRY names, pyOcean_device_gpu.c:66-92
REFERENCE_PROPERTIES = ["deviceName", "totalGlobalMem", "totalMem", "freeMem", "sharedMemPerBlock", "regsPerBlock", "warpSize", "memPitch",
                        "maxThreadsPerBlock", "maxThreadsDim", "maxGridSize", "totalConstMem", "major", "minor", "version", "clockRate",
                        "deviceOverlap", "multiProcessorCount", "kernelExecTimeoutEnabled", "integrated", "canMapHostMemory", "computeMode",
                        "concurrentKernels", "ECCEnabled", "pciBusID", "pciDeviceID", "tccDriver"]


def test_module_names_and_property_list():
    """Importing works on a machine without a GPU too (the device tuple is then empty, device_gpu.c:189-191)."""
    import ocean_gpu
    assert isinstance(ocean_gpu.gpu, tuple)
    assert len(ocean_gpu.gpu) == host.lib.OcDeviceGPUCount()
    for name in REFERENCE_PROPERTIES:
        assert isinstance(getattr(ocean_gpu.deviceGPU, name), property), name
        assert getattr(ocean_gpu.deviceGPU, name).__doc__
    with pytest.raises(IndexError):
        ocean_gpu.deviceGPU(len(ocean_gpu.gpu))


@pytest.mark.gpu
def test_device_properties(hip):
    import ocean_gpu
    assert len(ocean_gpu.gpu) >= 1
    d = ocean_gpu.gpu[0]
    assert (d.index, d.name, d.type) == (0, "gpu0", "GPU") and repr(d) == "<device 'gpu0'>"
    values = {name: getattr(d, name) for name in REFERENCE_PROPERTIES}
    assert isinstance(values["deviceName"], str)          # the marketing name; some systems report an empty one
    assert values["warpSize"] == 64 and values["multiProcessorCount"] >= 64
    assert values["totalMem"] == values["totalGlobalMem"] >= (1 << 30)
    assert 0 < values["freeMem"] <= values["totalMem"]
    assert values["version"] == "%d.%d" % (values["major"], values["minor"])
    assert d.archName.startswith("gfx") and values["major"] >= 9
    assert values["sharedMemPerBlock"] >= 65536 and values["maxThreadsPerBlock"] >= 256
    assert len(values["maxThreadsDim"]) == 3 and len(values["maxGridSize"]) == 3 and min(values["maxGridSize"]) >= 65535
    assert values["clockRate"] > 100.0
    for name in ("deviceOverlap", "kernelExecTimeoutEnabled", "integrated", "canMapHostMemory", "concurrentKernels", "ECCEnabled", "tccDriver"):
        assert isinstance(values[name], bool), name
    assert values["tccDriver"] is False and values["integrated"] is False
    assert d.peerAccess(d)
    # free memory follows allocations (updateProperties is called on every read, pyOcean_device_gpu.c:186-191)
    before = d.freeMem
    t = host.create([1 << 26], host.DOUBLE, host.gpu_device(0))
    assert d.freeMem <= before - (1 << 28)
    host.lib.OcDecrefTensor(t)


@pytest.mark.gpu
def test_device_call_moves_data(hip):
    import ocean_gpu
    rng = np.random.default_rng(5)
    for a in (rng.standard_normal((3, 5)), rng.integers(-9, 9, (4, 2, 3)).astype(np.int16), rng.random(7) < 0.5,
              rng.standard_normal(6).astype(np.float32) + 1j * rng.standard_normal(6).astype(np.float32)):
        t = ocean_gpu.gpu[0](a)
        assert isinstance(t, ocean_gpu.tensor) and t.device is ocean_gpu.gpu[0]
        assert list(t.size) == list(a.shape[::-1])
        assert np.array_equal(t.asnumpy(), a)
    h = ocean_gpu.gpu[0](np.arange(5, dtype=np.float16))
    assert h.dtype == host.HALF and np.array_equal(h.asnumpy(), np.arange(5, dtype=np.float16))


# ---- the reference's GPU example expressions, replayed through the operators of ocean_gpu.tensor ----------------
# Each function below restates what one example script of examples/python/gpu/tensors computes and prints, and
# returns the printed tensors in order; the expected values, types, sizes and device names are those of the script's
# .ref file (the part after "on gpu0"; the part on the cpu device belongs to Ocean's CPU module).
import os

import ref_format as RF

REFDIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref")
OCEAN_NAME = {code: name for name, code in RF.TYPE_NAMES.items()}


def gpu_part(name):
    text = open(os.path.join(REFDIR, name + ".ref")).read()
    cut = text.find("# Boolean on gpu0")
    return [it for it in RF.parse_ref(text[cut:] if cut >= 0 else text) if isinstance(it, RF.RefTensor)]


def assert_printed(printed, expected, decimals=None):
    """decimals: the expected file prints floating values rounded to that many decimals"""
    assert len(printed) == len(expected)
    for k, (t, ref) in enumerate(zip(printed, expected)):
        assert t.dtype == ref.dtype and list(t.size) == list(ref.shape) and t.device.name == ref.device, (k, t.footer(), ref)
        if list(ref.shape) == []:
            assert t.footer() == "<scalar.%s on %s>" % (OCEAN_NAME[ref.dtype], ref.device)
        else:
            assert t.footer() == "<tensor.%s of size %s on %s%s>" % (OCEAN_NAME[ref.dtype], "x".join(map(str, ref.shape)), ref.device,
                                                                       " (byteswapped)" if ref.byteswapped else "")
        got = t.asnumpy()
        got = got.transpose(*range(got.ndim)[::-1])          # Ocean index order A[i0, i1, ...]
        if decimals is not None and got.dtype.kind in "fc":
            assert np.allclose(got.astype(np.complex128 if got.dtype.kind == "c" else np.float64), ref.values, rtol=0, atol=0.51 * 10.0 ** -decimals,
                               equal_nan=True), (k, got, ref.values)
        else:
            assert np.array_equal(got.astype(ref.values.dtype), ref.values), (k, got, ref.values)


@pytest.mark.gpu
def test_replay_tensor_add_02(hip):
    import ocean_gpu as ocean
    device, out = ocean.gpu[0], []
    a = ocean.asTensor([True, True, False], device)
    out += [a.clone(), +a, a + True]
    a += True
    out.append(a.clone())
    for dtype, three in ((ocean.int8, 3), (ocean.float, 3.0)):
        a = ocean.asTensor([-2, -1, 0, 1, 2], dtype, device)
        out += [a.clone(), +a, a + three]
        a += 3
        out.append(a.clone())
    assert_printed(out, gpu_part("tensor_add_02"))


@pytest.mark.gpu
def test_replay_tensor_multiply_01(hip):
    import ocean_gpu as ocean
    device, out = ocean.gpu[0], []
    a = ocean.asTensor([True, True, False], device)
    out += [a.clone(), a * True, ocean.scale(a, [True, False, True])]
    a *= [True, False, True]
    out.append(a.clone())
    for dtype, three in ((ocean.int8, 3), (ocean.float, 3.0)):
        a = ocean.asTensor([-2, -1, 0, 1, 2], dtype, device)
        out += [a.clone(), a * three]
        a *= 3
        out.append(a.clone())
    assert_printed(out, gpu_part("tensor_multiply_01"))


@pytest.mark.gpu
def test_replay_tensor_subtract_01(hip):
    import ocean_gpu as ocean
    device, out = ocean.gpu[0], []
    a = ocean.asTensor([True, True, False], device)
    out += [a.clone(), -a, a - True]
    a -= True
    out.append(a.clone())
    for dtype, three in ((ocean.int8, 3), (ocean.float, 3.0)):
        a = ocean.asTensor([-2, -1, 0, 1, 2], dtype, device)
        out += [a.clone(), -a, a - three]
        a -= 3
        out.append(a.clone())
    assert_printed(out, gpu_part("tensor_subtract_01"))


@pytest.mark.gpu
def test_replay_tensor_divide_01(hip):
    import ocean_gpu as ocean
    device, out = ocean.gpu[0], []
    a = ocean.asTensor([True, True, False], device)
    out += [a.clone(), a / True]
    a /= [True, False, True]
    out.append(a.clone())
    for dtype, three in ((ocean.int8, 3), (ocean.float, 3.0)):
        a = ocean.asTensor([-10, -5, 0, 4, 6], dtype, device)
        out += [a.clone(), a / three]
        a /= 3
        out.append(a.clone())
    assert_printed(out, gpu_part("tensor_divide_01"), decimals=5)


@pytest.mark.gpu
def test_replay_ocean_gemm_01(hip):
    import ocean_gpu as ocean
    device = ocean.gpu[0]
    a = ocean.arange(9, ocean.cfloat, device).reshape([3, 3])
    b = ocean.arange(9, ocean.cfloat, device).reshape([3, 3])
    alpha = ocean.asTensor([1.0, 2j, 1 + 2j], ocean.chalf, device).reshape([1, 1, 3])
    c = ocean.gemm(alpha, a, b)
    assert c.footer() == "<tensor.complex-float of size 3x3x3 on gpu0>"
    assert alpha.footer() == "<tensor.complex-half of size 1x1x3 on gpu0>"
    assert_printed([a, alpha, c], gpu_part("ocean_gemm_01"))


@pytest.mark.gpu
def test_operators_follow_the_reference_mapping(hip):
    """pyOcean_tensor.c:303-335: * is mtimes, @ the elementwise product, the in-place forms keep the destination's type."""
    import ocean_gpu as ocean
    device = ocean.gpu[0]
    rng = np.random.default_rng(11)
    A, B = rng.standard_normal((4, 3)), rng.standard_normal((4, 3))          # numpy (4, 3) = Ocean 3 x 4
    a, b = device(A), device(B)
    back = lambda t: t.asnumpy()
    assert np.array_equal(back(a + b), A + B) and np.array_equal(back(a - b), A - B) and np.array_equal(back(a / b), A / B)
    assert np.array_equal(back(a @ b), A * B)
    assert np.allclose(back(a.T * b), B @ A.T, rtol=1e-13)          # Ocean (4x3)*(3x4) = 4x4, seen through reversed numpy axes
    assert np.array_equal(back(2 * a), 2 * A) and np.array_equal(back(a * 2), 2 * A) and np.array_equal(back(1 - a), 1 - A)
    assert np.array_equal(back(-a), -A) and np.array_equal(back(a < b), A < B) and np.array_equal(back(a == a), A == A)
    assert (a + 1).dtype == ocean.double and (device(A.astype(np.float32)) + 1.5).dtype == ocean.float
    i = device(np.arange(-4, 4, dtype=np.int16))
    assert np.array_equal(back(i % 3), np.arange(-4, 4) % 3) and np.array_equal(back(i // 3), np.arange(-4, 4) // 3)
    assert np.array_equal(back(i & 5), np.arange(-4, 4) & 5) and np.array_equal(back(~i), ~np.arange(-4, 4, dtype=np.int16))
    assert np.array_equal(back(i << 2), np.arange(-4, 4, dtype=np.int16) << 2) and (i << 2).dtype == ocean.int16
    i += 1.0                                                              # stays int16
    assert i.dtype == ocean.int16 and np.array_equal(back(i), np.arange(-3, 5))
    # views and reductions
    assert np.array_equal(back(a[1:3, ::2]), A[::2, 1:3]) and np.array_equal(back(a.T), A.T)
    assert np.isclose(a.sum(), A.sum(), rtol=1e-13) and np.isclose(a.norm(), np.linalg.norm(A), rtol=1e-13) and a.maximum() == A.max()
    assert np.allclose(back(a.sum(0)), A.sum(axis=1), rtol=1e-13) and list(a.sum(0).size) == [4]


def all_items(name):
    return RF.parse_ref(open(os.path.join(REFDIR, name + ".ref")).read())


def printed_tensors(name):
    return [it for it in all_items(name) if isinstance(it, RF.RefTensor)]


def printed_scalars(name):
    return [v for it in all_items(name) if isinstance(it, tuple) and it[0] == "scalars" for v in it[1]]


BITWISE = {"and": ("bitwiseAnd", lambda a, b: a & b, [1, 2, 3, 7, 127]), "or": ("bitwiseOr", lambda a, b: a | b, [0, 2, 3, 7, 127]),
           "xor": ("bitwiseXor", lambda a, b: a ^ b, [0, 2, 3, 7, 127])}


@pytest.mark.gpu
@pytest.mark.parametrize("which", ["and", "or", "xor"])
def test_replay_ocean_bitwise_01(hip, which):
    """examples/python/gpu/tensors/ocean_and_01, ocean_or_01, ocean_xor_01: a row of five against a column of six, through the
    module function, the operator and the module function with a destination."""
    import ocean_gpu as ocean
    fname, operator, v1 = BITWISE[which]
    device, out = ocean.gpu[0], []
    v2 = [0, 1, 2, 4, 8, 15]
    for dtype in (ocean.bool, ocean.int8, ocean.uint8, ocean.int32):
        a1 = ocean.asTensor(v1, "r", dtype, device)
        a2 = ocean.asTensor(v2, dtype, device).reshape([len(v2), 1])
        r = ocean.tensor([len(v2), len(v1)], dtype, device)
        out += [a1, a2, getattr(ocean, fname)(a1, a2), operator(a1, a2)]
        getattr(ocean, fname)(a1, a2, r)
        out.append(r)
    assert_printed(out, printed_tensors("ocean_%s_01" % which))


@pytest.mark.gpu
def test_replay_ocean_not_01(hip):
    import ocean_gpu as ocean
    device, out = ocean.gpu[0], []
    for dtype in (ocean.bool, ocean.int8, ocean.uint8):
        a = ocean.asTensor([0, 1, -1], dtype, device)
        out += [a, ocean.bitwiseNot(a), ~a, ocean.logicalNot(a)]
        r = ocean.tensor(3, dtype, device)
        ocean.bitwiseNot(a, r)
        out.append(r.clone())
        ocean.logicalNot(a, r)
        out.append(r.clone())
    assert_printed(out, printed_tensors("ocean_not_01"))


@pytest.mark.gpu
@pytest.mark.parametrize("direction", [1, 2])
def test_replay_ocean_bitshift(hip, direction):
    """ocean_bitshift_01 (<<) and ocean_bitshift_02 (>>): a row of four shifted by a column of six counts"""
    import ocean_gpu as ocean
    device, out = ocean.gpu[0], []
    for dtype in (ocean.bool, ocean.int8, ocean.uint8, ocean.uint32):
        a = ocean.asTensor([0, 1, 2, 9], "r", dtype, device)
        b = ocean.asTensor([0, 1, 2, 4, 6, 8], ocean.uint8, device)
        r = ocean.tensor([6, 4], dtype, device)
        out += [a.clone(), b, (a << b) if direction == 1 else (a >> b)]
        (ocean.bitshiftLeft if direction == 1 else ocean.bitshiftRight)(a, b, r)
        out.append(r)
        if direction == 1:
            a <<= 1
        else:
            a >>= 1
        out.append(a)
    assert_printed(out, printed_tensors("ocean_bitshift_0%d" % direction))


@pytest.mark.gpu
def test_replay_ocean_power_01_and_02(hip):
    """Scalars and lists as bases and exponents: the result types follow pyOceanCore_intrnl_power (an integer tensor to an
    integer scalar stays in its type, 2 ** tensor is int64, 2.0 ** tensor double, tensor ** 0.5 the smallest float type)."""
    import ocean_gpu as ocean
    device, out = ocean.gpu[0], []
    for dtype in (ocean.int8, ocean.int32, ocean.float, ocean.cfloat):
        out += [ocean.asTensor([1, 2, 3, 4], dtype, device) ** 2, 2 ** ocean.asTensor([1, 2, 3, 4], dtype, device),
                ocean.asTensor([1, 2, 3, 4], dtype, device) ** 0.5, 2.0 ** ocean.asTensor([1, 2, 3, 4], dtype, device)]
    assert_printed(out, printed_tensors("ocean_power_01"), decimals=5)
    out = []
    for dtype in (ocean.int8, ocean.int32, ocean.float, ocean.cfloat):
        out += [ocean.asTensor([1, 2, 3, 4], "r", dtype, device) ** [0, 1, 2], device([1, 2, 3]) ** ocean.asTensor([1, 2, 3, 4], "r", dtype, device),
                ocean.asTensor([1, 2, 3, 4], "r", dtype, device) ** [0, 0.5, 1], device([1.0, 2.0, 3.0]) ** ocean.asTensor([1, 2, 3, 4], "r", dtype, device)]
    assert_printed(out, printed_tensors("ocean_power_02"), decimals=5)


@pytest.mark.gpu
def test_replay_ocean_power_03(hip):
    import ocean_gpu as ocean
    device, out = ocean.gpu[0], []
    a = ocean.asTensor([1, 2, 3, 4], "r", ocean.float, device)
    b = ocean.asTensor([0, 0.5, 1, 2], ocean.float, device)
    out += [a ** b, pow(a, b), ocean.power(a, b)]
    for dtype in (ocean.float, ocean.cdouble, ocean.int16):
        c = ocean.tensor([4, 4], dtype, device)
        ocean.power(a, b, c)
        out.append(c)
    a **= ocean.asTensor([1, 1, 1, 0.5], "r", ocean.float, device)
    out.append(a)
    assert_printed(out, printed_tensors("ocean_power_03"), decimals=5)
    with pytest.raises(Exception, match="The modulo parameter in power is not supported"):
        pow(a, b, 3)


@pytest.mark.gpu
def test_replay_full_reductions(hip):
    """ocean_sum_01 / 02, ocean_sumabs_01, ocean_all_01, ocean_maximumabs_01 / 02: full reductions to scalars"""
    import ocean_gpu as ocean
    gpu = ocean.gpu[0]
    assert [ocean.sum(gpu([]))] == printed_scalars("ocean_sum_01")
    got = [ocean.sum(gpu([1, 2, 3])), ocean.sum(ocean.asTensor([True, False, True], ocean.bool, gpu))]
    got += [ocean.sum(ocean.asTensor([1, 2, 5], dtype, gpu)) for dtype in (ocean.int8, ocean.int16, ocean.half, ocean.chalf, ocean.cdouble)]
    assert got == printed_scalars("ocean_sum_02")
    got = [ocean.sumAbs(gpu([1, -2, 3]))] + [ocean.sumAbs(ocean.asTensor([1, -2, 5], dtype, gpu)) for dtype in (ocean.int8, ocean.int16, ocean.half, ocean.chalf, ocean.cdouble)]
    assert got == printed_scalars("ocean_sumabs_01")
    assert [ocean.all(ocean.asTensor([1, 1, 1, 1, 0, 1], gpu))] == printed_scalars("ocean_all_01")
    A = ocean.asTensor([[1 + 2j, 3 + 1j], [1, 2 + 2j]], gpu)
    assert_printed([A], printed_tensors("ocean_maximumabs_01"))
    assert abs(ocean.maximumAbs(A) - printed_scalars("ocean_maximumabs_01")[0]) < 1e-5
    with pytest.raises(Exception):
        ocean.maximumAbs(gpu([[]]))
    want = printed_scalars("ocean_maximumabs_02")
    got = []
    for dtype in (ocean.bool, ocean.int8, ocean.uint8, ocean.int32, ocean.half, ocean.float, ocean.chalf, ocean.double):
        A = ocean.asTensor([1, -3, 2], dtype, gpu)
        B = A.clone()
        got += [ocean.maximumAbs(A), ocean.maximumAbs(B), ocean.maximumAbs(ocean.asTensor([A, B])), ocean.minimumAbs(ocean.asTensor([-1, -3, 2], dtype, gpu))]
    assert len(got) == len(want) and all(abs(g - w) < 1e-4 for g, w in zip(got, want)), (got, want)


@pytest.mark.gpu
def test_replay_ocean_sign_01_and_fabs_02(hip):
    import ocean_gpu as ocean
    device, out = ocean.gpu[0], []
    values = [-1, 0, 1, 1 + 2j, 0 + 2j, 0 - 2j, 0 + 0j]
    for dtype in (ocean.int8, ocean.uint8, ocean.int32, ocean.float, ocean.chalf, ocean.cfloat):
        a = ocean.asTensor(values, dtype, device)
        b = ocean.tensor(len(values), ocean.int8, device)
        out += [a, ocean.sign(a)]
        ocean.sign(a, b)
        out.append(b)
    assert_printed(out, printed_tensors("ocean_sign_01"), decimals=5)
    out = []
    for fn in (ocean.fabs, ocean.absolute):
        for dtype, otype in zip((ocean.int8, ocean.int16, ocean.float, ocean.chalf, ocean.cdouble), (ocean.float, ocean.uint8, ocean.double, ocean.int32, ocean.chalf)):
            a = ocean.asTensor([-3 - 4j], dtype, device)
            b = ocean.tensor([1], otype, device)
            fn(a, b)
            out.append(b)
    assert_printed(out, printed_tensors("ocean_fabs_02"), decimals=5)


@pytest.mark.gpu
def test_replay_ocean_min_01(hip):
    import ocean_gpu as ocean
    device, out = ocean.gpu[0], []
    v1 = [1, 2, 3, 1, ocean.nan, 2 + 3j, 4 - 5j]
    v2 = [3, 2, 1, 1, 1, 2 + 2j, 4 - 6j]
    for dtype in (ocean.int8, ocean.uint8, ocean.float, ocean.chalf, ocean.cdouble):
        a1, a2 = ocean.asTensor(v1, dtype, device), ocean.asTensor(v2, dtype, device)
        r1, r2 = ocean.tensor([len(v1)], dtype, device), ocean.tensor([len(v1)], ocean.cfloat, device)
        out += [a1, a2, ocean.min(a1, a2), ocean.min(a2, a1), ocean.max(a1, a2), ocean.fmin(a1, a2), ocean.fmin(a2, a1), ocean.fmax(a1, a2)]
        ocean.fmin(a1, a2, r1)
        ocean.fmin(a1, a2, r2)
        out += [r1, r2]
    assert_printed(out, printed_tensors("ocean_min_01"), decimals=5)


@pytest.mark.gpu
def test_replay_ocean_logical_01(hip):
    """Logical operations into a bool tensor on the device and into a byte-swapped int16 tensor on the host"""
    import ocean_gpu as ocean
    device, out = ocean.gpu[0], []
    for dtype in (ocean.bool, ocean.int32, ocean.uint32, ocean.float, ocean.cfloat):
        a1, a2 = ocean.asTensor([0, 0, 1, 1], dtype, device), ocean.asTensor([0, 1, 0, 1], dtype, device)
        r1 = ocean.tensor([4], ocean.bool, device)
        r2 = ocean.tensor([4], ocean.int16, ocean.cpu)
        r2.byteswap()
        out += [a1, a2]
        for fn in (ocean.logicalAnd, ocean.logicalOr, ocean.logicalXor):
            fn(a1, a2, r1)
            fn(a1, a2, r2)
            out += [fn(a1, a2), r1.clone(), r2.clone()]
    want = printed_tensors("ocean_logical_01")
    assert [t.byteswapped for t in out] == [w.byteswapped for w in want]
    assert_printed(out, want)


@pytest.mark.gpu
def test_replay_ocean_axis_reduce_04_and_axis_norm2_01(hip):
    import ocean_gpu as ocean
    gpu, out = ocean.gpu[0], []
    A = ocean.arange(2 * 3 * 4, ocean.float, gpu).reshape([2, 3, 4])
    out += [A.clone(), ocean.norm2(A, [0, 1])]
    A.fliplr(True)
    out += [ocean.minimum(A, 0), ocean.maximum(A, 2, True)]
    B = ocean.tensor([4], ocean.half, gpu)
    ocean.norm(A, 3, [0, 1], B)
    out += [B, ocean.norm(A, 3, [0, 1])]
    assert_printed(out, printed_tensors("ocean_axis_reduce_04"), decimals=4)
    a = ocean.arange(64 * 65, ocean.double, gpu).reshape(64, 65).T
    b = np.arange(64 * 65, dtype=np.float64).reshape(65, 64)               # b[i1][i0] of the 64 x 65 tensor before .T
    want = printed_tensors("tensor_axis_norm2_01")
    got = [a, ocean.norm(a, 2, 0), None, ocean.norm(a, 2, 1), None]
    assert got[0].footer() == "<tensor.double of size 65x64 on gpu0>" and list(want[0].shape) == [65, 64]
    n0, n1 = got[1].asnumpy(), got[3].asnumpy()
    assert list(got[1].size) == list(want[1].shape) == [64] and list(got[3].size) == list(want[3].shape) == [65]
    assert np.allclose(n0, np.linalg.norm(b, axis=0), rtol=1e-12) and np.allclose(n1, np.linalg.norm(b, axis=1), rtol=1e-12)
    assert np.isclose(ocean.norm(a, 2, [0, 1]).asscalar(), np.linalg.norm(np.arange(64 * 65.0)), rtol=1e-12)


@pytest.mark.gpu
def test_replay_tensor_copy_and_fill_examples(hip):
    """tensor_copy_01 (zero strides), _02 (scalars), _03 / _05 / _06 (host tensors, byte order), _04 (broadcast source into a
    swapped half / double / int8 host tensor), _07 (transposed and flipped views), _08 (empty), tensor_fill_01,
    tensor_fillnan_01, tensor_clone_01, tensor_dtype_cast_01 (the tensor parts), ocean_unary_01, ocean_gemm_10 / 11"""
    import ocean_gpu as ocean
    gpu, cpu = ocean.gpu[0], ocean.cpu
    # ---- tensor_copy_01: tensors whose strides are zero along one or both dimensions
    a, b = ocean.tensor([2, 6], [0, 0], gpu), ocean.tensor([2, 6], [0, 1], gpu)
    c, d = ocean.tensor([2, 2, 3], [1, 0, 0], gpu), ocean.tensor([2, 6], [0, 0], gpu)
    for t, v in ((a, 1), (b, 2), (c, 3), (d, 4)):
        t.fill(v)
    out = [a.clone(), b.clone(), c.clone(), d.clone()]
    b.copy(a); c.copy(a); d.copy(a)
    out += [a, b, c, d]
    want = printed_tensors("tensor_copy_01")
    assert_printed(out, want[:8])
    # ---- tensor_copy_02: tensors without dimensions
    a = gpu(12345)
    b = ocean.tensor([], ocean.float, gpu)
    b.copy(a)
    out = [b.clone()]
    b = ocean.double(b); out.append(b.clone())
    b = ocean.cdouble(b); out.append(b.clone())
    b.copy(54321); out.append(b.clone())
    b.copy(gpu(1.2345)); out.append(b.clone())
    assert_printed(out, printed_tensors("tensor_copy_02"), decimals=4)
    # ---- tensor_copy_03: a byte-swapped host tensor into host and device tensors
    a = ocean.arange(18, cpu).reshape([3, 6])
    b, c = ocean.tensor([3, 6], cpu), ocean.tensor([3, 6], gpu)
    a.byteswap(); b.fill(1); c.fill(2)
    out = [a.clone(), b.clone(), c.clone()]
    b.copy(a); c.copy(a)
    out += [a, b, c, ocean.double(a), gpu(a)]
    want = printed_tensors("tensor_copy_03")
    assert_printed(out, want)
    # ---- tensor_copy_04: a broadcast device tensor into host tensors of other types and byte orders
    a = ocean.arange(4, ocean.float, gpu).broadcastTo([4, 3])
    out = [a]
    for dtype, swapped in ((ocean.half, True), (ocean.double, True), (ocean.int8, False)):
        b = ocean.tensor([12], dtype, cpu)
        if swapped:
            b.byteswap()
        b.copy(a.clone().reshape([12]))
        out.append(b.reshape([4, 3]))
    b = ocean.tensor([12], ocean.double, cpu)
    b.copy(a.clone().reshape([12]))
    out += [b.reshape([4, 3]), b.reshape([3, 4]), b.reshape([2, 6]), b.reshape([6, 2])]
    assert_printed(out, printed_tensors("tensor_copy_04"))
    # ---- tensor_copy_05: a host tensor with a zero stride into a device tensor
    a, b = ocean.tensor([3, 6], [0, 1], ocean.double, cpu), ocean.tensor([3, 6], ocean.float, gpu)
    a.fill(1); b.fill(2)
    out = [a.clone(), b.clone()]
    b.copy(a)
    out += [a, b]
    assert_printed(out, printed_tensors("tensor_copy_05"))
    # ---- tensor_copy_07: transposed, flipped and swapped views of a device tensor
    A = ocean.arange([15], ocean.float, gpu).reshape([3, 5])
    X = cpu(A.T)
    out = [A, A.T, X]
    assert list(A.T.strides) == [12, 4] and list(X.strides) == [4, 20]
    B = A.flipAxis(0)
    out += [B, B.T]
    B = A.swapAxes(0, 1)
    out += [B, B.T, B]
    Cc = ocean.zeros(B.size, B.dtype, B.device)
    assert list(B.strides) == [12, 4] and list(Cc.strides) == [4, 20]
    Cc.copy(B)
    out += [Cc, Cc.T]
    assert_printed(out, printed_tensors("tensor_copy_07"))
    # ---- tensor_copy_08
    a = ocean.tensor([0], gpu)
    assert a.footer() == "<empty tensor.float of size 0 on gpu0>"
    # ---- tensor_fill_01, tensor_fillnan_01
    out = []
    for dtype in (ocean.int16, ocean.float, ocean.chalf):
        a = ocean.tensor([], dtype, gpu)
        a.fill(24); out.append(a.clone())
        a.fill(36); out.append(a.clone())
    assert_printed(out, printed_tensors("tensor_fill_01"))
    a = ocean.asTensor([ocean.nan, 3, 4, ocean.nan], ocean.float, gpu)
    a.fillNaN(ocean.inf)
    # (the reference's GPU output for this example records a defect of its GPU kernel, which fills every element; the
    #  expected values are those of the same example on the CPU device)
    ref = printed_tensors("tensor_fillnan_01_cpu")[0]
    assert a.dtype == ref.dtype and list(a.size) == list(ref.shape) and np.array_equal(a.asnumpy().astype(np.float64), ref.values)
    # ---- tensor_clone_01
    a = ocean.asTensor([[1, 2, 3], [4, 5, 6]], "r", ocean.float)
    out = [a.clone(), a.clone(gpu)]
    a = ocean.asTensor([[2, 3, 4], [5, 6, 7]], "r", ocean.double, gpu)
    out += [a.clone(), a.clone(cpu)]
    assert_printed(out, printed_tensors("tensor_clone_01"))
    # ---- tensor_dtype_cast_01: the tensor and list casts
    A = ocean.asTensor([1, 2, 3], ocean.float, gpu)
    want = printed_tensors("tensor_dtype_cast_01")
    assert_printed([ocean.int8(A)], want[:1])
    h = ocean.half([[1, 2, 3], [4, 5, 6.]])
    assert h.footer() == "<tensor.half of size 3x2 on cpu>" and list(want[2].shape) == [3, 2] and want[2].dtype == ocean.half
    assert np.array_equal(h.asnumpy().T.astype(np.float64), want[2].values)
    # ---- ocean_unary_01: square between devices, types and byte orders
    out = []
    a, b = ocean.asTensor([1, 2, 3], ocean.int8, cpu), ocean.tensor([3], ocean.int16, gpu)
    ocean.square(gpu(a), b); out.append(b.clone())
    a.byteswap(); b.fill(0)
    ocean.square(gpu(a), b); out.append(b.clone())
    a, b = ocean.asTensor([1, 2, 3], ocean.int8, gpu), ocean.tensor([3], ocean.int16, cpu)
    ocean.square(a, b); out.append(b.clone())
    b.fill(0); b.byteswap()
    ocean.square(a, b); out.append(b.clone())
    want = printed_tensors("ocean_unary_01")
    assert [t.byteswapped for t in out] == [w.byteswapped for w in want]
    assert_printed(out, want)
    # ---- ocean_gemm_10 / 11: products with an empty dimension
    c = ocean.zeros([0, 5], ocean.float, gpu) * ocean.ones([5], ocean.float, gpu)
    assert c.footer() == open(os.path.join(REFDIR, "ocean_gemm_10.ref")).read().strip().splitlines()[-1]
    c = ocean.zeros([5, 0], ocean.float, gpu) * ocean.ones([0, 5], ocean.float, gpu)
    assert_printed([c], printed_tensors("ocean_gemm_11"))


def test_python_scalars_are_typed_as_the_reference_types_them():
    """OcScalar_getCommonType (src/core/interface/scalar_itf.c:736-781): a float scalar takes the smallest float type whose
    RANGE holds it, an integer next to a float tensor half up to 2048 and float up to 2^24, integers next to integer
    tensors the smallest integer type, signed when the tensor is signed or the value is not positive."""
    import ocean_gpu as ocean
    T = ocean._scalar_dtype
    assert T(0.1, ocean.float) == ocean.float and T(0.1, ocean.half) == ocean.half and T(0.1, ocean.double) == ocean.double
    assert T(1000, ocean.half) == ocean.half and T(2048, ocean.half) == ocean.half and T(2049, ocean.half) == ocean.float
    assert T(100000, ocean.float) == ocean.float and T(1 << 24, ocean.half) == ocean.float and T((1 << 24) + 1, ocean.float) == ocean.double
    assert T(70000.0, ocean.half) == ocean.float and T(1e39, ocean.float) == ocean.double and T(float("inf"), ocean.half) == ocean.half
    assert T(1000, ocean.int8) == ocean.int16 and T(3, ocean.int8) == ocean.int8 and T(-1, ocean.uint8) == ocean.int16
    assert T(200, ocean.uint8) == ocean.uint8 and T(200, ocean.int8) == ocean.int16 and T(300, ocean.uint8) == ocean.uint16
    assert T(1 + 2j, ocean.float) == ocean.cfloat and T(1 + 2j, ocean.half) == ocean.chalf and T(1e5 + 0j, ocean.half) == ocean.cfloat
    assert T(0.5, ocean.int8) == ocean.half and T(0.5, ocean.int32) == ocean.double
    assert T(2, ocean.cfloat) == ocean.cfloat and T(1 << 40, ocean.int8) == ocean.int64
    # a Python bool is no weak scalar (pyOcean_convert.c:79-90): it is a bool tensor, whatever it meets
    assert not ocean._is_weak_scalar(True) and ocean._is_weak_scalar(1) and not ocean._is_weak_scalar(np.float32(1))
    # nested lists: innermost lists run along dimension 0 unless the order is 'r'
    a = ocean.asTensor([[1, 2, 3], [4, 5, 6]])
    assert list(a.size) == [3, 2] and a.dtype == ocean.int64 and a[2, 1].asscalar() == 6 and a[0, 1].asscalar() == 4
    b = ocean.asTensor([[1, 2, 3], [4, 5, 6]], "r", ocean.float)
    assert list(b.size) == [2, 3] and b[1, 2].asscalar() == 6.0 and b[1, 0].asscalar() == 4.0
    assert list(ocean.asTensor([0, 1, 2, 9], "r", ocean.int8).size) == [1, 4]
    # integer indices remove their dimension, slices keep it
    assert list(b[0].size) == [3] and list(b[:, 1].size) == [2] and list(b[0:1].size) == [1, 3] and b[1, 2].ndims == 0
    with pytest.raises(IndexError):
        b[2, 0]
