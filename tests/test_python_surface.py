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
        assert t.footer() == "<tensor.%s of size %s on %s>" % (OCEAN_NAME[ref.dtype], "x".join(map(str, ref.shape)), ref.device)
        got = t.asnumpy()
        got = got.transpose(*range(got.ndim)[::-1])          # Ocean index order A[i0, i1, ...]
        if decimals is not None and got.dtype.kind == "f":
            assert np.allclose(got.astype(np.float64), ref.values, rtol=0, atol=0.51 * 10.0 ** -decimals), (k, got, ref.values)
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
