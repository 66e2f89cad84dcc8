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
        assert host.shape_of(t) == list(a.shape[::-1])
        back = host.to_numpy(t)
        assert np.array_equal(back.view(a.dtype) if a.dtype == np.bool_ else back, a)
        host.lib.OcDecrefTensor(t)
    h = ocean_gpu.gpu[0](np.arange(5, dtype=np.float16))
    assert h.contents.dtype == host.HALF and np.array_equal(host.to_numpy(h).view(np.float16), np.arange(5, dtype=np.float16))
    host.lib.OcDecrefTensor(h)
