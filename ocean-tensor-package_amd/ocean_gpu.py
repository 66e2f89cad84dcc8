"""Python surface of the GPU device module: what `import pyOcean_gpu` adds to Ocean
(interfaces/python/pyOcean/gpu/pyOcean_gpu.c:62-117, pyOcean_device_gpu.c:65-165).

Importing the module initialises the GPU package (OcInitGPU), and the module then holds
  deviceGPU   the device type, with the read-only properties of pyOcean_device_gpu.c:65-94 under the same
              names; the fields of cudaDeviceProp are filled from the HIP device properties (warpSize is the
              wavefront size, 64; multiProcessorCount the number of compute units; sharedMemPerBlock the LDS
              of a workgroup; major.minor the gfx version, 9.5 for gfx950)
  gpu         the tuple of devices, gpu[0] ... gpu[n-1]; empty on a machine without a GPU
A device is callable on a numpy array, as `ocean.gpu[0](tensor)` is: the data moves to the device and the
result is a tensor of the host layer (ocean_host), which `ocean_host.to_numpy` brings back.
"""
import ctypes as C

import ocean_hip as _hip
import ocean_host as _host

_host.lib.OcDeviceGPUByIndex.restype = C.c_void_p
_host.lib.OcDeviceGPUByIndex.argtypes = [C.c_int]
_host.lib.OcDeviceGPU_properties.restype = C.c_int
_host.lib.OcDeviceGPU_properties.argtypes = [C.c_void_p, C.c_void_p]
_host.lib.OcDeviceGPU_peerAccess.restype = C.c_int
_host.lib.OcDeviceGPU_peerAccess.argtypes = [C.c_int, C.c_int]


class deviceGPU(object):
    """One GPU of the machine (ocean.deviceGPU)."""

    def __init__(self, index):
        handle = _host.lib.OcDeviceGPUByIndex(index)
        if not handle:
            raise IndexError("GPU device index %d out of range" % index)
        self._handle = handle
        self._index = index

    def _prop(self):
        p = _hip.DeviceProp()
        _host.check(_host.lib.OcDeviceGPU_properties(self._handle, C.byref(p)))
        return p

    # attributes of the device base type
    index = property(lambda self: self._index, doc="device index")
    name = property(lambda self: "gpu%d" % self._index, doc="device name in Ocean")
    type = property(lambda self: "GPU", doc="device type")
    # pyOcean_device_gpu.c:65-94, in the same order
    deviceName = property(lambda self: self._prop().name.decode(), doc="device name")
    totalGlobalMem = property(lambda self: int(self._prop().total_global_mem), doc="total amount of global memory on the device in bytes")
    totalMem = totalGlobalMem
    freeMem = property(lambda self: int(self._prop().free_global_mem), doc="free amount of global memory on the device in bytes")
    sharedMemPerBlock = property(lambda self: int(self._prop().shared_mem_per_block), doc="maximum amount of shared memory available to a thread block")
    regsPerBlock = property(lambda self: self._prop().regs_per_block, doc="maximum number of 32-bit registers available to a thread block")
    warpSize = property(lambda self: self._prop().wavefront_size, doc="warp size in threads")
    memPitch = property(lambda self: int(self._prop().mem_pitch), doc="maximum pitch in bytes allows by the memory copy functions")
    maxThreadsPerBlock = property(lambda self: self._prop().max_threads_per_block, doc="maximum number of threads per block")
    maxThreadsDim = property(lambda self: list(self._prop().max_threads_dim), doc="maximum size of each dimension of a block")
    maxGridSize = property(lambda self: list(self._prop().max_grid_size), doc="maximum size of each dimension of a grid")
    totalConstMem = property(lambda self: int(self._prop().total_const_mem), doc="total amount of constant memory available on the device in bytes")
    major = property(lambda self: self._prop().major, doc="major revision number")
    minor = property(lambda self: self._prop().minor, doc="minor revision number")
    version = property(lambda self: "%d.%d" % (self._prop().major, self._prop().minor), doc="revision number")
    clockRate = property(lambda self: self._prop().clock_rate_khz / 1000.0, doc="clock frequency in megahertz")
    deviceOverlap = property(lambda self: self._prop().async_engine_count > 0, doc="True if the device can concurrently copy memory, False if not")
    multiProcessorCount = property(lambda self: self._prop().multiprocessor_count, doc="number of multiprocessors on the device")
    kernelExecTimeoutEnabled = property(lambda self: bool(self._prop().kernel_exec_timeout_enabled), doc="True if there is a run time limit for kernels, False if not")
    integrated = property(lambda self: bool(self._prop().integrated), doc="True if the device is integrated, False if not")
    canMapHostMemory = property(lambda self: bool(self._prop().can_map_host_memory), doc="True if the device can map host memory, False if not")
    computeMode = property(lambda self: self._prop().compute_mode, doc="compute mode that the device is currently in")
    concurrentKernels = property(lambda self: bool(self._prop().concurrent_kernels), doc="True if the device supports concurrent kernels, False if not")
    ECCEnabled = property(lambda self: bool(self._prop().ecc_enabled), doc="True if the device has ECC support turned on, False if not")
    pciBusID = property(lambda self: self._prop().pci_bus_id, doc="PCI bus identifier of the device")
    pciDeviceID = property(lambda self: self._prop().pci_device_id, doc="PCI device identifier of the device")
    tccDriver = property(lambda self: bool(self._prop().tcc_driver), doc="True if the device is using a TCC driver, False if not")
    # beyond the reference's list: what identifies the code object target
    archName = property(lambda self: self._prop().arch.decode(), doc="architecture name of the device, e.g. gfx950:sramecc+:xnack-")

    def peerAccess(self, other):
        """True if this device can access the memory of `other` directly (device_gpu.c:447-454)."""
        return bool(_host.lib.OcDeviceGPU_peerAccess(self._index, other.index))

    def __call__(self, array, dtype=None):
        """Copy of a numpy array on this device, as a tensor of the host layer."""
        import numpy as np
        a = np.asarray(array)
        if dtype is None:
            dtype = _host.dtype_of(a.dtype)
        return _host.from_numpy(a, dtype, device=self._handle)

    def __repr__(self):
        return "<device '%s'>" % self.name


_host.check(_host.lib.OcInitGPU())
gpu = tuple(deviceGPU(i) for i in range(_host.lib.OcDeviceGPUCount()))
