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
import builtins as _py
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
    # pyOcean_device_gpu.c:199-206: refreshed through OcDeviceGPU_updateProperties, then read from the device object
    freeMem = property(lambda self: int(_host.gpu_public_properties(self._handle, update=True).freeGlobalMem),
                       doc="free amount of global memory on the device in bytes")
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
    kernelExecTimeoutEnabled = property(lambda self: _py.bool(self._prop().kernel_exec_timeout_enabled), doc="True if there is a run time limit for kernels, False if not")
    integrated = property(lambda self: _py.bool(self._prop().integrated), doc="True if the device is integrated, False if not")
    canMapHostMemory = property(lambda self: _py.bool(self._prop().can_map_host_memory), doc="True if the device can map host memory, False if not")
    computeMode = property(lambda self: self._prop().compute_mode, doc="compute mode that the device is currently in")
    concurrentKernels = property(lambda self: _py.bool(self._prop().concurrent_kernels), doc="True if the device supports concurrent kernels, False if not")
    ECCEnabled = property(lambda self: _py.bool(self._prop().ecc_enabled), doc="True if the device has ECC support turned on, False if not")
    pciBusID = property(lambda self: self._prop().pci_bus_id, doc="PCI bus identifier of the device")
    pciDeviceID = property(lambda self: self._prop().pci_device_id, doc="PCI device identifier of the device")
    tccDriver = property(lambda self: _py.bool(self._prop().tcc_driver), doc="True if the device is using a TCC driver, False if not")
    # beyond the reference's list: what identifies the code object target
    archName = property(lambda self: self._prop().arch.decode(), doc="architecture name of the device, e.g. gfx950:sramecc+:xnack-")

    def peerAccess(self, other):
        """True if this device can access the memory of `other` directly (device_gpu.c:447-454)."""
        return _py.bool(_host.lib.OcDeviceGPU_peerAccess(self._index, other.index))

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


# ---------------------------------------------------------------------------------------------------------------
# Tensors with Ocean's operators (interfaces/python/pyOcean/cpu/pyOcean_tensor.c:295-345, 684-760): every operator
# goes through the front end (type promotion, broadcasting) into the GPU module's function table.
#   +  -  /  //  %  &  |  ^  <<  >>  **   elementwise (add, subtract, divide, floorDivide, mod, bitwise*, bitshift*, power)
#   @        elementwise product (scale)
#   *        mtimes: the product with a scalar, otherwise the matrix product of the first two dimensions
#   comparisons give bool tensors; += and the other in-place forms keep the tensor's type
# ---------------------------------------------------------------------------------------------------------------
import numpy as _np

_DTYPE_NAMES = ["bool", "uint8", "uint16", "uint32", "uint64", "int8", "int16", "int32", "int64", "half", "float", "double",
                "complex-half", "complex-float", "complex-double"]


class dtype(_py.int):
    """An Ocean data type (ocean.int8, ocean.float, ...): its number in Ocean's type list, with a name, and callable as a
    cast -- ocean.float(x) converts a tensor, a nested list or a number (pyOcean_dtype.c: the type objects' call)."""

    def __new__(cls, code):
        return _py.int.__new__(cls, code)

    name = property(lambda self: _DTYPE_NAMES[self])

    def __call__(self, data):
        if isinstance(data, tensor):
            return data.convert(self)
        return asTensor(data, self)

    def __repr__(self):
        return "<dtype '%s'>" % self.name


bool, uint8, uint16, uint32, uint64, int8, int16, int32, int64, half, float, double, chalf, cfloat, cdouble = [dtype(i) for i in range(15)]
nan, inf = _py.float("nan"), _py.float("inf")
_B = _hip.B          # names of the binary block of the table -> index
_U = _hip.U
_R = _hip.R
_host.lib.OcTensor_gemmTensors.argtypes = [_host.TP, _host.TP, C.c_char, _host.TP, C.c_char, _host.TP, C.POINTER(_host.TP)]
_host.lib.OcTensor_ensure.argtypes = [C.POINTER(_host.TP), C.c_int, C.c_void_p]
_host.lib.OcIncrefTensor.restype = _host.TP
_host.lib.OcIncrefTensor.argtypes = [_host.TP]
_host.lib.OcDType_getCommonType.restype = C.c_int
_host.lib.OcTensor_createFromStorage.restype = _host.TP
_host.lib.OcTensor_createFromStorage.argtypes = [C.POINTER(_host.Storage), C.c_int, _host._ss, _host._ss, C.c_ssize_t, C.c_int]
_host.lib.OcTensor_reduceLogical.argtypes = [C.c_int, _host.TP, C.POINTER(C.c_int)]
_host.lib.OcTensor_reduceCount.argtypes = [C.c_int, _host.TP, C.POINTER(C.c_uint64)]


class deviceCPU(object):
    """The host (ocean.cpu). Tensors live there on their way to and from a GPU; this module computes on GPUs only."""
    name, type, index = "cpu", "CPU", 0
    _handle = property(lambda self: _host.cpu_device().value)

    def __call__(self, data, dtype=None):
        if isinstance(data, tensor):
            return data if data.device is self and dtype is None else asTensor(data, dtype, self)
        return asTensor(data, dtype, self)

    def __repr__(self):
        return "<device 'cpu'>"


cpu = deviceCPU()


def _is_weak_scalar(value):
    """pyOcean_isWeakScalar (pyOcean_convert.c:79-90): Python integers, floats and complex numbers adapt their type to the
    tensor they meet; a Python bool and typed scalars (numpy's) are tensors of their own type."""
    return not isinstance(value, (_py.bool, _np.generic)) and isinstance(value, (_py.int, _py.float, _py.complex))


def _scalar_kind(value):
    """Ocean type of the scalar a Python value becomes (pyOcean_getScalar, pyOcean_convert.c:203-258): bool, int64,
    double or complex-double; numpy scalars keep their own type."""
    if isinstance(value, (_py.bool, _np.bool_)):
        return bool
    if isinstance(value, _np.generic):
        return dtype(_host.dtype_of(value.dtype))
    if isinstance(value, _py.int):
        return int64 if value < (1 << 63) else uint64
    if isinstance(value, _py.float):
        return double
    if isinstance(value, _py.complex):
        return cdouble
    raise TypeError("cannot use %r as a tensor operand" % (value,))


def _float_type_of(v):
    """OcDType_getTypeDouble (src/base/dtype.c:417-427): the smallest float type whose RANGE holds the value."""
    if v != v or v in (inf, -inf):
        return half
    v = _py.abs(v)
    if v <= 65504.0:
        return half
    return float if v <= 3.4028234663852886e38 else double


def _scalar_dtype(value, like):
    """Type of the tensor a scalar becomes next to a tensor of type `like`: OcScalar_getCommonType
    (src/core/interface/scalar_itf.c:736-781), the way pyOceanCore_intrnl_add and its siblings use it
    (pyOcean_core.c:200-213). A float value takes the smallest float type whose range holds it, an integer next to a
    float tensor half up to 2048 and float up to 2^24, an integer next to an integer tensor the smallest integer type
    that holds it (signed when the tensor's type is signed or the value is not positive); the result is the common type
    of that and the tensor's type."""
    kind = _scalar_kind(value)
    if kind >= half or like >= half:
        if kind < half:                                               # an integer or bool next to a float tensor
            v = _py.abs(_py.float(value))
            stype = half if v <= 2048 else (float if v <= 16777216 else double)
        elif kind < chalf:
            stype = _float_type_of(_py.float(value))
        else:
            c = _py.complex(value)
            stype = dtype(_py.max(_float_type_of(c.real), _float_type_of(c.imag)) + 3)
    elif kind >= int8:
        v = _py.int(value)
        if v <= 0 or like >= int8:
            stype = next(t for t, bits in ((int8, 8), (int16, 16), (int32, 32), (int64, 64)) if -(1 << (bits - 1)) <= v < (1 << (bits - 1)))
        else:
            stype = next(t for t, bits in ((uint8, 8), (uint16, 16), (uint32, 32), (uint64, 64)) if v < (1 << bits))
    else:
        v = _py.int(value)
        stype = next(t for t, bits in ((uint8, 8), (uint16, 16), (uint32, 32), (uint64, 64)) if v < (1 << bits))
    return dtype(_host.lib.OcDType_getCommonType(stype, like))


def _host_array(value, dt):
    """numpy array holding `value` in the storage type of Ocean type `dt` (half travels as its bit pattern)."""
    a = _np.asarray(value)
    if dt == half:
        return a.astype(_np.float16).view(_np.uint16)
    if dt == chalf:
        c = _np.asarray(a, dtype=_np.complex64)
        out = _np.empty(c.shape + (2,), _np.uint16)
        out[..., 0] = c.real.astype(_np.float16).view(_np.uint16); out[..., 1] = c.imag.astype(_np.float16).view(_np.uint16)
        return out
    if dt == bool:
        return (a != 0).view(_np.uint8)
    if a.dtype.kind == "c" and dt < chalf:
        a = a.real                                                    # complex to real: the imaginary part is dropped
    if a.dtype.kind == "f" and dt < half:
        with _np.errstate(invalid="ignore"):
            return a.astype(_np.int64).astype(_host.NUMPY[dt])
    return a.astype(_host.NUMPY[dt])


def _device_handle(device):
    return device._handle if device is not None else _host.cpu_device().value


def _host_ndarray(t):
    """numpy view (no copy) of the memory of a HOST tensor: axes are the tensor's dimensions reversed, strides and byte
    order as stored; half is seen as uint16, complex-half as uint16 with a last axis of two. The compute module of this
    build is the GPU's: what a host tensor needs on its own (filling, reading, converting copies between host tensors)
    is done here with numpy."""
    c = t._h.contents
    dt = dtype(c.dtype)
    es = _hip.TYPE_SIZE[dt]
    size = [c.size[i] for i in range(c.ndims)]
    strides = [c.strides[i] for i in range(c.ndims)]
    base = _np.dtype(_np.uint16 if dt in (half, chalf) else _host.NUMPY[dt])
    if t.byteswapped:
        base = base.newbyteorder()
    # the lowest and highest byte the view touches, to wrap exactly that range
    lo = _py.sum((n - 1) * st for n, st in zip(size, strides) if st < 0 and n > 0)
    hi = _py.sum((n - 1) * st for n, st in zip(size, strides) if st > 0 and n > 0) + es
    if c.nelem == 0:
        return _np.zeros(size[::-1] + ([2] if dt == chalf else []), base)
    raw = (C.c_uint8 * (hi - lo)).from_address(_host.data_address(t._h) + lo)
    if dt == chalf:
        return _np.ndarray(shape=size[::-1] + [2], dtype=base, buffer=raw, offset=-lo, strides=strides[::-1] + [2])
    return _np.ndarray(shape=size[::-1], dtype=base, buffer=raw, offset=-lo, strides=strides[::-1])


def _host_values(t):
    """The values of a host tensor as a native numpy array (numpy axes reversed): bool as bool, half as float16,
    complex-half as complex64."""
    v = _host_ndarray(t)
    dt = t.dtype
    if dt == bool:
        return v != 0
    if dt == half:
        return v.astype(_np.uint16).view(_np.float16)
    if dt == chalf:
        f = v.astype(_np.uint16).view(_np.float16).astype(_np.float32)
        return (f[..., 0] + 1j * f[..., 1]).astype(_np.complex64)
    return v.astype(v.dtype.newbyteorder("=")) if t.byteswapped else v.copy()


def _host_store(t, values):
    """Writes values (a numpy array broadcastable to the tensor, numpy axes reversed) into a host tensor, converted to its
    type and byte order."""
    v = _host_ndarray(t)
    dt = t.dtype
    if v.size == 0:
        return
    a = _host_array(_np.broadcast_to(values, v.shape[:-1] if dt == chalf else v.shape), dt)
    v[...] = a


class tensor(object):
    """A tensor on a GPU device (or on the host, for operands on their way there). ocean.tensor(size [, strides]
    [, dtype] [, device]) creates one (float on the host by default, strides in elements as in pyOcean_tensor.c's
    constructor); the functions of this module return them."""

    def __init__(self, *args):
        if len(args) == 1 and isinstance(args[0], _host.TP):
            self._h = args[0]
            return
        args = list(args)
        size = args.pop(0)
        size = [size] if isinstance(size, _py.int) else list(size)
        strides = None
        if args and isinstance(args[0], (list, tuple)):
            strides = list(args.pop(0))
        dt, device = float, None
        for a in args:
            if isinstance(a, dtype):
                dt = a
            elif isinstance(a, (deviceGPU, deviceCPU)):
                device = a
            else:
                raise TypeError("ocean.tensor: unexpected argument %r" % (a,))
        if strides is not None:
            if len(strides) != len(size):
                raise ValueError("ocean.tensor: size and strides differ in length")
            es = _hip.TYPE_SIZE[dt]
            strides = [st * es for st in strides]
        self._h = _host.create(size, dt, _device_handle(device), strides)

    def __del__(self):
        try:
            if self._h:
                _host.lib.OcDecrefTensor(self._h)
        except Exception:
            pass

    # ---- properties (pyOcean_tensor.c: dtype, device, size, strides, ndims, nelem, T) ----
    dtype = property(lambda self: dtype(self._h.contents.dtype))
    ndims = property(lambda self: self._h.contents.ndims)
    nelem = property(lambda self: self._h.contents.nelem)
    size = property(lambda self: tuple(self._h.contents.size[i] for i in range(self._h.contents.ndims)))
    strides = property(lambda self: tuple(self._h.contents.strides[i] for i in range(self._h.contents.ndims)))
    byteswapped = property(lambda self: (self._h.contents.flags & 0x1000) != 0)

    @property
    def device(self):
        for d in gpu:
            if d._handle == self._h.contents.device:
                return d
        return cpu

    def _view(self, size, strides, offset):
        t = self._h.contents
        out = tensor(_host._need(_host.lib.OcTensor_createFromStorage(t.storage, len(size), _host._arr(size), _host._arr(strides), offset, t.dtype)))
        if self.byteswapped:
            _host.lib.OcTensor_setByteswapped(out._h, 1)
        return out

    @property
    def T(self):
        return tensor(_host._need(_host.lib.OcTensor_transpose(self._h)))

    def swapAxes(self, a, b):
        size, strides = list(self.size), list(self.strides)
        size[a], size[b] = size[b], size[a]; strides[a], strides[b] = strides[b], strides[a]
        return self._view(size, strides, self._h.contents.offset)

    def flipAxis(self, axis, inplace=False):
        """The same elements with dimension `axis` running backwards: a view; in place the tensor itself changes."""
        size, strides = list(self.size), list(self.strides)
        offset = self._h.contents.offset + (size[axis] - 1) * strides[axis] if size[axis] > 0 else self._h.contents.offset
        strides[axis] = -strides[axis]
        v = self._view(size, strides, offset)
        if not inplace:
            return v
        old, self._h, v._h = self._h, v._h, self._h
        return None

    def fliplr(self, inplace=False):
        return self.flipAxis(1, inplace)

    def flipud(self, inplace=False):
        return self.flipAxis(0, inplace)

    def broadcastTo(self, size):
        return tensor(_host._need(_host.lib.OcTensor_broadcastTo(self._h, len(size), _host._arr(list(size)))))

    def reshape(self, *size):
        """A tensor of the same elements (dimension 0 fastest) with the given size; a view when this tensor is dense."""
        size = list(size[0]) if len(size) == 1 and not isinstance(size[0], _py.int) else list(size)
        if _py.int(_np.prod(size, dtype=_np.int64)) != self.nelem:
            raise ValueError("cannot reshape %d elements to size %s" % (self.nelem, size))
        src = self
        if not _host.lib.OcTensor_isContiguous(self._h):
            src = self.clone()
        t = src._h.contents
        out = tensor(_host._need(_host.lib.OcTensor_createFromStorage(t.storage, len(size), _host._arr(size), None, t.offset, t.dtype)))
        if src.byteswapped:
            _host.lib.OcTensor_setByteswapped(out._h, 1)
        out._keep = src
        return out

    def clone(self, device=None):
        dev = self._h.contents.device if device is None else _device_handle(device)
        out = tensor(_host.create(list(self.size), self.dtype, dev))
        if self.byteswapped and dev == self._h.contents.device:
            _host.lib.OcTensor_setByteswapped(out._h, 1)              # a clone keeps the byte order of its source
        out.copy(self)
        return out

    def copy(self, source):
        """tensor.copy(source): the elements of `source` (a tensor of any type and device, or data that asTensor takes)
        into this tensor, converted to its type; a source with fewer dimensions or dimensions of size one is repeated."""
        src = source if isinstance(source, tensor) else asTensor(list(source) if isinstance(source, range) else source,
                                                                   _scalar_dtype(source, self.dtype) if _is_weak_scalar(source) else None)
        if list(src.size) != list(self.size) and src.ndims <= self.ndims and _py.all(s == 1 or s == d for s, d in zip(src.size, self.size)):
            src = src.broadcastTo(self.size)
        if self.device is cpu and src.device is cpu:
            if src.nelem != self.nelem:
                raise ValueError("Mismatch in the number of elements in tensor copy")
            values = _host_values(src)
            _host_store(self, values if list(src.size) == list(self.size) else values.reshape(-1).reshape(list(self.size)[::-1]))
            return
        _host.check(_host.lib.OcTensor_copy(src._h, self._h))

    def fill(self, value):
        if self.device is cpu:
            _host_store(self, _np.asarray(value))
            return
        v = asTensor(value, self.dtype)
        raw = _np.zeros(16, _np.uint8)
        C.memmove(raw.ctypes.data, _host.data_address(v._h), _hip.TYPE_SIZE[self.dtype])
        s = _host.Scalar(); s.dtype = self.dtype
        C.memmove(C.byref(s.value), raw.ctypes.data, 16)
        _host.check(_host.lib.OcTensor_fill(self._h, C.byref(s)))

    def fillNaN(self, value):
        s = _host.scalar(_host.DOUBLE, _py.float(value)) if not isinstance(value, _py.complex) else _host.scalar(_host.CDOUBLE, value)
        _host.check(_host.lib.OcTensor_fillNaN(self._h, C.byref(s)))

    def sync(self):
        _host.to_numpy(self._h) if self.nelem == 0 else None
        return None

    def byteswap(self):
        """Reverses the bytes of every element in memory and flips the flag that says so: the values stay the same."""
        if self.device is not cpu:
            raise NotImplementedError("byteswap of a device tensor through this surface")
        v = _host_ndarray(self)
        if v.size:
            v[...] = v.byteswap()                                     # the same values, stored in the other order
        _host.lib.OcTensor_setByteswapped(self._h, 0 if self.byteswapped else 1)

    def asnumpy(self):
        """Dense numpy copy; numpy axes are Ocean's dimensions reversed. half comes back as float16, bool as bool."""
        if self.device is cpu:
            return _np.ascontiguousarray(_host_values(self))
        a = _host.to_numpy(self._h) if self.dtype != chalf else None
        if self.dtype == half:
            return a.view(_np.float16)
        if self.dtype == bool:
            return a.view(_np.bool_)
        if self.dtype == chalf:
            f = tensor._converted(self, cfloat)
            return f.asnumpy()
        return a

    def aslist(self):
        return self.asnumpy().tolist()

    def asscalar(self):
        if self.nelem != 1:
            raise ValueError("only tensors with one element convert to a scalar")
        return self.asnumpy().reshape(-1)[0].item()

    @staticmethod
    def _converted(t, dt, device=None):
        if t.device is cpu and (device is None or device == _host.cpu_device().value):
            if t.dtype == dt and not t.byteswapped:
                return t
            out = tensor(list(t.size), dtype(dt), cpu)              # host to host: converted here (see _host_ndarray)
            out.copy(t)
            return out
        h = _host.lib.OcIncrefTensor(t._h)
        _host.check(_host.lib.OcTensor_ensure(C.byref(h), dt, device if device is not None else t._h.contents.device))
        return tensor(h)

    def convert(self, dt):
        return tensor._converted(self, dt)

    # ---- operands ----
    def _operand(self, other, dt=None):
        """Tensor for the other operand of an operator. Python scalars are typed by OcScalar_getCommonType (see
        _scalar_dtype); lists and numpy arrays keep the type asTensor gives them. With `dt` the operand is given in that
        type (the in-place forms work in the type of their destination)."""
        if isinstance(other, tensor):
            if dt is None or other.dtype == dt:
                return other
            return tensor._converted(other, dt, self._h.contents.device)
        if dt is not None:
            return asTensor(other, dt)
        if _is_weak_scalar(other):
            return asTensor(other, _scalar_dtype(other, self.dtype))
        return asTensor(other)

    def _binary(self, name, other, out=None, swap=False):
        if name == "power" and out is None and _is_weak_scalar(other):
            # pyOceanCore_intrnl_power (pyOcean_core.c:283-303): scalar ** tensor keeps the scalar's own type, tensor ** integer
            # takes an int16 exponent when the tensor is an integer too
            kind = _scalar_kind(other)
            if swap:
                b = asTensor(other, kind)
            elif self.dtype < half and kind < half:
                b = asTensor(other, int16)
            else:
                b = asTensor(other, _scalar_dtype(other, self.dtype))
        else:
            b = self._operand(other, self.dtype if out is self and not name.startswith("bitshift") else None)
        x, y = (b, self) if swap else (self, b)
        dst = _host.TP() if out is None else out._h
        _host.check(_host.lib.OcTensor_binary(_B[name], x._h, y._h, C.byref(dst)))
        return out if out is not None else tensor(dst)

    def _unary(self, name, out=None):
        dst = _host.TP() if out is None else out._h
        _host.check(_host.lib.OcTensor_unary(_U[name], self._h, C.byref(dst)))
        return out if out is not None else tensor(dst)

    def _mtimes(self, other, swap=False):
        b = self._operand(other)
        x, y = (b, self) if swap else (self, b)
        if x.nelem == 1 or y.nelem == 1 or x.ndims < 2 or y.ndims < 2:
            if _is_weak_scalar(other) or (x.ndims == 0 or y.ndims == 0):
                return x._binary("multiply", y)              # product with a scalar: scale
        if x.ndims < 2 or y.ndims < 2:
            # a vector takes part as a matrix of one column (tensor_itf.c:6137-6170); the result loses that dimension again
            xm = x if x.ndims >= 2 else x.reshape([x.size[0], 1])
            ym = y if y.ndims >= 2 else y.reshape([y.size[0], 1])
            dst = _host.TP()
            _host.check(_host.lib.OcTensor_mtimes(xm._h, ym._h, C.byref(dst)))
            r = tensor(dst)
            return r.reshape([r.size[0]]) if y.ndims < 2 else r
        dst = _host.TP()
        _host.check(_host.lib.OcTensor_mtimes(x._h, y._h, C.byref(dst)))
        return tensor(dst)

    # ---- the number protocol ----
    def __pos__(self): return self.clone()
    def __neg__(self): return self._unary("negative")
    def __invert__(self): return self._unary("bitwise_not")
    def __abs__(self): return self._unary("absolute")
    def __add__(self, o): return self._binary("add", o)
    def __radd__(self, o): return self._binary("add", o, swap=True)
    def __sub__(self, o): return self._binary("subtract", o)
    def __rsub__(self, o): return self._binary("subtract", o, swap=True)
    def __mul__(self, o): return self._mtimes(o)
    def __rmul__(self, o): return self._mtimes(o, swap=True)
    def __matmul__(self, o): return self._binary("multiply", o)
    def __rmatmul__(self, o): return self._binary("multiply", o, swap=True)
    def __truediv__(self, o): return self._binary("divide", o)
    def __rtruediv__(self, o): return self._binary("divide", o, swap=True)
    def __floordiv__(self, o): return self._binary("floor_divide", o)
    def __rfloordiv__(self, o): return self._binary("floor_divide", o, swap=True)
    def __mod__(self, o): return self._binary("mod", o)
    def __rmod__(self, o): return self._binary("mod", o, swap=True)
    def __pow__(self, o, modulo=None):
        if modulo is not None:
            raise ValueError("The modulo parameter in power is not supported")
        return self._binary("power", o)
    def __rpow__(self, o): return self._binary("power", o, swap=True)
    def __and__(self, o): return self._binary("bitwise_and", o)
    def __rand__(self, o): return self._binary("bitwise_and", o, swap=True)
    def __or__(self, o): return self._binary("bitwise_or", o)
    def __ror__(self, o): return self._binary("bitwise_or", o, swap=True)
    def __xor__(self, o): return self._binary("bitwise_xor", o)
    def __rxor__(self, o): return self._binary("bitwise_xor", o, swap=True)
    def __lshift__(self, o): return self._binary("bitshift_left", o)
    def __rlshift__(self, o): return self._binary("bitshift_left", o, swap=True)
    def __rshift__(self, o): return self._binary("bitshift_right", o)
    def __rrshift__(self, o): return self._binary("bitshift_right", o, swap=True)
    def __iadd__(self, o): return self._binary("add", o, out=self)
    def __isub__(self, o): return self._binary("subtract", o, out=self)
    def __imul__(self, o): return self._binary("multiply", o, out=self)          # *= is iscale (pyOcean_tensor.c:743)
    def __imatmul__(self, o): return self._binary("multiply", o, out=self)
    def __itruediv__(self, o): return self._binary("divide", o, out=self)
    def __ifloordiv__(self, o): return self._binary("floor_divide", o, out=self)
    def __imod__(self, o): return self._binary("mod", o, out=self)
    def __ipow__(self, o): return self._binary("power", o, out=self)
    def __iand__(self, o): return self._binary("bitwise_and", o, out=self)
    def __ior__(self, o): return self._binary("bitwise_or", o, out=self)
    def __ixor__(self, o): return self._binary("bitwise_xor", o, out=self)
    def __ilshift__(self, o): return self._binary("bitshift_left", o, out=self)
    def __irshift__(self, o): return self._binary("bitshift_right", o, out=self)
    def __lt__(self, o): return self._binary("lt", o)
    def __le__(self, o): return self._binary("le", o)
    def __gt__(self, o): return self._binary("gt", o)
    def __ge__(self, o): return self._binary("ge", o)
    def __eq__(self, o): return self._binary("eq", o)
    def __ne__(self, o): return self._binary("ne", o)
    __hash__ = None

    # ---- indexing: views along the dimensions; a slice keeps its dimension, an integer removes it (pyOcean_tensor.c's
    # subscript: scalar indices give a tensor of fewer dimensions) ----
    def __getitem__(self, key):
        key = key if isinstance(key, tuple) else (key,)
        if len(key) > self.ndims:
            raise IndexError("too many indices for a tensor of %d dimensions" % self.ndims)
        size, strides, offset = [], [], self._h.contents.offset
        for axis in range(self.ndims):
            n, st = self.size[axis], self.strides[axis]
            k = key[axis] if axis < len(key) else _py.slice(None)
            if isinstance(k, (_py.int, _np.integer)):
                i = _py.int(k)
                if i < -n or i >= n:
                    raise IndexError("Tensor index (%d) out of range (%d) at dimension %d" % (i, n, axis))
                offset += (i + n if i < 0 else i) * st
                continue
            start, stop, step = k.indices(n)
            count = len(range(start, stop, step))
            offset += (start if count else 0) * st
            size.append(count); strides.append(st * step)
        return self._view(size, strides, offset)

    # ---- reductions ----
    def _reduce(self, name, p=0.0):
        which = _R[name]
        if which <= 4:
            r = C.c_int()
            _host.check(_host.lib.OcTensor_reduceLogical(which, self._h, C.byref(r)))
            return _py.bool(r.value)
        if which <= 6:
            r = C.c_uint64()
            _host.check(_host.lib.OcTensor_reduceCount(which, self._h, C.byref(r)))
            return r.value
        s = _host.Scalar()
        _host.check(_host.lib.OcTensor_reduceAll(which, self._h, p, C.byref(s)))
        return s.get()

    def sum(self, axis=None): return self._reduce("sum") if axis is None else self._axis("sum", axis)
    def prod(self, axis=None): return self._reduce("prod") if axis is None else self._axis("prod", axis)
    def maximum(self, axis=None): return self._reduce("maximum") if axis is None else self._axis("maximum", axis)
    def minimum(self, axis=None): return self._reduce("minimum") if axis is None else self._axis("minimum", axis)
    def norm(self, p=2, axis=None):
        if axis is not None:
            return self._axis("norm2" if p == 2 else "norm", axis, p)
        return self._reduce("norm2") if p == 2 else self._reduce("norm", _py.float(p))

    def _axis(self, name, axis, p=0.0, keepdims=False, out=None):
        axes = [axis] if isinstance(axis, _py.int) else list(axis)
        dst = _host.TP() if out is None else out._h
        _host.check(_host.lib.OcTensor_axisReduce(_R[name], self._h, len(axes), (C.c_int * len(axes))(*axes), 1 if keepdims else 0, _py.float(p), C.byref(dst)))
        return out if out is not None else tensor(dst)

    # ---- printing: the closing line is Ocean's (src/base/format.c), the values are numpy's rendering ----
    def footer(self):
        dev = self.device
        if self.ndims == 0:
            return "<scalar.%s on %s>" % (_DTYPE_NAMES[self.dtype], dev.name)
        return "<%stensor.%s of size %s on %s%s>" % ("empty " if self.nelem == 0 else "", _DTYPE_NAMES[self.dtype], "x".join(str(s) for s in self.size),
                                                     dev.name, " (byteswapped)" if self.byteswapped else "")

    def __repr__(self):
        return "%s\n%s" % (self.asnumpy().T if self.ndims <= 2 else self.asnumpy(), self.footer())


def _list_dtype(values):
    """Type ocean.asTensor gives a nested list without a dtype argument: bool, int64, double or complex-double by kind."""
    kind = _np.asarray(values).dtype.kind
    if kind not in "biufc":
        raise TypeError("cannot convert %r to a tensor" % (values,))
    return {"b": bool, "i": int64, "u": int64, "f": double, "c": cdouble}[kind]


def asTensor(data, *args):
    """ocean.asTensor(data [, order] [, dtype] [, device]) (pyOcean_module_core.c:823-866). In a nested list the innermost
    lists run along dimension 0 -- [[1, 2, 3], [4, 5, 6]] has size 3 x 2 and A[i, j] = data[j][i] -- unless order is 'r'
    ('R', 'C'), in which case lists are rows: size 2 x 3, A[i, j] = data[i][j], and a flat list is a row of size 1 x n.
    A numpy array gives the tensor whose dimensions are the array's axes reversed (its memory order as it is); scalars
    give tensors with no dimensions. A list of tensors stacks them along a new last dimension."""
    order, dt, device = "F", None, None
    for a in args:
        if isinstance(a, str):
            order = a.upper()
        elif isinstance(a, dtype):
            dt = a
        elif isinstance(a, (deviceGPU, deviceCPU)):
            device = a
        elif a is None:
            continue
        elif isinstance(a, _py.int):
            dt = dtype(a)
        else:
            raise TypeError("ocean.asTensor: unexpected argument %r" % (a,))
    if isinstance(data, tensor):
        t = data if dt is None else data.convert(dt)
        return t if device is None or device is t.device else t.clone(device)
    if isinstance(data, (list, tuple)) and data and _py.all(isinstance(x, tensor) for x in data):
        first = data[0]
        out = tensor(list(first.size) + [len(data)], first.dtype if dt is None else dt, first.device if device is None else device)
        for k, x in enumerate(data):
            out[(_py.slice(None),) * first.ndims + (k,)].copy(x)
        return out
    if isinstance(data, _np.ndarray):
        first_fastest = data
        if dt is None:
            dt = dtype(_host.dtype_of(data.dtype))
    else:
        a = _np.asarray(data)
        if dt is None:
            dt = _list_dtype(data)
        if order in ("R", "C"):
            # lists are rows: A[i0, i1, ...] = data[i0][i1]...; a flat list is one row (size 1 x n)
            rows = a.reshape(1, -1) if a.ndim == 1 else a
            first_fastest = rows.transpose(*range(rows.ndim)[::-1])
        else:
            first_fastest = a                                         # innermost list = dimension 0 = numpy's last axis
    flat = _np.ascontiguousarray(_host_array(first_fastest, dt))
    t = _host.create(list(first_fastest.shape[::-1]), dt, _host.cpu_device())
    C.memmove(_host.data_address(t), flat.ctypes.data, flat.nbytes)
    out = tensor(t)
    return out if device is None or device is cpu else out.clone(device)


def zeros(size, dt=float, device=None):
    t = tensor(size, dt, device if device is not None else cpu)
    if t.nelem:
        t.fill(0)
    return t


def ones(size, dt=float, device=None):
    t = tensor(size, dt, device if device is not None else cpu)
    if t.nelem:
        t.fill(1)
    return t


def arange(n, *args):
    dt, device = int64, None
    for a in args:
        if isinstance(a, dtype):
            dt = a
        elif isinstance(a, (deviceGPU, deviceCPU)):
            device = a
    n = n[0] if isinstance(n, (list, tuple)) else n
    return asTensor(_np.arange(n), dt, device)


def ensure(t, dt=None, device=None, inplace=False):
    """ocean.ensure(tensor [, dtype] [, device] [, inplace]): the tensor in the given type on the given device -- itself when
    it already is -- or, in place, the tensor object re-seated on the converted data."""
    if isinstance(dt, (deviceGPU, deviceCPU)):
        dt, device = None, dt
    r = tensor._converted(t, t.dtype if dt is None else dt, _device_handle(device) if device is not None else None)
    if not inplace:
        return r
    t._h, r._h = r._h, t._h
    return None


def _unary_function(name):
    def fn(a, out=None):
        a = a if isinstance(a, tensor) else asTensor(a)
        return a._unary(name, out)
    fn.__name__ = name
    return fn


def _binary_function(name):
    def fn(a, b, out=None):
        if not isinstance(a, tensor):
            if not isinstance(b, tensor):
                a = asTensor(a)
            else:
                return b._binary(name, a, out=out, swap=True)
        return a._binary(name, b, out=out)
    fn.__name__ = name
    return fn


def _reduce_function(name):
    def fn(a, axes=None, keepdims=False, out=None):
        a = a if isinstance(a, tensor) else asTensor(a)
        if isinstance(axes, tensor):
            axes, out = None, axes
        if axes is None:
            return a._reduce(name)
        return a._axis(name, axes, 0.0, keepdims, out)
    fn.__name__ = name
    return fn


# module functions under Ocean's names (pyOcean_module_core.c:120-330), each with an optional destination tensor
for _ocean, _op in (("negative", "negative"), ("bitwiseNot", "bitwise_not"), ("logicalNot", "logical_not"), ("conj", "conj"), ("reciprocal", "reciprocal"),
                    ("sin", "sin"), ("cos", "cos"), ("tan", "tan"), ("sinh", "sinh"), ("cosh", "cosh"), ("tanh", "tanh"), ("arcsin", "arcsin"),
                    ("arccos", "arccos"), ("arctan", "arctan"), ("arcsinh", "arcsinh"), ("arccosh", "arccosh"), ("arctanh", "arctanh"), ("sqrt", "sqrt"),
                    ("cbrt", "cbrt"), ("square", "square"), ("exp", "exp"), ("exp2", "exp2"), ("exp10", "exp10"), ("expm1", "expm1"), ("log", "log"),
                    ("log2", "log2"), ("log10", "log10"), ("log1p", "log1p"), ("absolute", "absolute"), ("fabs", "fabs"), ("sign", "sign"),
                    ("ceil", "ceil"), ("floor", "floor"), ("trunc", "trunc"), ("round", "round"), ("isinf", "isinf"), ("isnan", "isnan"),
                    ("isfinite", "isfinite"), ("isposinf", "isposinf"), ("isneginf", "isneginf")):
    globals()[_ocean] = _unary_function(_op)
for _ocean, _op in (("add", "add"), ("subtract", "subtract"), ("scale", "multiply"), ("multiply", "multiply"), ("divide", "divide"),
                    ("trueDivide", "true_divide"), ("floorDivide", "floor_divide"), ("power", "power"), ("mod", "mod"), ("fmod", "fmod"),
                    ("min", "min"), ("max", "max"), ("fmin", "fmin"), ("fmax", "fmax"), ("bitwiseAnd", "bitwise_and"), ("bitwiseOr", "bitwise_or"),
                    ("bitwiseXor", "bitwise_xor"), ("logicalAnd", "logical_and"), ("logicalOr", "logical_or"), ("logicalXor", "logical_xor"),
                    ("bitshiftLeft", "bitshift_left"), ("bitshiftRight", "bitshift_right")):
    globals()[_ocean] = _binary_function(_op)
for _ocean, _op in (("any", "any"), ("all", "all"), ("allFinite", "all_finite"), ("anyInf", "any_inf"), ("anyNaN", "any_nan"), ("nnz", "nnz"),
                    ("nnzNaN", "nnz_nan"), ("sum", "sum"), ("sumNaN", "sum_nan"), ("prod", "prod"), ("prodNaN", "prod_nan"), ("sumAbs", "sum_abs"),
                    ("sumAbsNaN", "sum_abs_nan"), ("maximum", "maximum"), ("minimum", "minimum"), ("maximumAbs", "maximum_abs"),
                    ("minimumAbs", "minimum_abs"), ("norm2", "norm2"), ("norm2NaN", "norm2_nan")):
    globals()[_ocean] = _reduce_function(_op)


def mtimes(a, b): return a * b


def norm(a, p=2, axes=None, keepdims=False, out=None):
    """ocean.norm(tensor [, p] [, axes [, keepdims]] [, out])"""
    if isinstance(keepdims, tensor):
        keepdims, out = False, keepdims
    if isinstance(axes, tensor):
        axes, out = None, axes
    if axes is None:
        return a.norm(p)
    return a._axis("norm2" if p == 2 else "norm", axes, p, keepdims, out)


def gemm(alpha, a, b, beta=None, c=None, transA="N", transB="N"):
    """ocean.gemm(alpha, A [, transA], B [, transB] [, beta, C]): alpha and beta are scalars or tensors with one element per
    product (size 1 x 1 x batch...)."""
    al = alpha if isinstance(alpha, tensor) else asTensor(alpha, _scalar_dtype(alpha, a.dtype))
    be = None if beta is None else (beta if isinstance(beta, tensor) else asTensor(beta, _scalar_dtype(beta, a.dtype)))
    dst = _host.TP() if c is None else c._h
    _host.check(_host.lib.OcTensor_gemmTensors(al._h, a._h, transA.encode(), b._h, transB.encode(), be._h if be is not None else None, C.byref(dst)))
    return c if c is not None else tensor(dst)


def _device_call(self, array, dt=None):
    """ocean.gpu[0](x): x on this device -- a tensor of this module moves (or stays), anything else goes through asTensor."""
    if isinstance(array, tensor):
        return array if array.device is self and dt is None else asTensor(array, dt, self)
    return asTensor(array, dt, self)


deviceGPU.__call__ = _device_call
