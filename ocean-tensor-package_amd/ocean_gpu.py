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

bool, uint8, uint16, uint32, uint64, int8, int16, int32, int64, half, float, double, chalf, cfloat, cdouble = range(15)
_DTYPE_NAMES = ["bool", "uint8", "uint16", "uint32", "uint64", "int8", "int16", "int32", "int64", "half", "float", "double",
                "complex-half", "complex-float", "complex-double"]
_B = _hip.B          # names of the binary block of the table -> index
_U = _hip.U
_R = _hip.R
_host.lib.OcTensor_gemmTensors.argtypes = [_host.TP, _host.TP, C.c_char, _host.TP, C.c_char, _host.TP, C.POINTER(_host.TP)]
_host.lib.OcTensor_ensure.argtypes = [C.POINTER(_host.TP), C.c_int, C.c_void_p]
_host.lib.OcIncrefTensor.restype = _host.TP
_host.lib.OcIncrefTensor.argtypes = [_host.TP]
_host.lib.OcDType_getCommonType.restype = C.c_int


def _scalar_dtype(value, like):
    """Ocean type of a Python scalar next to a tensor of type `like`: scalars are typed weakly -- the smallest type of
    their kind that holds the value exactly -- so that int8 + 3 stays int8 and float + 3.0 stays float."""
    if isinstance(value, (_py.bool, _np.bool_)):
        return bool
    if isinstance(value, (_py.int, _np.integer)):
        v = _py.int(value)
        if v >= 0 and uint8 <= like <= uint64:
            return next(t for t, bits in ((uint8, 8), (uint16, 16), (uint32, 32), (uint64, 64)) if v < (1 << bits))
        return next(t for t, bits in ((int8, 8), (int16, 16), (int32, 32), (int64, 64)) if -(1 << (bits - 1)) <= v < (1 << (bits - 1)))
    if isinstance(value, (_py.float, _np.floating)):
        v = _py.float(value)
        if v != v or v in (_py.float("inf"), -_py.float("inf")) or _py.float(_np.float16(v)) == v:
            return half
        return float if _py.float(_np.float32(v)) == v else double
    if isinstance(value, (_py.complex, _np.complexfloating)):
        re, im = _scalar_dtype(value.real, like), _scalar_dtype(value.imag, like)
        return {half: chalf, float: cfloat, double: cdouble}[max(re, im)]
    raise TypeError("cannot use %r as a tensor operand" % (value,))


def _host_array(value, dtype):
    """numpy array holding `value` in the storage type of Ocean type `dtype` (half travels as its bit pattern)."""
    a = _np.asarray(value)
    if dtype == half:
        return a.astype(_np.float16).view(_np.uint16)
    if dtype == chalf:
        c = _np.asarray(a, dtype=_np.complex64)
        out = _np.empty(c.shape + (2,), _np.uint16)
        out[..., 0] = c.real.astype(_np.float16).view(_np.uint16); out[..., 1] = c.imag.astype(_np.float16).view(_np.uint16)
        return out
    if dtype == bool:
        return a.astype(_np.bool_).view(_np.uint8)
    return a.astype(_host.NUMPY[dtype])


class tensor(object):
    """A tensor on a GPU device (or on the host, for operands on their way there). Wraps a tensor of the host layer."""

    def __init__(self, handle):
        self._h = handle

    def __del__(self):
        try:
            if self._h:
                _host.lib.OcDecrefTensor(self._h)
        except Exception:
            pass

    # ---- properties (pyOcean_tensor.c: dtype, device, size, strides, ndims, nelem, T) ----
    dtype = property(lambda self: self._h.contents.dtype)
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
        return "cpu"

    @property
    def T(self):
        return tensor(_host._need(_host.lib.OcTensor_transpose(self._h)))

    def reshape(self, size):
        """A tensor of the same elements (dimension 0 fastest) with the given size; a view when this tensor is dense."""
        size = list(size)
        if int(_np.prod(size, dtype=_np.int64)) != self.nelem:
            raise ValueError("cannot reshape %d elements to size %s" % (self.nelem, size))
        src = self
        if not _host.lib.OcTensor_isContiguous(self._h):
            src = self.clone()
        t = src._h.contents
        lib = _host.lib
        lib.OcTensor_createFromStorage.restype = _host.TP
        lib.OcTensor_createFromStorage.argtypes = [C.POINTER(_host.Storage), C.c_int, _host._ss, _host._ss, C.c_ssize_t, C.c_int]
        out = tensor(_host._need(lib.OcTensor_createFromStorage(t.storage, len(size), _host._arr(size), None, t.offset, t.dtype)))
        out._keep = src
        return out

    def clone(self, device=None):
        dev = self._h.contents.device if device is None else device._handle
        out = _host.create(list(self.size), self.dtype, dev)
        _host.check(_host.lib.OcTensor_copy(self._h, out))
        return tensor(out)

    def asnumpy(self):
        """Dense numpy copy; numpy axes are Ocean's dimensions reversed. half comes back as float16, bool as bool."""
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

    @staticmethod
    def _converted(t, dtype, device=None):
        h = _host.lib.OcIncrefTensor(t._h)
        _host.check(_host.lib.OcTensor_ensure(C.byref(h), dtype, device if device is not None else t._h.contents.device))
        return tensor(h)

    def convert(self, dtype):
        return tensor._converted(self, dtype)

    # ---- operands ----
    def _operand(self, other, dtype=None):
        """Tensor for the other operand of an operator. Python scalars are typed weakly (the smallest type of their kind
        that holds the value), so they do not widen the tensor's type; lists are typed by kind. With `dtype` the operand
        is given in that type (the in-place forms work in the type of their destination)."""
        if isinstance(other, tensor):
            if dtype is None or other.dtype == dtype:
                return other
            return tensor._converted(other, dtype, self._h.contents.device)
        if dtype is not None:
            return asTensor(other, dtype)
        if isinstance(other, _np.ndarray) and other.ndim > 0:
            return asTensor(other)                            # a numpy array keeps its own type
        if _np.ndim(other) == 0:
            return asTensor(other, _scalar_dtype(other, self.dtype))
        if _list_dtype(other) == bool:
            return asTensor(other, bool)
        flat = _np.asarray(other).reshape(-1).tolist()
        return asTensor(other, max(_scalar_dtype(v, self.dtype) for v in flat))

    def _binary(self, name, other, out=None, swap=False):
        b = self._operand(other, self.dtype if out is self and not name.startswith("bitshift") else None)
        x, y = (b, self) if swap else (self, b)
        dst = _host.TP() if out is None else out._h
        _host.check(_host.lib.OcTensor_binary(_B[name], x._h, y._h, C.byref(dst)))
        return out if out is not None else tensor(dst)

    def _unary(self, name):
        dst = _host.TP()
        _host.check(_host.lib.OcTensor_unary(_U[name], self._h, C.byref(dst)))
        return tensor(dst)

    def _mtimes(self, other, swap=False):
        b = self._operand(other)
        x, y = (b, self) if swap else (self, b)
        if x.nelem == 1 or y.nelem == 1 or x.ndims < 2 or y.ndims < 2:
            return x._binary("multiply", y)                  # product with a scalar: scale
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
    def __mod__(self, o): return self._binary("mod", o)
    def __pow__(self, o): return self._binary("power", o)
    def __and__(self, o): return self._binary("bitwise_and", o)
    def __or__(self, o): return self._binary("bitwise_or", o)
    def __xor__(self, o): return self._binary("bitwise_xor", o)
    def __lshift__(self, o): return self._binary("bitshift_left", o)
    def __rshift__(self, o): return self._binary("bitshift_right", o)
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

    # ---- slicing: views along the dimensions (start:stop:step per dimension, integers drop nothing here) ----
    def __getitem__(self, key):
        key = key if isinstance(key, tuple) else (key,)
        h = _host.lib.OcIncrefTensor(self._h)
        for axis, k in enumerate(key):
            n = self.size[axis]
            if isinstance(k, _py.int):
                k = _py.slice(k, k + 1 if k != -1 else None, 1)
            start, stop, step = k.indices(n)
            count = len(range(start, stop, step))
            v = _host._need(_host.lib.OcTensor_slice(h, axis, start if count else 0, count, step))
            _host.lib.OcDecrefTensor(h)
            h = v
        return tensor(h)

    # ---- reductions ----
    def _reduce(self, name, p=0.0):
        s = _host.Scalar()
        _host.check(_host.lib.OcTensor_reduceAll(_R[name], self._h, p, C.byref(s)))
        return s.get()

    def sum(self, axis=None): return self._reduce("sum") if axis is None else self._axis("sum", axis)
    def prod(self, axis=None): return self._reduce("prod") if axis is None else self._axis("prod", axis)
    def maximum(self, axis=None): return self._reduce("maximum") if axis is None else self._axis("maximum", axis)
    def minimum(self, axis=None): return self._reduce("minimum") if axis is None else self._axis("minimum", axis)
    def norm(self, p=2, axis=None):
        if axis is not None:
            return self._axis("norm2" if p == 2 else "norm", axis, p)
        return self._reduce("norm2") if p == 2 else self._reduce("norm", _py.float(p))

    def _axis(self, name, axis, p=0.0, keepdims=False):
        axes = [axis] if isinstance(axis, _py.int) else list(axis)
        dst = _host.TP()
        _host.check(_host.lib.OcTensor_axisReduce(_R[name], self._h, len(axes), (C.c_int * len(axes))(*axes), 1 if keepdims else 0, _py.float(p), C.byref(dst)))
        return tensor(dst)

    # ---- printing: the closing line is Ocean's (src/base/format.c), the values are numpy's rendering ----
    def footer(self):
        dev = self.device
        return "<tensor.%s of size %s on %s>" % (_DTYPE_NAMES[self.dtype], "x".join(str(s) for s in self.size), dev if isinstance(dev, str) else dev.name)

    def __repr__(self):
        return "%s\n%s" % (self.asnumpy().T if self.ndims <= 2 else self.asnumpy(), self.footer())


def _list_dtype(values):
    """Type ocean.asTensor gives a nested list without a dtype argument: bool, int64, double or complex-double by kind."""
    kind = _np.asarray(values).dtype.kind
    if kind not in "biufc":
        raise TypeError("cannot convert %r to a tensor" % (values,))
    return {"b": bool, "i": int64, "u": int64, "f": double, "c": cdouble}[kind]


def asTensor(data, dtype=None, device=None):
    """ocean.asTensor(data [, dtype] [, device]). Nested lists index as data[i0][i1]..., so [[1, 2, 3], [4, 5, 6]] has size
    2x3; a numpy array gives the tensor whose dimensions are the array's axes reversed (its memory order as it is);
    scalars give tensors with no dimensions."""
    if isinstance(dtype, deviceGPU):
        dtype, device = None, dtype
    if isinstance(data, tensor):
        t = data if dtype is None else data.convert(dtype)
        return t if device is None else t.clone(device)
    if isinstance(data, _np.ndarray):
        first_fastest = data
        if dtype is None:
            dtype = _host.dtype_of(data.dtype)
    else:
        first_fastest = _np.asarray(data).T
        if dtype is None:
            dtype = _list_dtype(data)
    flat = _np.ascontiguousarray(_host_array(first_fastest, dtype))
    t = _host.create(list(first_fastest.shape[::-1]), dtype, _host.cpu_device())
    C.memmove(_host.data_address(t), flat.ctypes.data, flat.nbytes)
    out = tensor(t)
    return out if device is None else out.clone(device)


def arange(n, dtype=int64, device=None):
    return asTensor(_np.arange(n), dtype, device)


def add(a, b): return a + b
def subtract(a, b): return a - b
def scale(a, b): return a._binary("multiply", b)
def mtimes(a, b): return a * b
def sum(a, axis=None): return a.sum(axis)
def maximum(a, axis=None): return a.maximum(axis)
def minimum(a, axis=None): return a.minimum(axis)
def norm(a, p=2, axis=None): return a.norm(p, axis)


def gemm(alpha, a, b, beta=None, c=None, transA="N", transB="N"):
    """ocean.gemm(alpha, A [, transA], B [, transB] [, beta, C]): alpha and beta are scalars or tensors with one element per
    product (size 1 x 1 x batch...)."""
    al = alpha if isinstance(alpha, tensor) else asTensor(alpha, _scalar_dtype(alpha, a.dtype))
    be = None if beta is None else (beta if isinstance(beta, tensor) else asTensor(beta, _scalar_dtype(beta, a.dtype)))
    dst = _host.TP() if c is None else c._h
    _host.check(_host.lib.OcTensor_gemmTensors(al._h, a._h, transA.encode(), b._h, transB.encode(), be._h if be is not None else None, C.byref(dst)))
    return c if c is not None else tensor(dst)


def _device_call(self, array, dtype=None):
    """ocean.gpu[0](x): x on this device -- a tensor of this module moves (or stays), anything else goes through asTensor."""
    if isinstance(array, tensor):
        return array if array.device is self and dtype is None else asTensor(array, dtype, self)
    return asTensor(array, dtype, self)


deviceGPU.__call__ = _device_call
