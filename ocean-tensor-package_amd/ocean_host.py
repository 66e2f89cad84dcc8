"""ctypes binding of host/libocean_host.so: Ocean's GPU device module and the small front end that
drives it (OcInitGPU, tensors as views over device storages, OcTensor_add/scale/..., reductions,
GEMM). Used by the tests; fails loudly when the library has not been built."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "host", "libocean_host.so")
if not os.path.exists(LIB_PATH):
    raise ImportError("%s is missing: build it with `make -C %s`" % (LIB_PATH, _HERE))
lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)

MAX_DIMS = 8
(BOOL, UINT8, UINT16, UINT32, UINT64, INT8, INT16, INT32, INT64, HALF, FLOAT, DOUBLE, CHALF, CFLOAT, CDOUBLE, NONE) = range(16)
NUMPY = {BOOL: np.uint8, UINT8: np.uint8, UINT16: np.uint16, UINT32: np.uint32, UINT64: np.uint64, INT8: np.int8, INT16: np.int16,
         INT32: np.int32, INT64: np.int64, HALF: np.uint16, FLOAT: np.float32, DOUBLE: np.float64, CFLOAT: np.complex64, CDOUBLE: np.complex128}


class Storage(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("event", C.c_void_p), ("data", C.c_void_p), ("dtype", C.c_int), ("size", C.c_ssize_t),
                ("capacity", C.c_ssize_t), ("nelem", C.c_ssize_t), ("elemsize", C.c_int), ("flags", C.c_uint32),
                ("refcount", C.c_long), ("finalize", C.c_void_p)]


class Tensor(C.Structure):
    _fields_ = [("ndims", C.c_int), ("capacity", C.c_int), ("size", C.POINTER(C.c_ssize_t)), ("strides", C.POINTER(C.c_ssize_t)),
                ("offset", C.c_ssize_t), ("storage", C.POINTER(Storage)), ("device", C.c_void_p), ("dtype", C.c_int),
                ("elemsize", C.c_int), ("nelem", C.c_ssize_t), ("blockOffset", C.c_ssize_t), ("blockExtent", C.c_ssize_t),
                ("refcount", C.c_long), ("flags", C.c_uint32)]


class ScalarValue(C.Union):
    _fields_ = [("u8", C.c_uint8), ("u16", C.c_uint16), ("u32", C.c_uint32), ("u64", C.c_uint64), ("i8", C.c_int8), ("i16", C.c_int16),
                ("i32", C.c_int32), ("i64", C.c_int64), ("f32", C.c_float), ("f64", C.c_double), ("c64", C.c_float * 2), ("c128", C.c_double * 2)]


class Scalar(C.Structure):
    _fields_ = [("dtype", C.c_int), ("value", ScalarValue)]

    def get(self):
        v = self.value
        if self.dtype == HALF:
            return float(np.array([v.u16], np.uint16).view(np.float16)[0])
        if self.dtype == CHALF:
            parts = np.array([v.u32 & 0xFFFF, v.u32 >> 16], np.uint16).view(np.float16)
            return complex(float(parts[0]), float(parts[1]))
        return {BOOL: v.u8, UINT8: v.u8, UINT16: v.u16, UINT32: v.u32, UINT64: v.u64, INT8: v.i8, INT16: v.i16, INT32: v.i32,
                INT64: v.i64, FLOAT: v.f32, DOUBLE: v.f64, CFLOAT: complex(*v.c64), CDOUBLE: complex(*v.c128)}[self.dtype]


def scalar(dtype, value):
    s = Scalar(); s.dtype = dtype
    if dtype == DOUBLE: s.value.f64 = value
    elif dtype == FLOAT: s.value.f32 = value
    elif dtype == CDOUBLE: s.value.c128[0], s.value.c128[1] = value.real, value.imag
    elif dtype == CFLOAT: s.value.c64[0], s.value.c64[1] = value.real, value.imag
    elif dtype in (INT8, INT16, INT32, INT64): s.value.i64 = int(value)
    else: s.value.u64 = int(value)
    return s


class ReduceAxis(C.Structure):
    """OcSolidReduceAxis (include/ocean/external/ocean-solid/ocean_solid.h:73-83)."""
    _fields_ = [("ndims", C.c_int), ("rdims", C.c_int), ("size", C.c_size_t * 8), ("rsize", C.c_size_t * 8), ("strides1", C.c_ssize_t * 8),
                ("strides2", C.c_ssize_t * 8), ("rstrides", C.c_ssize_t * 8), ("ptr1", C.c_void_p), ("ptr2", C.c_void_p)]


class DevicePropGPU(C.Structure):
    """OcDevicePropGPU (include/ocean_gpu_module.h; the reference's include/ocean/core/gpu/device_gpu.h:31-106)."""
    _fields_ = ([("name", C.c_char * 256), ("totalGlobalMem", C.c_size_t), ("freeGlobalMem", C.c_size_t), ("sharedMemPerBlock", C.c_size_t),
                 ("regsPerBlock", C.c_int), ("warpSize", C.c_int), ("memPitch", C.c_size_t), ("maxThreadsPerBlock", C.c_int),
                 ("maxThreadsDim", C.c_int * 3), ("maxGridSize", C.c_int * 3), ("clockRate", C.c_int), ("totalConstMem", C.c_size_t)]
                + [(n, C.c_int) for n in ("major", "minor", "deviceOverlap", "multiProcessorCount", "kernelExecTimeoutEnabled", "integrated",
                                          "canMapHostMemory", "computeMode", "concurrentKernels", "ECCEnabled", "pciBusID", "pciDeviceID",
                                          "pciDomainID", "tccDriver", "asyncEngineCount", "unifiedAddressing", "memoryClockRate",
                                          "memoryBusWidth", "l2CacheSize", "maxThreadsPerMultiProcessor", "streamPrioritiesSupported",
                                          "globalL1CacheSupported", "localL1CacheSupported")]
                + [("sharedMemPerMultiprocessor", C.c_size_t)]
                + [(n, C.c_int) for n in ("regsPerMultiprocessor", "managedMemSupported", "isMultiGpuBoard", "multiGpuBoardGroupID",
                                          "singleToDoublePrecisionPerfRatio", "pageableMemoryAccess", "concurrentManagedAccess",
                                          "hostNativeAtomicSupported", "maxBlocksPerMultiProcessor", "maxWarpsPerMultiProcessor",
                                          "maxSharedMemPerSM")])


def gpu_public_properties(device_handle, update=False):
    """The OcDevicePropGPU inside an OcDeviceGPU object (it follows the OcDevice head), read in place the way
    pyOcean_device_gpu.c:181-420 reads it; update=True calls OcDeviceGPU_updateProperties first (freeMem does)."""
    import json
    handle = device_handle.value if isinstance(device_handle, C.c_void_p) else device_handle
    if update:
        lib.OcDeviceGPU_updateProperties.argtypes = [C.c_void_p]
        check(lib.OcDeviceGPU_updateProperties(handle))
    head = json.loads(lib.OcHost_abiLayout())["sizeof(OcDevice)"]
    return DevicePropGPU.from_address(handle + head)


TP = C.POINTER(Tensor)
_ss = C.POINTER(C.c_ssize_t)
lib.OcError_lastMessage.restype = C.c_char_p
lib.OcHost_abiLayout.restype = C.c_char_p
lib.OcDType_getCommonType.argtypes = [C.c_int, C.c_int]
lib.OcTensor_create.restype = TP
lib.OcTensor_create.argtypes = [C.c_int, _ss, _ss, C.c_int, C.c_void_p]
for name in ("OcTensor_transpose", "OcTensor_shallowCopy"):
    getattr(lib, name).restype = TP
    getattr(lib, name).argtypes = [TP]
lib.OcTensor_slice.restype = TP
lib.OcTensor_slice.argtypes = [TP, C.c_int, C.c_ssize_t, C.c_ssize_t, C.c_ssize_t]
lib.OcTensor_broadcastTo.restype = TP
lib.OcTensor_broadcastTo.argtypes = [TP, C.c_int, _ss]
lib.OcTensor_setByteswapped.argtypes = [TP, C.c_int]
lib.OcDecrefTensor.argtypes = [TP]
lib.OcTensor_copy.argtypes = [TP, TP]
lib.OcTensor_binary.argtypes = [C.c_int, TP, TP, C.POINTER(TP)]
lib.OcTensor_unary.argtypes = [C.c_int, TP, C.POINTER(TP)]
lib.OcTensor_reduceAll.argtypes = [C.c_int, TP, C.c_double, C.POINTER(Scalar)]
lib.OcTensor_axisReduce.argtypes = [C.c_int, TP, C.c_int, C.POINTER(C.c_int), C.c_int, C.c_double, C.POINTER(TP)]
lib.OcTensor_gemm.argtypes = [C.POINTER(Scalar), TP, C.c_char, TP, C.c_char, C.POINTER(Scalar), C.POINTER(TP)]
lib.OcTensor_mtimes.argtypes = [TP, TP, C.POINTER(TP)]
lib.OcTensor_fill.argtypes = [TP, C.POINTER(Scalar)]
lib.OcTensor_fillNaN.argtypes = [TP, C.POINTER(Scalar)]
lib.OcTensor_maskedFill.argtypes = [TP, TP, C.POINTER(Scalar)]
lib.OcTensor_stepsInt64.argtypes = [TP, C.c_int64, C.c_int64]
lib.OcTensor_stepsDouble.argtypes = [TP, C.c_double, C.c_double]
lib.OcTensorGPU_projectColumns.argtypes = [TP, TP, TP]
lib.OcTensor_find.restype = TP
lib.OcTensor_find.argtypes = [TP]
lib.OcTensor_maskToOffset.restype = TP
lib.OcTensor_maskToOffset.argtypes = [TP, _ss]
lib.OcSolid_analyzeReduceAxis.restype = None
lib.OcSolid_analyzeReduceAxis.argtypes = [C.POINTER(ReduceAxis), TP, TP, C.c_int, C.POINTER(C.c_int), C.c_int]
lib.OcShape_extent.argtypes = [C.c_int, _ss, _ss, C.c_ssize_t, _ss, _ss]
lib.OcDeviceGPU_activity.argtypes = [C.c_void_p, C.POINTER(C.c_long), C.POINTER(C.c_long), C.POINTER(C.c_long)]
lib.OcFinalize.restype = None
lib.OcShape_sortStrides2.restype = None
lib.OcShape_mergeBlocks2.restype = None
lib.OcShape_sortStrides2.argtypes = [C.c_int, _ss, _ss, _ss]
lib.OcShape_mergeBlocks2.argtypes = [C.POINTER(C.c_int), _ss, _ss, _ss]


class OceanError(RuntimeError):
    pass


def check(status):
    if status != 0:
        raise OceanError(lib.OcError_lastMessage().decode())


def _need(ptr):
    if not ptr:
        raise OceanError(lib.OcError_lastMessage().decode())
    return ptr


def dtype_of(numpy_dtype):
    """Ocean data type of a numpy dtype (bool -> bool, float16 -> half; anything else by item type)."""
    dt = np.dtype(numpy_dtype)
    if dt == np.bool_:
        return BOOL
    if dt == np.float16:
        return HALF
    for code in (UINT8, UINT16, UINT32, UINT64, INT8, INT16, INT32, INT64, FLOAT, DOUBLE, CFLOAT, CDOUBLE):
        if np.dtype(NUMPY[code]) == dt:
            return code
    raise OceanError("no Ocean data type for numpy dtype %s" % dt)


def cpu_device():
    return C.c_void_p.in_dll(lib, "OcCPU")


def gpu_device(index=0):
    check(lib.OcInitGPU())
    devices = C.POINTER(C.c_void_p).in_dll(lib, "OcGPU")
    if index >= lib.OcDeviceGPUCount():
        raise OceanError("GPU device %d does not exist" % index)
    return C.c_void_p(devices[index])


def _arr(seq):
    return (C.c_ssize_t * max(len(seq), 1))(*seq)


def create(shape, dtype, device, strides=None):
    """Tensor of Ocean shape `shape` (first dimension fastest by default)."""
    return _need(lib.OcTensor_create(len(shape), _arr(shape), _arr(strides) if strides is not None else None, dtype, device))


def data_address(t):
    return t.contents.storage.contents.data + t.contents.offset


def from_numpy(a, dtype, device=None, byteswapped=False):
    """Host tensor holding a copy of numpy array `a`. Ocean dimensions are numpy's reversed (the last
    numpy axis is Ocean's dimension 0), so a C-contiguous array is a column-major Ocean tensor."""
    a = np.ascontiguousarray(a)
    t = create(list(a.shape[::-1]), dtype, cpu_device())
    C.memmove(data_address(t), a.ctypes.data, a.nbytes)
    if byteswapped:
        lib.OcTensor_setByteswapped(t, 1)
    if device is not None:
        d = create(list(a.shape[::-1]), dtype, device)
        if byteswapped:
            lib.OcTensor_setByteswapped(d, 1)
        check(lib.OcTensor_copy(t, d))
        lib.OcDecrefTensor(t)
        return d
    return t


def to_numpy(t):
    """Dense numpy copy (numpy axes = Ocean dimensions reversed) of any tensor, in native byte order."""
    tc = t.contents
    shape = [tc.size[i] for i in range(tc.ndims)]
    h = create(shape, tc.dtype, cpu_device())
    check(lib.OcTensor_copy(t, h))
    out = np.empty(shape[::-1], NUMPY[tc.dtype])
    C.memmove(out.ctypes.data, data_address(h), out.nbytes)
    lib.OcDecrefTensor(h)
    return out


def shape_of(t):
    return [t.contents.size[i] for i in range(t.contents.ndims)]
