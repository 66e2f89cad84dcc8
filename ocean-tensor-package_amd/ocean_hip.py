"""ctypes binding of csrc/libocean_hip.so (the C ABI declared in include/ocean_hip.h).

Used by the tests, the smoke check and the benchmark; the C host layer links the
library directly. There is no fallback: if the library is missing, importing this
module raises.
"""
import ctypes as C
import os
import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libocean_hip.so")
if not os.path.exists(LIB_PATH):
    raise ImportError("%s is missing: build it with `make -C %s` (or __graft_entry__.build())" % (LIB_PATH, _HERE))
lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)

MAX_DIMS = 8
(BOOL, UINT8, UINT16, UINT32, UINT64, INT8, INT16, INT32, INT64,
 HALF, FLOAT, DOUBLE, CHALF, CFLOAT, CDOUBLE) = range(15)
DTYPE_NAMES = ["bool", "uint8", "uint16", "uint32", "uint64", "int8", "int16", "int32", "int64",
               "half", "float", "double", "chalf", "cfloat", "cdouble"]
TYPE_SIZE = [1, 1, 2, 4, 8, 1, 2, 4, 8, 2, 4, 8, 4, 8, 16]
# numpy storage dtype per element type; half travels as its 16-bit pattern, chalf as two of them
NP_STORAGE = [np.uint8, np.uint8, np.uint16, np.uint32, np.uint64, np.int8, np.int16, np.int32, np.int64,
              np.uint16, np.float32, np.float64, np.dtype([("real", np.uint16), ("imag", np.uint16)]),
              np.complex64, np.complex128]

UNARY_OPS = ["negative", "bitwise_not", "logical_not", "conj", "reciprocal", "sin", "cos", "tan", "sinh", "cosh",
             "tanh", "arcsin", "arccos", "arctan", "arcsinh", "arccosh", "arctanh", "sqrt", "cbrt", "square",
             "exp", "exp2", "exp10", "expm1", "log", "log2", "log10", "log1p", "absolute", "fabs", "sign",
             "ceil", "floor", "trunc", "round", "isinf", "isnan", "isfinite", "isposinf", "isneginf"]
BINARY_OPS = ["add", "subtract", "multiply", "divide", "true_divide", "floor_divide", "power", "mod", "fmod",
              "min", "max", "fmin", "fmax", "lt", "le", "eq", "ne", "ge", "gt",
              "bitwise_and", "bitwise_or", "bitwise_xor", "logical_and", "logical_or", "logical_xor",
              "bitshift_left", "bitshift_right"]
REDUCE_OPS = ["any", "all", "all_finite", "any_inf", "any_nan", "nnz", "nnz_nan",
              "all_lt", "all_le", "all_gt", "all_ge", "all_gtlt", "all_gtle", "all_gelt", "all_gele",
              "sum", "sum_nan", "prod", "prod_nan", "sum_abs", "sum_abs_nan",
              "maximum", "minimum", "maximum_abs", "minimum_abs", "norm", "norm_nan", "norm2", "norm2_nan"]
U = {n: i for i, n in enumerate(UNARY_OPS)}
B = {n: i for i, n in enumerate(BINARY_OPS)}
R = {n: i for i, n in enumerate(REDUCE_OPS)}


class CHalf(C.Structure):
    _fields_ = [("real", C.c_uint16), ("imag", C.c_uint16)]


class CFloat(C.Structure):
    _fields_ = [("real", C.c_float), ("imag", C.c_float)]


class CDouble(C.Structure):
    _fields_ = [("real", C.c_double), ("imag", C.c_double)]


class ScalarUnion(C.Union):
    _fields_ = [("_bool", C.c_uint8), ("_uint8", C.c_uint8), ("_uint16", C.c_uint16), ("_uint32", C.c_uint32),
                ("_uint64", C.c_uint64), ("_int8", C.c_int8), ("_int16", C.c_int16), ("_int32", C.c_int32),
                ("_int64", C.c_int64), ("_half", C.c_uint16), ("_float", C.c_float), ("_double", C.c_double),
                ("_chalf", CHalf), ("_cfloat", CFloat), ("_cdouble", CDouble)]


class Scalar(C.Structure):
    """och_scalar as ctypes can pass it BY VALUE. libffi lays a ctypes Union out like a struct of all
    members, which breaks the x86-64 calling convention; the C union's two eightbytes classify as
    INTEGER and SSE, exactly like this two-field structure of the same 16 bytes."""
    _fields_ = [("lo", C.c_uint64), ("hi", C.c_double)]


def make_scalar(dtype, value):
    """Scalar holding `value` as element type `dtype` (half types take bit patterns)."""
    u = ScalarUnion()
    C.memset(C.byref(u), 0, C.sizeof(u))
    name = "_" + DTYPE_NAMES[dtype]
    if dtype in (CHALF, CFLOAT, CDOUBLE):
        re, im = (value if isinstance(value, tuple) else (value.real, value.imag))
        f = getattr(u, name)
        f.real, f.imag = re, im
    else:
        setattr(u, name, value)
    s = Scalar()
    C.memmove(C.byref(s), C.byref(u), C.sizeof(s))
    return s


class ElemwisePlan(C.Structure):
    _fields_ = [("ndims", C.c_int), ("size", C.c_size_t * 8), ("strides", (C.c_ssize_t * 8) * 3), ("offset", C.c_ssize_t * 3),
                ("kernel", C.c_int), ("vec", C.c_int), ("launches", C.c_int),
                ("div_d", C.c_uint * 8), ("div_m", C.c_uint * 8), ("div_s1", C.c_uint * 8), ("div_s2", C.c_uint * 8),
                ("row_units", C.c_uint), ("row_elements", C.c_size_t)]


KERNEL_WIDE, KERNEL_MIXED, KERNEL_SINGLE, KERNEL_TILED, KERNEL_ROWS = 0, 1, 2, 3, 4


def elemwise_analyze(elemsizes, size, strides_per_operand, addresses):
    """och_elemwise_analyze for operands given by element size, byte strides and base address."""
    n = len(elemsizes)
    es = (C.c_int * n)(*elemsizes)
    st = (_st * n)(*[strides(s) for s in strides_per_operand])
    pp = (_vp * n)(*addresses)
    plan = ElemwisePlan()
    check(lib.och_elemwise_analyze(n, es, len(size), sizes(size), st, pp, C.byref(plan)))
    return plan


class DeviceProp(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("arch", C.c_char * 64), ("total_global_mem", C.c_size_t),
                ("shared_mem_per_block", C.c_size_t), ("multiprocessor_count", C.c_int), ("wavefront_size", C.c_int),
                ("max_threads_per_block", C.c_int), ("max_threads_per_multiprocessor", C.c_int),
                ("clock_rate_khz", C.c_int), ("memory_clock_rate_khz", C.c_int), ("memory_bus_width", C.c_int),
                ("l2_cache_size", C.c_int), ("pci_bus_id", C.c_int), ("pci_device_id", C.c_int),
                ("pci_domain_id", C.c_int), ("concurrent_kernels", C.c_int), ("ecc_enabled", C.c_int),
                ("free_global_mem", C.c_size_t), ("total_const_mem", C.c_size_t), ("mem_pitch", C.c_size_t),
                ("regs_per_block", C.c_int), ("max_threads_dim", C.c_int * 3), ("max_grid_size", C.c_int * 3),
                ("major", C.c_int), ("minor", C.c_int), ("async_engine_count", C.c_int),
                ("kernel_exec_timeout_enabled", C.c_int), ("integrated", C.c_int), ("can_map_host_memory", C.c_int),
                ("compute_mode", C.c_int), ("tcc_driver", C.c_int)]


class ReduceAxisConfig(C.Structure):
    _fields_ = [("ndims", C.c_int), ("size", C.c_size_t * MAX_DIMS), ("strides1", C.c_ssize_t * MAX_DIMS),
                ("strides2", C.c_ssize_t * MAX_DIMS), ("rdims", C.c_int), ("rsize", C.c_size_t * MAX_DIMS),
                ("rstrides", C.c_ssize_t * MAX_DIMS), ("ptr1", C.c_void_p), ("ptr2", C.c_void_p),
                ("stream", C.c_void_p)]


_sz = C.POINTER(C.c_size_t)
_st = C.POINTER(C.c_ssize_t)
_vp = C.c_void_p
_i = C.c_int

# every symbol that include/ocean_hip.h declares, with its argument types
PROTOTYPES = {
    "och_last_error": (C.c_char_p, []),
    "och_status_check": (_i, []),
    "och_status_clear": (None, []),
    "och_reduce_cut_parts": (C.c_longlong, [_i, C.POINTER(C.c_size_t), C.c_size_t, C.c_longlong, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "och_reduce_set_part_limit": (None, [C.c_size_t]),
    "och_reduce_axis_set_output_limit": (None, [C.c_size_t]),
    "och_reduce_axis_set_range_limit": (None, [C.c_size_t]),
    "och_stream_release_workspace": (C.c_int, [C.c_void_p]),
    "och_elemwise_set_launch_limit": (C.c_int, [C.c_size_t]),
    "och_device_count": (_i, [C.POINTER(_i)]),
    "och_device_set": (_i, [_i]),
    "och_device_get": (_i, [C.POINTER(_i)]),
    "och_device_properties": (_i, [_i, C.POINTER(DeviceProp)]),
    "och_device_mem_info": (_i, [_i, _sz, _sz]),
    "och_device_can_access_peer": (_i, [_i, _i, C.POINTER(_i)]),
    "och_device_warmup": (_i, [_i]),
    "och_device_synchronize": (_i, []),
    "och_stream_create": (_i, [C.POINTER(_vp)]),
    "och_stream_destroy": (_i, [_vp]),
    "och_stream_synchronize": (_i, [_vp]),
    "och_stream_wait_event": (_i, [_vp, _vp]),
    "och_event_create": (_i, [C.POINTER(_vp), _i]),
    "och_event_destroy": (_i, [_vp]),
    "och_event_record": (_i, [_vp, _vp]),
    "och_event_synchronize": (_i, [_vp]),
    "och_event_elapsed_ms": (_i, [_vp, _vp, C.POINTER(C.c_float)]),
    "och_malloc_async": (_i, [C.POINTER(_vp), C.c_size_t, _vp]),
    "och_free_async": (_i, [_vp, _vp]),
    "och_malloc_host": (_i, [C.POINTER(_vp), C.c_size_t]),
    "och_free_host": (_i, [_vp]),
    "och_memcpy_dtod_async": (_i, [_vp, _vp, C.c_size_t, _vp]),
    "och_memcpy_peer_async": (_i, [_vp, _i, _vp, _i, C.c_size_t, _vp]),
    "och_memcpy_htod": (_i, [_vp, _vp, C.c_size_t, _vp]),
    "och_memcpy_dtoh": (_i, [_vp, _vp, C.c_size_t, _vp]),
    "och_memcpy_htod_async": (_i, [_vp, _vp, C.c_size_t, _vp]),
    "och_memcpy_dtoh_async": (_i, [_vp, _vp, C.c_size_t, _vp]),
    "och_memset_async": (_i, [_vp, _i, C.c_size_t, _vp]),
    "och_stream_begin_capture": (_i, [_vp]),
    "och_stream_end_capture": (_i, [_vp, C.POINTER(C.c_void_p)]),
    "och_graph_launch": (_i, [_vp, _vp]),
    "och_graph_destroy": (_i, [_vp]),
    "och_fill": (_i, [_i, _i, _sz, _st, _vp, Scalar, _vp]),
    "och_fill_nan": (_i, [_i, _i, _sz, _st, _vp, Scalar, _vp]),
    "och_masked_fill": (_i, [_i, _i, _sz, _st, _vp, _st, _vp, Scalar, _vp]),
    "och_steps_int64": (_i, [_i, _i, _sz, _st, _vp, C.c_int64, C.c_int64, _vp]),
    "och_steps_double": (_i, [_i, _i, _sz, _st, _vp, C.c_double, C.c_double, _vp]),
    "och_steps_cdouble": (_i, [_i, _i, _sz, _st, _vp, CDouble, CDouble, _vp]),
    "och_copy": (_i, [_i, _i, _i, _sz, _st, _vp, _i, _sz, _st, _vp, _vp]),
    "och_byteswap_copy": (_i, [_i, _i, _i, _sz, _st, _vp, _i, _sz, _st, _vp, _vp]),
    "och_byteswap": (_i, [_i, _i, _sz, _st, _vp, _vp]),
    "och_unary": (_i, [_i, _i, _i, _sz, _st, _vp, _st, _vp, _vp]),
    "och_unary_supported": (_i, [_i, _i]),
    "och_unary_result_dtype": (_i, [_i, _i]),
    "och_binary": (_i, [_i, _i, _i, _sz, _st, _vp, _st, _vp, _st, _vp, _vp]),
    "och_binary_supported": (_i, [_i, _i]),
    "och_binary_operand2_dtype": (_i, [_i, _i]),
    "och_binary_result_dtype": (_i, [_i, _i]),
    "och_reduce_all_buffer_size": (C.c_size_t, []),
    "och_reduce_supported": (_i, [_i, _i]),
    "och_reduce_result_dtype": (_i, [_i, _i]),
    "och_reduce_all": (_i, [_i, _i, _i, _sz, _st, _vp, C.POINTER(Scalar), C.POINTER(Scalar), C.c_double, _vp, _vp, _vp]),
    "och_reduce_all_device": (_i, [_i, _i, _i, _sz, _st, _vp, C.POINTER(Scalar), C.POINTER(Scalar), C.c_double, _vp, _vp, _vp]),
    "och_reduce_all_device_noalloc": (_i, [_i, _i, _i, _sz, _st, _vp, C.POINTER(Scalar), C.POINTER(Scalar), C.c_double, _vp, _vp]),
    "och_reduce_all_noalloc_max_elements": (C.c_size_t, []),
    "och_reduce_axis": (_i, [_i, _i, C.POINTER(ReduceAxisConfig), C.c_double]),
    "och_gemm": (_i, [_i, C.c_char, C.c_char, C.c_size_t, C.c_size_t, C.c_size_t, _vp, _vp, C.c_ssize_t, _vp, C.c_ssize_t,
                      _vp, _vp, C.c_ssize_t, _i, _vp]),
    "och_gemm_supported": (_i, [_i]),
    "och_gemm_batched": (_i, [_i, C.c_char, C.c_char, C.c_size_t, C.c_size_t, C.c_size_t, _vp, _vp, C.c_ssize_t, _vp, C.c_ssize_t,
                              _vp, _vp, C.c_ssize_t, _i, _sz, _st, _st, _st, _st, _st, _i, _vp]),
    "och_mgs_project": (_i, [_i, C.c_size_t, C.c_size_t, _vp, C.c_ssize_t, _vp, _vp, _vp]),
    "och_add_if_negative": (_i, [_i, _i, _sz, _st, _vp, Scalar, _vp]),
    "och_index_to_offset": (_i, [_i, _i, C.POINTER(C.c_int64), C.c_ssize_t, C.c_size_t, C.c_ssize_t, _vp, C.c_ssize_t, _vp, _vp]),
    "och_get_index": (_i, [_i, _i, _sz, C.POINTER(C.POINTER(C.c_int64)), _st, _vp, _st, _vp, _vp]),
    "och_set_index": (_i, [_i, _i, _sz, C.POINTER(C.POINTER(C.c_int64)), _st, _vp, _st, _vp, _vp]),
    "och_fill_index": (_i, [_i, _i, _sz, C.POINTER(C.POINTER(C.c_int64)), _st, _vp, Scalar, _vp]),
    "och_find_workspace_size": (C.c_size_t, [C.c_size_t]),
    "och_find_count": (_i, [_i, _sz, _st, _vp, _vp, C.POINTER(C.c_size_t), _vp]),
    "och_find_apply": (_i, [_i, _sz, _st, _vp, _vp, C.POINTER(C.c_int64), _vp, _vp]),
    "och_elemwise_analyze": (_i, [_i, C.POINTER(_i), _i, _sz, C.POINTER(_st), C.POINTER(_vp), C.c_void_p]),
    "och_elemwise_row_unit": (_i, [C.c_uint, _i, _i, _i, C.c_size_t, C.POINTER(C.c_longlong), C.POINTER(_i), C.POINTER(_i)]),
    "och_elemwise_row_units": (C.c_size_t, [C.c_size_t, _i, _i]),
    "och_gemm_set_kernel_choice": (_i, [_i]),
    "och_gemm_float_plan": (_i, [C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint]),
    "och_gemm_split_plan": (_i, [C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint, C.c_uint, C.c_uint, C.c_uint, C.c_uint, C.POINTER(C.c_double)]),
}


def bind(library=lib):
    """Attach prototypes; returns the names that the library does not export."""
    missing = []
    for name, (res, args) in PROTOTYPES.items():
        try:
            fn = getattr(library, name)
        except AttributeError:
            missing.append(name)
            continue
        fn.restype, fn.argtypes = res, args
    return missing


MISSING = bind()


class OceanHipError(RuntimeError):
    pass


def check(status):
    if status != 0:
        raise OceanHipError(lib.och_last_error().decode())


def sizes(seq):
    return (C.c_size_t * max(1, len(seq)))(*seq)


def strides(seq):
    return (C.c_ssize_t * max(1, len(seq)))(*seq)


class Stream:
    def __init__(self):
        self.handle = C.c_void_p()
        check(lib.och_stream_create(C.byref(self.handle)))

    def synchronize(self):
        check(lib.och_stream_synchronize(self.handle))

    def destroy(self):
        if self.handle:
            check(lib.och_stream_destroy(self.handle))
            self.handle = C.c_void_p()


class Event:
    def __init__(self, timing=True):
        self.handle = C.c_void_p()
        check(lib.och_event_create(C.byref(self.handle), 1 if timing else 0))

    def record(self, stream):
        check(lib.och_event_record(self.handle, stream.handle))

    def synchronize(self):
        check(lib.och_event_synchronize(self.handle))

    def elapsed_ms(self, stop):
        ms = C.c_float()
        check(lib.och_event_elapsed_ms(self.handle, stop.handle, C.byref(ms)))
        return ms.value

    def destroy(self):
        if self.handle:
            check(lib.och_event_destroy(self.handle))
            self.handle = C.c_void_p()


class DeviceBuffer:
    """Raw device allocation, stream-ordered on `stream`."""

    def __init__(self, nbytes, stream):
        self.nbytes, self.stream = int(nbytes), stream
        self.ptr = C.c_void_p()
        check(lib.och_malloc_async(C.byref(self.ptr), max(self.nbytes, 1), stream.handle))

    @property
    def address(self):
        return self.ptr.value or 0

    def upload(self, array, offset=0):
        a = np.ascontiguousarray(array)
        check(lib.och_memcpy_htod(C.c_void_p(self.address + offset), a.ctypes.data_as(C.c_void_p), a.nbytes, self.stream.handle))

    def download(self, dtype, count=None, offset=0):
        dt = np.dtype(dtype)
        n = (self.nbytes - offset) // dt.itemsize if count is None else count
        out = np.empty(n, dtype=dt)
        check(lib.och_memcpy_dtoh(out.ctypes.data_as(C.c_void_p), C.c_void_p(self.address + offset), out.nbytes, self.stream.handle))
        return out

    def free(self):
        if self.ptr:
            check(lib.och_free_async(self.ptr, self.stream.handle))
            self.ptr = C.c_void_p()


def to_device(array, stream):
    a = np.ascontiguousarray(array)
    buf = DeviceBuffer(a.nbytes, stream)
    if a.nbytes:
        buf.upload(a)
    return buf


def device_properties(device=0):
    p = DeviceProp()
    check(lib.och_device_properties(device, C.byref(p)))
    return p


def device_count():
    n = C.c_int()
    check(lib.och_device_count(C.byref(n)))
    return n.value
