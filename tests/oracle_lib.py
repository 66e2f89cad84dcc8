"""ctypes binding of the CPU oracle (oracle/liboracle.so). The library of the reference's own operation macros
(oracle/_ref/libocean_ref.so) is mapped only when load_ref() is called, which the CPU tests that pin the oracle
against it do; nothing that runs on a GPU machine calls it. Test infrastructure only."""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_PATH = os.path.join(ROOT, "oracle", "liboracle.so")
REF_PATH = os.path.join(ROOT, "oracle", "_ref", "libocean_ref.so")

if not os.path.exists(ORACLE_PATH):
    raise ImportError("oracle/liboracle.so is missing: run `make -C oracle`")
lib = C.CDLL(ORACLE_PATH)
_ref = None


def ref_built():
    return os.path.exists(REF_PATH)


def load_ref():
    """The reference-macro library, mapped on first use."""
    global _ref
    if _ref is None:
        _ref = C.CDLL(REF_PATH)
        for name in ("ref_binary", "ref_unary", "ref_reduce", "ref_assign", "ref_swap_assign"):
            getattr(_ref, name).restype = C.c_void_p
        _proto(_ref.ref_half_to_float, C.c_float, [C.c_uint16])
        _proto(_ref.ref_float_to_half, C.c_uint16, [C.c_float])
    return _ref

_sz = C.POINTER(C.c_size_t)
_st = C.POINTER(C.c_ssize_t)
_vp = C.c_void_p
_i = C.c_int


def _proto(fn, res, args):
    fn.restype, fn.argtypes = res, args


def setup(oh):
    """Declare prototypes (needs the Scalar / config structures of the product binding)."""
    S = oh.Scalar
    _proto(lib.oracle_max_threads, _i, [])
    _proto(lib.oracle_binary, _i, [_i, _i, _i, _sz, _st, _vp, _st, _vp, _st, _vp])
    _proto(lib.oracle_binary_supported, _i, [_i, _i])
    _proto(lib.oracle_unary, _i, [_i, _i, _i, _sz, _st, _vp, _st, _vp, _i])
    _proto(lib.oracle_unary_supported, _i, [_i, _i])
    _proto(lib.oracle_copy, _i, [_i, _i, _i, _sz, _st, _vp, _i, _sz, _st, _vp, _i])
    _proto(lib.oracle_byteswap_copy, _i, [_i, _i, _i, _sz, _st, _vp, _i, _sz, _st, _vp, _i])
    _proto(lib.oracle_byteswap, _i, [_i, _i, _sz, _st, _vp, _i])
    _proto(lib.oracle_fill, _i, [_i, _i, _sz, _st, _vp, S, _i])
    _proto(lib.oracle_fill_nan, _i, [_i, _i, _sz, _st, _vp, S, _i])
    _proto(lib.oracle_masked_fill, _i, [_i, _i, _sz, _st, _vp, _st, _vp, S, _i])
    _proto(lib.oracle_steps_int64, _i, [_i, _i, _sz, _st, _vp, C.c_int64, C.c_int64, _i])
    _proto(lib.oracle_steps_double, _i, [_i, _i, _sz, _st, _vp, C.c_double, C.c_double, _i])
    _proto(lib.oracle_steps_cdouble, _i, [_i, _i, _sz, _st, _vp, oh.CDouble, oh.CDouble, _i])
    _proto(lib.oracle_half_to_float, C.c_float, [C.c_uint16])
    _proto(lib.oracle_float_to_half, C.c_uint16, [C.c_float])
    for name, res, args in [
        ("oracle_reduce_all", _i, [_i, _i, _i, _sz, _st, _vp, C.POINTER(S), C.POINTER(S), C.c_double, _vp, _i]),
        ("oracle_reduce_supported", _i, [_i, _i]),
        ("oracle_reduce_result_dtype", _i, [_i, _i]),
        ("oracle_reduce_axis", _i, [_i, _i, C.POINTER(oh.ReduceAxisConfig), C.c_double]),
        ("oracle_reduce_axis_threads", _i, [_i, _i, C.POINTER(oh.ReduceAxisConfig), C.c_double, _i]),
        ("oracle_gemm", _i, [_i, C.c_char, C.c_char, C.c_size_t, C.c_size_t, C.c_size_t, _vp, _vp, C.c_ssize_t, _vp,
                            C.c_ssize_t, _vp, _vp, C.c_ssize_t, _i]),
        ("oracle_add_if_negative", _i, [_i, _i, _sz, _st, _vp, S]),
        ("oracle_index_to_offset", _i, [_i, _i, C.POINTER(C.c_int64), C.c_ssize_t, C.c_size_t, C.c_ssize_t, _vp, C.c_ssize_t, _vp]),
        ("oracle_get_index", _i, [_i, _i, _sz, C.POINTER(C.POINTER(C.c_int64)), _st, _vp, _st, _vp]),
        ("oracle_set_index", _i, [_i, _i, _sz, C.POINTER(C.POINTER(C.c_int64)), _st, _vp, _st, _vp]),
        ("oracle_fill_index", _i, [_i, _i, _sz, C.POINTER(C.POINTER(C.c_int64)), _st, _vp, S]),
        ("oracle_find", C.c_size_t, [_i, _sz, _st, _vp, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    ]:
        if hasattr(lib, name):
            _proto(getattr(lib, name), res, args)


def ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def byte_strides(a):
    return list(a.strides)
