"""ctypes binding of csrc/libocean_hip_bench.so (include/ocean_hip_bench.h): the streaming and matrix-core
micro-benchmarks that bench.py sets the library's kernels against. Measurement tools, not part of the product ABI."""
import ctypes as C
import os

import ocean_hip as _oh                      # the product library first: the benchmarks report errors through it

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libocean_hip_bench.so")
if not os.path.exists(LIB_PATH):
    raise ImportError("%s is missing: build it with `make -C %s`" % (LIB_PATH, _HERE))
lib = C.CDLL(LIB_PATH)
_i, _vp = C.c_int, C.c_void_p
lib.och_mfmabench.restype = _i
lib.och_mfmabench.argtypes = [_i, _i, _i, _i, _i, _i, C.POINTER(C.c_float), C.POINTER(C.c_double), _vp]
lib.och_membench.restype = _i
lib.och_membench.argtypes = [_i, _i, _i, _i, _i, _i, C.c_size_t, _i, _i, C.POINTER(C.c_float), C.POINTER(C.c_float), C.POINTER(C.c_size_t), _vp]
check = _oh.check
