"""CPU checks of the host layer (no GPU): struct layouts against the numbers taken from the
reference's headers (tests/golden/abi_layout.json), the order of the function table, type
promotion and the shape routines against the reference's own dtype.c / shape.c (compiled into
oracle/_ref/libocean_ref_base.so where the reference tree is present), and the axis-reduction
analysis against brute-force enumeration."""
import ctypes as C
import itertools
import json
import os

import numpy as np
import pytest

import ocean_host as host

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_BASE = os.path.join(ROOT, "oracle", "_ref", "libocean_ref_base.so")
needs_ref = pytest.mark.skipif(not os.path.exists(REF_BASE), reason="oracle/_ref/libocean_ref_base.so not built")
_ref_base = []


def ref_base():
    """The reference's dtype.c and shape.c, mapped by the first CPU test that compares against them."""
    if not _ref_base:
        _ref_base.append(C.CDLL(REF_BASE))
    return _ref_base[0]


def test_struct_layouts_match_reference_headers():
    golden = json.load(open(os.path.join(ROOT, "tests", "golden", "abi_layout.json")))
    mine = json.loads(host.lib.OcHost_abiLayout())
    keys = [k for k in golden if not k.startswith("_")]
    assert len(keys) > 200
    assert sorted(keys) == sorted(mine.keys())
    wrong = {k: (mine[k], golden[k]) for k in keys if mine[k] != golden[k]}
    assert not wrong, wrong
    # ctypes mirrors used by the tests agree too
    assert C.sizeof(host.Tensor) == golden["sizeof(OcTensor)"] and C.sizeof(host.Storage) == golden["sizeof(OcStorage)"]
    assert C.sizeof(host.Scalar) == golden["sizeof(OcScalar)"]


def test_table_order_matches_reference_lists():
    golden = json.load(open(os.path.join(ROOT, "tests", "golden", "abi_layout.json")))
    text = open(os.path.join(ROOT, "ocean-tensor-package_amd", "host", "oc_op_tables.h")).read()
    import re
    def table(name):
        body = text.split("#define %s(X)" % name)[1].split("\n\n")[0].split("#define")[0]
        return re.findall(r"X\((\w+), (\d+)\)", body)
    unary, binary = table("OC_UNARY_TABLE"), table("OC_BINARY_TABLE")
    assert [n for n, _ in unary] == golden["_unary_order"]
    assert [n for n, _ in binary] == golden["_binary_order"]
    assert [int(i) for _, i in unary] == list(range(40)) and [int(i) for _, i in binary] == list(range(27))


@needs_ref
def test_common_type_matches_reference():
    for a in range(16):
        for b in range(16):
            assert host.lib.OcDType_getCommonType(a, b) == ref_base().OcDType_getCommonType(a, b), (a, b)


def test_common_type_examples():
    # the promotions the benchmark configurations rely on (float64 with int32, float with int16)
    assert host.lib.OcDType_getCommonType(host.DOUBLE, host.INT32) == host.DOUBLE
    assert host.lib.OcDType_getCommonType(host.FLOAT, host.INT16) == host.FLOAT
    assert host.lib.OcDType_getCommonType(host.FLOAT, host.INT32) == host.DOUBLE
    assert host.lib.OcDType_getCommonType(host.INT8, host.UINT8) == host.INT16
    assert host.lib.OcDType_getCommonType(host.INT64, host.UINT64) == host.DOUBLE
    assert host.lib.OcDType_getCommonType(host.CFLOAT, host.DOUBLE) == host.CDOUBLE


@needs_ref
def test_shape_routines_match_reference():
    rng = np.random.default_rng(8)
    ss = C.POINTER(C.c_ssize_t)
    ref_base().OcShape_sortStrides2.argtypes = [C.c_int, ss, ss, ss]
    ref_base().OcShape_mergeBlocks2.argtypes = [C.POINTER(C.c_int), ss, ss, ss]
    for _ in range(500):
        nd = int(rng.integers(0, 9))
        size = rng.integers(1, 6, nd)
        s1 = rng.choice([0, 4, 8, 16, 32, 64, 128, 256], nd)
        s2 = rng.choice([0, 4, 8, 16, 32, 64, 128, 256], nd)
        def run(libx):
            a, b, c = host._arr(list(size)), host._arr(list(s1)), host._arr(list(s2))
            libx.OcShape_sortStrides2(nd, a, b, c)
            n = C.c_int(nd)
            libx.OcShape_mergeBlocks2(C.byref(n), a, b, c)
            return n.value, list(a)[:n.value], list(b)[:n.value], list(c)[:n.value]
        assert run(host.lib) == run(ref_base()), (size, s1, s2)


@needs_ref
def test_extent_convention_matches_reference():
    """OcShape_extent and the blockOffset / blockExtent of a tensor follow the reference's convention (shape.c:82-125):
    the offset is the NON-NEGATIVE number of bytes in front of the data pointer, whatever the signs of the strides;
    zero strides add nothing. Compared with the reference's own shape.c on random shapes with negative and zero strides,
    and with the lowest / highest address a brute-force enumeration touches."""
    rng = np.random.default_rng(88)
    ss = C.POINTER(C.c_ssize_t)
    ref_base().OcShape_extent.argtypes = [C.c_int, ss, ss, C.c_ssize_t, ss, ss]
    cpu = host.cpu_device()
    for _ in range(400):
        nd = int(rng.integers(0, 6))
        size = [int(x) for x in rng.integers(1, 5, nd)]
        strides = [int(x) for x in rng.choice([-64, -24, -8, 0, 8, 16, 40, 128], nd)]
        es = 8
        out = []
        for libx in (host.lib, ref_base()):
            off, ext = C.c_ssize_t(-1), C.c_ssize_t(-1)
            assert libx.OcShape_extent(nd, host._arr(size), host._arr(strides), es, C.byref(off), C.byref(ext)) == 0
            out.append((off.value, ext.value))
        assert out[0] == out[1], (size, strides, out)
        offs = _offsets(size, strides).reshape(-1)
        assert out[0] == (-int(offs.min()), int(offs.max() - offs.min()) + es), (size, strides)
        # a tensor over a storage large enough carries the same numbers
        t = host.create(size, host.DOUBLE, cpu, strides)
        assert (t.contents.blockOffset, t.contents.blockExtent) == out[0]
        assert t.contents.offset == out[0][0]                      # the data pointer sits blockOffset bytes into the block
        host.lib.OcDecrefTensor(t)


def test_device_module_compiles_against_the_reference_headers():
    """host/gpu_module.c is written against Ocean's base API only: with OC_REFERENCE_HEADERS it is compiled (syntax and
    types only; nothing is linked, run or kept) against the reference's own headers, which pins every signature, macro
    and field name the module relies on. Skipped where the reference tree is not present."""
    import subprocess
    if not os.path.isdir("/root/reference/include/ocean"):
        pytest.skip("reference tree not present")
    pkg = os.path.join(ROOT, "ocean-tensor-package_amd")
    r = subprocess.run(["make", "-C", pkg, "host-ref-check"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "host-ref-check: ok" in r.stdout


def _offsets(size, strides):
    tot = np.zeros([int(s) for s in size] or [1], dtype=np.int64)
    for d, (n, s) in enumerate(zip(size, strides)):
        shape = [1] * len(size); shape[d] = int(n)
        tot = tot + (np.arange(int(n), dtype=np.int64) * int(s)).reshape(shape)
    return tot


def test_axis_analysis_enumerates_the_same_elements():
    """For random strided sources, the (outer, reduced) decomposition must visit, for every destination
    element, exactly the source elements that the reduction over `axes` assigns to it."""
    rng = np.random.default_rng(21)
    cpu = host.cpu_device()
    for trial in range(200):
        nd = int(rng.integers(1, 5))
        shape = [int(x) for x in rng.integers(1, 5, nd)]
        perm = rng.permutation(nd)
        strides = [0] * nd; acc = 4
        for d in perm:
            sign = -1 if rng.integers(0, 4) == 0 else 1
            strides[d] = acc * sign; acc *= shape[d] * int(rng.integers(1, 3))
        src = host.create(shape, host.FLOAT, cpu, strides)
        k = int(rng.integers(1, nd + 1))
        axes = sorted(int(a) for a in rng.choice(nd, k, replace=False))
        keep = bool(rng.integers(0, 2))
        dshape = [1 if d in axes else shape[d] for d in range(nd)] if keep else [shape[d] for d in range(nd) if d not in axes]
        dst = host.create(dshape, host.FLOAT, cpu)
        cfg = host.ReduceAxis()
        host.lib.OcSolid_analyzeReduceAxis(C.byref(cfg), src, dst, k, (C.c_int * k)(*axes), 0)
        offset1, offset2 = cfg.ptr1 - host.data_address(src), cfg.ptr2 - host.data_address(dst)
        # expected: map destination offset -> sorted list of source offsets
        so = _offsets(shape, strides)
        dstrides = [dst.contents.strides[i] for i in range(dst.contents.ndims)]
        full_d = [0 if d in axes else dstrides[d if keep else [x for x in range(nd) if x not in axes].index(d)] for d in range(nd)]
        do = _offsets(shape, full_d)
        want = {}
        for s, d in zip(so.reshape(-1), do.reshape(-1)):
            want.setdefault(int(d), []).append(int(s))
        # got: enumerate the analysed configuration
        osz = [cfg.size[i] for i in range(cfg.ndims)]; o1 = [cfg.strides1[i] for i in range(cfg.ndims)]; o2 = [cfg.strides2[i] for i in range(cfg.ndims)]
        rsz = [cfg.rsize[i] for i in range(cfg.rdims)]; rs = [cfg.rstrides[i] for i in range(cfg.rdims)]
        outer1 = _offsets(osz, o1).reshape(-1) + offset1; outer2 = _offsets(osz, o2).reshape(-1) + offset2
        inner = _offsets(rsz, rs).reshape(-1)
        got = {int(d): sorted(int(s + i) for i in inner) for s, d in zip(outer1, outer2)}
        assert {k2: sorted(v) for k2, v in want.items()} == got, (shape, strides, axes, keep)
        host.lib.OcDecrefTensor(src); host.lib.OcDecrefTensor(dst)


def test_views_and_errors():
    cpu = host.cpu_device()
    t = host.create([4, 6], host.DOUBLE, cpu)
    tt = host.lib.OcTensor_transpose(t)
    assert host.shape_of(tt) == [6, 4] and [tt.contents.strides[i] for i in range(2)] == [32, 8]
    sl = host.lib.OcTensor_slice(t, 0, 1, 2, 2)
    assert host.shape_of(sl) == [2, 6] and sl.contents.offset == t.contents.offset + 8 and sl.contents.strides[0] == 16
    assert not host.lib.OcTensor_slice(t, 0, 3, 2, 2)            # out of range
    assert b"out of range" in host.lib.OcError_lastMessage()
    b = host.lib.OcTensor_broadcastTo(host.create([1, 6], host.DOUBLE, cpu), 2, host._arr([4, 6]))
    assert [b.contents.strides[i] for i in range(2)] == [0, 8]
    # without OcInitGPU no device module is registered for a made-up device
    with pytest.raises(host.OceanError):
        host.check(host.lib.OcTensor_binary(99, t, t, C.byref(host.TP())))


REF_GPU_HEADERS = "/root/reference/include/ocean/core/gpu"
# Names the reference's GPU headers export that this module deliberately does not, and why:
EXEMPT_EXPORTS = {
    "OcInitCuda": "cuda.h:30 -- CUDA runtime bring-up; the device library initialises HIP on first use",
    "OcCuda_setDevice": "cuda.h:33 -- takes no CUDA-typed argument, but belongs to the CUDA status helpers below; och_device_set",
    "OcCuda_setStatus": "cuda.h:36 -- argument is a cudaError_t; the device library keeps the first-error status (och_status_check)",
    "OcCuda_clearStatus": "cuda.h:37 -- same protocol, och_status_clear",
    "OcCuda_checkStatus": "cuda.h:38 -- same protocol, och_status_check",
    "OcModuleCoreGPU_cublasHandle": "module_core_gpu.h:40 -- returns a cublasHandle_t; the MFMA GEMM kernels need no handle",
}


def exported_symbols(path):
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", path], check=True, capture_output=True, text=True).stdout
    return {line.split()[-1] for line in out.splitlines() if line.strip()}


@pytest.mark.skipif(not os.path.isdir(REF_GPU_HEADERS), reason="reference tree not present")
def test_every_public_name_of_the_reference_gpu_headers_is_exported():
    """Every OC_API function of include/ocean/core/gpu/**/*.h is an exported symbol of the host library, except
    the CUDA-typed helpers listed above."""
    import re
    names = set()
    for folder, _, files in os.walk(REF_GPU_HEADERS):
        for f in files:
            if f.endswith(".h"):
                text = open(os.path.join(folder, f)).read()
                names.update(re.findall(r"OC_API\s+[\w\s\*]*?\b(\w+)\s*\(", text))
    assert len(names) >= 30 and "OcDeviceGPU_updateProperties" in names and "OcBufferGPU_zero" in names
    have = exported_symbols(host.LIB_PATH)
    missing = sorted(n for n in names if n not in have and n not in EXEMPT_EXPORTS)
    assert not missing, missing
    assert not [n for n in EXEMPT_EXPORTS if n not in names], "exemption for a name the reference does not have"
    assert "OcGPU" in have and "OcInitGPU" in have and "OcFinalizeGPU" in have           # include/ocean_gpu.h


def test_module_header_declares_what_the_library_exports():
    """include/ocean_gpu_module.h and the library agree: every function the header declares is exported."""
    import re
    text = open(os.path.join(ROOT, "include", "ocean_gpu_module.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(Oc\w+)\s*\(", text))
    assert {"OcInitGPU", "OcDeviceGPU_updateProperties", "OcInitDevicesGPU", "OcInitModuleCore_GPU", "OcRegisterStorageGPU",
            "OcBufferGPU_copyHostToStorage", "OcBufferGPU_copyStorageToHost", "OcRegisterTensorGPU"} <= declared
    have = exported_symbols(host.LIB_PATH)
    assert not sorted(declared - have), sorted(declared - have)


@pytest.mark.skipif(not os.path.isdir(REF_GPU_HEADERS), reason="reference tree not present")
def test_public_device_properties_have_the_reference_fields_in_order():
    """OcDevicePropGPU of include/ocean_gpu_module.h lists the live fields of the reference's struct
    (device_gpu.h:31-106) with the same types in the same order, and the ctypes mirror agrees with both."""
    import re

    def fields(text, closing):
        body = text[:text.index(closing)]
        body = body[body.rindex("typedef struct"):]
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        out = []
        for ctype, decl in re.findall(r"\b(char|size_t|int)\s+([^;]+);", body):
            for d in decl.split(","):
                m = re.match(r"\s*(\w+)\s*(\[\d+\])?\s*$", d)
                out.append((ctype, m.group(1), m.group(2) or ""))
        return out
    ref = fields(open(os.path.join(REF_GPU_HEADERS, "device_gpu.h")).read(), "} OcDevicePropGPU;")
    mine = fields(open(os.path.join(ROOT, "include", "ocean_gpu_module.h")).read(), "} OcDevicePropGPU;")
    assert len(ref) >= 45 and mine == ref
    assert [n for n, _ in host.DevicePropGPU._fields_] == [n for _, n, _ in ref]
    sizes = {"char": 1, "size_t": 8, "int": 4}
    for (ctype, name, dim), (fname, ftype) in zip(ref, host.DevicePropGPU._fields_):
        count = int(dim[1:-1]) if dim else 1
        assert C.sizeof(ftype) == sizes[ctype] * count, name
