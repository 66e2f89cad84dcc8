#!/usr/bin/env python3
"""Benchmark of the MI355X device module on the five reference workload configurations (one GPU).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only-step]

One "step" is one pass of configuration 2 through the device library, as Ocean's interface
layer would issue it for   Z = (A.T + r + I) * F   with
    A  float64 4096 x 4096, used through its transposed view (non-unit strides)
    r  float64 1 x 4096 row, broadcast along dimension 0 (zero stride)
    I  int32 4096 x 4096, auto-cast to float64 by a converting copy
    F  float32 4096 x 4096 stored byte-swapped, brought to native float64 by a swapping copy
i.e. five launches: add(A.T, r) -> Z ; copy(I) -> TI ; add(Z, TI) -> Z ; byteswap_copy(F) -> TF ;
multiply(Z, TF) -> Z.  Values are U(-10, 10) from a fixed seed; inputs are resident in HBM before
the timed region.  value = algorithmic bytes of the step / time (GB/s): every logical input element
read once, every output element written once, the broadcast row counted once.

Printed: ONE JSON line with the driver's fields plus
    roofline      dominant kernel of the step: algorithmic bytes per launch / mean launch time
                  (HIP events on the launch stream) against the 8 TB/s HBM peak
    kernels       the same figure for every kernel of the step
    configs       short measurements of configurations 1, 3, 4 and 5 (GB/s or TFLOP/s)
    cpu_baseline  the CPU oracle (a port of Ocean's CPU path with its threading policy:
                  binary operations serial, copies over all cores) timed on this host on the
                  same full-size step
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ocean-tensor-package_amd"))

HBM_PEAK_GBS = 8000.0
MFMA_PEAK = {"float": 157.3, "double": 78.6, "cfloat": 157.3, "cdouble": 78.6}

N2 = 4096


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="skip the graph-replay variant of the MGS window (rocprofv3's kernel tracing crashes inside hipGraphLaunch)")
    ap.add_argument("--only-step", action="store_true", help="time the configuration-2 step only (for profiling)")
    ap.add_argument("--only-gemm", action="store_true", help="run each configuration-5 GEMM twice and exit (for counter collection)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus %d is not supported (every figure here is a one-GPU figure)" % args.gpus)

    import numpy as np
    import ocean_hip as oh

    oh.check(oh.lib.och_device_set(0))
    oh.check(oh.lib.och_device_warmup(0))
    prop = oh.device_properties(0)
    stream = oh.Stream()
    lib = oh.lib
    B, R = oh.B, oh.R
    if args.only_gemm:
        rng = np.random.default_rng(5)
        for dt, es, nm, dim in ((oh.DOUBLE, 8, "double", 8192), (oh.FLOAT, 4, "float", 8192), (oh.CFLOAT, 8, "cfloat", 4096)):
            a, b, c = [oh.DeviceBuffer(es * dim * dim, stream) for _ in range(3)]
            block = rng.uniform(-1, 1, 1 << 22).astype(np.float32 if nm != "double" else np.float64)
            for buf in (a, b):
                for off in range(0, es * dim * dim, block.nbytes):
                    buf.upload(block[: (min(block.nbytes, es * dim * dim - off)) // block.itemsize], offset=off)
            one = np.array([1, 0], dtype=block.dtype); zero = np.zeros(2, dtype=block.dtype)
            for ta, tb in ((b"N", b"N"), (b"T", b"N"), (b"N", b"T")):
                for _ in range(2):
                    oh.check(lib.och_gemm(dt, ta, tb, dim, dim, dim, one.ctypes.data, a.ptr, dim, b.ptr, dim, zero.ctypes.data, c.ptr, dim, 1, stream.handle))
            stream.synchronize()
            for buf in (a, b, c):
                buf.free()
        print(json.dumps({"mode": "only-gemm"}))
        return
    F32, F64, I32, I16, CF, CD = oh.FLOAT, oh.DOUBLE, oh.INT32, oh.INT16, oh.CFLOAT, oh.CDOUBLE

    def time_launches(fn, reps=20, warm=3):
        """mean duration in ms of one call of fn(), measured with events on the launch stream"""
        for _ in range(warm):
            fn()
        e0, e1 = oh.Event(), oh.Event()
        e0.record(stream)
        for _ in range(reps):
            fn()
        e1.record(stream)
        e1.synchronize()
        ms = e0.elapsed_ms(e1) / reps
        e0.destroy(); e1.destroy()
        return ms

    # ------------------------------------------------------------------ configuration 2
    n = N2
    rng = np.random.default_rng(20240)
    hostA = rng.uniform(-10, 10, (n, n))
    hostR = rng.uniform(-10, 10, n)
    hostI = rng.integers(-10, 10, (n, n), endpoint=True).astype(np.int32)
    hostF = rng.uniform(-10, 10, (n, n)).astype(np.float32)
    hostFs = hostF.byteswap()
    NSETS = 3
    sets = []
    for _ in range(NSETS):
        s = {"A": oh.to_device(hostA, stream), "r": oh.to_device(hostR, stream), "I": oh.to_device(hostI, stream),
             "F": oh.to_device(hostFs, stream), "Z": oh.DeviceBuffer(8 * n * n, stream),
             "TI": oh.DeviceBuffer(8 * n * n, stream), "TF": oh.DeviceBuffer(8 * n * n, stream)}
        sets.append(s)
    shape = oh.sizes([n, n])
    st_f64, st_f64_T, st_row = oh.strides([8, 8 * n]), oh.strides([8 * n, 8]), oh.strides([0, 8])
    st_i32, st_f32 = oh.strides([4, 4 * n]), oh.strides([4, 4 * n])
    h = stream.handle

    def k_add_transposed(s):
        oh.check(lib.och_binary(B["add"], F64, 2, shape, st_f64_T, s["A"].ptr, st_row, s["r"].ptr, st_f64, s["Z"].ptr, h))

    def k_cast_i32(s):
        oh.check(lib.och_copy(I32, F64, 2, shape, st_i32, s["I"].ptr, 2, shape, st_f64, s["TI"].ptr, h))

    def k_add(s):
        oh.check(lib.och_binary(B["add"], F64, 2, shape, st_f64, s["Z"].ptr, st_f64, s["TI"].ptr, st_f64, s["Z"].ptr, h))

    def k_cast_swapped(s):
        oh.check(lib.och_byteswap_copy(F32, F64, 2, shape, st_f32, s["F"].ptr, 2, shape, st_f64, s["TF"].ptr, h))

    def k_multiply(s):
        oh.check(lib.och_binary(B["multiply"], F64, 2, shape, st_f64, s["Z"].ptr, st_f64, s["TF"].ptr, st_f64, s["Z"].ptr, h))

    nn = n * n
    step_kernels = [
        ("add f64: transposed view + row broadcast", k_add_transposed, 8 * nn * 2 + 8 * n),
        ("copy int32 -> f64", k_cast_i32, 12 * nn),
        ("add f64 contiguous", k_add, 24 * nn),
        ("byteswap_copy f32 (swapped) -> f64", k_cast_swapped, 12 * nn),
        ("multiply f64 contiguous", k_multiply, 24 * nn),
    ]
    step_bytes = sum(b for _, _, b in step_kernels)

    def step(i):
        s = sets[i % NSETS]
        for _, fn, _ in step_kernels:
            fn(s)

    for i in range(args.warmup):
        step(i)
    stream.synchronize()
    oh.check(lib.och_device_synchronize())
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    stream.synchronize()
    oh.check(lib.och_device_synchronize())
    ms_per_step = (time.perf_counter() - t0) * 1e3 / max(args.steps, 1)
    value = step_bytes / ms_per_step / 1e6

    result = {
        "metric": "elementwise/reduction HBM GB/s (% of peak); fp32/fp64 GEMM TFLOP/s",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64", "data": "synthetic",
        "config": {"workload": "config 2: Z = (A.T + r + I) * F, float64 4096x4096 transposed view + 1x4096 row broadcast, "
                               "int32 operand cast to float64, byteswapped float32 operand; 5 launches, %.1f MB algorithmic" % (step_bytes / 1e6),
                   "device": prop.arch.decode(), "compute_units": prop.multiprocessor_count,
                   "percent_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 1)},
    }
    if args.only_step:
        # one plain float64 -> float64 copy of known size (134.2 MB read, 134.2 MB written): the
        # yardstick that scales the FETCH_SIZE / WRITE_SIZE counters of a profiling run
        oh.check(lib.och_copy(F64, F64, 2, shape, st_f64, sets[0]["TI"].ptr, 2, shape, st_f64, sets[0]["TF"].ptr, h))
        stream.synchronize()
        print(json.dumps(result))
        return

    # per-kernel roofline of the step
    kernels = []
    for name, fn, nbytes in step_kernels:
        turn = [0]

        def rotating(fn=fn, turn=turn):          # alternate the buffer sets, as the step loop does
            turn[0] += 1
            fn(sets[turn[0] % NSETS])
        ms = time_launches(rotating)
        kernels.append({"kernel": name, "ms": round(ms, 4), "algorithmic_MB": round(nbytes / 1e6, 1),
                        "GBps": round(nbytes / ms / 1e6, 1), "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 3)})
    dom = max(kernels, key=lambda k: k["ms"])
    # HBM bytes per launch of that kernel as counted by rocprofv3 (FETCH_SIZE + WRITE_SIZE, scaled by a
    # copy kernel of known size; profiles/elementwise_config2_hbm_traffic.txt), over the same duration
    traffic, traffic_bytes = None, None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            t = json.load(f).get(dom["kernel"])
        if t:
            traffic_bytes = t["fetch_bytes"] + t["write_bytes"]
            traffic = round(traffic_bytes / dom["ms"] / 1e6, 1)
    result["roofline"] = {"bound": "hbm", "kernel": dom["kernel"], "achieved": dom["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(dom["GBps"] / HBM_PEAK_GBS, 3), "traffic": traffic,
                          "algorithmic_bytes_per_launch": next(b for nm, _, b in step_kernels if nm == dom["kernel"]),
                          "traffic_bytes_per_launch": traffic_bytes, "launch_ms": dom["ms"]}
    result["kernels"] = kernels
    for s in sets:
        for b in s.values():
            b.free()
    stream.synchronize()

    configs = {}

    def gbps(nbytes, ms):
        return {"ms": round(ms, 4), "GBps": round(nbytes / ms / 1e6, 1), "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 3)}

    # ------------------------------------------------------------------ configuration 1
    n1 = 1 << 24
    # six buffer sets (6 x 256 MB) so that successive launches never find their operands in the 256 MB Infinity Cache
    c1sets = []
    for i in range(6):
        bufs = [oh.DeviceBuffer(4 * n1, stream) for _ in range(4)]
        bufs[0].upload(rng.uniform(-1, 1, n1).astype(np.float32)); bufs[1].upload(rng.uniform(-1, 1, n1).astype(np.float32))
        c1sets.append(bufs)
    s1, st1 = oh.sizes([n1]), oh.strides([4])
    turn = [0]

    def c1_scale():
        x, y, t, z = c1sets[turn[0] % 6]; turn[0] += 1
        oh.check(lib.och_binary(B["multiply"], F32, 1, s1, st1, x.ptr, st1, y.ptr, st1, t.ptr, h))

    def c1_add():
        x, y, t, z = c1sets[turn[0] % 6]; turn[0] += 1
        oh.check(lib.och_binary(B["add"], F32, 1, s1, st1, t.ptr, st1, x.ptr, st1, z.ptr, h))
    ms_mul = time_launches(c1_scale, reps=30)
    ms_add = time_launches(c1_add, reps=30)
    configs["c1_scale_f32_2^24"] = gbps(12 * n1, ms_mul)
    configs["c1_add_f32_2^24"] = gbps(12 * n1, ms_add)
    for bufs in c1sets:
        for b in bufs:
            b.free()

    # ------------------------------------------------------------------ configuration 3
    n3 = 8192 * 8192
    for dt, es, nm in ((F32, 4, "f32"), (F64, 8, "f64")):
        rbufs = [oh.DeviceBuffer(es * n3, stream) for _ in range(2)]          # alternate: no reuse from the Infinity Cache
        chunk = rng.standard_normal(1 << 22).astype(np.float32 if es == 4 else np.float64)
        for buf in rbufs:
            for off in range(0, n3, 1 << 22):
                buf.upload(chunk, offset=off * es)
        rturn = [0]

        def next_buf():
            rturn[0] += 1
            return rbufs[rturn[0] % 2]
        dres = oh.DeviceBuffer(64, stream)
        s3, st3 = oh.sizes([n3]), oh.strides([es])
        for opn in ("sum", "norm2", "maximum"):
            ms = time_launches(lambda: oh.check(lib.och_reduce_all_device(R[opn], dt, 1, s3, st3, next_buf().ptr, None, None, 0.0, dres.ptr, None, h)), reps=10)
            configs["c3_%s_%s_8192^2" % (opn, nm)] = gbps(es * n3, ms)
        # two more axis reductions over the same dense 2^26 elements, outside the named configurations: few outputs with
        # a long strided reduced range (cut into pieces and folded by a second kernel), and many outputs of 8 elements each
        few = oh.DeviceBuffer(es * 64, stream); many = oh.DeviceBuffer(es * (1 << 23), stream)
        for label, osize, ostride, rsize, rstride, dest in (("64x2^20_axis1_few_outputs", 64, es, 1 << 20, 64 * es, few),
                                                            ("8x2^23_axis0_short_rows", 1 << 23, 8 * es, 8, es, many)):
            assert (osize - 1) * ostride + (rsize - 1) * rstride + es <= es * n3 and osize * es <= dest.nbytes
            ecfgs = []
            for buf in rbufs:
                cfg = oh.ReduceAxisConfig()
                cfg.ndims, cfg.rdims = 1, 1
                cfg.size[0], cfg.strides1[0], cfg.strides2[0] = osize, ostride, es
                cfg.rsize[0], cfg.rstrides[0] = rsize, rstride
                cfg.ptr1, cfg.ptr2, cfg.stream = buf.ptr.value, dest.ptr.value, h
                ecfgs.append(cfg)
            eturn = [0]

            def next_ecfg():
                eturn[0] += 1
                return ecfgs[eturn[0] % 2]
            ms = time_launches(lambda: oh.check(lib.och_reduce_axis(R["sum"], dt, C.byref(next_ecfg()), 0.0)), reps=10)
            configs["extra_axis_sum_%s_%s" % (nm, label)] = gbps(es * (n3 + osize), ms)
        few.free(); many.free()
        # axis reductions on a 512 x 512 x 256 view with padded pitches (no two dimensions merge);
        # the view lives in a parent of (512+4) x (512+2) x 256 elements
        d0, d1, d2 = 512, 512, 256
        p0, p1 = (d0 + 4) * es, (d0 + 4) * (d1 + 2) * es
        parent_bytes = p1 * d2
        extent = (d0 - 1) * es + (d1 - 1) * p0 + (d2 - 1) * p1 + es
        assert extent <= parent_bytes, "axis view exceeds its parent buffer"
        abufs = [oh.DeviceBuffer(parent_bytes, stream) for _ in range(2)]     # alternate: no reuse from the Infinity Cache
        for abuf in abufs:
            for off in range(0, parent_bytes, chunk.nbytes):
                m = min(chunk.nbytes, parent_bytes - off) // chunk.itemsize
                abuf.upload(chunk[:m], offset=off)
        out = oh.DeviceBuffer(es * d0 * d1, stream)
        for axis, keep in ((0, (d1, d2)), (1, (d0, d2))):
            cfgs = []
            for abuf in abufs:
                cfg = oh.ReduceAxisConfig()
                cfg.ndims = 2
                if axis == 0:
                    cfg.size[0], cfg.size[1] = d1, d2; cfg.strides1[0], cfg.strides1[1] = p0, p1
                    cfg.rsize[0], cfg.rstrides[0] = d0, es
                else:
                    cfg.size[0], cfg.size[1] = d0, d2; cfg.strides1[0], cfg.strides1[1] = es, p1
                    cfg.rsize[0], cfg.rstrides[0] = d1, p0
                cfg.strides2[0], cfg.strides2[1] = es, es * keep[0]
                assert es * keep[0] * keep[1] <= es * d0 * d1
                cfg.rdims = 1; cfg.ptr1, cfg.ptr2, cfg.stream = abuf.ptr.value, out.ptr.value, h
                cfgs.append(cfg)
            aturn = [0]

            def next_cfg():
                aturn[0] += 1
                return cfgs[aturn[0] % 2]
            for opn in ("sum", "minimum"):
                ms = time_launches(lambda: oh.check(lib.och_reduce_axis(R[opn], dt, C.byref(next_cfg()), 0.0)), reps=10)
                configs["c3_axis%d_%s_%s_512x512x256" % (axis, opn, nm)] = gbps(es * (d0 * d1 * d2 + keep[0] * keep[1]), ms)
        for b in rbufs + abufs + [dres, out]:
            b.free()

    # ------------------------------------------------------------------ configuration 4
    d0, d1, d2 = 1024, 1024, 64
    n4 = d0 * d1 * d2
    src = oh.DeviceBuffer(2 * 2 * n4, stream); dst = oh.DeviceBuffer(4 * n4, stream)
    chunk = rng.integers(-32768, 32767, 1 << 22, dtype=np.int16, endpoint=True)
    for off in range(0, 2 * n4, 1 << 22):
        src.upload(chunk, offset=off * 2)
    sz4 = oh.sizes([d0, d1, d2])
    st_src, st_dst = oh.strides([4, 4 * d0, 4 * d0 * d1]), oh.strides([4, 4 * d0, 4 * d0 * d1])
    ms = time_launches(lambda: oh.check(lib.och_byteswap_copy(I16, F32, 3, sz4, st_src, src.ptr, 3, sz4, st_dst, dst.ptr, h)), reps=10)
    configs["c4_int16_swapped_step2_to_f32_1024x1024x64"] = gbps(6 * n4, ms)
    src.free(); dst.free()
    n4b = 1 << 26
    src = oh.DeviceBuffer(8 * n4b, stream); dst = oh.DeviceBuffer(16 * n4b, stream)
    oh.check(lib.och_memset_async(src.ptr, 0, 8 * n4b, h))
    s4, sa, sb = oh.sizes([n4b]), oh.strides([8]), oh.strides([16])
    ms = time_launches(lambda: oh.check(lib.och_copy(CF, CD, 1, s4, sa, src.ptr, 1, s4, sb, dst.ptr, h)), reps=10)
    configs["c4_cfloat_to_cdouble_2^26"] = gbps(24 * n4b, ms)
    src.free(); dst.free()

    # ------------------------------------------------------------------ configuration 5 (GEMM)
    if "och_gemm" not in oh.MISSING:
        for dt, es, nm, dim, flop_per_mac in ((F64, 8, "double", 8192, 2), (F32, 4, "float", 8192, 2), (CF, 8, "cfloat", 4096, 8)):
            if not lib.och_gemm_supported(dt):
                continue
            a, b, c = [oh.DeviceBuffer(es * dim * dim, stream) for _ in range(3)]
            block = rng.uniform(-1, 1, 1 << 22).astype(np.float32 if nm != "double" else np.float64)
            for buf in (a, b):
                for off in range(0, es * dim * dim, block.nbytes):
                    buf.upload(block[: (min(block.nbytes, es * dim * dim - off)) // block.itemsize], offset=off)
            one = np.array([1, 0], dtype=block.dtype); zero = np.zeros(2, dtype=block.dtype)
            for ta, tb in ((b"N", b"N"), (b"T", b"N"), (b"N", b"T")):
                fn = lambda: oh.check(lib.och_gemm(dt, ta, tb, dim, dim, dim, one.ctypes.data, a.ptr, dim, b.ptr, dim,
                                                   zero.ctypes.data, c.ptr, dim, 1, h))
                ms = time_launches(fn, reps=3, warm=1)
                tf = flop_per_mac * dim ** 3 / ms / 1e9
                configs["c5_gemm_%s_%d_%s%s" % (nm, dim, ta.decode(), tb.decode())] = {
                    "ms": round(ms, 3), "TFLOPs": round(tf, 2), "frac": round(tf / MFMA_PEAK[nm], 3)}
            for buf in (a, b, c):
                buf.free()
        # beyond the named configurations: the half-precision product of the same size (float accumulation, one rounding)
        if lib.och_gemm_supported(oh.HALF):
            dim = 8192
            a, b, c = [oh.DeviceBuffer(2 * dim * dim, stream) for _ in range(3)]
            block = rng.uniform(-1, 1, 1 << 22).astype(np.float16)
            for buf in (a, b):
                for off in range(0, 2 * dim * dim, block.nbytes):
                    buf.upload(block, offset=off)
            one16 = np.array([0x3C00, 0], np.uint16); zero16 = np.zeros(2, np.uint16)
            for ta, tb in ((b"N", b"N"), (b"T", b"N"), (b"N", b"T")):
                fn = lambda: oh.check(lib.och_gemm(oh.HALF, ta, tb, dim, dim, dim, one16.ctypes.data, a.ptr, dim, b.ptr, dim,
                                                   zero16.ctypes.data, c.ptr, dim, 1, h))
                ms = time_launches(fn, reps=3, warm=1)
                tf = 2 * dim ** 3 / ms / 1e9
                configs["extra_gemm_half_%d_%s%s" % (dim, ta.decode(), tb.decode())] = {"ms": round(ms, 3), "TFLOPs": round(tf, 2), "frac": round(tf / 2500.0, 3)}
            for buf in (a, b, c):
                buf.free()
        if lib.och_gemm_supported(oh.INT8):
            dim = 8192
            a, b, c = [oh.DeviceBuffer(dim * dim, stream) for _ in range(3)]
            block = rng.integers(-128, 127, 1 << 22, endpoint=True).astype(np.int8)
            for buf in (a, b):
                for off in range(0, dim * dim, block.nbytes):
                    buf.upload(block, offset=off)
            one8 = np.array([1, 0], np.int8); zero8 = np.zeros(2, np.int8)
            for ta, tb in ((b"N", b"N"), (b"T", b"N")):
                fn = lambda: oh.check(lib.och_gemm(oh.INT8, ta, tb, dim, dim, dim, one8.ctypes.data, a.ptr, dim, b.ptr, dim,
                                                   zero8.ctypes.data, c.ptr, dim, 1, h))
                ms = time_launches(fn, reps=3, warm=1)
                tf = 2 * dim ** 3 / ms / 1e9
                configs["extra_gemm_int8_%d_%s%s" % (dim, ta.decode(), tb.decode())] = {"ms": round(ms, 3), "TOPs": round(tf, 2), "frac": round(tf / 5000.0, 3)}
            for buf in (a, b, c):
                buf.free()
        # MGS-QR pattern on a 4096 x 4096 float64 matrix: per (i, j) pair one dot product (gemm M = N = 1, result kept
        # on the device) and one rank-1 update reading that device scalar; window = the first 64 columns (2016 pairs)
        m = 4096
        q = oh.DeviceBuffer(8 * m * m, stream)
        blockq = rng.uniform(-1, 1, 1 << 22)
        for off in range(0, 8 * m * m, blockq.nbytes):
            q.upload(blockq, offset=off)
        rr = oh.DeviceBuffer(8 * 64 * 64, stream)
        consts = oh.to_device(np.array([1.0, 0.0, -1.0]), stream)
        c_one, c_zero, c_minus = [C.c_void_p(consts.address + 8 * i) for i in range(3)]
        col = lambda j: C.c_void_p(q.address + 8 * m * j)
        rij = lambda i, j: C.c_void_p(rr.address + 8 * (i + 64 * j))

        def mgs_window():
            for j in range(64):
                for i in range(j):
                    lib.och_gemm(F64, b"T", b"N", 1, 1, m, c_minus, col(i), m, col(j), m, c_zero, rij(i, j), 1, 0, h)
                    lib.och_gemm(F64, b"N", b"N", m, 1, 1, c_one, col(i), m, rij(i, j), 1, c_one, col(j), m, 0, h)
        mgs_window(); stream.synchronize()
        t0 = time.perf_counter(); mgs_window(); stream.synchronize(); dt_s = time.perf_counter() - t0
        pairs = 64 * 63 // 2
        configs["c5_mgs_qr_4096_first64cols"] = {"us_per_pair": round(dt_s / pairs * 1e6, 2), "launches_per_pair": 2,
                                                 "effective_GBps": round(pairs * (2 * 8 * m + 3 * 8 * m) / dt_s / 1e9, 1)}
        # the same window recorded once and replayed as a graph: no host work per operation
        if "och_graph_launch" not in oh.MISSING and not args.no_graph:
            oh.check(lib.och_stream_begin_capture(h))
            mgs_window()
            graph = C.c_void_p()
            oh.check(lib.och_stream_end_capture(h, C.byref(graph)))
            oh.check(lib.och_graph_launch(graph, h)); stream.synchronize()
            t0 = time.perf_counter()
            for _ in range(3):
                oh.check(lib.och_graph_launch(graph, h))
            stream.synchronize(); dt_g = (time.perf_counter() - t0) / 3
            oh.check(lib.och_graph_destroy(graph))
            configs["c5_mgs_qr_4096_first64cols_graph_replay"] = {"us_per_pair": round(dt_g / pairs * 1e6, 2), "launches_per_pair": 2,
                                                                  "effective_GBps": round(pairs * (2 * 8 * m + 3 * 8 * m) / dt_g / 1e9, 1)}
        # the same window through the fused projection: one launch per column instead of two per pair
        if "och_mgs_project" not in oh.MISSING:
            def mgs_fused():
                for j in range(1, 64):
                    lib.och_mgs_project(F64, m, j, q.ptr, m, col(j), C.c_void_p(rr.address + 8 * 64 * j), h)
            mgs_fused(); stream.synchronize()
            t0 = time.perf_counter()
            for _ in range(3):
                mgs_fused()
            stream.synchronize(); dt_f = (time.perf_counter() - t0) / 3
            configs["c5_mgs_qr_4096_first64cols_fused_projection"] = {"us_per_pair": round(dt_f / pairs * 1e6, 3), "launches_per_pair": round(63 / pairs, 4),
                                                                      "effective_GBps": round(pairs * (2 * 8 * m + 3 * 8 * m) / dt_f / 1e9, 1)}
        for b in (q, rr, consts):
            b.free()
    result["configs"] = configs

    # ------------------------------------------------------------------ CPU baseline (oracle, Ocean's threading policy)
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        import oracle_lib as orc
        orc.setup(oh)
        threads = orc.lib.oracle_max_threads()
        Z = np.empty((n, n)); TI = np.empty((n, n)); TF = np.empty((n, n))
        p = orc.ptr

        def cpu_step():
            assert orc.lib.oracle_binary(B["add"], F64, 2, shape, st_f64_T, p(hostA), st_row, p(hostR), st_f64, p(Z)) == 0
            assert orc.lib.oracle_copy(I32, F64, 2, shape, st_i32, p(hostI), 2, shape, st_f64, p(TI), threads) == 0
            assert orc.lib.oracle_binary(B["add"], F64, 2, shape, st_f64, p(Z), st_f64, p(TI), st_f64, p(Z)) == 0
            assert orc.lib.oracle_byteswap_copy(F32, F64, 2, shape, st_f32, p(hostFs), 2, shape, st_f64, p(TF), threads) == 0
            assert orc.lib.oracle_binary(B["multiply"], F64, 2, shape, st_f64, p(Z), st_f64, p(TF), st_f64, p(Z)) == 0

        cpu_step()
        reps, t0 = 0, time.perf_counter()
        while reps < 5 and (time.perf_counter() - t0) < 20:
            cpu_step(); reps += 1
        cpu_ms = (time.perf_counter() - t0) * 1e3 / reps
        result["cpu_baseline"] = {"value": round(step_bytes / cpu_ms / 1e6, 2), "unit": "GB/s", "cores": threads, "kind": "port",
                                  "sample": "%d full-size configuration-2 steps (binary operations serial, copies on %d threads, as in Ocean's CPU module)" % (reps, threads),
                                  "ms_per_step": round(cpu_ms, 1)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
