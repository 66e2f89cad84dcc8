#!/usr/bin/env python3
"""Benchmark of the MI355X device module on the five reference workload configurations (one GPU).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-graph]
                    [--only c1|c2|c3|c4|c5] [--ceiling]

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

Every per-kernel figure is taken from at least 20 timed samples (a sample = a few back-to-back
launches between two events on the launch stream, operand sets rotated so that no launch finds its
operands in the 256 MB last-level cache); the median and the best sample are reported.

Printed: ONE JSON line with the driver's fields plus
    roofline      dominant kernel of the step: algorithmic bytes per launch / median launch time
                  against the 8 TB/s HBM peak; traffic = HBM bytes per launch counted by rocprofv3
                  (profiles/traffic.json, from the counter runs recorded under profiles/)
    kernels       the same figure for every kernel of the step
    ceiling       what plain streaming kernels (och_membench) sustain on this device for the
                  same mixes of reads and writes, measured in the same run
    configs       measurements of configurations 1, 3, 4 and 5 (GB/s or TFLOP/s)
    cpu_baseline  the CPU oracle (a port of Ocean's CPU path with its threading policy) timed on
                  this host: the full-size step, and bounded samples of the other configurations

--only NAME runs one configuration with few samples and then a plain float64 copy of known size
(the yardstick that scales the FETCH_SIZE / WRITE_SIZE counters of a profiling run). In such a run a
one-byte fill (a single workgroup of fill_bytes_kernel) precedes every measured kernel, and the JSON
line lists the measured kernels in that order under "segments", so that the dispatches of a counter
run can be told apart.
--ceiling prints the whole sweep of the streaming micro-benchmark as a table.
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
MEMBENCH_KINDS = ["read", "write", "copy (1 read : 1 write)", "add float64 (2 reads : 1 write)",
                  "float32 -> float64 (8-byte loads, 16-byte stores)", "int16 step 2 -> float32 (16-byte loads)",
                  "float32 -> float64 (16-byte loads, lane exchange)", "int16 step 2 -> float32 (2-byte loads)"]
# bytes of the narrowest operand per launch: every launch moves 400 - 540 MB
MEMBENCH_BYTES = {0: 1 << 29, 1: 1 << 29, 2: 1 << 28, 3: 1 << 27, 4: 1 << 27, 5: 1 << 27, 6: 1 << 27, 7: 1 << 27}


def cpu_description():
    """CPU model, physical cores and logical CPUs visible to this process."""
    model, cores = "unknown", set()
    try:
        phys = core = None
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name") and model == "unknown":
                    model = line.split(":", 1)[1].strip()
                elif line.startswith("physical id"):
                    phys = line.split(":", 1)[1].strip()
                elif line.startswith("core id"):
                    core = line.split(":", 1)[1].strip()
                elif not line.strip():
                    if phys is not None and core is not None:
                        cores.add((phys, core))
                    phys = core = None
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    return {"model": model, "physical_cores": len(cores) or None, "logical_cpus": os.cpu_count(), "usable_cpus": usable}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="skip the graph-replay variant of the MGS window (rocprofv3's kernel tracing crashes inside hipGraphLaunch)")
    ap.add_argument("--only", default=None, choices=["c1", "c2", "c3", "c4", "c5"], help="run one configuration with few samples, then the yardstick copy (for profiling)")
    ap.add_argument("--ceiling", action="store_true", help="print the full sweep of the streaming micro-benchmark and exit")
    ap.add_argument("--samples", type=int, default=20, help="timed samples per figure (at least 20 unless --only is given)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus %d is not supported (every figure here is a one-GPU figure)" % args.gpus)

    import numpy as np
    import ocean_hip as oh
    import ocean_hip_bench as ohb

    oh.check(oh.lib.och_device_set(0))
    oh.check(oh.lib.och_device_warmup(0))
    prop = oh.device_properties(0)
    stream = oh.Stream()
    lib = oh.lib
    B, R = oh.B, oh.R
    h = stream.handle
    F32, F64, I32, I16, CF, CD = oh.FLOAT, oh.DOUBLE, oh.INT32, oh.INT16, oh.CFLOAT, oh.CDOUBLE
    profiling = args.only is not None
    SAMPLES = 3 if profiling else max(20, args.samples)
    rng = np.random.default_rng(20240)

    def membench(kind, unr, nt, mp, block, blocks, reps, nbytes=None):
        med, best, moved = C.c_float(), C.c_float(), C.c_size_t()
        oh.check(ohb.lib.och_membench(kind, unr, nt, mp, block, blocks, nbytes or MEMBENCH_BYTES[kind], 3, reps, C.byref(med), C.byref(best), C.byref(moved), h))
        return moved.value / med.value / 1e6, moved.value / best.value / 1e6

    if args.ceiling:
        import itertools
        print("# streaming micro-benchmark (och_membench), %s, %d compute units; GB/s of the bytes every launch moves" % (prop.arch.decode(), prop.multiprocessor_count))
        print("# columns: median, best of 20 samples of 10 back-to-back launches; 3 operand sets rotated")
        for kind, name in enumerate(MEMBENCH_KINDS):
            rows = []
            for unr, nt, block in itertools.product((1, 2, 4), (0, 1), (256, 512, 1024)):
                rows.append(membench(kind, unr, nt, 0, block, 0, 20) + ("one trip per thread, %d group(s) per thread, nontemporal %d, workgroup %d" % (unr, nt, block),))
            for unr, nt, block, blocks in itertools.product((2, 4), (0, 1), (256, 512), (1024, 4096)):
                rows.append(membench(kind, unr, nt, 1, block, blocks, 20) + ("persistent grid of %d workgroups, %d groups per trip, nontemporal %d, workgroup %d" % (blocks, unr, nt, block),))
            rows.sort(reverse=True)
            print("== %s: %.0f MB per launch" % (name, MEMBENCH_BYTES[kind] * {0: 1, 1: 1, 2: 2, 3: 3, 4: 3, 5: 3, 6: 3, 7: 3}[kind] / 1e6))
            for r in rows[:5]:
                print("   %7.1f  %7.1f   %s" % r)
            print("   ... %d forms measured; slowest: %7.1f  %7.1f   %s" % ((len(rows),) + rows[-1]))
            sys.stdout.flush()
        # matrix cores: a loop of nothing but MFMAs, and what other instructions of the same wave cost between them
        def mfmabench(typ, kind, per, waves, iters=4000):
            ms, flop = C.c_float(), C.c_double()
            oh.check(ohb.lib.och_mfmabench(typ, kind, per, waves, iters, 7, C.byref(ms), C.byref(flop), h))
            return ms.value, flop.value
        print("== matrix cores (och_mfmabench): 16 independent MFMAs per iteration, one block of 4 waves per compute unit (one wave per SIMD)")
        peaks = (("float 32x32x2", MFMA_PEAK["float"]), ("double 16x16x4", MFMA_PEAK["double"]), ("half 32x32x16", 2500.0), ("int8 32x32x32", 5000.0))
        for typ, (name, peak) in enumerate(peaks):
            mfmabench(typ, 0, 0, 4, 16000)                       # warm: the clock settles under this load
            ms, flop = mfmabench(typ, 0, 0, 4, 16000)
            ms1, flop1 = mfmabench(typ, 7, 0, 4, 16000)
            print("   %-16s MFMAs alone: %8.1f T/s = %.3f of the nominal %.1f on 16 pseudo-random operand pairs in turn; %8.1f T/s on one pair" % (name, flop / ms / 1e9, flop / ms / 1e9 / peak, peak, flop1 / ms1 / 1e9))
        print("   cost of an instruction between 64-cycle float MFMAs, in MFMA cycles (64 x time / time of the bare loop - 64) per instruction:")
        for waves in (4, 8):
            base, _ = mfmabench(0, 0, 0, waves)
            for kind, name in ((1, "v_mov_b32"), (2, "v_add_f32"), (3, "s_nop"), (4, "s_add_u32"), (5, "s_waitcnt"), (6, "ds_read_b128")):
                cells = []
                for per in (1, 2, 4):
                    ms, _ = mfmabench(0, kind, per, waves)
                    cells.append("%5.1f" % ((ms / base - 1.0) * 64.0 / per))
                print("   %d wave(s) per SIMD  %-13s 1 / 2 / 4 per MFMA: %s" % (waves // 4, name, "  ".join(cells)))
        sys.stdout.flush()
        # an independent implementation on the same sizes: PyTorch's own elementwise, copy and reduction kernels
        try:
            import torch
        except ImportError:
            return
        dev = torch.device("cuda:0")

        def torch_time(fn):
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            ts = []
            for _ in range(20):
                e0.record()
                for _ in range(10):
                    fn()
                e1.record(); torch.cuda.synchronize()
                ts.append(e0.elapsed_time(e1) / 10)
            ts.sort()
            return ts[len(ts) // 2], ts[0]
        print("== PyTorch %s on the same device, three operand sets rotated, random data (GB/s median, best)" % torch.__version__)
        n = 1 << 24
        sets = [[torch.randn(n, dtype=torch.float64, device=dev) for _ in range(3)] for _ in range(3)]
        turn = [0]

        def t_add():
            turn[0] += 1; a, b, c = sets[turn[0] % 3]; torch.add(a, b, out=c)

        def t_copy():
            turn[0] += 1; a, b, c = sets[turn[0] % 3]; c.copy_(a)
        med, best = torch_time(t_add); print("   %7.1f  %7.1f   torch.add, float64, 134 MB operands (2 reads : 1 write)" % (24 * n / med / 1e6, 24 * n / best / 1e6))
        med, best = torch_time(t_copy); print("   %7.1f  %7.1f   Tensor.copy_, float64, 134 MB operands (1 read : 1 write)" % (16 * n / med / 1e6, 16 * n / best / 1e6))
        del sets
        xs = [torch.randn(1 << 26, dtype=torch.float32, device=dev) for _ in range(3)]

        def t_sum():
            turn[0] += 1; return xs[turn[0] % 3].sum()
        med, best = torch_time(t_sum); print("   %7.1f  %7.1f   torch.sum, float32, 268 MB (read only)" % (4 * (1 << 26) / med / 1e6, 4 * (1 << 26) / best / 1e6))
        del xs
        # the vendor library's matrix products through torch.matmul / torch._int_mm at 8192^3 (T/s median, best): an
        # independent figure for what the matrix cores sustain on random and on constant operands
        print("== vendor GEMM through PyTorch at 8192^3, two operand sets alternating (TFLOP/s or TOP/s median, best)")
        dim = 8192

        def gemm_line(name, make, op, peak):
            for label, const in (("random operands", False), ("constant operands (1.0 / 1 everywhere)", True)):
                ops = [(make(const), make(const)) for _ in range(2)]
                gturn = [0]

                def run():
                    gturn[0] += 1
                    a_, b_ = ops[gturn[0] % 2]
                    return op(a_, b_)
                try:
                    med, best = torch_time(run)
                except Exception as e:                                  # a product the installed library does not offer
                    print("   %-28s %-40s not available: %s" % (name, label, str(e).splitlines()[0][:80]))
                    return
                flop = 2.0 * dim ** 3
                print("   %8.1f  %8.1f   %-28s %-40s (%.3f of the nominal %.0f)" % (flop / med / 1e9, flop / best / 1e9, name, label, flop / med / 1e9 / peak, peak))
                del ops
        gemm_line("float32 NN", lambda c: torch.ones(dim, dim, device=dev) if c else torch.rand(dim, dim, device=dev) * 2 - 1, torch.matmul, MFMA_PEAK["float"])
        gemm_line("float64 NN", lambda c: torch.ones(dim, dim, device=dev, dtype=torch.float64) if c else torch.rand(dim, dim, device=dev, dtype=torch.float64) * 2 - 1, torch.matmul, MFMA_PEAK["double"])
        gemm_line("float16 NN", lambda c: torch.ones(dim, dim, device=dev, dtype=torch.float16) if c else (torch.rand(dim, dim, device=dev) * 2 - 1).half(), torch.matmul, 2500.0)
        gemm_line("float16 TN (A.T @ B)", lambda c: torch.ones(dim, dim, device=dev, dtype=torch.float16) if c else (torch.rand(dim, dim, device=dev) * 2 - 1).half(),
                  lambda a_, b_: torch.matmul(a_.t(), b_), 2500.0)
        gemm_line("bfloat16 NN", lambda c: torch.ones(dim, dim, device=dev, dtype=torch.bfloat16) if c else (torch.rand(dim, dim, device=dev) * 2 - 1).bfloat16(), torch.matmul, 2500.0)
        gemm_line("int8 NN (torch._int_mm)", lambda c: torch.ones(dim, dim, device=dev, dtype=torch.int8) if c else torch.randint(-128, 128, (dim, dim), device=dev, dtype=torch.int8),
                  lambda a_, b_: torch._int_mm(a_, b_), 5000.0)
        gemm_line("int8 NT (torch._int_mm)", lambda c: torch.ones(dim, dim, device=dev, dtype=torch.int8) if c else torch.randint(-128, 128, (dim, dim), device=dev, dtype=torch.int8),
                  lambda a_, b_: torch._int_mm(a_, b_.t()), 5000.0)
        # the same library away from 8192^3, at the sizes of the extra_gemm_<type>_MxNxK lines of the default run
        print("== vendor GEMM through PyTorch at the sizes of the extra_gemm_ lines (NN, random operands, TFLOP/s median, microseconds)")
        for tdt, tname in ((torch.float32, "float32"), (torch.float64, "float64"), (torch.float16, "float16")):
            for m_, n_, k_ in ((1024, 1024, 1024), (1536, 1536, 1536), (2048, 2048, 2048), (3000, 3000, 3000), (4096, 4096, 4096), (8192, 8192, 64), (8192, 8192, 256)):
                ta_ = (torch.rand(m_, k_, device=dev) * 2 - 1).to(tdt)
                tb_ = (torch.rand(k_, n_, device=dev) * 2 - 1).to(tdt)
                tc_ = torch.empty(m_, n_, device=dev, dtype=tdt)
                med, best = torch_time(lambda: torch.matmul(ta_, tb_, out=tc_))
                print("   %8.1f  %8.1f us   %s %5d x %5d x %5d" % (2.0 * m_ * n_ * k_ / med / 1e9, med * 1e3, tname, m_, n_, k_))
                del ta_, tb_, tc_
        return

    def sample_launches(fn, samples=None, warm=3, target_ms=0.6):
        """median and best duration (ms) of one call of fn(): `samples` samples, each a few back-to-back calls between
        two events on the launch stream (so the events' own cost is spread; at least ~0.6 ms per sample)"""
        samples = samples or SAMPLES
        e0, e1 = oh.Event(), oh.Event()
        if profiling:
            # a one-byte fill in front of every measured kernel: in a counter run the dispatches between two of these
            # single-workgroup fills belong to one entry of "segments"
            oh.check(lib.och_memset_async(separator.ptr, 0, 1, h))
        for _ in range(warm):
            fn()
        e0.record(stream); fn(); fn(); e1.record(stream); e1.synchronize()
        est = max(e0.elapsed_ms(e1) / 2, 1e-3)
        inner = int(min(50, max(1, round(target_ms / est))))
        times = []
        for _ in range(samples):
            e0.record(stream)
            for _ in range(inner):
                fn()
            e1.record(stream)
            e1.synchronize()
            times.append(e0.elapsed_ms(e1) / inner)
        e0.destroy(); e1.destroy()
        times.sort()
        return times[len(times) // 2], times[0], inner

    def gbps(nbytes, timing, ceiling=None):
        med, best, inner = timing
        out = {"ms": round(med, 4), "best_ms": round(best, 4), "samples": SAMPLES, "launches_per_sample": inner,
               "algorithmic_MB": round(nbytes / 1e6, 1), "GBps": round(nbytes / med / 1e6, 1), "best_GBps": round(nbytes / best / 1e6, 1),
               "frac": round(nbytes / med / 1e6 / HBM_PEAK_GBS, 3)}
        if ceiling:
            out["frac_of_ceiling"] = round(nbytes / med / 1e6 / ceiling, 3)
        return out

    def upload_tiled(buf, block, nbytes):
        """fill a device buffer with copies of a host block of random values"""
        for off in range(0, nbytes, block.nbytes):
            m = min(block.nbytes, nbytes - off) // block.itemsize
            buf.upload(block[:m], offset=off)

    segments = []                      # names of the measured kernels in launch order (profiling runs)
    separator = oh.DeviceBuffer(256, stream)
    traffic_table = {}
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic_table = json.load(f)

    def with_traffic(entry, name):
        segments.append(name)
        t = traffic_table.get(name)
        if t:
            entry["traffic_MB"] = round((t["fetch_bytes"] + t["write_bytes"]) / 1e6, 1)
            entry["traffic_GBps"] = round((t["fetch_bytes"] + t["write_bytes"]) / entry["ms"] / 1e6, 1)
        return entry

    # ------------------------------------------------------------------ what the device sustains (plain streaming kernels)
    ceiling = {}
    if not profiling:
        # the same operand sizes as the library kernels they are set against (a launch of 200 MB loses more to its start
        # and its tail than one of 1.6 GB); the best form of each mix per the full sweep (--ceiling)
        for key, kind, unr, nt, block, nbytes in (("read_268MB", 0, 1, 1, 1024, 1 << 28), ("read_537MB", 0, 1, 1, 1024, 1 << 29), ("write_268MB", 1, 1, 0, 256, 1 << 28),
                                                  ("copy_134MB_operands", 2, 1, 1, 512, 1 << 27), ("add_134MB_operands", 3, 1, 1, 512, 1 << 27),
                                                  ("add_67MB_operands", 3, 1, 1, 512, 1 << 26), ("cast_4B_to_8B_67MB_source", 4, 1, 1, 512, 1 << 26),
                                                  ("cast_4B_to_8B_537MB_source", 4, 1, 1, 512, 1 << 29), ("int16_step2_to_f32_134MB_asked", 5, 1, 1, 512, 1 << 27)):
            med, best = membench(kind, unr, nt, 0, block, 0, SAMPLES, nbytes)
            ceiling[key] = {"GBps": round(med, 1), "best_GBps": round(best, 1), "frac": round(med / HBM_PEAK_GBS, 3)}

    def ceil_of(key):
        return ceiling[key]["GBps"] if key in ceiling else None

    result = {}
    configs = {}

    # ------------------------------------------------------------------ configuration 2 (the step)
    n = N2
    nn = n * n
    shape = oh.sizes([n, n])
    st_f64, st_f64_T, st_row = oh.strides([8, 8 * n]), oh.strides([8 * n, 8]), oh.strides([0, 8])
    st_i32, st_f32 = oh.strides([4, 4 * n]), oh.strides([4, 4 * n])
    hostA = rng.uniform(-10, 10, (n, n))
    hostR = rng.uniform(-10, 10, n)
    hostI = rng.integers(-10, 10, (n, n), endpoint=True).astype(np.int32)
    hostF = rng.uniform(-10, 10, (n, n)).astype(np.float32)
    hostFs = hostF.byteswap()
    if args.only in (None, "c2"):
        NSETS = 3
        sets = []
        for _ in range(NSETS):
            s = {"A": oh.to_device(hostA, stream), "r": oh.to_device(hostR, stream), "I": oh.to_device(hostI, stream),
                 "F": oh.to_device(hostFs, stream), "Z": oh.DeviceBuffer(8 * nn, stream),
                 "TI": oh.DeviceBuffer(8 * nn, stream), "TF": oh.DeviceBuffer(8 * nn, stream)}
            sets.append(s)

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

        step_kernels = [
            ("add f64: transposed view + row broadcast", k_add_transposed, 8 * nn * 2 + 8 * n, "copy_134MB_operands"),
            ("copy int32 -> f64", k_cast_i32, 12 * nn, "cast_4B_to_8B_67MB_source"),
            ("add f64 contiguous", k_add, 24 * nn, "add_134MB_operands"),
            ("byteswap_copy f32 (swapped) -> f64", k_cast_swapped, 12 * nn, "cast_4B_to_8B_67MB_source"),
            ("multiply f64 contiguous", k_multiply, 24 * nn, "add_134MB_operands"),
        ]
        step_bytes = sum(b for _, _, b, _ in step_kernels)

        def step(i):
            s = sets[i % NSETS]
            for _, fn, _, _ in step_kernels:
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
        # per-kernel roofline of the step
        kernels = []
        for name, fn, nbytes, mix in step_kernels:
            turn = [0]

            def rotating(fn=fn, turn=turn):          # alternate the operand sets, as the step loop does
                turn[0] += 1
                fn(sets[turn[0] % NSETS])
            entry = gbps(nbytes, sample_launches(rotating), ceil_of(mix))
            entry["kernel"] = name
            entry["ceiling_mix"] = mix
            kernels.append(with_traffic(entry, name))
        dom = max(kernels, key=lambda k: k["ms"])
        t = traffic_table.get(dom["kernel"])
        result["roofline"] = {"bound": "hbm", "kernel": dom["kernel"], "achieved": dom["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": round(dom["GBps"] / HBM_PEAK_GBS, 3),
                              "traffic": dom.get("traffic_GBps"),
                              "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `bench.py --only c1|c2|c3|c4`, scaled by a float64 copy of known size)" if t else None,
                              "algorithmic_bytes_per_launch": next(b for nm, _, b, _ in step_kernels if nm == dom["kernel"]),
                              "traffic_bytes_per_launch": (t["fetch_bytes"] + t["write_bytes"]) if t else None,
                              "launch_ms": dom["ms"], "best_launch_ms": dom["best_ms"], "samples": SAMPLES,
                              "device_ceiling_for_this_mix_GBps": ceil_of(dom["ceiling_mix"])}
        result["kernels"] = kernels
        result["ceiling"] = ceiling
        for s in sets:
            for b in s.values():
                b.free()
        stream.synchronize()

    # ------------------------------------------------------------------ configuration 1
    n1 = 1 << 24
    if args.only in (None, "c1"):
        # six operand sets (6 x 256 MB): successive launches never find their operands in the last-level cache
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
        for bufs in c1sets:                       # t must hold values before the add is timed
            oh.check(lib.och_binary(B["multiply"], F32, 1, s1, st1, bufs[0].ptr, st1, bufs[1].ptr, st1, bufs[2].ptr, h))
        configs["c1_scale_f32_2^24"] = with_traffic(gbps(12 * n1, sample_launches(c1_scale), ceil_of("add_67MB_operands")), "c1_scale_f32_2^24")
        configs["c1_add_f32_2^24"] = with_traffic(gbps(12 * n1, sample_launches(c1_add), ceil_of("add_67MB_operands")), "c1_add_f32_2^24")
        for bufs in c1sets:
            for b in bufs:
                b.free()

    # ------------------------------------------------------------------ configuration 3
    n3 = 8192 * 8192
    d0, d1, d2 = 512, 512, 256
    if args.only in (None, "c3"):
        for dt, es, nm in ((F32, 4, "f32"), (F64, 8, "f64")):
            rbufs = [oh.DeviceBuffer(es * n3, stream) for _ in range(2)]          # alternate: no reuse from the last-level cache
            chunk = rng.standard_normal(1 << 22).astype(np.float32 if es == 4 else np.float64)
            for buf in rbufs:
                upload_tiled(buf, chunk, es * n3)
            rturn = [0]

            def next_buf():
                rturn[0] += 1
                return rbufs[rturn[0] % 2]
            dres = oh.DeviceBuffer(64, stream)
            s3, st3 = oh.sizes([n3]), oh.strides([es])
            for opn in ("sum", "norm2", "maximum"):
                key = "c3_%s_%s_8192^2" % (opn, nm)
                timing = sample_launches(lambda: oh.check(lib.och_reduce_all_device(R[opn], dt, 1, s3, st3, next_buf().ptr, None, None, 0.0, dres.ptr, None, h)))
                configs[key] = with_traffic(gbps(es * n3, timing, ceil_of("read_268MB" if es == 4 else "read_537MB")), key)
            if not profiling:
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
                    timing = sample_launches(lambda: oh.check(lib.och_reduce_axis(R["sum"], dt, C.byref(next_ecfg()), 0.0)))
                    configs["extra_axis_sum_%s_%s" % (nm, label)] = gbps(es * (n3 + osize), timing, ceil_of("read_268MB" if es == 4 else "read_537MB"))
                few.free(); many.free()
            # axis reductions on a 512 x 512 x 256 view with padded pitches (no two dimensions merge);
            # the view lives in a parent of (512+4) x (512+2) x 256 elements
            p0, p1 = (d0 + 4) * es, (d0 + 4) * (d1 + 2) * es
            parent_bytes = p1 * d2
            extent = (d0 - 1) * es + (d1 - 1) * p0 + (d2 - 1) * p1 + es
            assert extent <= parent_bytes, "axis view exceeds its parent buffer"
            abufs = [oh.DeviceBuffer(parent_bytes, stream) for _ in range(2)]     # alternate: no reuse from the last-level cache
            for abuf in abufs:
                upload_tiled(abuf, chunk, parent_bytes)
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
                    key = "c3_axis%d_%s_%s_512x512x256" % (axis, opn, nm)
                    timing = sample_launches(lambda: oh.check(lib.och_reduce_axis(R[opn], dt, C.byref(next_cfg()), 0.0)))
                    configs[key] = with_traffic(gbps(es * (d0 * d1 * d2 + keep[0] * keep[1]), timing, ceil_of("read_268MB" if es == 4 else "read_537MB")), key)
            for b in rbufs + abufs + [dres, out]:
                b.free()

    # ------------------------------------------------------------------ configuration 4
    e0, e1, e2 = 1024, 1024, 64
    n4 = e0 * e1 * e2
    n4b = 1 << 26
    if args.only in (None, "c4"):
        # int16, uniform over the full range, stored byte-swapped, every second element of the first dimension -> float32;
        # two operand sets (2 x 537 MB) alternate
        chunk16 = rng.integers(-32768, 32767, 1 << 22, dtype=np.int16, endpoint=True)
        c4 = []
        for _ in range(2):
            src = oh.DeviceBuffer(2 * 2 * n4, stream); dst = oh.DeviceBuffer(4 * n4, stream)
            upload_tiled(src, chunk16, 2 * 2 * n4)
            c4.append((src, dst))
        sz4 = oh.sizes([e0, e1, e2])
        st_src, st_dst = oh.strides([4, 4 * e0, 4 * e0 * e1]), oh.strides([4, 4 * e0, 4 * e0 * e1])
        t4 = [0]

        def c4a():
            src, dst = c4[t4[0] % 2]; t4[0] += 1
            oh.check(lib.och_byteswap_copy(I16, F32, 3, sz4, st_src, src.ptr, 3, sz4, st_dst, dst.ptr, h))
        key = "c4_int16_swapped_step2_to_f32_1024x1024x64"
        configs[key] = with_traffic(gbps(6 * n4, sample_launches(c4a), ceil_of("int16_step2_to_f32_134MB_asked")), key)
        configs[key]["note"] = "the memory system moves the skipped int16 elements too: 8 bytes of traffic per 6 bytes asked for"
        for src, dst in c4:
            src.free(); dst.free()
        # complex64 -> complex128, 2^26 elements, real and imaginary parts U(-1, 1); two operand sets (2 x 1.6 GB) alternate
        chunkc = (rng.uniform(-1, 1, 1 << 21) + 1j * rng.uniform(-1, 1, 1 << 21)).astype(np.complex64)
        c4 = []
        for _ in range(2):
            src = oh.DeviceBuffer(8 * n4b, stream); dst = oh.DeviceBuffer(16 * n4b, stream)
            upload_tiled(src, chunkc, 8 * n4b)
            c4.append((src, dst))
        s4, sa, sb = oh.sizes([n4b]), oh.strides([8]), oh.strides([16])

        def c4b():
            src, dst = c4[t4[0] % 2]; t4[0] += 1
            oh.check(lib.och_copy(CF, CD, 1, s4, sa, src.ptr, 1, s4, sb, dst.ptr, h))
        key = "c4_cfloat_to_cdouble_2^26"
        configs[key] = with_traffic(gbps(24 * n4b, sample_launches(c4b), ceil_of("cast_4B_to_8B_537MB_source")), key)
        for src, dst in c4:
            src.free(); dst.free()

    # ------------------------------------------------------------------ beyond the named configurations: the other kernel families
    # (unary functions, arithmetic-heavy binary operations, the software half types, fill, gather / scatter / find): the same
    # sampling, two operand sets alternating, algorithmic bytes = every input element read once + every output written once
    if args.only is None:
        U = oh.U
        ne = 1 << 26
        HALF_T, CHALF_T, I64, I32 = oh.HALF, oh.CHALF, oh.INT64, oh.INT32

        def extra_sets(es_in, es_out, n_in, fill):
            """two sets of n_in inputs + 1 output of ne elements; fill(k) gives a host block for input k"""
            out = []
            for _ in range(2):
                ins = []
                for k in range(n_in):
                    b = oh.DeviceBuffer(es_in * ne, stream)
                    upload_tiled(b, fill(k), es_in * ne)
                    ins.append(b)
                out.append((ins, oh.DeviceBuffer(es_out * ne, stream)))
            return out

        def free_sets(sets_):
            for ins, o in sets_:
                for b in ins + [o]:
                    b.free()
        se = oh.sizes([ne])
        # unary functions
        for dt, es, nm, npt in ((F32, 4, "f32", np.float32), (F64, 8, "f64", np.float64)):
            sets_ = extra_sets(es, es, 1, lambda k: rng.uniform(0.5, 4.0, 1 << 22).astype(npt))
            stx = oh.strides([es]); ut = [0]
            for opn in ("sqrt", "exp", "sin", "tanh", "sinh", "cosh", "log1p", "arcsinh"):
                def un(opn=opn):
                    ins, o = sets_[ut[0] % 2]; ut[0] += 1
                    oh.check(lib.och_unary(U[opn], dt, 1, se, stx, ins[0].ptr, stx, o.ptr, h))
                configs["extra_unary_%s_%s_2^26" % (opn, nm)] = gbps(2 * es * ne, sample_launches(un), ceil_of("copy_134MB_operands"))
            free_sets(sets_)
        sets_ = extra_sets(8, 8, 1, lambda k: (rng.uniform(-2, 2, 1 << 21) + 1j * rng.uniform(-2, 2, 1 << 21)).astype(np.complex64))
        outr = [oh.DeviceBuffer(4 * ne, stream) for _ in range(2)]
        stc, stf = oh.strides([8]), oh.strides([4]); ut = [0]

        def un_cexp():
            ins, o = sets_[ut[0] % 2]; ut[0] += 1
            oh.check(lib.och_unary(U["exp"], CF, 1, se, stc, ins[0].ptr, stc, o.ptr, h))

        def un_cabs():
            ins, o = sets_[ut[0] % 2]; ut[0] += 1
            oh.check(lib.och_unary(U["absolute"], CF, 1, se, stc, ins[0].ptr, stf, outr[ut[0] % 2].ptr, h))
        configs["extra_unary_exp_cfloat_2^26"] = gbps(16 * ne, sample_launches(un_cexp), ceil_of("copy_134MB_operands"))
        configs["extra_unary_absolute_cfloat_to_f32_2^26"] = gbps(12 * ne, sample_launches(un_cabs), ceil_of("copy_134MB_operands"))
        free_sets(sets_)
        for b in outr:
            b.free()
        # binary operations with real arithmetic behind them: integer division and remainder (floor rules), powers
        def int_block(npt, k):
            v = rng.integers(-(1 << 20), 1 << 20, 1 << 22).astype(npt)
            if k == 1:
                v = rng.integers(1, 1000, 1 << 22).astype(npt) * rng.choice(np.array([-1, 1], npt), 1 << 22)
            return v
        for dt, es, nm, npt in ((I32, 4, "int32", np.int32), (I64, 8, "int64", np.int64)):
            sets_ = extra_sets(es, es, 2, lambda k: int_block(npt, k))
            stx = oh.strides([es]); bt = [0]
            for opn in ("divide", "mod"):
                def bn(opn=opn):
                    ins, o = sets_[bt[0] % 2]; bt[0] += 1
                    oh.check(lib.och_binary(B[opn], dt, 1, se, stx, ins[0].ptr, stx, ins[1].ptr, stx, o.ptr, h))
                configs["extra_binary_%s_%s_2^26" % (opn, nm)] = gbps(3 * es * ne, sample_launches(bn), ceil_of("add_134MB_operands"))
            free_sets(sets_)
        for dt, es, nm, fillf, es2 in ((I32, 4, "int32", lambda k: (rng.integers(-9, 9, 1 << 22) if k == 0 else rng.integers(0, 9, 1 << 22)).astype(np.int32 if k == 0 else np.int16), 2),
                                        (F32, 4, "f32", lambda k: rng.uniform(0.5, 2.0, 1 << 22).astype(np.float32), 4)):
            # integer powers take int16 exponents (the second operand type of the table's power entry)
            sets_ = []
            for _ in range(2):
                a_ = oh.DeviceBuffer(es * ne, stream); b_ = oh.DeviceBuffer(es2 * ne, stream); o_ = oh.DeviceBuffer(es * ne, stream)
                upload_tiled(a_, fillf(0), es * ne); upload_tiled(b_, fillf(1), es2 * ne)
                sets_.append(([a_, b_], o_))
            stx, stb = oh.strides([es]), oh.strides([es2]); bt = [0]

            def bp():
                ins, o = sets_[bt[0] % 2]; bt[0] += 1
                oh.check(lib.och_binary(B["power"], dt, 1, se, stx, ins[0].ptr, stb, ins[1].ptr, stx, o.ptr, h))
            configs["extra_binary_power_%s_2^26" % nm] = gbps((2 * es + es2) * ne, sample_launches(bp), ceil_of("add_134MB_operands"))
            free_sets(sets_)
        # the half types: storage is half, arithmetic is float, conversions by the library's own rounding rules
        for dt, es, nm in ((HALF_T, 2, "half"), (CHALF_T, 4, "chalf")):
            sets_ = extra_sets(es, es, 2, lambda k: rng.uniform(-2, 2, 1 << 22).astype(np.float16))
            stx = oh.strides([es]); bt = [0]
            for opn in ("add", "multiply"):
                def bh(opn=opn):
                    ins, o = sets_[bt[0] % 2]; bt[0] += 1
                    oh.check(lib.och_binary(B[opn], dt, 1, se, stx, ins[0].ptr, stx, ins[1].ptr, stx, o.ptr, h))
                configs["extra_binary_%s_%s_2^26" % (opn, nm)] = gbps(3 * es * ne, sample_launches(bh), ceil_of("add_67MB_operands"))
            free_sets(sets_)
        # fill and masked fill, float32
        fbufs = [oh.DeviceBuffer(4 * ne, stream) for _ in range(2)]
        mbufs = [oh.to_device((rng.random(ne) < 0.5).astype(np.uint8), stream) for _ in range(2)]
        fval = oh.make_scalar(F32, 1.5); ft = [0]

        def k_fill():
            ft[0] += 1
            oh.check(lib.och_fill(F32, 1, se, stf, fbufs[ft[0] % 2].ptr, fval, h))

        def k_masked_fill():
            ft[0] += 1
            oh.check(lib.och_masked_fill(F32, 1, se, stf, fbufs[ft[0] % 2].ptr, oh.strides([1]), mbufs[ft[0] % 2].ptr, fval, h))
        configs["extra_fill_f32_2^26"] = gbps(4 * ne, sample_launches(k_fill), ceil_of("write_268MB"))
        e = gbps(9 * ne, sample_launches(k_masked_fill), ceil_of("copy_134MB_operands"))
        e["note"] = ("half of the mask set at random, so every 16-byte group holds kept and replaced elements: the result is where(mask, value, old) -- "
                     "the mask (1 byte) and the old element (4 bytes) are read, the element (4 bytes) is written: 9 bytes per element")
        configs["extra_masked_fill_f32_2^26_half_set"] = e
        for b in fbufs + mbufs:
            b.free()
        # gather / scatter of 65536 rows of 8 KB through an offset table, 16M random 8-byte elements, and find on a 64M-element mask
        rows_n, row_bytes = 65536, 8192
        gsrc = [oh.DeviceBuffer(rows_n * row_bytes, stream) for _ in range(2)]
        gdst = [oh.DeviceBuffer(rows_n * row_bytes, stream) for _ in range(2)]
        for b in gsrc:
            upload_tiled(b, rng.standard_normal(1 << 21), rows_n * row_bytes)
        perm = rng.permutation(rows_n).astype(np.int64) * row_bytes
        dperm = oh.to_device(perm, stream)
        tabs = (C.POINTER(C.c_int64) * 2)(None, C.cast(dperm.ptr, C.POINTER(C.c_int64)))
        gsz = oh.sizes([row_bytes // 8, rows_n]); gst1 = oh.strides([8, 0]); gst2 = oh.strides([8, row_bytes]); gt = [0]

        def k_gather():
            gt[0] += 1
            oh.check(lib.och_get_index(F64, 2, gsz, tabs, gst1, gsrc[gt[0] % 2].ptr, gst2, gdst[gt[0] % 2].ptr, h))

        def k_scatter():
            gt[0] += 1
            oh.check(lib.och_set_index(F64, 2, gsz, tabs, gst1, gdst[gt[0] % 2].ptr, gst2, gsrc[gt[0] % 2].ptr, h))
        configs["extra_gather_65536_rows_of_8KB"] = gbps(2 * rows_n * row_bytes, sample_launches(k_gather), ceil_of("copy_134MB_operands"))
        configs["extra_scatter_65536_rows_of_8KB"] = gbps(2 * rows_n * row_bytes, sample_launches(k_scatter), ceil_of("copy_134MB_operands"))
        nr = 1 << 24
        eperm = (rng.integers(0, rows_n * row_bytes // 8, nr).astype(np.int64)) * 8
        deperm = oh.to_device(eperm, stream)
        tab1 = (C.POINTER(C.c_int64) * 1)(C.cast(deperm.ptr, C.POINTER(C.c_int64)))

        def k_gather_elements():
            gt[0] += 1
            oh.check(lib.och_get_index(F64, 1, oh.sizes([nr]), tab1, oh.strides([0]), gsrc[gt[0] % 2].ptr, oh.strides([8]), gdst[gt[0] % 2].ptr, h))
        e = gbps(16 * nr, sample_launches(k_gather_elements))
        e["Gelements_per_s"] = round(nr / e["ms"] / 1e6, 1)
        e["note"] = "16M random 8-byte elements out of 537 MB: every element costs the memory system a whole sector"
        configs["extra_gather_16M_random_8B_elements"] = e
        for b in gsrc + gdst + [dperm, deperm]:
            b.free()
        nm_ = 1 << 26
        masks = [oh.to_device((rng.random(nm_) < 0.3).astype(np.uint8), stream) for _ in range(2)]
        work = oh.DeviceBuffer(lib.och_find_workspace_size(nm_), stream)
        fout = oh.DeviceBuffer(8 * nm_ // 2, stream)
        nnz = C.c_size_t(); fsz, fst = oh.sizes([nm_]), oh.strides([1]); fturn = [0]

        def k_find():
            fturn[0] += 1
            m_ = masks[fturn[0] % 2]
            oh.check(lib.och_find_count(1, fsz, fst, m_.ptr, work.ptr, C.byref(nnz), h))
            oh.check(lib.och_find_apply(1, fsz, fst, m_.ptr, work.ptr, None, fout.ptr, h))
        k_find()
        e = gbps(2 * nm_ + 8 * nnz.value, sample_launches(k_find))
        e["note"] = "count (with its read-back of the total) + apply on a 64M-element mask, 30 %% set: the mask read twice, %d positions of 8 bytes written" % nnz.value
        configs["extra_find_64M_mask_30pct"] = e
        for b in masks + [work, fout]:
            b.free()

    # ------------------------------------------------------------------ configuration 5 (GEMM)
    if args.only in (None, "c5"):
        def tflops(flop, timing, peak):
            med, best, inner = timing
            return {"ms": round(med, 3), "best_ms": round(best, 3), "samples": SAMPLES, "launches_per_sample": inner,
                    "TFLOPs": round(flop / med / 1e9, 2), "best_TFLOPs": round(flop / best / 1e9, 2), "frac": round(flop / med / 1e9 / peak, 3)}
        for dt, es, nm, dim, flop_per_mac in ((F64, 8, "double", 8192, 2), (F32, 4, "float", 8192, 2), (CF, 8, "cfloat", 4096, 8)):
            a, b, c = [oh.DeviceBuffer(es * dim * dim, stream) for _ in range(3)]
            block = rng.uniform(-1, 1, 1 << 22).astype(np.float32 if nm != "double" else np.float64)
            for buf in (a, b):
                upload_tiled(buf, block, es * dim * dim)
            one = np.array([1, 0], dtype=block.dtype); zero = np.zeros(2, dtype=block.dtype)
            for ta, tb in ((b"N", b"N"), (b"T", b"N"), (b"N", b"T")):
                fn = lambda: oh.check(lib.och_gemm(dt, ta, tb, dim, dim, dim, one.ctypes.data, a.ptr, dim, b.ptr, dim,
                                                   zero.ctypes.data, c.ptr, dim, 1, h))
                configs["c5_gemm_%s_%d_%s%s" % (nm, dim, ta.decode(), tb.decode())] = tflops(flop_per_mac * dim ** 3, sample_launches(fn, warm=2), MFMA_PEAK[nm])
            for buf in (a, b, c):
                buf.free()
        if True:
            # beyond the named configurations: complex double of the complex-float size; a float product whose sizes are
            # not multiples of any tile
            dim = 4096
            a, b, c = [oh.DeviceBuffer(16 * dim * dim, stream) for _ in range(3)]
            block = rng.uniform(-1, 1, 1 << 22)
            for buf in (a, b):
                upload_tiled(buf, block, 16 * dim * dim)
            onez = np.array([1.0, 0.0]); zeroz = np.zeros(2)
            for ta, tb in ((b"N", b"N"), (b"T", b"N"), (b"N", b"T")):
                fn = lambda: oh.check(lib.och_gemm(CD, ta, tb, dim, dim, dim, onez.ctypes.data, a.ptr, dim, b.ptr, dim,
                                                   zeroz.ctypes.data, c.ptr, dim, 1, h))
                configs["extra_gemm_cdouble_%d_%s%s" % (dim, ta.decode(), tb.decode())] = tflops(8 * dim ** 3, sample_launches(fn, warm=2), MFMA_PEAK["cdouble"])
            for buf in (a, b, c):
                buf.free()
            dim = 7000
            a, b, c = [oh.DeviceBuffer(4 * dim * dim, stream) for _ in range(3)]
            block = rng.uniform(-1, 1, 1 << 22).astype(np.float32)
            for buf in (a, b):
                upload_tiled(buf, block, 4 * dim * dim)
            onef = np.array([1, 0], np.float32); zerof = np.zeros(2, np.float32)
            fn = lambda: oh.check(lib.och_gemm(F32, b"N", b"N", dim, dim, dim, onef.ctypes.data, a.ptr, dim, b.ptr, dim,
                                               zerof.ctypes.data, c.ptr, dim, 1, h))
            configs["extra_gemm_float_%d_NN" % dim] = tflops(2 * dim ** 3, sample_launches(fn, warm=2), MFMA_PEAK["float"])
            for buf in (a, b, c):
                buf.free()
            # away from 8192^3: products of one or a few rounds of the compute units, and products with a short K (whose
            # blocks spend as long on their first loads and on writing C as in their loop)
            for dt, es, nm, npt in ((F32, 4, "float", np.float32), (F64, 8, "double", np.float64)):
                cap = 8192 * 8192
                a, b, c = [oh.DeviceBuffer(es * cap, stream) for _ in range(3)]
                block = rng.uniform(-1, 1, 1 << 22).astype(npt)
                for buf in (a, b):
                    upload_tiled(buf, block, es * cap)
                one_, zero_ = np.array([1, 0], npt), np.zeros(2, npt)
                for m_, n_, k_ in ((1024, 1024, 1024), (1536, 1536, 1536), (2048, 2048, 2048), (3000, 3000, 3000), (4096, 4096, 4096), (8192, 8192, 64), (8192, 8192, 256)):
                    fn = lambda: oh.check(lib.och_gemm(dt, b"N", b"N", m_, n_, k_, one_.ctypes.data, a.ptr, m_, b.ptr, k_, zero_.ctypes.data, c.ptr, m_, 1, h))
                    configs["extra_gemm_%s_%dx%dx%d_NN" % (nm, m_, n_, k_)] = tflops(2.0 * m_ * n_ * k_, sample_launches(fn, warm=2), MFMA_PEAK[nm])
                for buf in (a, b, c):
                    buf.free()
            # half-precision and 8-bit products of the size of the named configurations on the matrix cores
            dim = 8192
            a, b, c = [oh.DeviceBuffer(2 * dim * dim, stream) for _ in range(3)]
            block = rng.uniform(-1, 1, 1 << 22).astype(np.float16)
            for buf in (a, b):
                upload_tiled(buf, block, 2 * dim * dim)
            one16 = np.array([0x3C00, 0], np.uint16); zero16 = np.zeros(2, np.uint16)
            for ta, tb in ((b"N", b"N"), (b"T", b"N"), (b"N", b"T")):
                fn = lambda: oh.check(lib.och_gemm(oh.HALF, ta, tb, dim, dim, dim, one16.ctypes.data, a.ptr, dim, b.ptr, dim,
                                                   zero16.ctypes.data, c.ptr, dim, 1, h))
                configs["extra_gemm_half_%d_%s%s" % (dim, ta.decode(), tb.decode())] = tflops(2 * dim ** 3, sample_launches(fn, warm=2), 2500.0)
            # the same products on operands that are 1.0 everywhere: the same instructions at the same addresses, but hardly a
            # bit changes from one MFMA to the next, the matrix cores draw less power and the clock stays up -- how much of
            # the distance to nominal peak is the power limit and how much the kernel
            block = np.full(1 << 22, 0x3C00, np.uint16)
            for buf in (a, b):
                upload_tiled(buf, block, 2 * dim * dim)
            for ta, tb in ((b"N", b"N"), (b"T", b"N")):
                fn = lambda: oh.check(lib.och_gemm(oh.HALF, ta, tb, dim, dim, dim, one16.ctypes.data, a.ptr, dim, b.ptr, dim,
                                                   zero16.ctypes.data, c.ptr, dim, 1, h))
                configs["extra_gemm_half_%d_%s%s_constant_operands" % (dim, ta.decode(), tb.decode())] = tflops(2 * dim ** 3, sample_launches(fn, warm=2), 2500.0)
            for buf in (a, b, c):
                buf.free()
            a, b, c = [oh.DeviceBuffer(dim * dim, stream) for _ in range(3)]
            block = rng.integers(-128, 127, 1 << 22, endpoint=True).astype(np.int8)
            for buf in (a, b):
                upload_tiled(buf, block, dim * dim)
            one8 = np.array([1, 0], np.int8); zero8 = np.zeros(2, np.int8)
            for ta, tb in ((b"N", b"N"), (b"T", b"N"), (b"N", b"T")):
                fn = lambda: oh.check(lib.och_gemm(oh.INT8, ta, tb, dim, dim, dim, one8.ctypes.data, a.ptr, dim, b.ptr, dim,
                                                   zero8.ctypes.data, c.ptr, dim, 1, h))
                e = tflops(2 * dim ** 3, sample_launches(fn, warm=2), 5000.0)
                e["TOPs"] = e.pop("TFLOPs"); e["best_TOPs"] = e.pop("best_TFLOPs")
                configs["extra_gemm_int8_%d_%s%s" % (dim, ta.decode(), tb.decode())] = e
            for buf in (a, b, c):
                buf.free()
        # MGS-QR pattern on a 4096 x 4096 float64 matrix: per (i, j) pair one dot product (gemm M = N = 1, result kept
        # on the device) and one rank-1 update reading that device scalar, per column a norm and a division; window =
        # the first 64 columns (2016 pairs). The window is re-run on its own output: after the first pass the columns
        # are orthonormal, the arithmetic and the launches stay the same.
        m = 4096
        q = oh.DeviceBuffer(8 * m * m, stream)
        upload_tiled(q, rng.uniform(-1, 1, 1 << 22), 8 * m * m)
        rr = oh.DeviceBuffer(8 * 64 * 64, stream)
        consts = oh.to_device(np.array([1.0, 0.0, -1.0]), stream)
        c_one, c_zero, c_minus = [C.c_void_p(consts.address + 8 * i) for i in range(3)]
        col = lambda j: C.c_void_p(q.address + 8 * m * j)
        rij = lambda i, j: C.c_void_p(rr.address + 8 * (i + 64 * j))
        pairs = 64 * 63 // 2

        sm, stm, st0 = oh.sizes([m]), oh.strides([8]), oh.strides([0])

        # the pointers are made once: what is timed is the calls, not the construction of their arguments
        cols = [col(j) for j in range(64)]
        rijs = [[rij(i, j) for j in range(64)] for i in range(64)]
        gemm, mode_t, mode_n = lib.och_gemm, b"T", b"N"

        def mgs_window():
            for j in range(64):
                cj = cols[j]
                for i in range(j):
                    ci, r = cols[i], rijs[i][j]
                    gemm(F64, mode_t, mode_n, 1, 1, m, c_minus, ci, m, cj, m, c_zero, r, 1, 0, h)
                    gemm(F64, mode_n, mode_n, m, 1, 1, c_one, ci, m, r, 1, c_one, cj, m, 0, h)
                # column j is finished: its norm into a device scalar, the column divided by it (2 launches per column)
                lib.och_reduce_all_device(R["norm2"], F64, 1, sm, stm, cj, None, None, 0.0, rijs[j][j], None, h)
                lib.och_binary(B["divide"], F64, 1, sm, stm, cj, st0, rijs[j][j], stm, cj, h)

        def wall(fn, reps):
            fn(); stream.synchronize()
            ts = []
            for _ in range(reps):
                t0 = time.perf_counter(); fn(); stream.synchronize(); ts.append(time.perf_counter() - t0)
            ts.sort()
            return ts[len(ts) // 2], ts[0]

        def mgs_entry(med, best, launches_per_pair):
            return {"us_per_pair": round(med / pairs * 1e6, 3), "best_us_per_pair": round(best / pairs * 1e6, 3), "launches_per_pair": launches_per_pair,
                    "effective_GBps": round(pairs * (2 * 8 * m + 3 * 8 * m) / med / 1e9, 1)}
        wreps = 2 if profiling else 5
        configs["c5_mgs_qr_4096_first64cols"] = mgs_entry(*wall(mgs_window, wreps), round(2 + 128 / pairs, 3))
        # the same window recorded once and replayed as a graph: no host work per operation
        if not args.no_graph:
            oh.check(lib.och_stream_begin_capture(h))
            mgs_window()
            graph = C.c_void_p()
            oh.check(lib.och_stream_end_capture(h, C.byref(graph)))
            configs["c5_mgs_qr_4096_first64cols_graph_replay"] = mgs_entry(*wall(lambda: oh.check(lib.och_graph_launch(graph, h)), wreps), round(2 + 128 / pairs, 3))
            oh.check(lib.och_graph_destroy(graph))
        # the same window through the fused projection: one launch per column instead of two per pair

        def mgs_fused():
            for j in range(64):
                if j:
                    lib.och_mgs_project(F64, m, j, q.ptr, m, col(j), C.c_void_p(rr.address + 8 * 64 * j), h)
                lib.och_reduce_all_device(R["norm2"], F64, 1, sm, stm, col(j), None, None, 0.0, rij(j, j), None, h)
                lib.och_binary(B["divide"], F64, 1, sm, stm, col(j), st0, rij(j, j), stm, col(j), h)
        configs["c5_mgs_qr_4096_first64cols_fused_projection"] = mgs_entry(*wall(mgs_fused, wreps), round((63 + 128) / pairs, 4))
        for b in (q, rr, consts):
            b.free()
    result["configs"] = configs

    if profiling:
        # one plain float64 -> float64 copy of known size (134.2 MB read, 134.2 MB written): the
        # yardstick that scales the FETCH_SIZE / WRITE_SIZE counters of a profiling run
        ya, yb = oh.DeviceBuffer(8 * nn, stream), oh.DeviceBuffer(8 * nn, stream)
        oh.check(lib.och_memset_async(ya.ptr, 1, 8 * nn, h))
        oh.check(lib.och_copy(F64, F64, 2, shape, st_f64, ya.ptr, 2, shape, st_f64, yb.ptr, h))
        stream.synchronize()
        result["mode"] = "only " + args.only
        result["segments"] = segments
        print(json.dumps(result))
        return

    # ------------------------------------------------------------------ CPU baseline (oracle, Ocean's threading policy)
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        import oracle_lib as orc
        orc.setup(oh)
        threads = orc.lib.oracle_max_threads()
        p = orc.ptr

        def cpu_time(fn, budget_s, max_reps=3):
            """seconds per call: one untimed call, then up to max_reps timed calls within the budget"""
            fn()
            reps, t0 = 0, time.perf_counter()
            while reps < max_reps and (reps == 0 or time.perf_counter() - t0 < budget_s):
                fn(); reps += 1
            return (time.perf_counter() - t0) / reps, reps

        Z = np.empty((n, n)); TI = np.empty((n, n)); TF = np.empty((n, n))

        def cpu_step():
            assert orc.lib.oracle_binary(B["add"], F64, 2, shape, st_f64_T, p(hostA), st_row, p(hostR), st_f64, p(Z)) == 0
            assert orc.lib.oracle_copy(I32, F64, 2, shape, st_i32, p(hostI), 2, shape, st_f64, p(TI), threads) == 0
            assert orc.lib.oracle_binary(B["add"], F64, 2, shape, st_f64, p(Z), st_f64, p(TI), st_f64, p(Z)) == 0
            assert orc.lib.oracle_byteswap_copy(F32, F64, 2, shape, st_f32, p(hostFs), 2, shape, st_f64, p(TF), threads) == 0
            assert orc.lib.oracle_binary(B["multiply"], F64, 2, shape, st_f64, p(Z), st_f64, p(TF), st_f64, p(Z)) == 0

        sec, reps = cpu_time(cpu_step, 6.0, 5)
        others = {}
        result["cpu_baseline"] = {"value": round(step_bytes / sec / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
                                  "sample": "%d full-size configuration-2 steps (binary operations serial, copies on %d threads, as in Ocean's CPU module)" % (reps, threads),
                                  "ms_per_step": round(sec * 1e3, 1), "cpu": cpu_description(),
                                  "threading": "Ocean's rules: three-operand loops serial (apply_elemwise3.h:36,40), copies / casts and full reductions "
                                               "over all threads in contiguous index ranges (template_copy.c:37, reduce_all.h:64-83), axis reductions "
                                               "with the outputs dealt to the threads (reduce_axis.h:65-104)",
                                  "other_configs": others}
        del Z, TI, TF
        # configuration 1, full size: z = x * y + x, two serial three-operand loops
        x1 = rng.uniform(-1, 1, n1).astype(np.float32); y1 = rng.uniform(-1, 1, n1).astype(np.float32)
        t1 = np.empty(n1, np.float32); z1 = np.empty(n1, np.float32)
        s1, st1 = oh.sizes([n1]), oh.strides([4])

        def cpu_c1():
            assert orc.lib.oracle_binary(B["multiply"], F32, 1, s1, st1, p(x1), st1, p(y1), st1, p(t1)) == 0
            assert orc.lib.oracle_binary(B["add"], F32, 1, s1, st1, p(t1), st1, p(x1), st1, p(z1)) == 0
        sec, reps = cpu_time(cpu_c1, 2.0)
        others["c1_scale_and_add_f32_2^24"] = {"GBps": round(2 * 12 * n1 / sec / 1e9, 2), "ms": round(sec * 1e3, 1), "threads": 1, "sample": "%d full-size passes" % reps}
        del x1, y1, t1, z1
        # configuration 3, full size: full reductions over all threads, axis reductions with the outputs dealt to the threads
        for dt, es, nm, npt in ((F32, 4, "f32", np.float32), (F64, 8, "f64", np.float64)):
            nparent = (d0 + 4) * (d1 + 2) * d2                      # the padded parent of the 512 x 512 x 256 view
            v3 = rng.standard_normal(max(n3, nparent), dtype=npt)
            s3, st3 = oh.sizes([n3]), oh.strides([es])
            out = np.zeros(2, npt)
            for opn in ("sum", "norm2", "maximum"):
                sec, reps = cpu_time(lambda: orc.lib.oracle_reduce_all(R[opn], dt, 1, s3, st3, p(v3), None, None, 0.0, p(out), threads), 1.0)
                others["c3_%s_%s_8192^2" % (opn, nm)] = {"GBps": round(es * n3 / sec / 1e9, 2), "ms": round(sec * 1e3, 1), "threads": threads, "sample": "%d full-size passes" % reps}
            p0, p1 = (d0 + 4) * es, (d0 + 4) * (d1 + 2) * es
            parent = v3[:nparent]
            outa = np.empty(d0 * d1, npt)
            for axis, keep in ((0, (d1, d2)), (1, (d0, d2))):
                cfg = oh.ReduceAxisConfig()
                cfg.ndims = 2
                if axis == 0:
                    cfg.size[0], cfg.size[1] = d1, d2; cfg.strides1[0], cfg.strides1[1] = p0, p1
                    cfg.rsize[0], cfg.rstrides[0] = d0, es
                else:
                    cfg.size[0], cfg.size[1] = d0, d2; cfg.strides1[0], cfg.strides1[1] = es, p1
                    cfg.rsize[0], cfg.rstrides[0] = d1, p0
                cfg.strides2[0], cfg.strides2[1] = es, es * keep[0]
                cfg.rdims = 1; cfg.ptr1, cfg.ptr2 = parent.ctypes.data, outa.ctypes.data
                for opn in ("sum", "minimum"):
                    sec, reps = cpu_time(lambda: orc.lib.oracle_reduce_axis_threads(R[opn], dt, C.byref(cfg), 0.0, threads), 1.0)
                    others["c3_axis%d_%s_%s_512x512x256" % (axis, opn, nm)] = {"GBps": round(es * (d0 * d1 * d2 + keep[0] * keep[1]) / sec / 1e9, 2), "ms": round(sec * 1e3, 1),
                                                                                 "threads": threads, "sample": "%d full-size passes" % reps}
            del v3, parent, outa
        # configuration 4, full size: converting copies over all threads
        src16 = rng.integers(-32768, 32767, 2 * n4, dtype=np.int16, endpoint=True); dst32 = np.empty(n4, np.float32)
        sz4 = oh.sizes([e0, e1, e2])
        st_src, st_dst = oh.strides([4, 4 * e0, 4 * e0 * e1]), oh.strides([4, 4 * e0, 4 * e0 * e1])
        sec, reps = cpu_time(lambda: orc.lib.oracle_byteswap_copy(I16, F32, 3, sz4, st_src, p(src16), 3, sz4, st_dst, p(dst32), threads), 2.0)
        others["c4_int16_swapped_step2_to_f32_1024x1024x64"] = {"GBps": round(6 * n4 / sec / 1e9, 2), "ms": round(sec * 1e3, 1), "threads": threads, "sample": "%d full-size passes" % reps}
        del src16, dst32
        srcc = rng.uniform(-1, 1, 2 * n4b).astype(np.float32); dstc = np.empty(2 * n4b, np.float64)
        s4, sa, sb = oh.sizes([n4b]), oh.strides([8]), oh.strides([16])
        sec, reps = cpu_time(lambda: orc.lib.oracle_copy(CF, CD, 1, s4, sa, p(srcc), 1, s4, sb, p(dstc), threads), 2.0)
        others["c4_cfloat_to_cdouble_2^26"] = {"GBps": round(24 * n4b / sec / 1e9, 2), "ms": round(sec * 1e3, 1), "threads": threads, "sample": "%d full-size passes" % reps}
        del srcc, dstc
        # configuration 5: Ocean's built-in GEMM (ocean_custom_blas.c, a plain triple loop) at a reduced size; the full-size
        # time is an extrapolation by the flop count and is labelled so
        for dt, nm, npt, dim, full, flop_per_mac in ((F64, "double", np.float64, 1024, 8192, 2), (F32, "float", np.float32, 1024, 8192, 2), (CF, "cfloat", np.complex64, 512, 4096, 8)):
            if nm == "cfloat":
                a = (rng.uniform(-1, 1, (dim, dim)) + 1j * rng.uniform(-1, 1, (dim, dim))).astype(npt); b = a.T.copy()
            else:
                a = rng.uniform(-1, 1, (dim, dim)).astype(npt); b = rng.uniform(-1, 1, (dim, dim)).astype(npt)
            c = np.zeros((dim, dim), npt)
            one = np.array([1, 0], dtype=a.real.dtype); zero = np.zeros(2, dtype=a.real.dtype)
            sec, reps = cpu_time(lambda: orc.lib.oracle_gemm(dt, b"N", b"N", dim, dim, dim, p(one), p(a), dim, p(b), dim, p(zero), p(c), dim, threads), 2.0, 2)
            gf = flop_per_mac * dim ** 3 / sec / 1e9
            others["c5_gemm_%s_%d_NN" % (nm, dim)] = {"GFLOPs": round(gf, 2), "ms": round(sec * 1e3, 1), "threads": threads, "sample": "%d products of %d^3" % (reps, dim),
                                                      "extrapolated_seconds_at_%d^3" % full: round(flop_per_mac * full ** 3 / gf / 1e9, 1)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
