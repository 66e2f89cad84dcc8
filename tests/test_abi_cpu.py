"""CPU-side checks of the C-ABI library and its host logic (no GPU needed):
  * the shared library loads and exports every function that include/ocean_hip.h declares,
    and the Python binding declares a prototype for each of them;
  * the support / result-type tables agree with the oracle's, which follow the reference's
    function tables (solid_core_gpu.src:42-439 lists the same (operation, type) pairs as the CPU);
  * the launch analysis (normalisation: drop, flip, sort, merge; kernel choice; chunking) keeps
    the set of element offsets of every operand, checked by brute-force enumeration, and its
    multiply-shift division constants divide exactly.
"""
import ctypes as C
import itertools
import os
import re

import numpy as np
import pytest

import helpers as H
import ocean_hip as oh

orc = H.orc
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "ocean_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(och_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_function():
    names = declared_functions()
    assert len(names) >= 58
    raw = C.CDLL(oh.LIB_PATH)
    missing = [n for n in names if not hasattr(raw, n)]
    assert not missing, "not exported: %s" % missing
    assert oh.MISSING == []
    unbound = [n for n in names if n not in oh.PROTOTYPES]
    assert not unbound, "no prototype in the binding: %s" % unbound
    stale = [n for n in oh.PROTOTYPES if n not in names]
    assert not stale, "binding declares functions the header does not: %s" % stale


def test_type_sizes_and_error_message():
    sizes = (C.c_int * 15).in_dll(oh.lib, "och_type_size")
    assert list(sizes) == [1, 1, 2, 4, 8, 1, 2, 4, 8, 2, 4, 8, 4, 8, 16]
    assert oh.lib.och_binary_supported(999, 0) == 0
    assert oh.lib.och_gemm_supported(H.CHALF) == 0
    plan = oh.ElemwisePlan()
    assert oh.lib.och_elemwise_analyze(4, None, 0, None, None, None, C.byref(plan)) != 0
    assert len(oh.lib.och_last_error()) > 0


def test_support_tables_match_oracle():
    for op in range(len(oh.BINARY_OPS)):
        for dt in H.ALL_TYPES:
            assert bool(oh.lib.och_binary_supported(op, dt)) == bool(orc.lib.oracle_binary_supported(op, dt)), (oh.BINARY_OPS[op], dt)
    for op in range(len(oh.UNARY_OPS)):
        for dt in H.ALL_TYPES:
            assert bool(oh.lib.och_unary_supported(op, dt)) == bool(orc.lib.oracle_unary_supported(op, dt)), (oh.UNARY_OPS[op], dt)
    for op in range(len(oh.REDUCE_OPS)):
        for dt in H.ALL_TYPES:
            sup = bool(oh.lib.och_reduce_supported(op, dt))
            assert sup == bool(orc.lib.oracle_reduce_supported(op, dt)), (oh.REDUCE_OPS[op], dt)
            if sup:
                assert oh.lib.och_reduce_result_dtype(op, dt) == orc.lib.oracle_reduce_result_dtype(op, dt)


def fastdiv(n, d, m, s1, s2):
    t = (m * n) >> 32
    return (t + ((n - t) >> s1)) >> s2


def test_division_constants_exact():
    """The kernels divide by dimension sizes with q = (t + ((n - t) >> s1)) >> s2, t = mulhi(m, n)."""
    rng = np.random.default_rng(1)
    divisors = [1, 2, 3, 4, 5, 7, 255, 256, 257, 641, 65535, 65536, 65537, (1 << 31) - 1, 1 << 31, (1 << 31) + 1, (1 << 32) - 1]
    divisors += [int(x) for x in rng.integers(1, 1 << 32, 40)]
    for d in divisors:
        # a 2-D shape whose first dimension cannot merge with the second: dim 0 keeps size d
        if d > 0x7FFF0000 or d < 2:             # (the whole shape must stay below 2^32 elements for one launch)
            continue
        plan = oh.elemwise_analyze([1], [d, 2], [[1, 2 * d + 3]], [0x10000])
        assert plan.ndims == 2 and plan.launches == 1
        for i in range(plan.ndims):
            dd, m, s1, s2 = plan.div_d[i], plan.div_m[i], plan.div_s1[i], plan.div_s2[i]
            assert dd >= 1
            probes = [0, 1, dd - 1, dd, dd + 1, 2 * dd - 1, 2 * dd, (1 << 32) - 1, (1 << 32) - dd, (1 << 31)] + [int(x) for x in rng.integers(0, 1 << 32, 200)]
            for n in probes:
                if 0 <= n < (1 << 32):
                    assert fastdiv(n, dd, m, s1, s2) == n // dd, (n, dd)
    # exhaustive for small divisors over a 16-bit range plus the top of the 32-bit range
    for d in range(1, 70):
        plan = oh.elemwise_analyze([1], [d * 16, 2], [[1, 16 * d + 16]], [0x10000])
        dd, m, s1, s2 = plan.div_d[0], plan.div_m[0], plan.div_s1[0], plan.div_s2[0]
        n = np.concatenate([np.arange(0, 1 << 16, dtype=np.uint64), np.arange((1 << 32) - (1 << 12), 1 << 32, dtype=np.uint64)])
        t = (np.uint64(m) * n) >> np.uint64(32)
        q = (t + ((n - t) >> np.uint64(s1))) >> np.uint64(s2)
        assert np.array_equal(q, n // np.uint64(dd)), dd


def offsets_of(size, strides, base=0):
    """Multiset of byte offsets visited by a strided operand."""
    off = np.zeros([1] * 0, dtype=np.int64) + base
    grids = np.meshgrid(*[np.arange(n, dtype=np.int64) for n in size], indexing="ij") if size else []
    total = np.zeros(tuple(size), dtype=np.int64) + base
    for g, s in zip(grids, strides):
        total = total + g * s
    return total


def joint_offsets(size, strides_list, bases):
    """Set of offset tuples (one entry per operand) visited together."""
    cols = [offsets_of(size, st, b).reshape(-1) for st, b in zip(strides_list, bases)]
    rows = np.stack(cols, axis=1)
    return rows[np.lexsort(rows.T[::-1])]


CASES = []
_rng = np.random.default_rng(99)
for _ in range(300):
    nd = int(_rng.integers(0, 6))
    size = [int(x) for x in _rng.choice([1, 1, 2, 3, 4, 5, 8, 16], size=nd)]
    nops = int(_rng.integers(1, 4))
    es = [int(x) for x in _rng.choice([1, 2, 4, 8, 16], size=nops)]
    strides_list = []
    for k in range(nops):
        # a permuted, possibly padded, possibly reversed or broadcast layout
        perm = _rng.permutation(nd)
        st = [0] * nd
        acc = es[k]
        for d in perm:
            mode = _rng.integers(0, 8)
            if mode == 0 and k < nops - 1:
                st[d] = 0                      # broadcast (inputs only)
            else:
                st[d] = acc * (-1 if mode == 1 else 1)
                acc *= size[d] * (2 if mode == 2 else 1)
        strides_list.append(st)
    CASES.append((size, es, strides_list))


@pytest.mark.parametrize("case", range(len(CASES)))
def test_normalisation_preserves_offsets(case):
    size, es, strides_list = CASES[case]
    bases = [1 << 20] * len(es)
    plan = oh.elemwise_analyze(es, size, strides_list, bases)
    nelem = int(np.prod(size)) if size else 1
    if nelem == 0:
        assert plan.ndims == 0
        return
    nsize = [plan.size[d] for d in range(plan.ndims)]
    assert int(np.prod(nsize)) == nelem
    nstr = [[plan.strides[k][d] for d in range(plan.ndims)] for k in range(len(es))]
    nbase = [bases[k] + plan.offset[k] for k in range(len(es))]
    assert np.array_equal(joint_offsets(size, strides_list, bases), joint_offsets(nsize, nstr, nbase))
    # canonical form: no unit dimensions (unless scalar), destination strides ascending and non-negative
    key = nstr[-1]
    if plan.ndims > 1:
        assert all(n > 1 for n in nsize)
    assert all(s >= 0 for s in key) or plan.ndims == 1
    assert key == sorted(key)
    # no two neighbouring dimensions are still mergeable
    for d in range(plan.ndims - 1):
        assert not all(nstr[k][d + 1] == nstr[k][d] * nsize[d] for k in range(len(es)))
    assert plan.kernel in (oh.KERNEL_WIDE, oh.KERNEL_MIXED, oh.KERNEL_SINGLE, oh.KERNEL_TILED, oh.KERNEL_ROWS)
    if plan.kernel == oh.KERNEL_ROWS:
        assert nstr[-1][0] == es[-1] and nsize[0] * es[-1] >= 24 and plan.row_elements == nsize[0]
        assert plan.row_units == oh.lib.och_elemwise_row_units(nsize[0], es[-1], plan.vec)
    elif plan.kernel != oh.KERNEL_SINGLE:
        assert nsize[0] % plan.vec == 0 or plan.ndims == 1


def test_kernel_choice():
    a = 1 << 20
    n = 4096
    # contiguous float64 add: wide, 2 elements per access
    p = oh.elemwise_analyze([8, 8, 8], [n, n], [[8, 8 * n]] * 3, [a, a, a])
    assert (p.ndims, p.kernel, p.vec, p.launches) == (1, oh.KERNEL_WIDE, 2, 1)
    # transposed input + row broadcast: tiled
    p = oh.elemwise_analyze([8, 8, 8], [n, n], [[8 * n, 8], [0, 8], [8, 8 * n]], [a, a, a])
    assert (p.ndims, p.kernel) == (2, oh.KERNEL_TILED)
    # step-2 source: mixed
    p = oh.elemwise_analyze([2, 4], [1024, 64], [[4, 4096], [4, 4096]], [a, a])
    assert p.kernel == oh.KERNEL_MIXED and p.vec == 4
    # odd length: vector body + scalar tail
    p = oh.elemwise_analyze([4, 4, 4], [4099], [[4]] * 3, [a, a, a])
    assert (p.kernel, p.launches) == (oh.KERNEL_WIDE, 2)
    # misaligned pointer of a unit-stride operand: aligned units of the destination, inputs read where they lie
    p = oh.elemwise_analyze([4, 4, 4], [4096], [[4]] * 3, [a + 4, a, a])
    assert p.kernel == oh.KERNEL_ROWS and p.vec == 4 and p.row_units == (12 + 4096 * 4 + 15) // 16
    # odd width of a sub-matrix, odd pitch, start inside a unit: rows
    p = oh.elemwise_analyze([1, 1], [999, 37], [[1, 1001], [1, 1001]], [a + 3, a + 5])
    assert p.kernel == oh.KERNEL_ROWS and p.vec == 16 and p.row_elements == 999 and p.row_units == (15 + 999 + 15) // 16
    # rows shorter than 24 bytes stay with one element per thread; a destination that is not unit-stride too
    p = oh.elemwise_analyze([1, 1], [21, 37], [[1, 64], [1, 64]], [a, a])
    assert p.kernel == oh.KERNEL_SINGLE
    p = oh.elemwise_analyze([2, 2], [999, 37], [[2, 2048], [4, 4096]], [a, a])
    assert p.kernel == oh.KERNEL_SINGLE
    # a broadcast input next to aligned operands is no reason for rows
    p = oh.elemwise_analyze([4, 4, 4], [4096, 8], [[4, 16384], [0, 4], [4, 16384]], [a, a, a])
    assert p.kernel == oh.KERNEL_MIXED
    # more than 2^32 elements: several launches
    p = oh.elemwise_analyze([1], [1 << 33], [[1]], [a])
    assert p.launches == 8 and p.kernel == oh.KERNEL_WIDE
    # first dimension equal to the vector width (one group per row: divisor 1)
    p = oh.elemwise_analyze([4, 4], [4, 5], [[4, 32], [4, 16]], [a, a])
    assert p.div_d[0] == 1 and fastdiv(12345, 1, p.div_m[0], p.div_s1[0], p.div_s2[0]) == 12345


def test_gemm_kernel_choice_knob_checks_its_argument():
    """och_gemm_set_kernel_choice touches no device: 0 to 4 are accepted, anything else is refused with a message."""
    import ocean_hip as oh
    for choice in (1, 2, 3, 4, 0):
        assert oh.lib.och_gemm_set_kernel_choice(choice) == 0
    for choice in (-1, 5, 99):
        assert oh.lib.och_gemm_set_kernel_choice(choice) != 0
        assert b"kernel choice" in oh.lib.och_last_error()
    assert oh.lib.och_gemm_set_kernel_choice(0) == 0


def test_float_products_and_the_tile_the_model_gives_them():
    """och_gemm_float_plan is host arithmetic on 256 compute units when there is no device. The expectations are the
    winners of measurements on an MI355X (TFLOP/s, NN products; tiled kernels / 128 x 128 / 64 x 64 tiles):
    512^3 10 / 7 / 16, 768^3 26 / 17 / 41, 1024^3 49 / 53 / 69, 1536^3 65 / 75 / 107, 1792^3 71 / 104 / 98,
    2048^3 91 / 136 / 125, 1024 x 2048 x 1024 65 / 92 / 102, 1024 x 1024 x 4096 63 / 104 / 97."""
    import ocean_hip as oh
    plan = oh.lib.och_gemm_float_plan
    assert oh.lib.och_gemm_set_kernel_choice(0) == 0
    for m, n, k, tile in [(512, 512, 512, 64), (768, 768, 768, 64), (1024, 1024, 1024, 64), (1536, 1536, 1536, 64),
                          (1024, 2048, 1024, 64), (1792, 1792, 1792, 128), (2048, 2048, 2048, 128), (1024, 1024, 4096, 128),
                          (4096, 4096, 4096, 256), (8192, 8192, 8192, 256), (8192, 8192, 64, 128)]:
        assert plan(m, n, k, 1) == tile, (m, n, k)
    # what the pipelined kernel does not take: M or N below 128 or not a multiple of 4, K below a slab
    for m, n, k in [(64, 4096, 4096), (4096, 126, 4096), (1026, 1024, 1024), (1024, 1024, 16)]:
        assert plan(m, n, k, 1) == 0, (m, n, k)
    # a batch of small products counts its tiles over all entries
    assert plan(256, 256, 256, 100) in (64, 128)
    # the knob overrides the model
    for choice, tile in [(1, 256), (2, 128), (3, 0), (4, 64)]:
        assert oh.lib.och_gemm_set_kernel_choice(choice) == 0
        try:
            assert plan(1024, 1024, 1024, 1) == tile
        finally:
            assert oh.lib.och_gemm_set_kernel_choice(0) == 0


def test_cutting_the_last_round_of_a_product_along_k():
    """och_gemm_split_plan (host arithmetic only): known answers, and for shapes from a fixed seed the rules a cut has to
    keep -- only a last round that is at most half full is cut, at most 8 shares per tile (64 for a product of less than
    one round), every share at least 8 slabs and none empty, the shares of the round within the compute units and within
    the 64 MB workspace, no cut that leaves most units idle, and a cost between the whole rounds and the rounds rounded up."""
    import ocean_hip as oh
    workspace = 1 << 26

    def plan(M, N, K, tm, tn, slab, es, units=256):
        rounds = C.c_double(-1.0)
        shares = oh.lib.och_gemm_split_plan(M, N, K, tm, tn, slab, es, units, C.byref(rounds))
        assert shares == oh.lib.och_gemm_split_plan(M, N, K, tm, tn, slab, es, units, None)
        return shares, rounds.value
    assert plan(8192, 8192, 8192, 256, 256, 32, 4) == (1, 4.0)                  # whole rounds: nothing to cut
    shares, rounds = plan(3000, 3000, 3000 - 3000 % 32, 128, 128, 32, 4)        # 576 tiles = 2 rounds + 64 tiles, 93 slabs
    assert shares == 4 and abs(rounds - (2 + (24 + 6 + 0.02 * 99) / 99)) < 1e-12
    assert plan(512, 512, 65536, 256, 256, 32, 4)[0] == 64                      # four tiles and a long K
    assert plan(128, 128, 262144, 128, 128, 32, 4)[0] == 1                      # one tile: 64 shares would leave 3/4 idle
    assert plan(2176, 2048, 1024, 128, 128, 16, 8)[0] == 8                      # 272 tiles: 16 in the last round, 64 slabs
    assert plan(2176, 2048, 240, 128, 128, 16, 8)[0] == 1                       # 15 slabs: too short to cut
    assert plan(4352, 4096, 8192, 256, 256, 32, 4, units=0) == (1, 0.0)         # nothing to plan for
    rng = np.random.default_rng(77)
    tiles_of = [(256, 256, 32, 4), (128, 128, 32, 4), (256, 128, 16, 8), (128, 128, 16, 8), (128, 128, 32, 8), (128, 64, 16, 16)]
    cut = 0
    for n in range(4000):
        tm, tn, slab, es = tiles_of[n % len(tiles_of)]
        units = (256, 304, 64, 1)[(n // 7) % 4]
        M, N = int(rng.integers(1, 9000)), int(rng.integers(1, 9000))
        K = int(rng.integers(1, 3000 if n % 2 else 300)) * slab
        shares, rounds = plan(M, N, K, tm, tn, slab, es, units)
        tiles = -(-M // tm) * -(-N // tn)
        rest, slabs = tiles % units, K // slab
        assert 1 <= shares <= (64 if tiles < units else 8), (M, N, K, shares)
        assert tiles // units <= rounds <= -(-tiles // units) + 1e-12
        if rest == 0 or rest * 2 > units or slabs < 16:
            assert shares == 1
        if shares == 1:
            assert rounds == -(-tiles // units)
            continue
        cut += 1
        length = -(-slabs // shares)
        assert length >= 8 and length * (shares - 1) < slabs, "a share shorter than 8 slabs, or an empty one"
        assert rest * shares <= units and rest * shares * 2 >= units
        assert rest * shares * tm * tn * es <= workspace
        assert rounds < -(-tiles // units)
    assert cut > 200


def test_cutting_a_large_reduction_into_launches():
    """och_reduce_cut_parts (host arithmetic only): the boxes are disjoint, cover the tensor, hold at most `limit` elements
    each, and never cut dimension 0; a dimension 0 beyond the limit is refused."""
    import ocean_hip as oh
    rng = np.random.default_rng(12)
    cases = [([64, 20, 12, 9], 2304), ([64, 20, 12, 9], 997), ([63, 280], 64), ([5, 3, 2, 2, 3], 7), ([7], 7), ([4, 1, 6], 4),
             ([1 << 20, 1 << 13, 1 << 5], 0xFFFF0000), ([1 << 31, 3, 40], 0xFFFF0000), ([3, 1 << 33], 0xFFFF0000)]
    cases += [([int(v) for v in rng.integers(1, 9, rng.integers(2, 6))], int(rng.integers(8, 200))) for _ in range(200)]
    for size, limit in cases:
        nd, cap = len(size), 4096
        starts, counts = (C.c_size_t * (cap * nd))(), (C.c_size_t * (cap * nd))()
        n = oh.lib.och_reduce_cut_parts(nd, oh.sizes(size), limit, cap, starts, counts)
        if size[0] > limit:
            assert n == -1
            continue
        assert 1 <= n <= cap, (size, limit, n)
        total = 0
        small = int(np.prod(size, dtype=np.float64)) <= 1 << 20
        seen = np.zeros(size[::-1], np.int32) if small else None
        for k in range(n):
            st, ct = [starts[k * nd + d] for d in range(nd)], [counts[k * nd + d] for d in range(nd)]
            assert st[0] == 0 and ct[0] == size[0], "dimension 0 is never cut"
            assert all(ct[d] >= 1 and st[d] + ct[d] <= size[d] for d in range(nd))
            vol = 1
            for c in ct:
                vol *= c
            assert vol <= limit, (size, limit, st, ct)
            total += vol
            if small:
                seen[tuple(slice(st[d], st[d] + ct[d]) for d in range(nd - 1, -1, -1))] += 1
        want = 1
        for v in size:
            want *= v
        assert total == want, (size, limit)
        if small:
            assert (seen == 1).all(), (size, limit)
        # a full run holds more than half the limit and at most one run per outer index is partial: under four times the minimum
        assert n <= 4 * -(-want // limit), (size, limit, n)


def test_units_of_a_row_partition_it():
    """The row kernels' work items: for every width, element size and placement of a row the ranges [lo, hi) of its units
    cover the row exactly once; units that take the one-access path (lo = 0, hi = vec) start on an aligned address; no
    unit reaches outside the row; the number of units given to every row is enough for the worst placement."""
    first, lo, hi = C.c_longlong(), C.c_int(), C.c_int()
    for es in (1, 2, 4, 8):
        for vec in {16 // es, max(1, 8 // es), max(1, 4 // es)} - {1}:
            wd = vec * es
            for n0 in list(range(1, 70)) + [255, 256, 257, 1000, 1001, 4097]:
                units = oh.lib.och_elemwise_row_units(n0, es, vec)
                for m in range(0, wd, es):
                    covered = np.zeros(n0, np.int32)
                    for c in range(units + 2):
                        any_ = oh.lib.och_elemwise_row_unit(c, m, es, vec, n0, C.byref(first), C.byref(lo), C.byref(hi))
                        if not any_:
                            assert hi.value <= lo.value
                            continue
                        assert c < units, (es, vec, n0, m, c)
                        assert 0 <= lo.value < hi.value <= vec
                        a, b = first.value + lo.value, first.value + hi.value
                        assert 0 <= a and b <= n0
                        covered[a:b] += 1
                        if lo.value == 0 and hi.value == vec:
                            assert (m + first.value * es) % wd == 0
                    assert (covered == 1).all(), (es, vec, n0, m)


def test_elementwise_launch_limit_cuts_calls_into_runs():
    """och_elemwise_set_launch_limit lowers the number of elements per launch, so that the cutting of tensors above
    2^32 - 2^16 elements can be seen on small ones: och_elemwise_analyze reports the launches of a call without a GPU."""
    import ocean_hip as oh
    a = 1 << 20
    try:
        assert oh.lib.och_elemwise_set_launch_limit(63) == -1 and oh.lib.och_elemwise_set_launch_limit((1 << 32) + 5) == -1
        assert oh.lib.och_elemwise_set_launch_limit(1000) == 0
        # one dimension: runs of the largest multiple of 64 below the limit (960), 5000 = 5 * 960 + 200
        p = oh.elemwise_analyze([4, 4], [5000], [[4], [4]], [a, a])
        assert p.launches == 6 and p.kernel == oh.KERNEL_WIDE
        # one dimension whose last run is not a whole number of vectors: body + tail in that run only
        p = oh.elemwise_analyze([4, 4], [5003], [[4], [4]], [a, a])
        assert p.launches == 7
        # two dimensions that do not merge: runs of whole indices of the outer one (1000 // 48 = 20 of 45 -> 3 launches)
        p = oh.elemwise_analyze([4, 4], [48, 45], [[4, 256], [4, 192]], [a, a])
        assert p.launches == 3 and p.ndims == 2
        # one index of the outer dimension is still too long: walked index by index, each cut inside (3 x 3 runs)
        p = oh.elemwise_analyze([4, 4], [2560, 3], [[4, 16384], [4, 10240]], [a, a])
        assert p.launches == 9
        assert oh.lib.och_elemwise_set_launch_limit(0) == 0
        p = oh.elemwise_analyze([4, 4], [5000], [[4], [4]], [a, a])
        assert p.launches == 1
    finally:
        oh.lib.och_elemwise_set_launch_limit(0)


PIPELINED_GEMM_SOURCES = ["och_gemm_f32p.hip", "och_gemm_f64p.hip", "och_gemm_c32p.hip", "och_gemm_c64p.hip"]


@pytest.mark.parametrize("source", PIPELINED_GEMM_SOURCES)
def test_m0_is_used_by_the_loads_to_lds_only(source):
    """The pipelined GEMM kernels pass the LDS target of `global_load_lds_dwordx4` in M0 from inline assembly without
    the compiler knowing. That is sound only while the compiler itself keeps nothing in M0 across those statements
    (dynamic register indexing, LDS-direct reads, s_sendmsg and v_readlane with M0 would): every mention of M0 in the
    generated code of these kernels must be the `s_mov_b32 m0, <sgpr>` of such a load, followed by the load within the
    next two instructions."""
    import re
    import shutil
    import subprocess
    import tempfile
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc is not available")
    src = os.path.join(ROOT, "ocean-tensor-package_amd", "csrc", source)
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k.s")
        subprocess.run([hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
                        "-packed-fp32-ops", "-Wno-unused-command-line-argument", "--cuda-device-only", "-S", src, "-o", out],
                       check=True, capture_output=True)
        lines = [ln.split(";")[0].strip() for ln in open(out)]
    code = [ln for ln in lines if ln and not ln.startswith(".") and not ln.endswith(":")]
    uses = [i for i, ln in enumerate(code) if re.search(r"\bm0\b", ln)]
    assert len(uses) >= 8, "no load to LDS found in %s" % source
    for i in uses:
        assert re.fullmatch(r"s_mov_b32 m0, s\d+", code[i]), code[i]
        assert any(c.startswith("global_load_lds_dwordx4") for c in code[i + 1:i + 3]), code[i:i + 3]


def library_kernel_metadata():
    """(kernel name, scratch bytes per lane, vector registers) of every gfx950 kernel in csrc/libocean_hip.so, read from the
    notes of the code objects it carries: the .hip_fatbin section is a row of clang offload bundles (magic, entry count,
    then per entry offset, size and target triple), each holding one translation unit's code object."""
    import shutil
    import struct
    import subprocess
    import tempfile
    tools = "/opt/rocm/llvm/bin"
    objcopy, readelf = os.path.join(tools, "llvm-objcopy"), os.path.join(tools, "llvm-readelf")
    if not (os.path.exists(objcopy) and os.path.exists(readelf)):
        pytest.skip("the LLVM binary tools of ROCm are not available")
    magic = b"__CLANG_OFFLOAD_BUNDLE__"
    kernels = []
    with tempfile.TemporaryDirectory() as tmp:
        fat = os.path.join(tmp, "fat.bin")
        subprocess.run([objcopy, "-O", "binary", "--only-section=.hip_fatbin", oh.LIB_PATH, fat], check=True, capture_output=True)
        blob = open(fat, "rb").read()
        at = blob.find(magic)
        while at >= 0:
            (entries,) = struct.unpack_from("<Q", blob, at + len(magic))
            pos = at + len(magic) + 8
            for _ in range(entries):
                offset, size, tlen = struct.unpack_from("<QQQ", blob, pos)
                triple = blob[pos + 24:pos + 24 + tlen].decode()
                pos += 24 + tlen
                if "gfx950" not in triple or size == 0:
                    continue
                co = os.path.join(tmp, "k.co")
                with open(co, "wb") as out:
                    out.write(blob[at + offset:at + offset + size])
                notes = subprocess.run([readelf, "--notes", co], check=True, capture_output=True, text=True).stdout
                name = scratch = vgprs = None
                for line in notes.splitlines():
                    line = line.strip()
                    if line.startswith(".name:"):
                        name = line.split(":", 1)[1].strip()
                    elif line.startswith(".private_segment_fixed_size:"):
                        scratch = int(line.split(":")[1])
                    elif line.startswith(".vgpr_count:"):
                        vgprs = int(line.split(":")[1])
                    elif line.startswith(".wavefront_size:") and name is not None and scratch is not None:
                        kernels.append((name, scratch, vgprs))
                        name = scratch = vgprs = None
            at = blob.find(magic, at + len(magic))
    return kernels


def test_no_kernel_of_the_library_lives_in_scratch_memory():
    """A change far from a kernel (a conversion routine in a shared header, say) can cost a kernel with hundreds of live
    accumulators its registers without any test of results noticing: the half GEMM once went from 1100 to 50 TFLOP/s that
    way, with a kilobyte and more of scratch per lane. So the scratch every kernel of the built library asks for is held
    to what it is known to need: nothing for the float, double and complex pipelined GEMM kernels beyond a few spilled
    registers, at most 128 bytes per lane for the 8-bit kernels and the half kernels of whole tiles, 320 for the half
    kernels of ragged ones, 768 for the fused projection, 32 for the per-thread axis reduction, none for anything
    else (every elementwise, copy, fill, index and other reduction kernel)."""
    kernels = library_kernel_metadata()
    assert len(kernels) > 5000
    limits = [("gemm_float_pipe_kernel", 32), ("gemm_double_pipe", 32), ("gemm_cfloat_pipe", 64), ("gemm_cdouble_pipe", 64),
              ("Li128ELi128ELi2ELi2ELi64E", 128),          # the half kernels of whole 256 x 256 tiles: waves of 128 x 128
              ("gemm_half_kernel", 320), ("gemm_byte_kernel", 128), ("mgs_project_kernel", 768), ("axis_thread_kernel", 32),
              ("", 0)]                                        # every elementwise, copy, fill, index and other reduction kernel: none
    seen = set()
    for name, scratch, _ in kernels:
        prefix, limit = next((p, l) for p, l in limits if p in name)
        seen.add(prefix)
        assert scratch <= limit, "%s: %d bytes of scratch per lane (limit %d)" % (name, scratch, limit)
    assert seen == {p for p, _ in limits}


def test_microbenchmarks_live_in_their_own_library():
    """The product header declares no measurement tool; the two micro-benchmarks are declared in include/ocean_hip_bench.h and
    exported by csrc/libocean_hip_bench.so only."""
    import ocean_hip_bench as ohb
    assert not [n for n in declared_functions() if "bench" in n]
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "ocean_hip_bench.h")).read(), flags=re.S)
    names = sorted(set(re.findall(r"\b(och_[a-z0-9_]+)\s*\(", text)))
    assert names == ["och_membench", "och_mfmabench"]
    raw = C.CDLL(ohb.LIB_PATH)
    assert all(hasattr(raw, n) for n in names)
    product = C.CDLL(oh.LIB_PATH)
    assert not any(hasattr(product, n) for n in names)
