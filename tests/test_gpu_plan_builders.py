"""The row side of a plan put in order two ways: by the counting sorts written for this layout (per column
panel over the heavy rows' ranks, then by row for the light rows) and by one library radix sort of
(key, position) pairs. Both must give the same plan, array for array, on patterns that exercise every
branch: no heavy rows, only heavy rows, one panel, empty columns and rows, unsorted and repeated rows inside
a column, columns of length one, tiny segments, row counts that need one, two and three light passes.
"""
import ctypes as C
import zlib

import numpy as np
import pytest

from bidmat_amd import gen, hip_abi
from bidmat_amd.device import DeviceArray
from util import random_csc

pytestmark = pytest.mark.gpu

ARRAYS = ("pc", "perm", "segstart", "segrow", "rowseg", "rowptr")
SCALARS = ("nseg", "nheavy", "npanels", "panel_cols", "seglen") + tuple("xcd_start%d" % i for i in range(9))


def export(hip, plan):
    out = {}
    for name in SCALARS:
        out[name] = hip.bidmat_plan_info(plan, name.encode())
    for name in ARRAYS:
        p, n = C.c_void_p(), C.c_longlong()
        hip_abi.check(hip.bidmat_plan_array(plan, name.encode(), C.byref(p), C.byref(n)), name)
        a = np.empty(n.value, np.int32)
        if n.value:
            hip_abi.check(hip.bidmat_memcpy_d2h(a.ctypes.data, p, 4 * n.value))
        out[name] = a
    return out


def both_builders(hip, nrows, ncols, ir, jc, k, **opts):
    nnz = int(ir.size)
    d_ir, d_jc = DeviceArray.from_numpy(ir), DeviceArray.from_numpy(jc)
    old = {o: hip.bidmat_get_option(o.encode()) for o in list(opts) + ["plan_builder"]}
    got = []
    try:
        for o, v in opts.items():
            hip_abi.check(hip.bidmat_set_option(o.encode(), v), o)
        for builder in (1, 0):
            hip_abi.check(hip.bidmat_set_option(b"plan_builder", builder))
            plan = C.c_void_p()
            hip_abi.check(hip.bidmat_plan_create(nrows, ncols, nnz, d_ir.ptr, d_jc.ptr, k, C.byref(plan)), "plan_create")
            got.append(export(hip, plan))
            hip_abi.check(hip.bidmat_plan_destroy(plan))
    finally:
        for o, v in old.items():
            hip_abi.check(hip.bidmat_set_option(o.encode(), v), o)
        d_ir.free(); d_jc.free()
    ref, new = got
    for name in SCALARS:
        assert ref[name] == new[name], "%s: %d (sorted) vs %d (binned)" % (name, ref[name], new[name])
    for name in ARRAYS:
        assert ref[name].size == new[name].size, name
        if not np.array_equal(ref[name], new[name]):
            bad = np.flatnonzero(ref[name] != new[name])
            raise AssertionError("%s differs at %d of %d positions, first %d: %d vs %d" %
                                 (name, bad.size, ref[name].size, bad[0], ref[name][bad[0]], new[name][bad[0]]))
    # the order itself: a permutation of the positions, grouped as the plan says
    assert np.array_equal(np.sort(new["perm"]), np.arange(nnz, dtype=np.int32))
    return new


def zipf_rows(rng, nrows, n, s=1.1):
    p = 1.0 / np.arange(1, nrows + 1) ** s
    p /= p.sum()
    return rng.choice(nrows, size=n, p=p).astype(np.int32)


@pytest.mark.parametrize("case", ["zipf_heavy", "all_light", "one_panel", "empty_cols", "length_one_cols",
                                  "single_row", "many_rows_three_passes", "tiny_segments", "wide_panels"])
def test_binned_builder_gives_the_sorted_builder_plan(hip, case):
    rng = np.random.default_rng(zlib.crc32(case.encode()))
    k, opts = 64, {}
    if case == "zipf_heavy":            # heavy and light rows, unsorted rows with repeats inside columns
        nrows, ncols = 3000, 5000
        lengths = rng.integers(0, 80, size=ncols)
        jc = np.zeros(ncols + 1, np.int32); jc[1:] = np.cumsum(lengths)
        ir = zipf_rows(rng, nrows, int(jc[-1]))
        opts = dict(panel_kb=64, heavy_min=2, seglen=256)
    elif case == "all_light":           # uniform rows: nothing reaches the heavy threshold
        nrows, ncols = 50000, 4000
        _, ir, jc = random_csc(rng, nrows, ncols, lengths=rng.integers(0, 30, size=ncols))
        opts = dict(panel_kb=64)
    elif case == "one_panel":           # fewer than two panels: every row is light, rows with thousands of nonzeros
        nrows, ncols = 40, 500
        _, ir, jc = random_csc(rng, nrows, ncols, lengths=rng.integers(0, 40, size=ncols))
    elif case == "empty_cols":          # runs of empty columns, at the start, at panel borders, at the end
        nrows, ncols = 700, 6000
        lengths = rng.integers(0, 50, size=ncols)
        lengths[:300] = 0; lengths[1000:1400] = 0; lengths[-500:] = 0; lengths[rng.integers(0, ncols, 2000)] = 0
        jc = np.zeros(ncols + 1, np.int32); jc[1:] = np.cumsum(lengths)
        ir = zipf_rows(rng, nrows, int(jc[-1]), 1.3)
        opts = dict(panel_kb=32, heavy_min=1)
    elif case == "length_one_cols":     # a wave's 64 entries span 64 columns
        nrows, ncols = 500, 70000
        jc = np.arange(ncols + 1, dtype=np.int32)
        ir = zipf_rows(rng, nrows, ncols)
        opts = dict(panel_kb=256, heavy_min=4)
    elif case == "single_row":          # every nonzero in one row: one key per panel, long runs of equal keys
        nrows, ncols = 9, 3000
        lengths = rng.integers(1, 4, size=ncols)
        jc = np.zeros(ncols + 1, np.int32); jc[1:] = np.cumsum(lengths)
        ir = np.full(int(jc[-1]), 5, np.int32)
        opts = dict(panel_kb=16, heavy_min=1, seglen=64)
    elif case == "many_rows_three_passes":   # 2^23 rows: three light passes of 8 bits
        nrows, ncols = 1 << 23, 3000
        lengths = rng.integers(0, 200, size=ncols)
        jc = np.zeros(ncols + 1, np.int32); jc[1:] = np.cumsum(lengths)
        ir = rng.integers(0, nrows, size=int(jc[-1])).astype(np.int32)
        ir[::7] = rng.integers(0, 50, size=ir[::7].size)          # and a few heavy rows
        opts = dict(panel_kb=16, heavy_min=2)
    elif case == "tiny_segments":       # heavy rows whose panel runs are cut at global multiples of seglen
        nrows, ncols = 200, 20000
        lengths = rng.integers(20, 60, size=ncols)
        jc = np.zeros(ncols + 1, np.int32); jc[1:] = np.cumsum(lengths)
        ir = zipf_rows(rng, nrows, int(jc[-1]), 1.5)
        opts = dict(panel_kb=128, heavy_min=1, seglen=64)
    else:                               # wide_panels: few columns per tile
        nrows, ncols = 5000, 900
        lengths = rng.integers(500, 3000, size=ncols)
        jc = np.zeros(ncols + 1, np.int32); jc[1:] = np.cumsum(lengths)
        ir = zipf_rows(rng, nrows, int(jc[-1]), 1.05)
        opts = dict(panel_kb=16, heavy_min=8)
    plan = both_builders(hip, nrows, ncols, ir, jc, k, **opts)
    if case in ("zipf_heavy", "tiny_segments", "wide_panels", "length_one_cols"):
        assert plan["nheavy"] > 0
    if case in ("all_light", "one_panel"):
        assert plan["nheavy"] == 0


@pytest.mark.timeout(600)
def test_binned_builder_on_the_headline_pattern(hip):
    """100 M nonzeros, 5 139 heavy rows, 168 panels: the whole plan, array for array."""
    nrows, ncols = 100000, 500000
    ir, jc = gen.pattern(nrows, ncols, ("poisson", 200), ("zipf", 1.1), 2)
    plan = both_builders(hip, nrows, ncols, ir, jc, 256)
    assert plan["nheavy"] > 1000 and plan["nseg"] > 1000000


@pytest.mark.timeout(600)
def test_binned_builder_at_k128_with_a_million_rows(hip):
    """A fifth of configs[4] (80 M nonzeros, a million rows, two light passes, thousands of heavy rows)."""
    nrows, ncols = 1000000, 200000
    ir, jc = gen.pattern(nrows, ncols, ("poisson", 400), ("zipf", 1.05), 5)
    plan = both_builders(hip, nrows, ncols, ir, jc, 128)
    assert plan["nheavy"] > 1000
