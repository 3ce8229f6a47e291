"""A *^ S with the densest rows of the pattern multiplied as a dense block on the matrix cores.

The dense block changes the order of the additions of those rows only, so the bar is the path's tolerance
against the oracle's float64 arbiter, for every row; rows outside the block must keep the bits of the plain walk
over the plan. What must not change at all: values of A that are not finite (an absent entry's zero may not turn
them into a NaN of that row), patterns with repeated entries (no dense block), and the bits from run to run.
"""
import ctypes as C

import numpy as np
import pytest

import oracle
from bidmat_amd import hip_abi
from util import Dev, make_plan

pytestmark = pytest.mark.gpu


def power_law_csc(rng, nrows, ncols, mean_len, a=1.1, sort_rows=True, shuffle_rows=False):
    p = 1.0 / np.arange(1, nrows + 1) ** a
    p /= p.sum()
    names = rng.permutation(nrows) if shuffle_rows else np.arange(nrows)      # frequent rows need not carry small indices
    lens = rng.poisson(mean_len, size=ncols)
    cols = []
    for c in range(ncols):
        rows = np.unique(rng.choice(nrows, size=int(lens[c]), p=p))
        rows = names[rows]
        rows = np.sort(rows) if sort_rows else rng.permutation(rows)
        cols.append(rows.astype(np.int32))
    jc = np.zeros(ncols + 1, np.int32)
    jc[1:] = np.cumsum([x.size for x in cols])
    return np.concatenate(cols).astype(np.int32), jc


@pytest.fixture()
def dense_options(hip):
    """Dense blocks for small patterns too; everything back to the defaults afterwards."""
    names = ("dense_rows", "dense_min_pct", "dense_min_nnz", "dense_cb")
    before = {n: hip.bidmat_get_option(n.encode()) for n in names}
    hip_abi.check(hip.bidmat_set_option(b"dense_min_nnz", 0))
    yield hip
    for n, v in before.items():
        hip_abi.check(hip.bidmat_set_option(n.encode(), v))


def plan_info(hip, plan, name):
    return int(hip.bidmat_plan_info(plan, name.encode()))


def run(hip, plan, k, dA, dv, dG, beta=0):
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, dA.ptr, dv.ptr, dG.ptr, beta, None))
    hip_abi.check(hip.bidmat_synchronize())
    return dG.numpy()


# k: both widths of the kernel (up to 128 and up to 256), odd tails, not a multiple of 4 (no 128-bit stores)
@pytest.mark.parametrize("k", [65, 96, 128, 130, 200, 256])
@pytest.mark.parametrize("shape", [(3000, 4001, 60, 0), (900, 1500, 150, 16), (2000, 2050, 80, 0)],
                         ids=["4001cols", "cb16", "2050cols"])
def test_dense_block_against_the_oracle(dense_options, k, shape):
    hip = dense_options
    nrows, ncols, mean_len, cb = shape
    hip_abi.check(hip.bidmat_set_option(b"dense_cb", cb))
    rng = np.random.default_rng(17 * k + nrows)
    ir, jc = power_law_csc(rng, nrows, ncols, mean_len, shuffle_rows=True, sort_rows=(k % 2 == 0))
    nnz = ir.size
    A = rng.standard_normal(k * ncols).astype(np.float32)
    v = (1.0 - rng.random(nnz)).astype(np.float32)
    d = Dev(ir=ir, jc=jc, A=A, v=v)
    d.zeros("G", k * nrows); d.zeros("G0", k * nrows)
    plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
    nd = plan_info(hip, plan, "dense_rows")
    assert nd >= 32 and nd % 32 == 0, "the pattern has rows in more than 15 %% of the columns: %d dense rows" % nd
    got = run(hip, plan, k, d.A, d.v, d.G)
    ref64, sa = oracle.fsmultT_f64(A, k, nrows, v, ir, jc, nthreads=8)
    ok, worst = oracle.within_tolerance(got, ref64, sa, 1e-4)
    assert ok, "A *^ S with %d dense rows differs from the oracle: %.3e" % (nd, worst)
    # the walk over all segments (the option switched off at call time) agrees on every other row, bit for bit
    hip_abi.check(hip.bidmat_set_option(b"dense_rows", 0))
    plain = run(hip, plan, k, d.A, d.v, d.G0)
    hip_abi.check(hip.bidmat_set_option(b"dense_rows", 128))
    ok0, worst0 = oracle.within_tolerance(plain, ref64, sa, 1e-4)
    assert ok0, worst0
    drow = np.empty(nd, np.int32)
    ptr, cnt = C.c_void_p(), C.c_longlong()
    hip_abi.check(hip.bidmat_plan_array(plan, b"drow", C.byref(ptr), C.byref(cnt)))
    assert cnt.value == nd
    hip_abi.check(hip.bidmat_memcpy_d2h(drow.ctypes.data, ptr, 4 * nd))
    counts = np.bincount(ir, minlength=nrows)
    assert counts[drow].min() >= 0.1 * ncols, "dense rows are frequent rows"
    assert np.all(np.diff(counts[drow].astype(np.int64)) <= 0), "ranked by count (these patterns are counted in full)"
    mask = np.ones(nrows, bool); mask[drow] = False
    g2, p2 = got.reshape(nrows, k), plain.reshape(nrows, k)
    assert np.array_equal(g2[mask], p2[mask]), "rows outside the dense block changed"
    assert not np.array_equal(g2[~mask], p2[~mask]) or nnz == 0, "the dense rows took the same path"
    # accumulate (beta = 1) and a second run: same bits
    again = run(hip, plan, k, d.A, d.v, d.G0)
    assert np.array_equal(again, got), "two runs differ"
    twice = run(hip, plan, k, d.A, d.v, d.G0, beta=1)
    ok2, worst2 = oracle.within_tolerance(twice, 2 * ref64, 2 * sa, 1e-4)
    assert ok2, "beta = 1 does not add to what was there: %.3e" % worst2
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


def test_values_that_are_not_finite_fall_back_to_the_segments(dense_options):
    hip = dense_options
    nrows, ncols, k = 2000, 3000, 256
    rng = np.random.default_rng(5)
    ir, jc = power_law_csc(rng, nrows, ncols, 80)
    nnz = ir.size
    A = rng.standard_normal(k * ncols).astype(np.float32)
    v = (1.0 - rng.random(nnz)).astype(np.float32)
    A2 = A.copy()
    A2[k * 1234 + 7] = np.inf           # one element of one column
    A2[k * 77 + 200] = np.nan
    d = Dev(ir=ir, jc=jc, A=A2, v=v)
    d.zeros("G", k * nrows); d.zeros("G0", k * nrows)
    plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
    assert plan_info(hip, plan, "dense_rows") >= 32
    got = run(hip, plan, k, d.A, d.v, d.G)
    hip_abi.check(hip.bidmat_set_option(b"dense_rows", 0))
    plain = run(hip, plan, k, d.A, d.v, d.G0)
    hip_abi.check(hip.bidmat_set_option(b"dense_rows", 128))
    assert np.array_equal(got, plain, equal_nan=True), "non-finite values of A spread differently with the dense block"
    # only the rows with a nonzero in those columns see them
    G = got.reshape(nrows, k)
    rows_inf = set(ir[jc[1234]:jc[1235]].tolist())
    bad = np.where(~np.isfinite(G[:, 7]))[0]
    assert set(bad.tolist()) == rows_inf
    # and with finite values again the dense block is back (the flag is per call)
    d.put("A", A)
    got2 = run(hip, plan, k, d.A, d.v, d.G)
    ref64, sa = oracle.fsmultT_f64(A, k, nrows, v, ir, jc, nthreads=8)
    ok, worst = oracle.within_tolerance(got2, ref64, sa, 1e-4)
    assert ok, worst
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


def test_repeated_entries_get_no_dense_block(dense_options):
    hip = dense_options
    nrows, ncols, k = 500, 800, 128
    rng = np.random.default_rng(9)
    ir, jc = power_law_csc(rng, nrows, ncols, 60)
    # repeat the first entry of every tenth column (the most frequent row, as a rule)
    cols = [ir[jc[c]:jc[c + 1]] for c in range(ncols)]
    for c in range(0, ncols, 10):
        if cols[c].size:
            cols[c] = np.concatenate([cols[c], cols[c][:1]])
    jc2 = np.zeros(ncols + 1, np.int32)
    jc2[1:] = np.cumsum([x.size for x in cols])
    ir2 = np.concatenate(cols).astype(np.int32)
    nnz = ir2.size
    A = rng.standard_normal(k * ncols).astype(np.float32)
    v = (1.0 - rng.random(nnz)).astype(np.float32)
    d = Dev(ir=ir2, jc=jc2, A=A, v=v)
    d.zeros("G", k * nrows)
    plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
    assert plan_info(hip, plan, "dense_rows") == 0
    got = run(hip, plan, k, d.A, d.v, d.G)
    ref64, sa = oracle.fsmultT_f64(A, k, nrows, v, ir2, jc2, nthreads=8)
    ok, worst = oracle.within_tolerance(got, ref64, sa, 1e-4)
    assert ok, worst
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


def test_patterns_without_dense_rows_and_other_k_keep_the_plain_walk(dense_options):
    hip = dense_options
    nrows, ncols = 4000, 3000
    rng = np.random.default_rng(11)
    # uniform rows: nothing is in 15 % of the columns
    lens = rng.poisson(30, size=ncols)
    cols = [np.sort(rng.choice(nrows, size=int(n), replace=False)).astype(np.int32) for n in lens]
    jc = np.zeros(ncols + 1, np.int32); jc[1:] = np.cumsum([x.size for x in cols])
    ir = np.concatenate(cols).astype(np.int32)
    d = Dev(ir=ir, jc=jc)
    plan = make_plan(hip, nrows, ncols, ir.size, d.ir, d.jc, 256)
    assert plan_info(hip, plan, "dense_rows") == 0
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()
    # a plan with a dense block, called with k outside (64, 256]: the plain walk, same as with the option off
    ir, jc = power_law_csc(rng, 1000, 1500, 60)
    nnz = ir.size
    for k in (32, 512):
        A = rng.standard_normal(k * 1500).astype(np.float32)
        v = (1.0 - rng.random(nnz)).astype(np.float32)
        d = Dev(ir=ir, jc=jc, A=A, v=v)
        d.zeros("G", k * 1000); d.zeros("G0", k * 1000)
        plan = make_plan(hip, 1000, 1500, nnz, d.ir, d.jc, 256)
        assert plan_info(hip, plan, "dense_rows") >= 32
        got = run(hip, plan, k, d.A, d.v, d.G)
        hip_abi.check(hip.bidmat_set_option(b"dense_rows", 0))
        plain = run(hip, plan, k, d.A, d.v, d.G0)
        hip_abi.check(hip.bidmat_set_option(b"dense_rows", 128))
        assert np.array_equal(got, plain)
        hip_abi.check(hip.bidmat_plan_destroy(plan))
        d.free()


def test_the_other_walks_over_the_plan_are_untouched(dense_options):
    """Row sums, stored values and the fused chain use the segments of all rows, dense block or not."""
    hip = dense_options
    nrows, ncols, k = 1500, 2500, 128
    rng = np.random.default_rng(13)
    ir, jc = power_law_csc(rng, nrows, ncols, 70)
    nnz = ir.size
    A = (0.01 + rng.random(k * nrows)).astype(np.float32)
    B = (0.01 + rng.random(k * ncols)).astype(np.float32)
    v = (1.0 - rng.random(nnz)).astype(np.float32)
    d = Dev(ir=ir, jc=jc, A=A, B=B, v=v)
    for name, n in (("s1", nrows), ("s2", nrows), ("G1", k * nrows), ("G2", k * nrows), ("G3", k * nrows)):
        d.zeros(name, n)
    plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
    assert plan_info(hip, plan, "dense_rows") >= 32
    hip_abi.check(hip.bidmat_spsum_rows_plan(plan, d.v.ptr, d.s1.ptr, 0, None))
    ref = np.bincount(ir, weights=v.astype(np.float64), minlength=nrows)
    assert np.allclose(d.s1.numpy(), ref, rtol=1e-5)
    # stored values: the plain walk (values in plan order); against the dense block within tolerance
    hip_abi.check(hip.bidmat_plan_set_values(plan, d.v.ptr, None))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.B.ptr, None, d.G1.ptr, 0, None))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.B.ptr, d.v.ptr, d.G2.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    ref64, sa = oracle.fsmultT_f64(B, k, nrows, v, ir, jc, nthreads=8)
    for name, got in (("stored", d.G1.numpy()), ("passed", d.G2.numpy())):
        ok, worst = oracle.within_tolerance(got, ref64, sa, 1e-4)
        assert ok, (name, worst)
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


def test_graph_replay_with_the_dense_block(dense_options):
    """A *^ S with a dense block recorded into a HIP graph: every replay gives what the eager call gives, also the
    replay whose A holds a value that is not finite (the fall-back to the segments is decided on the device)."""
    hip = dense_options
    nrows, ncols, k = 1200, 2000, 256
    rng = np.random.default_rng(21)
    ir, jc = power_law_csc(rng, nrows, ncols, 70)
    nnz = ir.size
    A = rng.standard_normal(k * ncols).astype(np.float32)
    v = (1.0 - rng.random(nnz)).astype(np.float32)
    d = Dev(ir=ir, jc=jc, A=A, v=v)
    d.zeros("G", k * nrows); d.zeros("G2", k * nrows)
    plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
    assert plan_info(hip, plan, "dense_rows") >= 32
    st = C.c_void_p()
    hip_abi.check(hip.bidmat_stream_create(C.byref(st)))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, d.v.ptr, d.G.ptr, 0, st))       # sizes the stream's scratch
    hip_abi.check(hip.bidmat_stream_synchronize(st))
    hip_abi.check(hip.bidmat_graph_begin_capture(st))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, d.v.ptr, d.G.ptr, 0, st))
    gx = C.c_void_p()
    hip_abi.check(hip.bidmat_graph_end_capture(st, C.byref(gx)))
    for rep in range(4):
        newA = rng.standard_normal(k * ncols).astype(np.float32)
        if rep == 2:
            newA[k * 5 + 3] = -np.inf
        hip_abi.check(hip.bidmat_memcpy_h2d(d.A.ptr, newA.ctypes.data, newA.nbytes))
        hip_abi.check(hip.bidmat_memset(d.G.ptr, 0xFF, d.G.nbytes))
        hip_abi.check(hip.bidmat_graph_launch(gx, st))
        hip_abi.check(hip.bidmat_stream_synchronize(st))
        hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, d.v.ptr, d.G2.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
        assert np.array_equal(d.G.numpy().view(np.int32), d.G2.numpy().view(np.int32)), "replay %d" % rep
        if rep == 2:
            hip_abi.check(hip.bidmat_set_option(b"dense_rows", 0))
            hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, d.v.ptr, d.G2.ptr, 0, None))
            hip_abi.check(hip.bidmat_synchronize())
            hip_abi.check(hip.bidmat_set_option(b"dense_rows", 128))
            assert np.array_equal(d.G.numpy().view(np.int32), d.G2.numpy().view(np.int32)), "the replay with -inf in A"
    hip_abi.check(hip.bidmat_graph_destroy(gx))
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    hip_abi.check(hip.bidmat_stream_destroy(st))
    d.free()


@pytest.mark.parametrize("k", [96, 256, 130])
def test_values_stored_in_the_plan_take_the_dense_block_too(dense_options, k):
    """bidmat_plan_set_values keeps the dense rows' values in the layout of the block's position table: a call without
    Sdata multiplies the same numbers in the same order as a call that passes them, so the results agree bit for bit,
    also after the values have been set anew, and a value of A that is not finite falls back to the segments."""
    hip = dense_options
    nrows, ncols = 2500, 3500
    rng = np.random.default_rng(40 + k)
    ir, jc = power_law_csc(rng, nrows, ncols, 90, shuffle_rows=True)
    nnz = ir.size
    A = rng.standard_normal(k * ncols).astype(np.float32)
    v = rng.standard_normal(nnz).astype(np.float32)
    d = Dev(ir=ir, jc=jc, A=A, v=v)
    d.zeros("G", k * nrows); d.zeros("G0", k * nrows)
    plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
    nd = plan_info(hip, plan, "dense_rows")
    assert nd >= 32
    before = hip.bidmat_plan_bytes(plan)
    for rep in range(2):
        passed = run(hip, plan, k, d.A, d.v, d.G)
        hip_abi.check(hip.bidmat_plan_set_values(plan, d.v.ptr, None))
        hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, None, d.G0.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
        stored = d.G0.numpy()
        assert np.array_equal(stored.view(np.uint32), passed.view(np.uint32)), "stored and passed values differ (round %d)" % rep
        if rep == 0:
            assert hip.bidmat_plan_bytes(plan) >= before + 4 * nnz + 4 * ncols * nd, "the plan counts what it stores"
            ref64, sa = oracle.fsmultT_f64(A, k, nrows, v, ir, jc, nthreads=8)
            ok, worst = oracle.within_tolerance(stored, ref64, sa, 1e-4)
            assert ok, worst
            v = rng.standard_normal(nnz).astype(np.float32)         # other values: set again
            d.v.upload(v)
    # the stored values without the dense block (option at call time): the walk over every row's segments
    hip_abi.check(hip.bidmat_set_option(b"dense_rows", 0))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, None, d.G.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    hip_abi.check(hip.bidmat_set_option(b"dense_rows", 128))
    walk = d.G.numpy()
    ref64, sa = oracle.fsmultT_f64(A, k, nrows, v, ir, jc, nthreads=8)
    ok, worst = oracle.within_tolerance(walk, ref64, sa, 1e-4)
    assert ok, worst
    assert not np.array_equal(walk, stored), "the dense rows took the same path"
    # a value of A that is not finite: the call falls back to exactly that walk
    A2 = A.copy(); A2[k * 17 + 3] = -np.inf
    d.A.upload(A2)
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, None, d.G0.ptr, 0, None))
    hip_abi.check(hip.bidmat_set_option(b"dense_rows", 0))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, None, d.G.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    hip_abi.check(hip.bidmat_set_option(b"dense_rows", 128))
    assert np.array_equal(d.G0.numpy(), d.G.numpy(), equal_nan=True)
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()
