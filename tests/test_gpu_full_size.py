"""Parity at the full sizes of the benchmark configurations, where the oracle cannot run the
whole problem in seconds: size-independent properties (the Frobenius identity that ties the
three products together, linearity, sum-of-sums) plus oracle checks on random samples of
columns / rows / nonzeros of the full-size result.
"""
import ctypes as C

import numpy as np
import pytest

import oracle
from bidmat_amd import gen, hip_abi
from bidmat_amd.device import DeviceArray
from util import make_plan

pytestmark = pytest.mark.gpu
RTOL = 1e-4


def close(x, ref64, sa, what):
    ok, worst = oracle.within_tolerance(x, ref64, sa, RTOL)
    assert ok, "%s: worst error measure %.3e" % (what, worst)


def sub_csc(ir, jc, vals, cols):
    """CSC restricted to the given columns (kept in the given order)."""
    lens = jc[cols + 1] - jc[cols]
    sjc = np.zeros(cols.size + 1, dtype=np.int32)
    sjc[1:] = np.cumsum(lens)
    idx = np.concatenate([np.arange(jc[c], jc[c + 1]) for c in cols]) if cols.size else np.zeros(0, np.int64)
    return (vals[idx] if vals is not None else None), ir[idx], sjc, idx


def rows_sub_csc(ir, jc, vals, rows):
    """All nonzeros of the given rows, as a CSC over all columns with rows renumbered 0..len-1."""
    pos = np.full(int(ir.max()) + 1, -1, dtype=np.int64)
    pos[rows] = np.arange(rows.size)
    keep = np.flatnonzero(pos[ir] >= 0)
    ic = np.searchsorted(jc, keep, side="right") - 1
    sjc = np.zeros(jc.size, dtype=np.int32)
    sjc[1:] = np.cumsum(np.bincount(ic, minlength=jc.size - 1))
    return vals[keep], pos[ir[keep]].astype(np.int32), sjc


@pytest.mark.timeout(600)
def test_headline_pattern_dds_dsmult_dsmultT(hip):
    """configs[1] (DDS) and configs[2] (A*^S) at full size, plus A*S on the same pattern."""
    cfg = gen.config("HEAD", 1.0)
    k, nrows, ncols = cfg["k"], cfg["nrows"], cfg["ncols"]
    ir, jc, vals = cfg["ir"], cfg["jc"], cfg["vals"]
    nnz = int(ir.size)
    assert 0.9e8 < nnz < 1.1e8
    assert oracle.check(nrows, ncols, nnz, ir, jc, 0)[0] == 0
    A, B, AT = cfg["A"], cfg["B"], cfg["A_T"]
    dA, dB, dAT = DeviceArray.from_numpy(A), DeviceArray.from_numpy(B), DeviceArray.from_numpy(AT)
    dv, dir_, djc = DeviceArray.from_numpy(vals), DeviceArray.from_numpy(ir), DeviceArray.from_numpy(jc)
    dP, dC, dG = DeviceArray(nnz, np.float32), DeviceArray(k * ncols, np.float32), DeviceArray(k * nrows, np.float32)
    plan = make_plan(hip, nrows, ncols, nnz, dir_, djc, k)
    hip_abi.check(hip.bidmat_dds_csc(k, ncols, nnz, dA.ptr, dB.ptr, dir_.ptr, djc.ptr, dP.ptr, 0, None))
    hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, nnz, dA.ptr, dv.ptr, dir_.ptr, djc.ptr, dC.ptr, 0, None))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, dAT.ptr, dv.ptr, dG.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    P, Cm, G = dP.numpy(), dC.numpy(), dG.numpy()
    # pattern arrays untouched, bit for bit
    assert np.array_equal(dir_.numpy(), ir) and np.array_equal(djc.numpy(), jc)

    # --- every value of all three results against the fp64-accumulated oracle
    ref64, sa = oracle.dds_f64(A, B, k, ir, jc, nthreads=oracle.max_threads())
    close(P, ref64, sa, "DDS, all %d values" % nnz)
    # A, B ~ U(0,1): every term is positive, so the plain relative error is well defined
    assert float(np.max(np.abs(P - ref64) / ref64)) <= RTOL
    ref64, sa = oracle.fsmult_f64(A, k, vals, ir, jc, nthreads=oracle.max_threads())
    close(Cm, ref64, sa, "A*S, all %d values" % Cm.size)
    nzc = ref64 > 0                                  # columns of S are never empty here, but be exact
    assert float(np.max(np.abs(Cm[nzc] - ref64[nzc]) / ref64[nzc])) <= RTOL
    ref64, sa = oracle.fsmultT_f64(AT, k, nrows, vals, ir, jc, nthreads=oracle.max_threads())
    close(G, ref64, sa, "A*^S, all %d values" % G.size)
    del ref64, sa
    # the plan-taking forms (class-ordered DDS, A*S in passes over row classes) on the same data
    dP2, dC2 = DeviceArray(nnz, np.float32), DeviceArray(k * ncols, np.float32)
    hip_abi.check(hip.bidmat_dds_plan(plan, k, dA.ptr, dB.ptr, dir_.ptr, djc.ptr, None, 0, dP2.ptr, 0, None))
    hip_abi.check(hip.bidmat_dsmult_plan(plan, k, dA.ptr, dv.ptr, dir_.ptr, djc.ptr, dC2.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    assert np.array_equal(dP2.numpy(), P)            # DDS: bit-identical whichever kernel the plan selects
    C2 = dC2.numpy()
    assert float(np.max(np.abs(C2.astype(np.float64) - Cm) / np.abs(Cm))) <= 2e-5    # A*S: another fixed order of the same sums
    del C2
    dP2.free(), dC2.free()
    # A*^S at full size by the other ways to fetch a value: a gather per lane instead of scalar loads, and the values
    # stored in the plan (plan order, the dense rows' in the layout of the dense block): the same bits each time
    dG2 = DeviceArray(k * nrows, np.float32)
    assert hip.bidmat_get_option(b"scalar_values") == 1
    hip_abi.check(hip.bidmat_set_option(b"scalar_values", 0))
    try:
        hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, dAT.ptr, dv.ptr, dG2.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
    finally:
        hip_abi.check(hip.bidmat_set_option(b"scalar_values", 1))
    assert np.array_equal(dG2.numpy().view(np.uint32), G.view(np.uint32)), "A*^S: scalar loads and gathered values differ"
    hip_abi.check(hip.bidmat_plan_set_values(plan, dv.ptr, None))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, dAT.ptr, None, dG2.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    assert np.array_equal(dG2.numpy().view(np.uint32), G.view(np.uint32)), "A*^S: stored and passed values differ"
    dG2.free()
    rng = np.random.default_rng(0)
    # --- the three products agree: <A*S, B> == sum_j v_j * DDS_j ; <B*^S, A> checked with A_T's own DDS
    f1 = np.dot(Cm.astype(np.float64), B.astype(np.float64))
    f2 = np.dot(P.astype(np.float64), vals.astype(np.float64))
    assert abs(f1 - f2) <= 1e-6 * abs(f2)
    hip_abi.check(hip.bidmat_dds_csc(k, ncols, nnz, dA.ptr, dAT.ptr, dir_.ptr, djc.ptr, dP.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    f3 = np.dot(G.astype(np.float64), A.astype(np.float64))
    f4 = np.dot(dP.numpy().astype(np.float64), vals.astype(np.float64))
    scale = np.dot(np.abs(G).astype(np.float64), np.abs(A).astype(np.float64))
    assert abs(f3 - f4) <= 1e-6 * scale

    # --- sparse sums on the same pattern: sum of column sums == sum of row sums == sum of values
    dcs, drs = DeviceArray(ncols, np.float32), DeviceArray(nrows, np.float32)
    hip_abi.check(hip.bidmat_spsum_cols(ncols, nnz, dv.ptr, djc.ptr, dcs.ptr, 0, None))
    hip_abi.check(hip.bidmat_spsum_rows_plan(plan, dv.ptr, drs.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    total = vals.sum(dtype=np.float64)
    assert abs(dcs.numpy().sum(dtype=np.float64) - total) <= 1e-6 * total
    assert abs(drs.numpy().sum(dtype=np.float64) - total) <= 1e-6 * total
    ref64, sa = oracle.spsum_f64(nrows, vals, ir, jc, 2)
    close(drs.numpy(), ref64, sa, "row sums")
    hip_abi.check(hip.bidmat_plan_destroy(plan))


@pytest.mark.timeout(600)
def test_config4_wide_k_power_law_columns(hip):
    """configs[3]: k=1024, Pareto column lengths clipped to [1,50000] (split-column path),
    output 1024 x 1 000 000 (4.1 GB)."""
    cfg = gen.config("C4", 1.0)
    k, nrows, ncols = cfg["k"], cfg["nrows"], cfg["ncols"]
    ir, jc, vals, A = cfg["ir"], cfg["jc"], cfg["vals"], cfg["A"]
    nnz = int(ir.size)
    lens = np.diff(jc)
    assert lens.max() > 10000 and 25e6 < nnz < 60e6
    dA, dv = DeviceArray.from_numpy(A), DeviceArray.from_numpy(vals)
    dir_, djc = DeviceArray.from_numpy(ir), DeviceArray.from_numpy(jc)
    dC = DeviceArray(k * ncols, np.float32)
    hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, nnz, dA.ptr, dv.ptr, dir_.ptr, djc.ptr, dC.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    rng = np.random.default_rng(4)
    longest = np.argsort(lens)[-5:]
    cols = np.unique(np.concatenate([rng.integers(0, ncols, 100), longest, [0, ncols - 1]]))
    got = np.concatenate([dC_slice(dC, c, k) for c in cols])
    sv, sir, sjc, _ = sub_csc(ir, jc, vals, cols)
    ref64, sa = oracle.fsmult_f64(A, k, sv, sir, sjc, nthreads=8)
    close(got, ref64, sa, "C4 sampled + longest columns")
    # the form bench.py times: through a plan (the plan holds the table of the 3 391 extra segments of the long
    # columns; uniform rows get no class ordering), the whole 4.1 GB output bit for bit
    plan = make_plan(hip, nrows, ncols, nnz, dir_, djc, k)
    assert hip.bidmat_plan_overflow_segments(plan) > 1000
    dCp = DeviceArray(k * ncols, np.float32)
    hip_abi.check(hip.bidmat_dsmult_plan(plan, k, dA.ptr, dv.ptr, dir_.ptr, djc.ptr, dCp.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    step = 1 << 28
    for off in range(0, k * ncols, step):                 # 1 GiB at a time
        n = min(step, k * ncols - off)
        a, b = np.empty(n, np.float32), np.empty(n, np.float32)
        hip_abi.check(hip.bidmat_memcpy_d2h(a.ctypes.data, dC.ptr + 4 * off, 4 * n))
        hip_abi.check(hip.bidmat_memcpy_d2h(b.ctypes.data, dCp.ptr + 4 * off, 4 * n))
        assert np.array_equal(a, b), "bidmat_dsmult_plan differs from bidmat_dsmult_csc in floats %d.." % off
    dCp.free()
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    # linearity in the values: A*(2S) == 2*(A*S) exactly (scaling by 2 is exact in fp32)
    dv2 = DeviceArray.from_numpy(vals * np.float32(2))
    dC2 = DeviceArray(k * 4096, np.float32)
    hip_abi.check(hip.bidmat_dsmult_csc(k, 4096, int(jc[4096]), dA.ptr, dv2.ptr, dir_.ptr, djc.ptr, dC2.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    assert np.array_equal(dC2.numpy(), 2 * dC.numpy(k * 4096))


def dC_slice(d, c, k):
    out = np.empty(k, dtype=np.float32)
    hip_abi.check(d.lib.bidmat_memcpy_d2h(out.ctypes.data, d.ptr + 4 * k * int(c), 4 * k))
    return out


@pytest.mark.timeout(900)
def test_config5_nmf_step(hip):
    """configs[4]: R = DDS(W,H,V); Q = V./R on the nonzeros; G = H *^ Q; rs = sum(H,2), k=128,
    V 1M x 1M with ~400M nonzeros."""
    cfg = gen.config("C5", 1.0)
    k, nrows, ncols = cfg["k"], cfg["nrows"], cfg["ncols"]
    ir, jc, vals, W, H = cfg["ir"], cfg["jc"], cfg["vals"], cfg["W"], cfg["H"]
    nnz = int(ir.size)
    assert 3.5e8 < nnz < 4.5e8
    dW, dH, dv = DeviceArray.from_numpy(W), DeviceArray.from_numpy(H), DeviceArray.from_numpy(vals)
    dir_, djc = DeviceArray.from_numpy(ir), DeviceArray.from_numpy(jc)
    dR, dG, drs = DeviceArray(nnz, np.float32), DeviceArray(k * nrows, np.float32), DeviceArray(k, np.float32)
    plan = make_plan(hip, nrows, ncols, nnz, dir_, djc, k)
    hip_abi.check(hip.bidmat_dds_csc(k, ncols, nnz, dW.ptr, dH.ptr, dir_.ptr, djc.ptr, dR.ptr, 0, None))
    hip_abi.check(hip.bidmat_applyop_flat(dv.ptr, dR.ptr, dR.ptr, nnz, 3, None))          # Q = V ./ R in place
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, dH.ptr, dR.ptr, dG.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    hip_abi.check(hip.bidmat_reduce2op(k, ncols, dH.ptr, drs.ptr, 0.0, 0))
    Q, G = dR.numpy(), dG.numpy()
    rng = np.random.default_rng(5)
    # sampled columns: Q against the oracle (DDS then an IEEE division)
    cols = np.unique(rng.integers(0, ncols, 200))
    sv, sir, sjc, idx = sub_csc(ir, jc, vals, cols)
    r32, _, _ = oracle.dds(W, H.reshape(ncols, k)[cols].ravel(), k, sir, sjc, nthreads=8)
    r64, sa = oracle.dds_f64(W, H.reshape(ncols, k)[cols].ravel(), k, sir, sjc, nthreads=8)
    np.testing.assert_allclose(Q[idx], sv.astype(np.float64) / r64, rtol=2e-4)
    np.testing.assert_allclose(Q[idx], sv / r32, rtol=2e-5)
    # sampled rows: G against the oracle fed with the device's own Q
    rows = np.unique(np.concatenate([rng.integers(0, nrows, 100), [0, 1, nrows - 1]]))
    rv, rir, rjc = rows_sub_csc(ir, jc, Q, rows)
    ref64, sa = oracle.fsmultT_f64(H, k, rows.size, rv, rir, rjc, nthreads=8)
    close(G.reshape(nrows, k)[rows].ravel(), ref64, sa, "NMF G sampled rows")
    # dense row sums of H
    ref = H.reshape(ncols, k).astype(np.float64).sum(axis=0)
    np.testing.assert_allclose(drs.numpy(), ref, rtol=1e-5)
    # the forms bench.py times: V stored in the plan once, Q = V ./ DDS in ONE launch of the class-ordered kernel
    # (hot rows of every class in LDS, persistent workgroups), G = H *^ Q fed by it: the same bits as the chain above
    hip_abi.check(hip.bidmat_plan_set_values(plan, dv.ptr, None))
    dQ2, dG2 = DeviceArray(nnz, np.float32), DeviceArray(k * nrows, np.float32)
    hip_abi.check(hip.bidmat_dds_plan_stored(plan, k, dW.ptr, dH.ptr, dir_.ptr, djc.ptr, 3, dQ2.ptr, None))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, dH.ptr, dQ2.ptr, dG2.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    assert np.array_equal(dQ2.numpy(), Q), "bidmat_dds_plan_stored(op_div) differs from DDS + V./R"
    assert np.array_equal(dG2.numpy(), G)
    # ... and with the caller's V instead of the stored copy (the fused step reads V through the class order)
    hip_abi.check(hip.bidmat_dds_plan(plan, k, dW.ptr, dH.ptr, dir_.ptr, djc.ptr, dv.ptr, 3, dQ2.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    assert np.array_equal(dQ2.numpy(), Q)
    # ... and the whole chain in one walk over the plan's rows (what bench.py times for this configuration), with the
    # stored V and with the caller's, with and without the products written: the same bits again
    # (the one walk adds every row's terms in the plan's order; bidmat_dsmultT_plan does so too once the plan's dense
    # block, which reorders the sums of the most frequent rows, is switched off: that is the G the bits are held against,
    # the G with the dense block having been checked against the oracle above, rows 0 and 1 among the sampled ones)
    dense_rows = int(hip.bidmat_plan_info(plan, b"dense_rows"))
    assert dense_rows >= 32, "this pattern's most frequent rows are in most columns"
    hip_abi.check(hip.bidmat_set_option(b"dense_rows", 0))
    try:
        hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, dH.ptr, dR.ptr, dG2.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
    finally:
        hip_abi.check(hip.bidmat_set_option(b"dense_rows", 128))
    G_plain = dG2.numpy()
    drow = np.empty(dense_rows, np.int32)
    ptr, cnt = C.c_void_p(), C.c_longlong()
    hip_abi.check(hip.bidmat_plan_array(plan, b"drow", C.byref(ptr), C.byref(cnt)))
    hip_abi.check(hip.bidmat_memcpy_d2h(drow.ctypes.data, ptr, 4 * dense_rows))
    others = np.ones(nrows, bool); others[drow] = False
    assert np.array_equal(G_plain.reshape(nrows, k)[others], G.reshape(nrows, k)[others]), "rows outside the dense block changed"
    np.testing.assert_allclose(G.reshape(nrows, k)[drow], G_plain.reshape(nrows, k)[drow], rtol=1e-5)
    G = G_plain
    for vptr, qptr in ((None, dQ2.ptr), (dv.ptr, None)):
        hip_abi.check(hip.bidmat_memset(dQ2.ptr, 0, dQ2.nbytes))
        hip_abi.check(hip.bidmat_memset(dG2.ptr, 0, dG2.nbytes))
        hip_abi.check(hip.bidmat_dds_dsmultT_plan(plan, k, dW.ptr, dH.ptr, vptr, 3, qptr, dG2.ptr, 0, None), "fused chain")
        hip_abi.check(hip.bidmat_synchronize())
        assert np.array_equal(dG2.numpy(), G), "bidmat_dds_dsmultT_plan differs from the two calls"
        if qptr:
            assert np.array_equal(dQ2.numpy(), Q)
    dQ2.free(), dG2.free()
    hip_abi.check(hip.bidmat_plan_destroy(plan))


@pytest.mark.timeout(300)
def test_large_pattern_with_one_bad_row_index_is_refused(hip):
    """From 16 M nonzeros on the plan build counts rows on a sample of the nonzeros (the counts only
    steer performance choices), but every row index is still checked: one index outside the matrix,
    placed where the sampled histogram does not look (chunk 1 of 256 nonzeros: the top three bits of
    1 * 0x9E3779B1 are not zero), must make bidmat_plan_create fail, and the sound pattern must build."""
    nrows, ncols = 50000, 100000
    ir, jc = gen.pattern(nrows, ncols, ("const", 200), ("zipf", 1.1), 77)
    nnz = int(ir.size)
    assert nnz >= (16 << 20)
    assert ((1 * 0x9E3779B1) & 0xFFFFFFFF) >> 29 != 0
    djc = DeviceArray.from_numpy(jc)
    for bad in (nrows, -1):
        broken = ir.copy()
        broken[300] = bad
        dbad = DeviceArray.from_numpy(broken)
        plan = C.c_void_p()
        rc = hip.bidmat_plan_create(nrows, ncols, nnz, dbad.ptr, djc.ptr, 256, C.byref(plan))
        assert rc == 1 and not plan.value, "bad row index %d accepted (rc %d)" % (bad, rc)
        dbad.free()
    dir_ = DeviceArray.from_numpy(ir)
    plan = make_plan(hip, nrows, ncols, nnz, dir_, djc, 256)
    # the sampled counts still find the heavy rows: row sums through the plan equal the oracle's
    vals = gen.uniform_open0(nnz, 5)
    dv, dout = DeviceArray.from_numpy(vals), DeviceArray(nrows, np.float32)
    hip_abi.check(hip.bidmat_spsum_rows_plan(plan, dv.ptr, dout.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    ref = np.bincount(ir, weights=vals.astype(np.float64), minlength=nrows)
    assert np.allclose(dout.numpy(), ref, rtol=RTOL, atol=0)
    hip_abi.check(hip.bidmat_plan_destroy(plan))


@pytest.mark.timeout(300)
def test_very_long_columns_keep_their_accuracy_through_the_plan(hip):
    """Pareto column lengths up to 60 000 nonzeros on Zipf rows, all terms positive: A*S through the plan must stay as
    close to the fp64 result as the plain entry (columns this long are never added up in one running sum), DDS through
    the plan must equal the plain entry bit for bit, and A*^S must meet the same bound."""
    k, nrows, ncols = 512, 300000, 60000
    ir, jc = gen.pattern(nrows, ncols, ("pareto", 20.0, 1.1, 1, 60000), ("zipf", 1.2), 107)
    nnz = int(ir.size)
    assert int(np.diff(jc).max()) > 30000
    A, B, vals = gen.uniform(k * nrows, 8), gen.uniform(k * ncols, 9), gen.uniform_open0(nnz, 10)
    dA, dB, dv = DeviceArray.from_numpy(A), DeviceArray.from_numpy(B), DeviceArray.from_numpy(vals)
    dir_, djc = DeviceArray.from_numpy(ir), DeviceArray.from_numpy(jc)
    old = hip.bidmat_get_option(b"col_classes")
    hip_abi.check(hip.bidmat_set_option(b"col_classes", 1))          # force the class ordering onto the plan
    try:
        plan = make_plan(hip, nrows, ncols, nnz, dir_, djc, k)
    finally:
        hip_abi.check(hip.bidmat_set_option(b"col_classes", old))
    C1, C2 = DeviceArray(k * ncols, np.float32), DeviceArray(k * ncols, np.float32)
    hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, nnz, dA.ptr, dv.ptr, dir_.ptr, djc.ptr, C1.ptr, 0, None))
    hip_abi.check(hip.bidmat_dsmult_plan(plan, k, dA.ptr, dv.ptr, dir_.ptr, djc.ptr, C2.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    ref64, _ = oracle.fsmult_f64(A, k, vals, ir, jc, nthreads=oracle.max_threads())
    nz = ref64 > 0
    e_plain = float(np.max(np.abs(C1.numpy()[nz] - ref64[nz]) / ref64[nz]))
    e_plan = float(np.max(np.abs(C2.numpy()[nz] - ref64[nz]) / ref64[nz]))
    assert e_plain <= 5e-6 and e_plan <= 5e-6, (e_plain, e_plan)
    C1.free(); C2.free()
    P1, P2 = DeviceArray(nnz, np.float32), DeviceArray(nnz, np.float32)
    hip_abi.check(hip.bidmat_dds_csc(k, ncols, nnz, dA.ptr, dB.ptr, dir_.ptr, djc.ptr, P1.ptr, 0, None))
    hip_abi.check(hip.bidmat_dds_plan(plan, k, dA.ptr, dB.ptr, dir_.ptr, djc.ptr, None, 0, P2.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    assert np.array_equal(P1.numpy(), P2.numpy())
    G = DeviceArray(k * nrows, np.float32)
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, dB.ptr, dv.ptr, G.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    ref64, _ = oracle.fsmultT_f64(B, k, nrows, vals, ir, jc, nthreads=oracle.max_threads())
    nz = ref64 > 0
    assert float(np.max(np.abs(G.numpy()[nz] - ref64[nz]) / ref64[nz])) <= 5e-6
    hip_abi.check(hip.bidmat_plan_destroy(plan))


@pytest.mark.timeout(900)
def test_three_fresh_100M_patterns_through_the_reference_shaped_dsmultT(hip):
    """What BIDMach does with every minibatch: a pattern the library has not seen, handed to the reference-shaped
    A*^S (no plan handle, per-nonzero column array). Three different ~100 M-nonzero patterns one after the other
    through a fingerprint cache of two entries (so the third evicts the first, 0.8 GB of plan each), then the first
    again (rebuilt): sampled rows of every result against the oracle, the repeat bit-equal to the first run; the
    reference-shaped row sums and DDS on the way."""
    k, nrows, ncols = 256, 100000, 500000
    rng = np.random.default_rng(6)
    AT = gen.normal(k * ncols, 31)
    dAT = DeviceArray.from_numpy(AT)
    old = hip.bidmat_get_option(b"cache_plans")
    hip_abi.check(hip.bidmat_release_caches())
    hip_abi.check(hip.bidmat_set_option(b"cache_plans", 2))
    try:
        first = None
        for seed in (2, 202, 302, 2):
            ir, jc = gen.pattern(nrows, ncols, ("poisson", 200), ("zipf", 1.1), seed)
            nnz = int(ir.size)
            assert 0.9e8 < nnz < 1.1e8
            vals = gen.uniform_open0(nnz, seed + 30)
            dir_, djc, dv = DeviceArray.from_numpy(ir), DeviceArray.from_numpy(jc), DeviceArray.from_numpy(vals)
            dic = DeviceArray(nnz, np.int32)
            hip_abi.check(hip.bidmat_csc_expand_cols(ncols, nnz, djc.ptr, dic.ptr, None))
            dG, drs = DeviceArray.zeros(k * nrows), DeviceArray.zeros(nrows)
            hip_abi.check(hip.bidmat_dsmultT(k, ncols, nnz, dAT.ptr, dv.ptr, dir_.ptr, dic.ptr, dG.ptr), "dsmultT seed %d" % seed)
            hip_abi.check(hip.bidmat_spsum(nrows, ncols, nnz, dir_.ptr, dic.ptr, dv.ptr, drs.ptr, 2), "spsum seed %d" % seed)
            G = dG.numpy()
            rows = np.unique(np.concatenate([rng.integers(0, nrows, 200), [0, 1, 2, int(ir.max())]]))
            rv, rir, rjc = rows_sub_csc(ir, jc, vals, rows)
            ref64, sa = oracle.fsmultT_f64(AT, k, rows.size, rv, rir, rjc, nthreads=oracle.max_threads())
            close(G.reshape(nrows, k)[rows].ravel(), ref64, sa, "bidmat_dsmultT on a fresh pattern (seed %d), sampled rows" % seed)
            ref = np.bincount(ir, weights=vals.astype(np.float64), minlength=nrows)
            assert np.allclose(drs.numpy(), ref, rtol=RTOL, atol=0)
            if seed == 2 and first is None:
                first = G
            elif seed == 2:
                assert np.array_equal(first, G)          # the evicted plan, rebuilt: a function of the pattern only
            for d in (dir_, djc, dv, dic, dG, drs):
                d.free()
    finally:
        hip_abi.check(hip.bidmat_set_option(b"cache_plans", old))
        hip_abi.check(hip.bidmat_release_caches())
