"""Pins the CPU oracle (oracle/bidmat_oracle.c) without a GPU.

The reference holds no golden files for this path, so the oracle is pinned by
  - the committed fixtures of tests/golden (scipy/numpy float64, made without the oracle),
  - the relations the reference's own tests assert (A*S == A*full(S): SMatTest.scala:42-53,
    GSMatTest.scala:64-71; A*^S == A*full(S)^T: SMatTest.scala:55-61; sums by explicit loops:
    GSMatTest.scala:283-316) at the reference's sizes and its 1e-4 absolute eps,
  - what the mathematics fixes: one-hot gather (bit-exact), identity, single-nonzero columns,
    transpose identity, dense-pattern DDS == A^T B, the Frobenius identity across the three
    products, bincount for the sums, brute-force loops on tiny inputs.
Each check is chosen so that a dropped term, a swapped operand or a wrong index base fails it.
"""
import os

import numpy as np
import pytest

import oracle
from util import dense_full, expand_cols, random_csc

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "sparse_dense_golden.npz"))
CASES = sorted({k.split("__")[0] for k in GOLD.files})


def gold(case):
    return {k.split("__")[1]: GOLD[k] for k in GOLD.files if k.startswith(case + "__")}


def close(x, ref64, sa):
    ok, worst = oracle.within_tolerance(x, ref64, sa, 1e-4)
    assert ok, worst


# ------------------------------------------------------------------ golden fixtures
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("ioff", [0, 1])
def test_fixture_products(case, ioff):
    g = gold(case)
    k, nrows, ncols = int(g["k"]), int(g["nrows"]), int(g["ncols"])
    ir, jc = g["ir"] + ioff, g["jc"] + ioff       # the reference's host matrices are 1-based by default
    # A * S
    ref64, sa = oracle.fsmult_f64(g["A"], k, g["data"], ir, jc, ioff)
    np.testing.assert_allclose(ref64, g["AS"], rtol=1e-12, atol=1e-12)
    close(oracle.fsmult(g["A"], k, g["data"], ir, jc, ioff), g["AS"], sa)
    # B *^ S
    ref64, sa = oracle.fsmultT_f64(g["B"], k, nrows, g["data"], ir, jc, ioff)
    np.testing.assert_allclose(ref64, g["BSt"], rtol=1e-12, atol=1e-12)
    close(oracle.fsmultT(g["B"], k, nrows, g["data"], ir, jc, ioff), g["BSt"], sa)
    # DDS
    ref64, sa = oracle.dds_f64(g["A"], g["B"], k, ir, jc, ioff)
    np.testing.assert_allclose(ref64, g["P"], rtol=1e-12, atol=1e-12)
    vals, oir, ojc = oracle.dds(g["A"], g["B"], k, ir, jc, ioff)
    close(vals, g["P"], sa)
    assert np.array_equal(oir, ir) and np.array_equal(ojc, jc)      # pattern copied bit for bit


@pytest.mark.parametrize("case", CASES)
def test_fixture_sums(case):
    g = gold(case)
    k, nrows, ncols = int(g["k"]), int(g["nrows"]), int(g["ncols"])
    for dim, want in ((1, g["colsum"]), (2, g["rowsum"])):
        ref64, sa = oracle.spsum_f64(nrows, g["data"], g["ir"], g["jc"], dim)
        np.testing.assert_allclose(ref64, want, rtol=1e-12, atol=1e-12)
        close(oracle.spsum(nrows, g["data"], g["ir"], g["jc"], dim), want, sa)
    sa1 = np.abs(g["A"].reshape(nrows, k)).sum(axis=1)
    close(oracle.dsum(g["A"], k, nrows, 1), g["dsum1"], sa1)
    close(oracle.dsum(g["A"], k, nrows, 2), g["dsum2"], np.abs(g["A"].reshape(nrows, k)).sum(axis=0))
    np.testing.assert_allclose(oracle.dsum_f64(g["A"], k, nrows, 1), g["dsum1"], rtol=1e-12)
    np.testing.assert_allclose(oracle.dsum_f64(g["A"], k, nrows, 2), g["dsum2"], rtol=1e-12)


# ------------------------------------------------------------------ the reference's own relations
def test_reference_relation_dense_product():
    rng = np.random.default_rng(1)
    nr, nc, nk = 10, 20, 30
    data, ir, jc = random_csc(rng, nk, nc, 0.2)
    A = rng.random(nr * nk).astype(np.float32)
    got = oracle.fsmult(A, nr, data, ir, jc).reshape(nc, nr).T
    want = A.reshape(nk, nr).T.astype(np.float64) @ dense_full(nk, nc, data, ir, jc)
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-4)
    data, ir, jc = random_csc(rng, nc, nk, 0.2)       # b = sprand(nc, nk): a *^ b
    got = oracle.fsmultT(A, nr, nc, data, ir, jc).reshape(nc, nr).T
    want = A.reshape(nk, nr).T.astype(np.float64) @ dense_full(nc, nk, data, ir, jc).T
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-4)


# ------------------------------------------------------------------ what the mathematics fixes
def test_onehot_identity_and_single_nonzero_are_bit_exact():
    rng = np.random.default_rng(2)
    k, nrows, ncols = 7, 11, 13
    A = rng.standard_normal(k * nrows).astype(np.float32)
    ir = rng.integers(0, nrows, size=ncols).astype(np.int32)
    jc = np.arange(ncols + 1, dtype=np.int32)
    ones = np.ones(ncols, dtype=np.float32)
    assert np.array_equal(oracle.fsmult(A, k, ones, ir, jc).reshape(ncols, k), A.reshape(nrows, k)[ir])
    # identity
    eye_ir = np.arange(nrows, dtype=np.int32)
    eye_jc = np.arange(nrows + 1, dtype=np.int32)
    assert np.array_equal(oracle.fsmult(A, k, np.ones(nrows, np.float32), eye_ir, eye_jc), A)
    assert np.array_equal(oracle.fsmultT(A, k, nrows, np.ones(nrows, np.float32), eye_ir, eye_jc), A)
    # one nonzero per column: a scaled copy, exactly fl(A*v)
    v = (1.0 - rng.random(ncols)).astype(np.float32)
    assert np.array_equal(oracle.fsmult(A, k, v, ir, jc).reshape(ncols, k), A.reshape(nrows, k)[ir] * v[:, None])
    # one-hot S^T: a segmented column sum
    B = rng.standard_normal(k * ncols).astype(np.float32)
    want = np.zeros((nrows, k), dtype=np.float64)
    np.add.at(want, ir, B.reshape(ncols, k).astype(np.float64))
    np.testing.assert_allclose(oracle.fsmultT(B, k, nrows, ones, ir, jc).reshape(nrows, k), want, rtol=1e-5, atol=1e-6)


def test_transpose_identity():
    """dsmultT(A, S) == dsmult(A, S^T) with S^T built independently (scipy)."""
    import scipy.sparse as sp
    rng = np.random.default_rng(3)
    k, nrows, ncols = 5, 23, 31
    data, ir, jc = random_csc(rng, nrows, ncols, 0.15)
    A = rng.standard_normal(k * ncols).astype(np.float32)
    St = sp.csc_matrix((data, ir, jc), shape=(nrows, ncols)).T.tocsc()
    St.sort_indices()
    a = oracle.fsmultT(A, k, nrows, data, ir, jc)
    b = oracle.fsmult(A, k, St.data, St.indices.astype(np.int32), St.indptr.astype(np.int32))
    # same terms per output, both added in ascending column order of S: identical bits
    assert np.array_equal(a, b)


def test_brute_force_tiny():
    rng = np.random.default_rng(4)
    k, nrows, ncols = 3, 4, 5
    data, ir, jc = random_csc(rng, nrows, ncols, 0.5)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    B = rng.standard_normal(k * ncols).astype(np.float32)
    AS = np.zeros((k, ncols), np.float32)
    BSt = np.zeros((k, nrows), np.float32)
    P = np.zeros(ir.size, np.float32)
    for c in range(ncols):
        for j in range(jc[c], jc[c + 1]):
            dot = np.float32(0)
            for i in range(k):
                AS[i, c] = np.float32(AS[i, c] + np.float32(A[i + k * ir[j]] * data[j]))
                BSt[i, ir[j]] = np.float32(BSt[i, ir[j]] + np.float32(B[i + k * c] * data[j]))
                dot = np.float32(dot + np.float32(A[i + k * ir[j]] * B[i + k * c]))
            P[j] = dot
    assert np.array_equal(oracle.fsmult(A, k, data, ir, jc).reshape(ncols, k).T, AS)
    assert np.array_equal(oracle.fsmultT(B, k, nrows, data, ir, jc).reshape(nrows, k).T, BSt)
    assert np.array_equal(oracle.dds(A, B, k, ir, jc)[0], P)


def test_dds_dense_pattern_is_At_B_and_frobenius_identity():
    rng = np.random.default_rng(5)
    k, nrows, ncols = 30, 10, 20
    A = rng.random(k * nrows).astype(np.float32)
    B = rng.random(k * ncols).astype(np.float32)
    jc = (np.arange(ncols + 1) * nrows).astype(np.int32)
    ir = np.tile(np.arange(nrows, dtype=np.int32), ncols)
    P = oracle.dds(A, B, k, ir, jc)[0].reshape(ncols, nrows).T
    want = A.reshape(nrows, k).astype(np.float64) @ B.reshape(ncols, k).astype(np.float64).T
    np.testing.assert_allclose(P, want, rtol=0, atol=1e-4)
    # <A*S, B>_F == sum_j v_j DDS_j == <B*^S, A>_F  (fp64 arbiters: equal to rounding)
    data, ir, jc = random_csc(rng, nrows, ncols, 0.3)
    f1 = np.dot(oracle.fsmult_f64(A, k, data, ir, jc)[0], B.astype(np.float64))
    f2 = np.dot(oracle.dds_f64(A, B, k, ir, jc)[0], data.astype(np.float64))
    f3 = np.dot(oracle.fsmultT_f64(B, k, nrows, data, ir, jc)[0], A.astype(np.float64))
    assert abs(f1 - f2) < 1e-10 * abs(f2) and abs(f3 - f2) < 1e-10 * abs(f2)


def test_sparse_sums_against_bincount_and_axis_rule():
    rng = np.random.default_rng(6)
    nrows, ncols = 10, 20
    data, ir, jc = random_csc(rng, nrows, ncols, 0.2)
    ic = expand_cols(jc)
    cs = np.bincount(ic, weights=data.astype(np.float64), minlength=ncols)
    rs = np.bincount(ir, weights=data.astype(np.float64), minlength=nrows)
    np.testing.assert_allclose(oracle.spsum(nrows, data, ir, jc, 1), cs, rtol=1e-6)
    np.testing.assert_allclose(oracle.spsum(nrows, data, ir, jc, 2), rs, rtol=1e-6)
    assert abs(cs.sum() - rs.sum()) < 1e-9
    # n == 0: columns, unless the matrix is a single row / column (then one total)
    np.testing.assert_allclose(oracle.spsum(nrows, data, ir, jc, 0), cs, rtol=1e-6)
    d1, i1, j1 = random_csc(rng, 1, 9, 0.7)
    tot = oracle.spsum(1, d1, i1, j1, 0)
    assert tot.size == 1 and abs(tot[0] - d1.sum(dtype=np.float64)) < 1e-5
    with pytest.raises(RuntimeError):
        oracle.spsum(nrows, data, ir, jc, 3)
    # column sums of a one-hot pattern are exactly 1
    oh_ir = rng.integers(0, nrows, size=ncols).astype(np.int32)
    assert np.array_equal(oracle.spsum(nrows, np.ones(ncols, np.float32), oh_ir, np.arange(ncols + 1, dtype=np.int32), 1),
                          np.ones(ncols, np.float32))


def test_index_base_and_thread_count_do_not_change_bits():
    rng = np.random.default_rng(7)
    k, nrows, ncols = 96, 50, 2000       # k*nnz > 100000 so the threaded branches are taken
    data, ir, jc = random_csc(rng, nrows, ncols, 0.1)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    B = rng.standard_normal(k * ncols).astype(np.float32)
    base = oracle.fsmult(A, k, data, ir, jc, 0, nthreads=1)
    assert np.array_equal(base, oracle.fsmult(A, k, data, ir + 1, jc + 1, 1, nthreads=8))
    assert np.array_equal(base, oracle.fsmult(A, k, data, ir + 1, jc + 1, native=True, nthreads=4))   # smcscm: base from jc[0]
    baseT = oracle.fsmultT(B, k, nrows, data, ir, jc, 0, nthreads=1)
    assert np.array_equal(baseT, oracle.fsmultT(B, k, nrows, data, ir + 1, jc + 1, 1, nthreads=8))
    assert np.array_equal(baseT, oracle.fsmultT(B, k, nrows, data, ir + 1, jc + 1, native=True))
    based = oracle.dds(A, B, k, ir, jc, 0, nthreads=1)[0]
    assert np.array_equal(based, oracle.dds(A, B, k, ir + 1, jc + 1, 1, nthreads=8)[0])


def test_madd_accumulates_into_existing_output():
    rng = np.random.default_rng(8)
    k, nrows, ncols = 4, 6, 5
    data, ir, jc = random_csc(rng, nrows, ncols, 0.4)
    A = rng.random(k * nrows).astype(np.float32)
    C0 = rng.random(k * ncols).astype(np.float32)
    once = oracle.fsmult(A, k, data, ir, jc)
    acc = oracle.fsmult(A, k, data, ir, jc, out=C0.copy())
    np.testing.assert_allclose(acc, C0 + once, rtol=1e-6)


# ------------------------------------------------------------------ structure helpers
def test_check_every_rule():
    ir = np.array([0, 2, 1, 3], dtype=np.int32)
    jc = np.array([0, 2, 2, 4], dtype=np.int32)
    assert oracle.check(4, 3, 4, ir, jc)[0] == 0
    assert oracle.check(4, 3, 4, ir + 1, jc + 1, ioff=1)[0] == 0
    assert oracle.check(4, 3, 4, ir, jc + 1)[0] == 1                                       # jc(0) != ioff
    assert oracle.check(4, 3, 4, np.arange(4, dtype=np.int32), np.array([0, 3, 2, 4], np.int32))[0] == 2   # jc out of order
    assert oracle.check(4, 3, 4, np.array([2, 0, 1, 3], np.int32), jc)[0] == 3             # rows not increasing
    assert oracle.check(4, 3, 4, np.array([0, 0, 1, 3], np.int32), jc)[0] == 3             # duplicate row
    assert oracle.check(4, 3, 4, np.array([-1, 2, 1, 3], np.int32), jc)[0] == 4            # too small
    assert oracle.check(3, 3, 4, ir, jc)[0] == 5                                           # out of range
    assert oracle.check(4, 3, 5, ir, jc)[0] == 6                                           # jc(ncols) != nnz
    assert oracle.check(4, 3, 4, None, jc)[0] == 0                                         # ir == null branch


def test_compress_and_uncompress_inds():
    rng = np.random.default_rng(9)
    ncols = 50
    lengths = rng.integers(0, 5, size=ncols)
    lengths[:3] = 0
    lengths[-2:] = 0
    jc = np.zeros(ncols + 1, dtype=np.int32)
    jc[1:] = np.cumsum(lengths)
    ic = np.repeat(np.arange(ncols), lengths).astype(np.int32)
    assert np.array_equal(oracle.uncompress_inds(jc), ic)
    assert np.array_equal(oracle.compress_inds(ic, ncols), jc)
    assert np.array_equal(oracle.compress_inds(ic, ncols), np.searchsorted(ic, np.arange(ncols + 1), side="left"))
    assert np.array_equal(oracle.compress_inds(ic, ncols, ioff=1), jc + 1)
    assert np.array_equal(oracle.uncompress_inds(jc + 1, ioff=1), ic)


def test_applyop_matches_numpy():
    rng = np.random.default_rng(10)
    a = rng.random(100).astype(np.float32) + 0.1
    b = rng.random(100).astype(np.float32) + 0.1
    b[::5] = a[::5]
    want = {0: a + b, 1: a - b, 2: a * b, 3: a / b, 4: a > b, 5: a < b, 6: a == b, 7: a >= b, 8: a <= b,
            9: a != b, 10: np.maximum(a, b), 11: np.minimum(a, b), 14: np.where(a > 0, b, 0)}
    for opn, w in want.items():
        assert np.array_equal(oracle.applyop(a, b, opn), w.astype(np.float32)), opn
    np.testing.assert_allclose(oracle.applyop(a, b, 12), np.arctan2(a, b), rtol=1e-6)
    np.testing.assert_allclose(oracle.applyop(a, b, 13), np.power(a, b), rtol=1e-6)
    with pytest.raises(RuntimeError):
        oracle.applyop(a, b, 15)


def _lanes_reduce(x, op):
    """The reference's reduce kernels, lane by lane (Operators.cu:650-671): lane t of L = min(n, 32) folds
    x[t], x[t+32], ... from the left; then for i = 1, 2, 4, ... every lane t with t + i < L takes
    op(own, value of lane t+i before the step)."""
    n = len(x)
    L = min(n, 32)
    v = []
    for t in range(L):
        acc = x[t]
        for e in range(t + 32, n, 32):
            acc = op(acc, x[e])
        v.append(acc)
    i = 1
    while i < L:
        v = [op(v[t], v[t + i]) if t + i < L else v[t] for t in range(L)]
        i *= 2
    return v[0]


def test_reduce_tree_against_a_lane_by_lane_simulation_and_closed_forms():
    """oracle.reduce_tree (every op, both directions) against a literal simulation of the reference's lanes; for the
    associative ops against numpy; for sub against its closed form: lane t's partial is x[t] - x[t+32] - ..., and
    the tree gives lane t the sign (-1)^popcount(t) (checked in exact integer arithmetic)."""
    rng = np.random.default_rng(91)
    f32 = np.float32
    ops = {0: lambda a, b: f32(a + b), 1: lambda a, b: f32(a - b), 2: lambda a, b: f32(a * b), 3: lambda a, b: f32(a / b),
           4: lambda a, b: f32(a > b), 5: lambda a, b: f32(a < b), 6: lambda a, b: f32(a == b), 7: lambda a, b: f32(a >= b),
           8: lambda a, b: f32(a <= b), 9: lambda a, b: f32(a != b), 10: lambda a, b: max(a, b), 11: lambda a, b: min(a, b),
           14: lambda a, b: b if a > 0 else f32(0)}
    for nrows, ncols in ((1, 1), (3, 5), (31, 4), (32, 3), (33, 3), (70, 2), (5, 100), (2, 64), (129, 1)):
        A = rng.integers(-4, 5, size=nrows * ncols).astype(np.float32)
        A[A == 0] = 1                                     # no division by zero
        M = A.reshape(ncols, nrows).T                     # M[r, c]
        for opn, op in ops.items():
            got1, got2 = oracle.reduce_tree(A, nrows, ncols, opn, 1), oracle.reduce_tree(A, nrows, ncols, opn, 2)
            want1 = np.array([_lanes_reduce(list(M[:, c]), op) for c in range(ncols)], dtype=np.float32)
            want2 = np.array([_lanes_reduce(list(M[r, :]), op) for r in range(nrows)], dtype=np.float32)
            assert np.array_equal(got1, want1), (nrows, ncols, opn)
            assert np.array_equal(got2, want2), (nrows, ncols, opn)
        # small integers: sums, maxima and minima are exact whatever the order
        assert np.array_equal(oracle.reduce_tree(A, nrows, ncols, 0, 1), M.sum(axis=0))
        assert np.array_equal(oracle.reduce_tree(A, nrows, ncols, 10, 2), M.max(axis=1))
        assert np.array_equal(oracle.reduce_tree(A, nrows, ncols, 11, 1), M.min(axis=0))
        # sub, closed form
        L = min(nrows, 32)
        part = np.array([[M[t, c] - M[t + 32::32, c].sum() for t in range(L)] for c in range(ncols)])
        sign = np.array([(-1) ** bin(t).count("1") for t in range(L)])
        assert np.array_equal(oracle.reduce_tree(A, nrows, ncols, 1, 1), (part * sign).sum(axis=1).astype(np.float32))
    # n == 0: the initial value
    assert np.array_equal(oracle.reduce_tree(np.zeros(0, np.float32), 0, 3, 1, 1, initv=7.0), np.full(3, 7.0, np.float32))
    with pytest.raises(RuntimeError):
        oracle.reduce_tree(np.ones(4, np.float32), 2, 2, 15, 1)


def test_tolerance_rule():
    ref = np.array([1.0, 0.0, 1e-9])
    sa = np.array([1.0, 10.0, 10.0])
    assert oracle.within_tolerance(ref + np.array([5e-5, 5e-4, 5e-4]), ref, sa)[0]      # cancellation-safe
    assert not oracle.within_tolerance(ref + np.array([5e-4, 0, 0]), ref, sa)[0]
    assert not oracle.within_tolerance(np.array([np.nan, 0, 0]), ref, sa)[0]


def test_tile_products_against_dense_windows():
    """tileMult / tileMultNT (FMat.scala:1200-1303): windows of A, S and C."""
    rng = np.random.default_rng(11)
    anr, anc, snr, snc, cnr, cnc = 12, 40, 35, 30, 15, 33
    A = rng.standard_normal(anr * anc).astype(np.float32)
    data, ir, jc = random_csc(rng, snr, snc, 0.3)
    S = dense_full(snr, snc, data, ir, jc)
    A2 = A.reshape(anc, anr).T.astype(np.float64)
    for ioff in (0, 1):
        # C[croff:+nr, ccoff:+nc] += A[aroff:+nr, acoff:+kk] * S[broff:+kk, bcoff:+nc]
        nr, nc, kk, aroff, acoff, broff, bcoff, croff, ccoff = 7, 9, 11, 3, 5, 6, 4, 2, 8
        C0 = rng.standard_normal(cnr * cnc).astype(np.float32)
        Cm = C0.copy()
        ref, sa = oracle.fsmult_tile(A, anr, aroff, acoff, nr, nc, kk, data, ir + ioff, jc + ioff, broff, bcoff,
                                     Cm, cnr, croff, ccoff, ioff=ioff)
        want = A2[aroff:aroff + nr, acoff:acoff + kk] @ S[broff:broff + kk, bcoff:bcoff + nc]
        np.testing.assert_allclose(ref.reshape(nc, nr).T, want, rtol=1e-12, atol=1e-12)
        full_want = C0.reshape(cnc, cnr).T.astype(np.float64).copy()
        full_want[croff:croff + nr, ccoff:ccoff + nc] += want
        np.testing.assert_allclose(Cm.reshape(cnc, cnr).T, full_want, rtol=1e-5, atol=1e-5)   # nothing outside the tile moved
        # C[.., ccoff:+nc] += A[aroff:+nr, acoff:+kk] * S[broff:+nc, bcoff:+kk]^T
        nr, nc, kk, aroff, acoff, broff, bcoff, croff, ccoff = 6, 10, 8, 1, 7, 5, 9, 4, 3
        Cm = C0.copy()
        ref, sa = oracle.fsmult_tile(A, anr, aroff, acoff, nr, nc, kk, data, ir + ioff, jc + ioff, broff, bcoff,
                                     Cm, cnr, croff, ccoff, ioff=ioff, transposed=True)
        want = A2[aroff:aroff + nr, acoff:acoff + kk] @ S[broff:broff + nc, bcoff:bcoff + kk].T
        np.testing.assert_allclose(ref.reshape(nc, nr).T, want, rtol=1e-12, atol=1e-12)
        full_want = C0.reshape(cnc, cnr).T.astype(np.float64).copy()
        full_want[croff:croff + nr, ccoff:ccoff + nc] += want
        np.testing.assert_allclose(Cm.reshape(cnc, cnr).T, full_want, rtol=1e-5, atol=1e-5)
    # a tile that covers everything is the plain product, bit for bit
    k = 5
    Af = rng.standard_normal(k * snr).astype(np.float32)
    Cm = np.zeros(k * snc, dtype=np.float32)
    oracle.fsmult_tile(Af, k, 0, 0, k, snc, snr, data, ir, jc, 0, 0, Cm, k, 0, 0)
    assert np.array_equal(Cm, oracle.fsmult(Af, k, data, ir, jc))
