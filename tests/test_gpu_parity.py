"""GPU parity: every C-ABI entry point of the path against the CPU oracle on the same seeded
inputs. Integer outputs bit-exact; fp32 values within 1e-4 (relative, or relative to the sum
of |terms| where a sum cancels) of the fp64-accumulated arbiter; the oracle's own fp32 result
must pass the same bar, so a failure points at the kernel, not at the tolerance.
"""
import ctypes as C

import numpy as np
import pytest

import oracle
from bidmat_amd import hip_abi
from util import Dev, dense_full, expand_cols, make_plan, random_csc

pytestmark = pytest.mark.gpu

RTOL = 1e-4


def assert_close(x, ref64, sumabs, what):
    ok, worst = oracle.within_tolerance(x, ref64, sumabs, RTOL)
    assert ok, "%s: worst error measure %.3e > %.1e" % (what, worst, RTOL)


def opt(lib, name, value):
    old = lib.bidmat_get_option(name.encode())
    hip_abi.check(lib.bidmat_set_option(name.encode(), value), "set_option")
    return old


# k values: below a vector, odd, every lane-group width, two- and four-vector shapes, a
# non-multiple of the tile, and one that needs several passes over k.
K_VALUES = [1, 3, 10, 32, 33, 64, 100, 128, 256, 260, 512, 1024, 1100, 4200]


# ------------------------------------------------------------------------------ A * S
@pytest.mark.parametrize("k", K_VALUES)
@pytest.mark.parametrize("beta", [0, 1])
def test_dsmult_csc(hip, k, beta):
    rng = np.random.default_rng(100 + k)
    nrows, ncols = 30, 20          # the reference's own test sizes (GSMatTest.scala:13-16)
    data, ir, jc = random_csc(rng, nrows, ncols, 0.2)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    C0 = rng.standard_normal(k * ncols).astype(np.float32)
    d = Dev(A=A, data=data, ir=ir, jc=jc, Cm=C0)
    hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, ir.size, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr, d.Cm.ptr, beta, None))
    hip_abi.check(hip.bidmat_synchronize())
    got = d.Cm.numpy()
    ref64, sa = oracle.fsmult_f64(A, k, data, ir, jc)
    ref32 = oracle.fsmult(A, k, data, ir, jc, out=(C0.copy() if beta else None))
    if beta:
        ref64 = ref64 + C0
        sa = sa + np.abs(C0)
    assert_close(ref32, ref64, sa, "oracle fp32")
    assert_close(got, ref64, sa, "dsmult_csc k=%d beta=%d" % (k, beta))
    d.free()


def test_dsmult_reference_shape_entry(hip):
    """bidmat_dsmult takes (ir, ic) like the reference launcher and accumulates into C."""
    rng = np.random.default_rng(7)
    k, nrows, ncols = 10, 30, 20
    data, ir, jc = random_csc(rng, nrows, ncols, 0.2)
    ic = expand_cols(jc)
    A = rng.random(k * nrows).astype(np.float32)
    C0 = rng.random(k * ncols).astype(np.float32)
    d = Dev(A=A, data=data, ir=ir, ic=ic, Cm=C0)
    hip_abi.check(hip.bidmat_dsmult(k, ncols, ir.size, d.A.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, d.Cm.ptr))
    got = d.Cm.numpy().reshape(ncols, k).T
    # the reference's own check: A * S == A * full(S)  (GSMatTest.scala:64-71), eps 1e-4 absolute
    want = A.reshape(nrows, k).T.astype(np.float64) @ dense_full(nrows, ncols, data, ir, jc) + C0.reshape(ncols, k).T
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-4)
    d.free()


def test_dsmult_onehot_is_a_gather_bit_exact(hip):
    rng = np.random.default_rng(8)
    k, nrows, ncols = 256, 500, 3000
    ir = rng.integers(0, nrows, size=ncols).astype(np.int32)
    jc = np.arange(ncols + 1, dtype=np.int32)
    data = np.ones(ncols, dtype=np.float32)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    d = Dev(A=A, data=data, ir=ir, jc=jc)
    d.zeros("Cm", k * ncols)
    hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, ncols, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr, d.Cm.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    got = d.Cm.numpy().reshape(ncols, k)
    assert np.array_equal(got, A.reshape(nrows, k)[ir])
    d.free()


@pytest.mark.parametrize("k", [32, 256, 1024])
def test_dsmult_long_columns_split_path(hip, k):
    """Columns far longer than seglen: overflow segments + ordered second-stage sum; plus empty
    columns, unsorted rows and duplicate rows inside a column."""
    rng = np.random.default_rng(9 + k)
    nrows, ncols = 400, 37
    lengths = rng.integers(0, 12, size=ncols)
    lengths[3] = 1500
    lengths[4] = 0
    lengths[20] = 129
    lengths[36] = 700
    data, ir, jc = random_csc(rng, nrows, ncols, lengths=lengths, sort_rows=False, unique=False)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    old = opt(hip, "seglen", 64)
    try:
        for beta in (0, 1):
            C0 = rng.standard_normal(k * ncols).astype(np.float32)
            d = Dev(A=A, data=data, ir=ir, jc=jc, Cm=C0)
            hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, ir.size, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr, d.Cm.ptr, beta, None))
            hip_abi.check(hip.bidmat_synchronize())
            got = d.Cm.numpy()
            ref64, sa = oracle.fsmult_f64(A, k, data, ir, jc)
            if beta:
                ref64, sa = ref64 + C0, sa + np.abs(C0)
            assert_close(got, ref64, sa, "split-path dsmult k=%d beta=%d" % (k, beta))
            d.free()
    finally:
        opt(hip, "seglen", old)


def test_dsmult_config1(hip):
    """Benchmark configuration 1: A 32x4096 N(0,1), S 4096x8192 with exactly 50 nnz per column."""
    from bidmat_amd import gen
    c = gen.config("C1")
    k, ncols = c["k"], c["ncols"]
    d = Dev(A=c["A"], data=c["vals"], ir=c["ir"], jc=c["jc"])
    d.zeros("Cm", k * ncols)
    hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, c["ir"].size, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr, d.Cm.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    got = d.Cm.numpy()
    ref64, sa = oracle.fsmult_f64(c["A"], k, c["vals"], c["ir"], c["jc"], nthreads=8)
    ref32 = oracle.fsmult(c["A"], k, c["vals"], c["ir"], c["jc"], nthreads=8)
    assert_close(ref32, ref64, sa, "oracle fp32 C1")
    assert_close(got, ref64, sa, "dsmult C1")
    d.free()


# ------------------------------------------------------------------------------ A *^ S
@pytest.mark.parametrize("k", K_VALUES)
@pytest.mark.parametrize("beta", [0, 1])
def test_dsmultT_plan(hip, k, beta):
    rng = np.random.default_rng(200 + k)
    nrows, ncols = 20, 30
    data, ir, jc = random_csc(rng, nrows, ncols, 0.2)
    A = rng.standard_normal(k * ncols).astype(np.float32)
    C0 = rng.standard_normal(k * nrows).astype(np.float32)
    d = Dev(A=A, data=data, ir=ir, jc=jc, Cm=C0)
    plan = make_plan(hip, nrows, ncols, ir.size, d.ir, d.jc, k)
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, d.data.ptr, d.Cm.ptr, beta, None))
    hip_abi.check(hip.bidmat_synchronize())
    got = d.Cm.numpy()
    ref64, sa = oracle.fsmultT_f64(A, k, nrows, data, ir, jc)
    ref32 = oracle.fsmultT(A, k, nrows, data, ir, jc, out=(C0.copy() if beta else None))
    if beta:
        ref64, sa = ref64 + C0, sa + np.abs(C0)
    assert_close(ref32, ref64, sa, "oracle fp32")
    assert_close(got, ref64, sa, "dsmultT_plan k=%d beta=%d" % (k, beta))
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


def test_dsmultT_reference_shape_entry_and_plan_cache(hip):
    """bidmat_dsmultT builds its plan from (ir, ic); a second pattern written into the SAME device
    buffers must not meet the first pattern's plan."""
    rng = np.random.default_rng(21)
    k, nrows, ncols = 10, 20, 30
    A = rng.random(k * ncols).astype(np.float32)
    d = Dev(A=A)
    nnz = None
    for rep in range(3):
        data, ir, jc = random_csc(rng, nrows, ncols, lengths=np.full(ncols, 4))
        ic = expand_cols(jc)
        if nnz is None:
            nnz = ir.size
            d.put("data", data), d.put("ir", ir), d.put("ic", ic)
        else:
            d.data.upload(data), d.ir.upload(ir), d.ic.upload(ic)
        d.zeros("Cm", k * nrows)
        for _ in range(2):      # second call hits the cached plan and accumulates again
            hip_abi.check(hip.bidmat_dsmultT(k, ncols, nnz, d.A.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, d.Cm.ptr))
        got = d.Cm.numpy()[: k * (ir.max() + 1)].reshape(-1, k).T
        # the reference's own check: A *^ S == A * full(S)^T  (GSMatTest.scala:74-83)
        want = 2 * (A.reshape(ncols, k).T.astype(np.float64) @ dense_full(nrows, ncols, data, ir, jc).T)
        np.testing.assert_allclose(got, want[:, : got.shape[1]], rtol=0, atol=1e-4)
    d.free()


@pytest.mark.parametrize("k", [32, 256])
def test_dsmultT_heavy_rows_panels_and_segments(hip, k):
    """A pattern with a few very heavy rows (cut by column panels and by seglen), empty rows,
    duplicates and unsorted rows."""
    rng = np.random.default_rng(22 + k)
    nrows, ncols = 300, 2000
    lengths = rng.integers(0, 6, size=ncols)
    data, ir, jc = random_csc(rng, nrows, ncols, lengths=lengths, sort_rows=False, unique=False)
    # rows 0..2 appear in most columns: overwrite the first entry of most columns
    for c in range(ncols):
        if jc[c + 1] > jc[c] and rng.random() < 0.9:
            ir[jc[c]] = rng.integers(0, 3)
    ir[ir == 17] = 18                      # row 17 stays empty
    A = rng.standard_normal(k * ncols).astype(np.float32)
    old_seg, old_panel = opt(hip, "seglen", 64), opt(hip, "panel_kb", 16)
    try:
        d = Dev(A=A, data=data, ir=ir, jc=jc)
        d.zeros("Cm", k * nrows)
        plan = make_plan(hip, nrows, ncols, ir.size, d.ir, d.jc, k)
        assert hip.bidmat_plan_segments(plan) > nrows      # heavy rows were cut
        for beta in (0, 1):
            hip_abi.check(hip.bidmat_memset(d.Cm.ptr, 0, d.Cm.nbytes))
            C0 = rng.standard_normal(k * nrows).astype(np.float32)
            d.Cm.upload(C0)
            hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, d.data.ptr, d.Cm.ptr, beta, None))
            hip_abi.check(hip.bidmat_synchronize())
            got = d.Cm.numpy()
            ref64, sa = oracle.fsmultT_f64(A, k, nrows, data, ir, jc)
            if beta:
                ref64, sa = ref64 + C0, sa + np.abs(C0)
            assert_close(got, ref64, sa, "heavy-row dsmultT k=%d beta=%d" % (k, beta))
            if not beta:
                assert np.all(got.reshape(nrows, k)[17] == 0)     # empty row is written as zeros
        # determinism: a second plan over the same pattern gives the same bits
        plan2 = make_plan(hip, nrows, ncols, ir.size, d.ir, d.jc, k)
        d.zeros("C2", k * nrows)
        hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, d.data.ptr, d.Cm.ptr, 0, None))
        hip_abi.check(hip.bidmat_dsmultT_plan(plan2, k, d.A.ptr, d.data.ptr, d.C2.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
        assert np.array_equal(d.Cm.numpy(), d.C2.numpy())
        hip_abi.check(hip.bidmat_plan_destroy(plan))
        hip_abi.check(hip.bidmat_plan_destroy(plan2))
        d.free()
    finally:
        opt(hip, "seglen", old_seg), opt(hip, "panel_kb", old_panel)


# ------------------------------------------------------------------------------ DDS
@pytest.mark.parametrize("k", K_VALUES)
@pytest.mark.parametrize("beta", [0, 1])
def test_dds_csc(hip, k, beta):
    rng = np.random.default_rng(300 + k)
    nrows, ncols = 30, 20
    _, ir, jc = random_csc(rng, nrows, ncols, 0.3)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    B = rng.standard_normal(k * ncols).astype(np.float32)
    P0 = rng.standard_normal(ir.size).astype(np.float32)
    d = Dev(A=A, B=B, ir=ir, jc=jc, P=P0)
    hip_abi.check(hip.bidmat_dds_csc(k, ncols, ir.size, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.P.ptr, beta, None))
    hip_abi.check(hip.bidmat_synchronize())
    got = d.P.numpy()
    ref64, sa = oracle.dds_f64(A, B, k, ir, jc)
    ref32, oir, ojc = oracle.dds(A, B, k, ir, jc)
    assert np.array_equal(oir, ir) and np.array_equal(ojc, jc)
    if beta:
        ref64, sa, ref32 = ref64 + P0, sa + np.abs(P0), ref32 + P0
    assert_close(ref32, ref64, sa, "oracle fp32")
    assert_close(got, ref64, sa, "dds_csc k=%d beta=%d" % (k, beta))
    # the pattern arrays are inputs only: still bit-identical on the device
    assert np.array_equal(d.ir.numpy(), ir) and np.array_equal(d.jc.numpy(), jc)
    d.free()


def test_dds_reference_shape_entry_dense_pattern(hip):
    """bidmat_dds with (ir, ic); a fully dense pattern must give A^T B (MatFunctions.scala:1660)."""
    rng = np.random.default_rng(31)
    k, nrows, ncols = 30, 10, 20
    jc = (np.arange(ncols + 1) * nrows).astype(np.int32)
    ir = np.tile(np.arange(nrows, dtype=np.int32), ncols)
    ic = expand_cols(jc)
    A = rng.random(k * nrows).astype(np.float32)
    B = rng.random(k * ncols).astype(np.float32)
    d = Dev(A=A, B=B, ir=ir, ic=ic)
    d.zeros("P", ir.size)
    hip_abi.check(hip.bidmat_dds(k, ir.size, d.A.ptr, d.B.ptr, d.ir.ptr, d.ic.ptr, d.P.ptr))
    got = d.P.numpy().reshape(ncols, nrows).T
    want = A.reshape(nrows, k).astype(np.float64) @ B.reshape(ncols, k).astype(np.float64).T
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-4)
    d.free()


@pytest.mark.parametrize("k", [32, 256])
def test_dds_long_columns_split_path(hip, k):
    rng = np.random.default_rng(32 + k)
    nrows, ncols = 500, 23
    lengths = rng.integers(0, 9, size=ncols)
    lengths[0] = 0
    lengths[5] = 1000
    lengths[22] = 321
    _, ir, jc = random_csc(rng, nrows, ncols, lengths=lengths, sort_rows=False, unique=False)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    B = rng.standard_normal(k * ncols).astype(np.float32)
    old = opt(hip, "seglen", 64)
    try:
        d = Dev(A=A, B=B, ir=ir, jc=jc)
        d.zeros("P", ir.size)
        hip_abi.check(hip.bidmat_dds_csc(k, ncols, ir.size, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.P.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
        ref64, sa = oracle.dds_f64(A, B, k, ir, jc)
        assert_close(d.P.numpy(), ref64, sa, "split-path dds k=%d" % k)
        d.free()
    finally:
        opt(hip, "seglen", old)


# ------------------------------------------------------------------------------ cross-kernel identity
def test_three_kernels_agree_frobenius(hip):
    """<A*S, B>_F == sum_j v[j]*DDS(A,B,S)[j] == <B*^S, A>_F ties the three kernels together."""
    rng = np.random.default_rng(40)
    k, nrows, ncols = 64, 300, 500
    data, ir, jc = random_csc(rng, nrows, ncols, 0.05)
    A = rng.random(k * nrows).astype(np.float32)
    B = rng.random(k * ncols).astype(np.float32)
    d = Dev(A=A, B=B, data=data, ir=ir, jc=jc)
    d.zeros("AS", k * ncols), d.zeros("P", ir.size), d.zeros("BSt", k * nrows)
    plan = make_plan(hip, nrows, ncols, ir.size, d.ir, d.jc, k)
    hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, ir.size, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr, d.AS.ptr, 0, None))
    hip_abi.check(hip.bidmat_dds_csc(k, ncols, ir.size, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.P.ptr, 0, None))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.B.ptr, d.data.ptr, d.BSt.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    f1 = np.dot(d.AS.numpy().astype(np.float64), B.astype(np.float64))
    f2 = np.dot(d.P.numpy().astype(np.float64), data.astype(np.float64))
    f3 = np.dot(d.BSt.numpy().astype(np.float64), A.astype(np.float64))
    assert abs(f1 - f2) <= 1e-5 * abs(f2) and abs(f3 - f2) <= 1e-5 * abs(f2)
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


# ------------------------------------------------------------------------------ sums
@pytest.mark.parametrize("n", [1, 2])
def test_spsum_reference_shape_entry(hip, n):
    rng = np.random.default_rng(50 + n)
    nrows, ncols = 10, 20                       # GSMatTest.scala testReduce2D sizes
    data, ir, jc = random_csc(rng, nrows, ncols, 0.2)
    ic = expand_cols(jc)
    d = Dev(data=data, ir=ir, ic=ic)
    nout = ncols if n == 1 else nrows
    d.zeros("out", nout)
    hip_abi.check(hip.bidmat_spsum(nrows, ncols, ir.size, d.ir.ptr, d.ic.ptr, d.data.ptr, d.out.ptr, n))
    got = d.out.numpy()
    ref32 = oracle.spsum(nrows, data, ir, jc, n)
    ref64, sa = oracle.spsum_f64(nrows, data, ir, jc, n)
    assert_close(ref32, ref64, sa, "oracle fp32")
    assert_close(got, ref64, sa, "spsum n=%d" % n)
    d.free()


def test_spsum_large_with_plan(hip):
    rng = np.random.default_rng(53)
    nrows, ncols = 3000, 5000
    data, ir, jc = random_csc(rng, nrows, ncols, lengths=rng.integers(0, 40, size=ncols))
    d = Dev(data=data, ir=ir, jc=jc)
    d.zeros("cs", ncols), d.zeros("rs", nrows)
    plan = make_plan(hip, nrows, ncols, ir.size, d.ir, d.jc, 0)
    hip_abi.check(hip.bidmat_spsum_cols(ncols, ir.size, d.data.ptr, d.jc.ptr, d.cs.ptr, 0, None))
    hip_abi.check(hip.bidmat_spsum_rows_plan(plan, d.data.ptr, d.rs.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    for n, got in ((1, d.cs.numpy()), (2, d.rs.numpy())):
        ref64, sa = oracle.spsum_f64(nrows, data, ir, jc, n)
        assert_close(got, ref64, sa, "spsum large n=%d" % n)
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


@pytest.mark.parametrize("shape", [(10, 20), (1, 50), (50, 1), (128, 3000), (300, 7), (3, 100000), (70000, 3), (1, 300000), (300000, 1)])
@pytest.mark.parametrize("opn,initv", [(0, 0.0), (2, 1.0), (10, -3.4e38), (11, 3.4e38)])
def test_dense_reduce(hip, shape, opn, initv):
    nrows, ncols = shape
    rng = np.random.default_rng(60 + nrows + ncols)
    if opn == 2:
        # factors exp(N(0,1)/sqrt(n)): products of n of them stay near 1 whatever the length
        A = np.exp(rng.standard_normal(nrows * ncols) / np.sqrt(max(nrows, ncols))).astype(np.float32)
    else:
        A = rng.standard_normal(nrows * ncols).astype(np.float32)
    d = Dev(A=A)
    d.zeros("c", ncols), d.zeros("r", nrows)
    hip_abi.check(hip.bidmat_reduce1op(nrows, ncols, d.A.ptr, d.c.ptr, initv, opn))
    hip_abi.check(hip.bidmat_reduce2op(nrows, ncols, d.A.ptr, d.r.ptr, initv, opn))
    M = A.reshape(ncols, nrows).T.astype(np.float64)
    fn = {0: np.sum, 2: np.prod, 10: np.max, 11: np.min}[opn]
    want_c, want_r = fn(M, axis=0), fn(M, axis=1)
    if opn in (10, 11):
        assert np.array_equal(d.c.numpy(), want_c.astype(np.float32))
        assert np.array_equal(d.r.numpy(), want_r.astype(np.float32))
    else:
        sa_c, sa_r = np.abs(M).sum(axis=0), np.abs(M).sum(axis=1)
        if opn == 2:
            sa_c, sa_r = np.abs(want_c), np.abs(want_r)
        assert_close(d.c.numpy(), want_c, sa_c, "reduce1op")
        assert_close(d.r.numpy(), want_r, sa_r, "reduce2op")
        if opn == 0:   # the oracle's sequential fp32 sums pass the same bar
            assert_close(oracle.dsum(A, nrows, ncols, 1), want_c, sa_c, "oracle dsum 1")
            assert_close(oracle.dsum(A, nrows, ncols, 2), want_r, sa_r, "oracle dsum 2")
    d.free()


def test_dense_reduce_rejects_unknown_op(hip):
    d = Dev(A=np.ones(6, dtype=np.float32))
    d.zeros("c", 3)
    assert hip.bidmat_reduce1op(2, 3, d.A.ptr, d.c.ptr, 0.0, 15) == 1
    assert hip.bidmat_reduce2op(2, 3, d.A.ptr, d.c.ptr, 0.0, -1) == 1
    d.free()


@pytest.mark.parametrize("shape", [(10, 20), (1, 50), (50, 1), (33, 7), (7, 33), (100, 65), (64, 1000), (2000, 3), (5, 4097)])
@pytest.mark.parametrize("opn", [1, 3, 4, 5, 6, 7, 8, 9, 12, 13, 14])
def test_dense_reduce_with_every_other_op_follows_the_reference_tree(hip, shape, opn):
    """The ops that BIDMat's own reductions never issue (sub, div, the comparisons, atan2, pow, ifpos) are not
    associative: the result is defined by the order of the reference's kernels (Operators.cu:650-671,828-851),
    which the oracle restates. Bit for bit, except atan2 / pow (device and host libm differ in the last bit)."""
    nrows, ncols = shape
    rng = np.random.default_rng(70 + 31 * nrows + ncols + opn)
    if opn in (3, 13):
        A = (0.5 + rng.random(nrows * ncols)).astype(np.float32)           # near 1: quotients / powers stay finite
    elif opn in (4, 5, 6, 7, 8, 9):
        A = rng.integers(0, 3, size=nrows * ncols).astype(np.float32)       # ties happen
    else:
        A = rng.standard_normal(nrows * ncols).astype(np.float32)
    d = Dev(A=A)
    d.zeros("c", ncols), d.zeros("r", nrows)
    hip_abi.check(hip.bidmat_reduce1op(nrows, ncols, d.A.ptr, d.c.ptr, 0.0, opn))
    hip_abi.check(hip.bidmat_reduce2op(nrows, ncols, d.A.ptr, d.r.ptr, 0.0, opn))
    want_c, want_r = oracle.reduce_tree(A, nrows, ncols, opn, 1), oracle.reduce_tree(A, nrows, ncols, opn, 2)
    if opn in (12, 13):
        np.testing.assert_allclose(d.c.numpy(), want_c, rtol=2e-5, atol=1e-6)
        np.testing.assert_allclose(d.r.numpy(), want_r, rtol=2e-5, atol=1e-6)
    else:
        assert np.array_equal(d.c.numpy(), want_c, equal_nan=True), "reduce1op op %d" % opn
        assert np.array_equal(d.r.numpy(), want_r, equal_nan=True), "reduce2op op %d" % opn
    d.free()


# ------------------------------------------------------------------------------ elementwise
@pytest.mark.parametrize("opn", list(range(15)))
def test_applyop_full_all_ops(hip, opn):
    rng = np.random.default_rng(70 + opn)
    nr, nc = 37, 29
    A = (rng.random(nr * nc).astype(np.float32) + 0.1)
    B = (rng.random(nr * nc).astype(np.float32) + 0.1)
    B[::7] = A[::7]                       # make eq/ge/le meaningful
    d = Dev(A=A, B=B)
    d.zeros("Cm", nr * nc)
    hip_abi.check(hip.bidmat_applyop(d.A.ptr, nr, nc, d.B.ptr, nr, nc, d.Cm.ptr, opn))
    got = d.Cm.numpy()
    want = oracle.applyop(A, B, opn)
    if opn in (12, 13):                   # atan2f / powf: libm vs device libm
        np.testing.assert_allclose(got, want, rtol=1e-5)
    else:                                 # IEEE add/sub/mul/div and comparisons: bit-exact
        assert np.array_equal(got, want)
    d.free()


def test_applyop_broadcast_modes(hip):
    rng = np.random.default_rng(90)
    nr, nc = 13, 17
    M = rng.random((nr, nc)).astype(np.float32) + 0.5
    col = rng.random((nr, 1)).astype(np.float32) + 0.5
    row = rng.random((1, nc)).astype(np.float32) + 0.5
    val = rng.random((1, 1)).astype(np.float32) + 0.5
    cases = [(M, col), (M, row), (col, M), (row, M), (M, val), (val, M)]
    for a, b in cases:
        da, db = Dev(x=np.asfortranarray(a).ravel(order="F")), Dev(x=np.asfortranarray(b).ravel(order="F"))
        out = Dev()
        out.zeros("c", nr * nc)
        hip_abi.check(hip.bidmat_applyop(da.x.ptr, a.shape[0], a.shape[1], db.x.ptr, b.shape[0], b.shape[1], out.c.ptr, 3))
        got = out.c.numpy().reshape(nc, nr).T
        assert np.array_equal(got, (a / b).astype(np.float32))
        da.free(), db.free(), out.free()
    # incompatible shapes are rejected
    d = Dev(x=np.ones(12, dtype=np.float32))
    assert hip.bidmat_applyop(d.x.ptr, 3, 4, d.x.ptr, 4, 3, d.x.ptr, 0) == 1
    d.free()


def test_applyop_flat_div_on_values(hip):
    """The V./R step: elementwise division of two nonzero-value arrays."""
    rng = np.random.default_rng(91)
    n = 1_000_003
    V = rng.exponential(size=n).astype(np.float32)
    R = (rng.random(n).astype(np.float32) + 0.01)
    d = Dev(V=V, R=R)
    d.zeros("Q", n)
    hip_abi.check(hip.bidmat_applyop_flat(d.V.ptr, d.R.ptr, d.Q.ptr, n, 3, None))
    hip_abi.check(hip.bidmat_synchronize())
    assert np.array_equal(d.Q.numpy(), V / R)
    d.free()


@pytest.mark.parametrize("n", [1, 3, 5, 4 * 1023, 4 * 1024, 4 * 1024 + 4, 4 * 1025 + 1, 4 * 2048, 4 * 2048 + 7,
                               4 * 1024 * 16384 + 4 * 100 + 2])
def test_applyop_flat_tile_edges(hip, n):
    """Sizes around the 4 x 256-vector tiles of the streaming kernel, and one larger than the grid."""
    rng = np.random.default_rng(n % 1000)
    A = rng.random(n).astype(np.float32)
    B = rng.random(n).astype(np.float32) + 0.5
    d = Dev(A=A, B=B)
    d.zeros("Cm", n)
    hip_abi.check(hip.bidmat_applyop_flat(d.A.ptr, d.B.ptr, d.Cm.ptr, n, 1, None))
    hip_abi.check(hip.bidmat_synchronize())
    assert np.array_equal(d.Cm.numpy(), A - B)
    d.free()


# ------------------------------------------------------------------------------ CSC utilities
def test_expand_and_compress_cols(hip):
    rng = np.random.default_rng(95)
    ncols = 5000
    lengths = rng.integers(0, 50, size=ncols)
    lengths[:10] = 0
    lengths[-5:] = 0
    jc = np.zeros(ncols + 1, dtype=np.int32)
    jc[1:] = np.cumsum(lengths)
    nnz = int(jc[-1])
    d = Dev(jc=jc)
    d.zeros("ic", nnz, np.int32), d.zeros("jc2", ncols + 1, np.int32)
    hip_abi.check(hip.bidmat_csc_expand_cols(ncols, nnz, d.jc.ptr, d.ic.ptr, None))
    hip_abi.check(hip.bidmat_coo_compress_cols(ncols, nnz, d.ic.ptr, d.jc2.ptr, None))
    hip_abi.check(hip.bidmat_synchronize())
    assert np.array_equal(d.ic.numpy(), oracle.uncompress_inds(jc))
    assert np.array_equal(d.jc2.numpy(), jc)
    assert np.array_equal(oracle.compress_inds(oracle.uncompress_inds(jc), ncols), jc)
    d.free()


def test_colslice_copy_and_zero_copy_column_ranges(hip):
    """bidmat_csc_colslice against numpy slicing (bit-exact), and the zero-copy form: the product
    entries take Sjc + col1 with the unsliced index / value arrays."""
    rng = np.random.default_rng(96)
    k, nrows, ncols = 64, 300, 2000
    lengths = rng.integers(0, 40, size=ncols)
    lengths[777] = 3000                                         # a split column inside the range
    data, ir, jc = random_csc(rng, nrows, ncols, lengths=lengths, unique=False)
    nnz = int(ir.size)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    B = rng.standard_normal(k * ncols).astype(np.float32)
    d = Dev(A=A, B=B, data=data, ir=ir, jc=jc)
    ref, sa = oracle.fsmult_f64(A, k, data, ir, jc)
    pref, psa = oracle.dds_f64(A, B, k, ir, jc)
    for c1, c2 in [(0, ncols), (500, 1200), (776, 778), (1999, 2000), (100, 100)]:
        start, n = C.c_int(-1), C.c_int(-1)
        hip_abi.check(hip.bidmat_csc_colslice_range(ncols, c1, c2, d.jc.ptr, C.byref(start), C.byref(n)))
        assert (start.value, n.value) == (int(jc[c1]), int(jc[c2] - jc[c1]))
        nc, n = c2 - c1, n.value
        o = Dev()
        o.zeros("jc", nc + 1, np.int32), o.zeros("ir", max(n, 1), np.int32), o.zeros("ic", max(n, 1), np.int32)
        o.zeros("data", max(n, 1))
        hip_abi.check(hip.bidmat_csc_colslice(c1, c2, start.value, n, d.jc.ptr, d.ir.ptr, d.data.ptr,
                                              o.jc.ptr, o.ir.ptr, o.ic.ptr, o.data.ptr, None))
        hip_abi.check(hip.bidmat_synchronize())
        lo, hi = int(jc[c1]), int(jc[c2])
        assert np.array_equal(o.jc.numpy(), jc[c1:c2 + 1] - jc[c1])
        assert np.array_equal(o.ir.numpy(n), ir[lo:hi]) and np.array_equal(o.data.numpy(n), data[lo:hi])
        assert np.array_equal(o.ic.numpy(n), np.repeat(np.arange(nc, dtype=np.int32), np.diff(jc[c1:c2 + 1])))
        if nc:
            # zero-copy: column pointers are absolute positions, so a range of them is a matrix
            o.zeros("AS", k * nc), o.zeros("P", nnz)
            hip_abi.check(hip.bidmat_dsmult_csc(k, nc, nnz, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr + 4 * c1,
                                                o.AS.ptr, 0, None))
            hip_abi.check(hip.bidmat_dds_csc(k, nc, nnz, d.A.ptr, d.B.ptr + 4 * k * c1, d.ir.ptr, d.jc.ptr + 4 * c1,
                                             o.P.ptr, 0, None))
            hip_abi.check(hip.bidmat_synchronize())
            assert_close(o.AS.numpy(), ref[k * c1:k * c2], sa[k * c1:k * c2], "A*S on a column range")
            P = o.P.numpy()                                     # P keeps absolute nonzero positions
            assert_close(P[lo:hi], pref[lo:hi], psa[lo:hi], "DDS on a column range")
            assert not P[:lo].any() and not P[hi:].any()
        o.free()
    assert hip.bidmat_csc_colslice_range(ncols, 5, 4, d.jc.ptr, C.byref(start), C.byref(C.c_int())) == 1
    assert hip.bidmat_csc_colslice_range(ncols, 0, ncols + 1, d.jc.ptr, C.byref(start), C.byref(C.c_int())) == 1
    d.free()


def test_two_streams_do_not_share_scratch(hip):
    """Products with split columns enqueued back to back on two streams (each needs its own
    overflow table and partial sums while the other is still running)."""
    rng = np.random.default_rng(97)
    k = 128
    cases = []
    for nrows, ncols in [(3000, 6000), (2500, 5000)]:
        lengths = rng.integers(0, 30, size=ncols)
        lengths[rng.integers(0, ncols, size=40)] = 5000          # many split columns
        data, ir, jc = random_csc(rng, nrows, ncols, lengths=lengths, unique=False)
        A = rng.standard_normal(k * nrows).astype(np.float32)
        B = rng.standard_normal(k * ncols).astype(np.float32)
        d = Dev(A=A, B=B, data=data, ir=ir, jc=jc)
        d.zeros("AS", k * ncols), d.zeros("P", ir.size)
        st = C.c_void_p()
        hip_abi.check(hip.bidmat_stream_create(C.byref(st)))
        cases.append((d, st, A, B, data, ir, jc, ncols))
    for rep in range(3):
        for d, st, A, B, data, ir, jc, ncols in cases:
            hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, ir.size, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr, d.AS.ptr, 0, st))
            hip_abi.check(hip.bidmat_dds_csc(k, ncols, ir.size, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.P.ptr, 0, st))
    for d, st, A, B, data, ir, jc, ncols in cases:
        hip_abi.check(hip.bidmat_stream_synchronize(st))
        assert_close(d.AS.numpy(), *oracle.fsmult_f64(A, k, data, ir, jc), "A*S on its own stream")
        assert_close(d.P.numpy(), *oracle.dds_f64(A, B, k, ir, jc), "DDS on its own stream")
        hip_abi.check(hip.bidmat_stream_destroy(st))              # frees that stream's scratch as well
        d.free()


def test_graph_replay_of_the_three_products(hip):
    """A*S, DDS and A*^S recorded into one HIP graph; every replay (with eager work and
    synchronisations in between, and with new values in the same buffers) must give exactly what
    the eager calls give."""
    rng = np.random.default_rng(98)
    k, nrows, ncols = 64, 400, 3000
    lengths = rng.integers(0, 25, size=ncols)
    lengths[11] = 2500                                           # overflow segments inside the graph
    data, ir, jc = random_csc(rng, nrows, ncols, lengths=lengths, unique=False)
    nnz = int(ir.size)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    B = rng.standard_normal(k * ncols).astype(np.float32)
    d = Dev(A=A, B=B, data=data, ir=ir, jc=jc)
    for name, n in (("AS", k * ncols), ("P", nnz), ("G", k * nrows), ("AS2", k * ncols), ("P2", nnz), ("G2", k * nrows)):
        d.zeros(name, n)
    plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
    st = C.c_void_p()
    hip_abi.check(hip.bidmat_stream_create(C.byref(st)))

    def step(AS, P, G, stream):
        hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, nnz, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr, AS.ptr, 0, stream))
        hip_abi.check(hip.bidmat_dds_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, P.ptr, 0, stream))
        hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.B.ptr, d.data.ptr, G.ptr, 0, stream))

    step(d.AS, d.P, d.G, st)                                      # warm-up: sizes the stream's scratch
    hip_abi.check(hip.bidmat_stream_synchronize(st))
    hip_abi.check(hip.bidmat_graph_begin_capture(st))
    step(d.AS, d.P, d.G, st)
    gx = C.c_void_p()
    hip_abi.check(hip.bidmat_graph_end_capture(st, C.byref(gx)))
    for rep in range(4):
        if rep:                                                   # new values in the same buffers
            newA = rng.standard_normal(k * nrows).astype(np.float32)
            newv = (1.0 - rng.random(nnz)).astype(np.float32)
            hip_abi.check(hip.bidmat_memcpy_h2d(d.A.ptr, newA.ctypes.data, newA.nbytes))
            hip_abi.check(hip.bidmat_memcpy_h2d(d.data.ptr, newv.ctypes.data, newv.nbytes))
        for buf in (d.AS, d.P, d.G):
            hip_abi.check(hip.bidmat_memset(buf.ptr, 0xFF, buf.nbytes))
        hip_abi.check(hip.bidmat_graph_launch(gx, st))
        hip_abi.check(hip.bidmat_stream_synchronize(st))
        step(d.AS2, d.P2, d.G2, None)                             # eager, default stream
        hip_abi.check(hip.bidmat_synchronize())
        for got, want, what in ((d.AS, d.AS2, "A*S"), (d.P, d.P2, "DDS"), (d.G, d.G2, "A*^S")):
            assert np.array_equal(got.numpy().view(np.int32), want.numpy().view(np.int32)), "%s replay %d" % (what, rep)
    hip_abi.check(hip.bidmat_graph_destroy(gx))
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    hip_abi.check(hip.bidmat_stream_destroy(st))
    d.free()


# ------------------------------------------------------------------------------ error behaviour
def test_argument_validation(hip):
    d = Dev(x=np.ones(16, dtype=np.float32), i=np.zeros(16, dtype=np.int32))
    assert hip.bidmat_dsmult(-1, 1, 1, d.x.ptr, d.x.ptr, d.i.ptr, d.i.ptr, d.x.ptr) == 1
    assert hip.bidmat_dsmult(2, 2, 2, None, d.x.ptr, d.i.ptr, d.i.ptr, d.x.ptr) == 1
    assert hip.bidmat_dsmult_csc(2, 2, 2, d.x.ptr, d.x.ptr, d.i.ptr, d.i.ptr, d.x.ptr, 2, None) == 1
    assert hip.bidmat_dds(2, -1, d.x.ptr, d.x.ptr, d.i.ptr, d.i.ptr, d.x.ptr) == 1
    assert hip.bidmat_dsmultT_plan(None, 2, d.x.ptr, d.x.ptr, d.x.ptr, 0, None) == 1
    assert hip.bidmat_dsmult(0, 0, 0, None, None, None, None, None) == 0          # empty product is a no-op
    assert b"invalid" in hip.bidmat_error_string(1).lower()
    # a row index outside the matrix is caught when the plan is built
    bad_ir = np.array([0, 5, 99], dtype=np.int32)
    jc = np.array([0, 2, 3], dtype=np.int32)
    e = Dev(ir=bad_ir, jc=jc)
    p = C.c_void_p()
    assert hip.bidmat_plan_create(10, 2, 3, e.ir.ptr, e.jc.ptr, 0, C.byref(p)) == 1
    e.free(), d.free()


# ------------------------------------------------------------------------------ tile variants
@pytest.mark.parametrize("nr", [5, 32, 64, 256, 300])
@pytest.mark.parametrize("transposed", [False, True])
def test_dsmult_tile(hip, nr, transposed):
    """bidmat_dsmultTile / TileT: windows of A, S and C with their parents' strides, aligned
    and unaligned window origins, accumulate into C, nothing outside the tile touched."""
    rng = np.random.default_rng(400 + nr + int(transposed))
    snr, snc = 90, 70
    lengths = rng.integers(0, 25, size=snc)
    lengths[11] = 0
    data, ir, jc = random_csc(rng, snr, snc, lengths=lengths, sort_rows=False)
    ir[(ir > 2) & (rng.random(ir.size) < 0.3)] = 1          # a heavy row
    ic = expand_cols(jc)
    old_seg, old_panel = opt(hip, "seglen", 64), opt(hip, "panel_kb", 16)
    try:
        for (aroff, croff) in ((0, 0), (3, 5), (4, 8)):
            anr, cnr = nr + aroff + 2, nr + croff + 3
            if transposed:
                nc, kk, broff, bcoff = 40, 33, 17, 9          # rows 17..56 of S, columns 9..41
            else:
                nc, kk, broff, bcoff = 29, 50, 13, 21         # rows 13..62 of S, columns 21..49
            acoff, ccoff = 2, 1
            anc, cnc = kk + acoff + 1, nc + ccoff + 2
            A = rng.standard_normal(anr * anc).astype(np.float32)
            C0 = rng.standard_normal(cnr * cnc).astype(np.float32)
            d = Dev(A=A, data=data, ir=ir, ic=ic, Cm=C0)
            fn = hip.bidmat_dsmultTileT if transposed else hip.bidmat_dsmultTile
            hip_abi.check(fn(nr, nc, kk, ir.size, d.A.ptr + 4 * (aroff + acoff * anr), anr, d.data.ptr, d.ir.ptr,
                             d.ic.ptr, broff, bcoff, d.Cm.ptr + 4 * (croff + ccoff * cnr), cnr))
            got = d.Cm.numpy().reshape(cnc, cnr).T
            Cref = C0.copy()
            ref64, sa = oracle.fsmult_tile(A, anr, aroff, acoff, nr, nc, kk, data, ir, jc, broff, bcoff, Cref, cnr,
                                           croff, ccoff, transposed=transposed)
            c0 = C0.reshape(cnc, cnr).T
            win = (slice(croff, croff + nr), slice(ccoff, ccoff + nc))
            want = ref64.reshape(nc, nr).T + c0[win]
            assert_close(got[win].ravel(), want.ravel(), (sa.reshape(nc, nr).T + np.abs(c0[win])).ravel(),
                         "tile nr=%d T=%s off=%d" % (nr, transposed, aroff))
            assert_close(Cref.reshape(cnc, cnr).T[win].ravel(), want.ravel(),
                         (sa.reshape(nc, nr).T + np.abs(c0[win])).ravel(), "oracle fp32 tile")
            mask = np.ones_like(got, dtype=bool)
            mask[win] = False
            assert np.array_equal(got[mask], c0[mask])            # outside the tile: untouched
            d.free()
    finally:
        opt(hip, "seglen", old_seg), opt(hip, "panel_kb", old_panel)


def test_dsmult_tile_whole_matrix_equals_plain_product(hip):
    rng = np.random.default_rng(450)
    k, nrows, ncols = 64, 200, 300
    data, ir, jc = random_csc(rng, nrows, ncols, 0.05)
    ic = expand_cols(jc)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    B = rng.standard_normal(k * ncols).astype(np.float32)
    d = Dev(A=A, B=B, data=data, ir=ir, ic=ic)
    d.zeros("C1", k * ncols), d.zeros("C2", k * ncols), d.zeros("G1", k * nrows), d.zeros("G2", k * nrows)
    hip_abi.check(hip.bidmat_dsmult(k, ncols, ir.size, d.A.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, d.C1.ptr))
    hip_abi.check(hip.bidmat_dsmultTile(k, ncols, nrows, ir.size, d.A.ptr, k, d.data.ptr, d.ir.ptr, d.ic.ptr, 0, 0, d.C2.ptr, k))
    assert np.array_equal(d.C1.numpy(), d.C2.numpy())
    hip_abi.check(hip.bidmat_dsmultT(k, ncols, ir.size, d.B.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, d.G1.ptr))
    hip_abi.check(hip.bidmat_dsmultTileT(k, nrows, ncols, ir.size, d.B.ptr, k, d.data.ptr, d.ir.ptr, d.ic.ptr, 0, 0, d.G2.ptr, k))
    assert np.array_equal(d.G1.numpy(), d.G2.numpy())
    d.free()


# ------------------------------------------------------------------------------ sparse x dense
@pytest.mark.parametrize("p", [1, 7, 64, 200])
def test_sparse_times_dense(hip, p):
    """S*A and S^T*A through the C ABI, windows via lda / ldc, against fp64 dense products."""
    rng = np.random.default_rng(500 + p)
    m, n = 150, 230
    data, ir, jc = random_csc(rng, m, n, 0.06)
    S = dense_full(m, n, data, ir, jc)
    d = Dev(data=data, ir=ir, jc=jc)
    plan = make_plan(hip, m, n, ir.size, d.ir, d.jc, p)
    # S * A: A is n x p inside a parent with leading dimension n + 3
    lda, ldc = n + 3, m + 2
    Ap = rng.standard_normal(lda * p).astype(np.float32)
    d.put("A", Ap), d.put("Cm", np.full(ldc * p, 7.0, dtype=np.float32))
    hip_abi.check(hip.bidmat_sdmult_plan(plan, p, d.data.ptr, d.A.ptr, lda, d.Cm.ptr, ldc, None))
    hip_abi.check(hip.bidmat_synchronize())
    got = d.Cm.numpy().reshape(p, ldc).T
    A2 = Ap.reshape(p, lda).T[:n].astype(np.float64)
    want, sa = S @ A2, np.abs(S) @ np.abs(A2)
    assert_close(got[:m].ravel(), want.ravel(), sa.ravel(), "S*A p=%d" % p)
    assert np.all(got[m:] == 7.0)                       # padding rows of the parent untouched
    # S^T * A: A is m x p
    lda, ldc = m + 1, n + 5
    Ap = rng.standard_normal(lda * p).astype(np.float32)
    d.put("A2", Ap), d.put("C2", np.full(ldc * p, 7.0, dtype=np.float32))
    hip_abi.check(hip.bidmat_sdtmult_csc(m, n, ir.size, p, d.data.ptr, d.ir.ptr, d.jc.ptr, d.A2.ptr, lda, d.C2.ptr, ldc, None))
    hip_abi.check(hip.bidmat_synchronize())
    got = d.C2.numpy().reshape(p, ldc).T
    A2 = Ap.reshape(p, lda).T[:m].astype(np.float64)
    want, sa = S.T @ A2, np.abs(S).T @ np.abs(A2)
    assert_close(got[:n].ravel(), want.ravel(), sa.ravel(), "S^T*A p=%d" % p)
    assert np.all(got[n:] == 7.0)
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


def test_transpose(hip):
    rng = np.random.default_rng(510)
    for (nr_, nc_) in ((1, 1), (5, 70), (33, 31), (257, 64), (64, 1000)):
        a = rng.standard_normal((nr_, nc_)).astype(np.float32)
        d = Dev(a=np.asfortranarray(a).ravel(order="F"))
        d.zeros("t", nr_ * nc_)
        hip_abi.check(hip.bidmat_transpose(nr_, nc_, d.a.ptr, nr_, d.t.ptr, nc_, None))
        hip_abi.check(hip.bidmat_synchronize())
        assert np.array_equal(d.t.numpy().reshape(nr_, nc_).T, a.T)
        d.free()
