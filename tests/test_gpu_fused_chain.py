"""bidmat_dds_dsmultT_plan: Q = op(V, DDS(A, B, S)) and G = B *^ Q in one walk over the plan's rows.

The fused entry promises the bits of the two calls it replaces (bidmat_dds_plan with the fused elementwise
op, then bidmat_dsmultT_plan), so the parity bar is array equality with that chain, which the other GPU
tests hold against the oracle; one case is also checked against the oracle's float64 arbiter directly.
"""
import numpy as np
import pytest

import oracle
from bidmat_amd import hip_abi
from util import Dev, make_plan

pytestmark = pytest.mark.gpu

OP_DIV = 3


def zipf_csc(rng, nrows, ncols, mean_len, a=1.1):
    p = 1.0 / np.arange(1, nrows + 1) ** a
    p /= p.sum()
    lens = rng.poisson(mean_len, size=ncols)
    cols = []
    for c in range(ncols):
        cols.append(np.unique(rng.choice(nrows, size=int(lens[c]), p=p)).astype(np.int32))
    jc = np.zeros(ncols + 1, np.int32)
    jc[1:] = np.cumsum([x.size for x in cols])
    ir = np.concatenate(cols) if cols else np.zeros(0, np.int32)
    return ir.astype(np.int32), jc


def chain(hip, plan, k, d, nnz, nrows, op, stored):
    """The two calls: Q through the class-ordered / plain DDS with the op fused, G through the plan."""
    d.zeros("Q1", max(nnz, 1))
    d.zeros("G1", k * nrows)
    if stored:
        hip_abi.check(hip.bidmat_dds_plan_stored(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, op, d.Q1.ptr, None))
    else:
        hip_abi.check(hip.bidmat_dds_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, op, d.Q1.ptr, 0, None))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.B.ptr, d.Q1.ptr, d.G1.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    return d.Q1.numpy()[:nnz], d.G1.numpy()


# k: a single lane group, odd, every group width, the headline's and configs[4]'s, several vectors per lane,
# the largest that fits one pass; nrows/ncols/mean length keep every case to well under a second
CASES = [(1, 40, 60, 8), (3, 40, 60, 8), (10, 300, 500, 20), (32, 300, 500, 20), (33, 300, 500, 20), (64, 2000, 3000, 30),
         (100, 2000, 3000, 30), (128, 5000, 20000, 60), (256, 5000, 20000, 60), (250, 300, 500, 20), (512, 1000, 2000, 40),
         (1024, 500, 1000, 40)]


@pytest.mark.parametrize("k,nrows,ncols,mean_len", CASES)
@pytest.mark.parametrize("stored", [False, True], ids=["values_passed", "values_in_plan"])
def test_fused_chain_has_the_bits_of_the_two_calls(hip, k, nrows, ncols, mean_len, stored):
    rng = np.random.default_rng(1000 * k + nrows)
    ir, jc = zipf_csc(rng, nrows, ncols, mean_len)
    nnz = ir.size
    A = (0.01 + rng.random(k * nrows)).astype(np.float32)
    B = (0.01 + rng.random(k * ncols)).astype(np.float32)
    v = rng.gamma(1.0, 1.0, size=nnz).astype(np.float32)
    d = Dev(A=A, B=B, v=v, ir=ir, jc=jc)
    plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
    if stored:
        hip_abi.check(hip.bidmat_plan_set_values(plan, d.v.ptr, None))
    Q1, G1 = chain(hip, plan, k, d, nnz, nrows, OP_DIV, stored)
    d.put("Q2", np.full(max(nnz, 1), -5.0, np.float32))
    G0 = rng.standard_normal(k * nrows).astype(np.float32)
    d.put("G2", np.zeros(k * nrows, np.float32))
    hip_abi.check(hip.bidmat_dds_dsmultT_plan(plan, k, d.A.ptr, d.B.ptr, None if stored else d.v.ptr, OP_DIV, d.Q2.ptr,
                                              d.G2.ptr, 0, None), "fused")
    hip_abi.check(hip.bidmat_synchronize())
    Q2, G2 = d.Q2.numpy()[:nnz], d.G2.numpy()
    assert np.array_equal(Q2.view(np.uint32), Q1.view(np.uint32)), "Q differs in %d places" % int((Q2 != Q1).sum())
    assert np.array_equal(G2.view(np.uint32), G1.view(np.uint32)), "G differs in %d places" % int((G2 != G1).sum())
    if not stored:
        # the values by a gather per lane instead of scalar loads (what k <= 128 takes anyway): the same bits
        hip_abi.check(hip.bidmat_set_option(b"scalar_values", 0))
        try:
            d.put("Q5", np.full(max(nnz, 1), -5.0, np.float32))
            d.put("G5", np.zeros(k * nrows, np.float32))
            hip_abi.check(hip.bidmat_dds_dsmultT_plan(plan, k, d.A.ptr, d.B.ptr, d.v.ptr, OP_DIV, d.Q5.ptr, d.G5.ptr, 0, None))
            hip_abi.check(hip.bidmat_synchronize())
        finally:
            hip_abi.check(hip.bidmat_set_option(b"scalar_values", 1))
        assert np.array_equal(d.Q5.numpy()[:nnz].view(np.uint32), Q2.view(np.uint32))
        assert np.array_equal(d.G5.numpy().view(np.uint32), G2.view(np.uint32))
    # without the product output, accumulating into G
    d.put("G3", G0)
    hip_abi.check(hip.bidmat_dds_dsmultT_plan(plan, k, d.A.ptr, d.B.ptr, None if stored else d.v.ptr, OP_DIV, None,
                                              d.G3.ptr, 1, None), "fused beta=1")
    d.put("G4", G0)
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.B.ptr, d.Q1.ptr, d.G4.ptr, 1, None))
    hip_abi.check(hip.bidmat_synchronize())
    assert np.array_equal(d.G3.numpy().view(np.uint32), d.G4.numpy().view(np.uint32))
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


def test_fused_chain_against_the_oracle(hip):
    """Q = V ./ DDS and G = B *^ Q from the CPU restatement (oracle.dds, oracle.fsmultT), fp32 tolerance 1e-4
    against the float64 arbiter."""
    rng = np.random.default_rng(77)
    k, nrows, ncols = 48, 200, 300
    ir, jc = zipf_csc(rng, nrows, ncols, 15)
    nnz = ir.size
    A = (0.01 + rng.random(k * nrows)).astype(np.float32)
    B = (0.01 + rng.random(k * ncols)).astype(np.float32)
    v = rng.gamma(1.0, 1.0, size=nnz).astype(np.float32)
    d = Dev(A=A, B=B, v=v, ir=ir, jc=jc)
    d.zeros("Q", nnz), d.zeros("G", k * nrows)
    plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
    hip_abi.check(hip.bidmat_dds_dsmultT_plan(plan, k, d.A.ptr, d.B.ptr, d.v.ptr, OP_DIV, d.Q.ptr, d.G.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    A2, B2 = A.reshape(nrows, k).astype(np.float64), B.reshape(ncols, k).astype(np.float64)
    ic = np.repeat(np.arange(ncols), np.diff(jc))
    dots = np.einsum("ij,ij->i", A2[ir], B2[ic])
    q64 = v.astype(np.float64) / dots
    assert np.allclose(d.Q.numpy(), q64, rtol=1e-4, atol=0)
    g64 = np.zeros((nrows, k))
    np.add.at(g64, ir, q64[:, None] * B2[ic])
    sa = np.zeros((nrows, k))
    np.add.at(sa, ir, np.abs(q64[:, None] * B2[ic]))
    ok, worst = oracle.within_tolerance(d.G.numpy(), g64.ravel(), sa.ravel(), 1e-4)
    assert ok, worst
    # and the oracle's own fp32 chain passes the same bar
    q32 = (v / oracle.dds(A, B, k, ir, jc)[0]).astype(np.float32)
    assert np.allclose(q32, q64, rtol=1e-4, atol=0)
    g32 = oracle.fsmultT(B, k, nrows, q32, ir, jc)
    ok, worst = oracle.within_tolerance(g32, g64.ravel(), sa.ravel(), 1e-4)
    assert ok, worst
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


def test_fused_chain_refuses_what_it_cannot_do(hip):
    rng = np.random.default_rng(3)
    nrows, ncols = 50, 80
    ir, jc = zipf_csc(rng, nrows, ncols, 6)
    nnz = ir.size
    for k in (1028, 260):                       # more than one pass: aligned beyond 1024, unaligned beyond 256
        d = Dev(A=rng.random(k * nrows).astype(np.float32), B=rng.random(k * ncols).astype(np.float32),
                v=rng.random(nnz).astype(np.float32), ir=ir, jc=jc)
        d.zeros("G", k * nrows)
        plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
        off = 0 if k == 1028 else 4             # k = 260 with a misaligned B takes the scalar shape
        rc = hip.bidmat_dds_dsmultT_plan(plan, k, d.A.ptr, d.B.ptr + off, d.v.ptr, OP_DIV, None, d.G.ptr, 0, None)
        assert rc == 1, (k, rc)
        assert hip.bidmat_dds_dsmultT_plan(plan, k, d.A.ptr, d.B.ptr, d.v.ptr, 99, None, d.G.ptr, 0, None) == 1
        assert hip.bidmat_dds_dsmultT_plan(plan, k, d.A.ptr, d.B.ptr, None, OP_DIV, None, d.G.ptr, 0, None) == 1  # no stored values
        hip_abi.check(hip.bidmat_plan_destroy(plan))
        d.free()


# ------------------------------------------------------------------ the chain by columns
COL_CASES = [(1, 40, 60, 8), (3, 40, 60, 8), (10, 300, 500, 20), (32, 300, 500, 20), (33, 300, 500, 20), (64, 2000, 3000, 30),
             (100, 2000, 3000, 30), (128, 5000, 20000, 60), (256, 5000, 20000, 60), (250, 300, 500, 20), (512, 1000, 2000, 40),
             (1024, 500, 1000, 40)]


@pytest.mark.parametrize("k,nrows,ncols,mean_len", COL_CASES)
@pytest.mark.parametrize("seglen", [1024, 64], ids=["whole_columns", "columns_cut_into_segments"])
def test_column_chain_has_the_bits_of_the_two_calls(hip, k, nrows, ncols, mean_len, seglen):
    """bidmat_dds_dsmult_csc against bidmat_dds_csc_op + bidmat_dsmult_csc; seglen = 64 cuts every longer column into
    overflow segments with partial sums."""
    rng = np.random.default_rng(2000 * k + nrows)
    ir, jc = zipf_csc(rng, nrows, ncols, mean_len * (4 if seglen == 64 else 1))
    nnz = ir.size
    A = (0.01 + rng.random(k * nrows)).astype(np.float32)
    B = (0.01 + rng.random(k * ncols)).astype(np.float32)
    v = rng.gamma(1.0, 1.0, size=nnz).astype(np.float32)
    C0 = rng.standard_normal(k * ncols).astype(np.float32)
    old = hip.bidmat_get_option(b"seglen")
    hip_abi.check(hip.bidmat_set_option(b"seglen", seglen))
    try:
        for beta in (0, 1):
            d = Dev(A=A, B=B, v=v, ir=ir, jc=jc, C1=C0, C2=C0)
            d.zeros("Q1", max(nnz, 1))
            d.put("Q2", np.full(max(nnz, 1), -5.0, np.float32))
            hip_abi.check(hip.bidmat_dds_csc_op(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, d.Q1.ptr, None))
            hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, nnz, d.A.ptr, d.Q1.ptr, d.ir.ptr, d.jc.ptr, d.C1.ptr, beta, None))
            hip_abi.check(hip.bidmat_dds_dsmult_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV,
                                                    d.Q2.ptr, d.C2.ptr, beta, None), "column chain")
            hip_abi.check(hip.bidmat_synchronize())
            assert np.array_equal(d.Q2.numpy()[:nnz].view(np.uint32), d.Q1.numpy()[:nnz].view(np.uint32))
            assert np.array_equal(d.C2.numpy().view(np.uint32), d.C1.numpy().view(np.uint32)), "beta %d" % beta
            # without the products, and in place (Q == V)
            d.put("C3", C0)
            hip_abi.check(hip.bidmat_dds_dsmult_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV,
                                                    None, d.C3.ptr, beta, None))
            hip_abi.check(hip.bidmat_synchronize())
            assert np.array_equal(d.C3.numpy().view(np.uint32), d.C1.numpy().view(np.uint32))
            d.put("C4", C0)
            hip_abi.check(hip.bidmat_dds_dsmult_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV,
                                                    d.v.ptr, d.C4.ptr, beta, None))
            hip_abi.check(hip.bidmat_synchronize())
            assert np.array_equal(d.C4.numpy().view(np.uint32), d.C1.numpy().view(np.uint32))
            assert np.array_equal(d.v.numpy()[:nnz].view(np.uint32), d.Q1.numpy()[:nnz].view(np.uint32))
            d.free()
    finally:
        hip_abi.check(hip.bidmat_set_option(b"seglen", old))


def test_column_chain_against_the_oracle_and_refusals(hip):
    rng = np.random.default_rng(78)
    k, nrows, ncols = 48, 200, 300
    ir, jc = zipf_csc(rng, nrows, ncols, 15)
    nnz = ir.size
    A = (0.01 + rng.random(k * nrows)).astype(np.float32)
    B = (0.01 + rng.random(k * ncols)).astype(np.float32)
    v = rng.gamma(1.0, 1.0, size=nnz).astype(np.float32)
    d = Dev(A=A, B=B, v=v, ir=ir, jc=jc)
    d.zeros("Q", nnz), d.zeros("C", k * ncols)
    hip_abi.check(hip.bidmat_dds_dsmult_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, d.Q.ptr, d.C.ptr, 0, None))
    hip_abi.check(hip.bidmat_synchronize())
    q32 = (v / oracle.dds(A, B, k, ir, jc)[0]).astype(np.float32)
    assert np.allclose(d.Q.numpy(), q32, rtol=2e-5, atol=0)
    ref64, sa = oracle.fsmult_f64(A, k, q32, ir, jc)
    ok, worst = oracle.within_tolerance(d.C.numpy(), ref64, sa, 1e-4)
    assert ok, worst
    # refusals: an op code outside the table, products that overlap the values at another offset, k beyond one pass
    assert hip.bidmat_dds_dsmult_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, 15, None, d.C.ptr, 0, None) == 1
    assert hip.bidmat_dds_dsmult_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, d.v.ptr + 4, d.C.ptr, 0, None) == 1
    assert hip.bidmat_dds_dsmult_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, None, d.C.ptr, 2, None) == 1
    d.free()
    k = 1028
    d = Dev(A=rng.random(k * nrows).astype(np.float32), B=rng.random(k * ncols).astype(np.float32), v=v, ir=ir, jc=jc)
    d.zeros("C", k * ncols)
    assert hip.bidmat_dds_dsmult_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, None, d.C.ptr, 0, None) == 1
    d.free()


# ------------------------------------------------------------------ the chain by columns through a plan
@pytest.mark.parametrize("k,nrows,ncols,mean_len", [(32, 300, 500, 20), (64, 2000, 3000, 30), (100, 2000, 3000, 30), (128, 3000, 5000, 60),
                                                    (256, 5000, 20000, 60), (250, 300, 500, 20), (512, 1000, 2000, 40), (1024, 500, 1000, 40)])
@pytest.mark.parametrize("classes,phases", [(1, 2), (1, 4), (1, 8), (1, 1), (0, 2)], ids=["2passes", "4passes", "8passes", "1pass", "no_class_order"])
def test_column_chain_through_a_plan_has_the_bits_of_the_two_plan_calls(hip, k, nrows, ncols, mean_len, classes, phases):
    """bidmat_dds_dsmult_plan against bidmat_dds_plan (with the op) + bidmat_dsmult_plan on the same plan: Q and C bit for bit,
    whether the plan has a class order (then both forms add a column's terms pass by pass, class by class) or not."""
    rng = np.random.default_rng(3000 * k + nrows + phases)
    ir, jc = zipf_csc(rng, nrows, ncols, mean_len)
    nnz = ir.size
    A = (0.01 + rng.random(k * nrows)).astype(np.float32)
    B = (0.01 + rng.random(k * ncols)).astype(np.float32)
    v = rng.gamma(1.0, 1.0, size=nnz).astype(np.float32)
    C0 = rng.standard_normal(k * ncols).astype(np.float32)
    old = {n: hip.bidmat_get_option(n) for n in (b"col_classes", b"class_phases", b"class_hot")}
    hip_abi.check(hip.bidmat_set_option(b"col_classes", classes))
    hip_abi.check(hip.bidmat_set_option(b"class_phases", phases))
    hip_abi.check(hip.bidmat_set_option(b"class_hot", 0))        # no hot-row ranks in the class order: the passes apply for every k
    try:
        d = Dev(A=A, B=B, v=v, ir=ir, jc=jc)
        plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
        assert int(hip.bidmat_plan_info(plan, b"col_classes")) == (8 if classes else 0)
        for beta in (0, 1):
            d.put("C1", C0); d.put("C2", C0); d.put("C3", C0)
            d.zeros("Q1", max(nnz, 1))
            d.put("Q2", np.full(max(nnz, 1), -5.0, np.float32))
            hip_abi.check(hip.bidmat_dds_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, d.Q1.ptr, 0, None))
            hip_abi.check(hip.bidmat_dsmult_plan(plan, k, d.A.ptr, d.Q1.ptr, d.ir.ptr, d.jc.ptr, d.C1.ptr, beta, None))
            hip_abi.check(hip.bidmat_dds_dsmult_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, d.Q2.ptr,
                                                     d.C2.ptr, beta, None), "column chain through the plan")
            hip_abi.check(hip.bidmat_dds_dsmult_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, None,
                                                     d.C3.ptr, beta, None), "without the products")
            hip_abi.check(hip.bidmat_synchronize())
            assert np.array_equal(d.Q2.numpy()[:nnz].view(np.uint32), d.Q1.numpy()[:nnz].view(np.uint32)), "Q, beta %d" % beta
            assert np.array_equal(d.C2.numpy().view(np.uint32), d.C1.numpy().view(np.uint32)), "C, beta %d" % beta
            assert np.array_equal(d.C3.numpy().view(np.uint32), d.C1.numpy().view(np.uint32)), "C without Q, beta %d" % beta
        # in place (Q == V), then against the oracle
        vq = d.put("vq", v)
        d.zeros("C4", k * ncols)
        hip_abi.check(hip.bidmat_dds_dsmult_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, vq.ptr, OP_DIV, vq.ptr, d.C4.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
        assert np.array_equal(vq.numpy()[:nnz].view(np.uint32), d.Q1.numpy()[:nnz].view(np.uint32))
        q32 = d.Q1.numpy()[:nnz]
        ref64, sa = oracle.fsmult_f64(A, k, q32, ir, jc, nthreads=8)
        ok, worst = oracle.within_tolerance(d.C4.numpy(), ref64, sa, 1e-4)
        assert ok, worst
        r32 = oracle.dds(A, B, k, ir, jc, nthreads=8)[0]
        assert np.allclose(q32, v / r32, rtol=2e-5, atol=0)
        # refusals: a plan without a column side, an op code outside the table, overlapping V and Q, k beyond one pass
        assert hip.bidmat_dds_dsmult_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, 15, None, d.C4.ptr, 0, None) == 1
        if nnz > 1:
            assert hip.bidmat_dds_dsmult_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, d.v.ptr + 4, d.C4.ptr, 0, None) == 1
        hip_abi.check(hip.bidmat_plan_destroy(plan))
        d.free()
    finally:
        for n, val in old.items():
            hip_abi.check(hip.bidmat_set_option(n, val))


def test_column_chain_through_a_plan_with_long_columns_and_refusals(hip):
    """Columns longer than a wave segment (the plan's table of extra segments, no passes) and k beyond one pass."""
    rng = np.random.default_rng(91)
    k, nrows, ncols = 64, 3000, 200
    ir, jc = zipf_csc(rng, nrows, ncols, 400)
    nnz = ir.size
    A = (0.01 + rng.random(k * nrows)).astype(np.float32)
    B = (0.01 + rng.random(k * ncols)).astype(np.float32)
    v = rng.gamma(1.0, 1.0, size=nnz).astype(np.float32)
    old = {n: hip.bidmat_get_option(n) for n in (b"seglen", b"col_classes")}
    hip_abi.check(hip.bidmat_set_option(b"seglen", 64))
    hip_abi.check(hip.bidmat_set_option(b"col_classes", 0))
    try:
        d = Dev(A=A, B=B, v=v, ir=ir, jc=jc)
        d.zeros("Q1", nnz); d.zeros("Q2", nnz); d.zeros("C1", k * ncols); d.zeros("C2", k * ncols)
        plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
        assert hip.bidmat_plan_overflow_segments(plan) > 0
        hip_abi.check(hip.bidmat_dds_dsmult_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, d.Q1.ptr, d.C1.ptr, 0, None))
        hip_abi.check(hip.bidmat_dds_dsmult_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, d.Q2.ptr, d.C2.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
        assert np.array_equal(d.Q2.numpy().view(np.uint32), d.Q1.numpy().view(np.uint32))
        assert np.array_equal(d.C2.numpy().view(np.uint32), d.C1.numpy().view(np.uint32))
        hip_abi.check(hip.bidmat_plan_destroy(plan))
        # k beyond one pass
        d.free()
        kk = 1028
        d = Dev(A=rng.random(kk * nrows).astype(np.float32), B=rng.random(kk * ncols).astype(np.float32), v=v, ir=ir, jc=jc)
        d.zeros("C", kk * ncols)
        plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, kk)
        assert hip.bidmat_dds_dsmult_plan(plan, kk, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, OP_DIV, None, d.C.ptr, 0, None) == 1
        hip_abi.check(hip.bidmat_plan_destroy(plan))
        d.free()
    finally:
        for n, val in old.items():
            hip_abi.check(hip.bidmat_set_option(n, val))
