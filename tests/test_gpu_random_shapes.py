"""Randomised shapes: k, matrix sizes, column-length distributions and the library's split
thresholds are drawn at random (seeded) and every product is checked against the fp64 arbiter
of the oracle. Catches shape-dependent indexing mistakes that fixed-size tests miss."""
import numpy as np
import pytest

import oracle
from bidmat_amd import hip_abi
from util import Dev, make_plan, random_csc

pytestmark = pytest.mark.gpu


def close(x, ref64, sa, what):
    ok, worst = oracle.within_tolerance(x, ref64, sa, 1e-4)
    assert ok, "%s: worst error measure %.3e" % (what, worst)


@pytest.mark.parametrize("seed", range(24))
def test_random_case(hip, seed):
    rng = np.random.default_rng(9000 + seed)
    k = int(rng.choice([1, 2, 5, 8, 12, 31, 32, 48, 64, 96, 127, 128, 192, 255, 256, 320, 384, 500, 768, 1000, 1536, 2050]))
    nrows = int(rng.integers(1, 400))
    ncols = int(rng.integers(1, 300))
    style = seed % 4
    if style == 0:
        lengths = rng.binomial(nrows, rng.uniform(0.01, 0.5), size=ncols)
    elif style == 1:                                      # power-law column lengths
        lengths = np.minimum((rng.pareto(1.2, size=ncols) * 3).astype(np.int64), 2000)
    elif style == 2:                                      # mostly empty
        lengths = (rng.random(ncols) < 0.1) * rng.integers(1, 50, size=ncols)
    else:                                                 # one giant column
        lengths = rng.integers(0, 5, size=ncols)
        lengths[rng.integers(0, ncols)] = 3000
    unique = bool(style == 0)
    if unique:
        lengths = np.minimum(lengths, nrows)
    data, ir, jc = random_csc(rng, nrows, ncols, lengths=lengths, sort_rows=bool(seed % 2), unique=unique)
    if ir.size and seed % 3 == 0:                         # a dominant row
        ir[rng.random(ir.size) < 0.4] = int(rng.integers(0, nrows))
    nnz = int(ir.size)
    seglen = int(rng.choice([64, 100, 256, 1024]))
    panel_kb = int(rng.choice([16, 64, 3072]))
    heavy_min = int(rng.choice([1, 4, 8]))
    olds = [(n, hip.bidmat_get_option(n.encode())) for n in ("seglen", "panel_kb", "heavy_min")]
    for n, v in (("seglen", seglen), ("panel_kb", panel_kb), ("heavy_min", heavy_min)):
        hip_abi.check(hip.bidmat_set_option(n.encode(), v))
    try:
        A = rng.standard_normal(k * nrows).astype(np.float32)
        B = rng.standard_normal(k * ncols).astype(np.float32)
        d = Dev(A=A, B=B, data=data, ir=ir, jc=jc)
        d.zeros("AS", k * ncols), d.zeros("P", max(nnz, 1)), d.zeros("BSt", k * nrows)
        d.zeros("cs", ncols), d.zeros("rs", nrows)
        plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
        hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, nnz, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr, d.AS.ptr, 0, None))
        hip_abi.check(hip.bidmat_dds_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.P.ptr, 0, None))
        hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.B.ptr, d.data.ptr, d.BSt.ptr, 0, None))
        hip_abi.check(hip.bidmat_spsum_cols(ncols, nnz, d.data.ptr, d.jc.ptr, d.cs.ptr, 0, None))
        hip_abi.check(hip.bidmat_spsum_rows_plan(plan, d.data.ptr, d.rs.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
        tag = "seed=%d k=%d %dx%d nnz=%d seglen=%d panel=%d heavy=%d" % (seed, k, nrows, ncols, nnz, seglen, panel_kb, heavy_min)
        close(d.AS.numpy(), *oracle.fsmult_f64(A, k, data, ir, jc), "A*S " + tag)
        if nnz:
            close(d.P.numpy(nnz), *oracle.dds_f64(A, B, k, ir, jc), "DDS " + tag)
        close(d.BSt.numpy(), *oracle.fsmultT_f64(B, k, nrows, data, ir, jc), "A*^S " + tag)
        close(d.cs.numpy(), *oracle.spsum_f64(nrows, data, ir, jc, 1), "colsum " + tag)
        close(d.rs.numpy(), *oracle.spsum_f64(nrows, data, ir, jc, 2), "rowsum " + tag)
        hip_abi.check(hip.bidmat_plan_destroy(plan))
        d.free()
    finally:
        for n, v in olds:
            hip_abi.check(hip.bidmat_set_option(n.encode(), v))


@pytest.mark.parametrize("seed", range(8))
def test_random_medium_case(hip, seed):
    """Thousands of columns and rows: several workgroups in the overflow table, plans with many
    panels (a multiple of 8 of them) and segment lengths adapted to the pattern size."""
    rng = np.random.default_rng(9500 + seed)
    k = int(rng.choice([32, 100, 128, 256, 512]))
    nrows = int(rng.integers(500, 6000))
    ncols = int(rng.integers(2000, 30000))
    lengths = rng.poisson(rng.uniform(2, 25), size=ncols).astype(np.int64)
    for c in rng.integers(0, ncols, size=5):              # a few long columns
        lengths[c] = int(rng.integers(1500, 6000))
    jc = np.zeros(ncols + 1, dtype=np.int32)
    jc[1:] = np.cumsum(lengths)
    nnz = int(jc[-1])
    # Zipf-like rows (repeats inside a column allowed), unsorted for odd seeds
    w = 1.0 / np.arange(1, nrows + 1) ** rng.uniform(0.8, 1.3)
    ir = rng.choice(nrows, size=nnz, p=w / w.sum()).astype(np.int32)
    if seed % 2 == 0:
        ic = np.repeat(np.arange(ncols), lengths)
        ir = ir[np.lexsort((ir, ic))]
    data = (1.0 - rng.random(nnz)).astype(np.float32)
    seglen = int(rng.choice([64, 256, 1024]))
    panel_kb = int(rng.choice([16, 256, 3072]))
    heavy_min = int(rng.choice([1, 8]))
    olds = [(n, hip.bidmat_get_option(n.encode())) for n in ("seglen", "panel_kb", "heavy_min")]
    for n, v in (("seglen", seglen), ("panel_kb", panel_kb), ("heavy_min", heavy_min)):
        hip_abi.check(hip.bidmat_set_option(n.encode(), v))
    try:
        A = rng.standard_normal(k * nrows).astype(np.float32)
        B = rng.standard_normal(k * ncols).astype(np.float32)
        d = Dev(A=A, B=B, data=data, ir=ir, jc=jc)
        d.zeros("AS", k * ncols), d.zeros("P", nnz), d.zeros("BSt", k * nrows)
        d.zeros("cs", ncols), d.zeros("rs", nrows)
        plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
        hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, nnz, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr, d.AS.ptr, 0, None))
        hip_abi.check(hip.bidmat_dds_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.P.ptr, 0, None))
        hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.B.ptr, d.data.ptr, d.BSt.ptr, 0, None))
        hip_abi.check(hip.bidmat_spsum_cols(ncols, nnz, d.data.ptr, d.jc.ptr, d.cs.ptr, 0, None))
        hip_abi.check(hip.bidmat_spsum_rows_plan(plan, d.data.ptr, d.rs.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
        tag = "seed=%d k=%d %dx%d nnz=%d seglen=%d panel=%d heavy=%d" % (seed, k, nrows, ncols, nnz, seglen, panel_kb, heavy_min)
        close(d.AS.numpy(), *oracle.fsmult_f64(A, k, data, ir, jc), "A*S " + tag)
        close(d.P.numpy(nnz), *oracle.dds_f64(A, B, k, ir, jc), "DDS " + tag)
        close(d.BSt.numpy(), *oracle.fsmultT_f64(B, k, nrows, data, ir, jc), "A*^S " + tag)
        close(d.cs.numpy(), *oracle.spsum_f64(nrows, data, ir, jc, 1), "colsum " + tag)
        close(d.rs.numpy(), *oracle.spsum_f64(nrows, data, ir, jc, 2), "rowsum " + tag)
        hip_abi.check(hip.bidmat_plan_destroy(plan))
        d.free()
    finally:
        for n, v in olds:
            hip_abi.check(hip.bidmat_set_option(n.encode(), v))
