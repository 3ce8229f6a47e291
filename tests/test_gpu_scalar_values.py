"""A *^ S over a plan with each nonzero's value fetched by a scalar load (option "scalar_values").

Where a value comes from does not change what is multiplied or the order of the additions: the results must have the
bits of the form that gathers the values lane by lane, for every k and shape of segment (full chunks of 64 nonzeros,
short tails, segments shorter than a round of 8, empty rows), and both must agree with the oracle's float64 arbiter
(reference: the product of BIDMat's dsmultT, jni/src/Arith.cu:206-248).
"""
import numpy as np
import pytest

import oracle
from bidmat_amd import hip_abi
from util import Dev, make_plan
from test_gpu_dense_rows import power_law_csc

pytestmark = pytest.mark.gpu


@pytest.fixture()
def options(hip):
    names = ("scalar_values", "dense_rows", "heavy_min", "seglen")
    before = {n: hip.bidmat_get_option(n.encode()) for n in names}
    yield hip
    for n, v in before.items():
        hip_abi.check(hip.bidmat_set_option(n.encode(), v))


def product(hip, plan, k, d, out, scalar, beta=0):
    hip_abi.check(hip.bidmat_set_option(b"scalar_values", scalar))
    hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.A.ptr, d.v.ptr, out.ptr, beta, None))
    hip_abi.check(hip.bidmat_synchronize())
    return out.numpy()


# k: every layout in which a nonzero's row takes the whole wave (1 to 4 vectors of 4 floats per lane; k % 4 != 0 takes
# one float per lane, from k = 33 on) and both sides of the limits below which the values stay with the gather
@pytest.mark.parametrize("k", [7, 32, 33, 64, 100, 128, 130, 132, 256, 300, 512, 1028])
@pytest.mark.parametrize("shape", [(700, 900, 40), (90, 3000, 25), (5000, 300, 150)], ids=["700x900", "90x3000", "5000x300"])
def test_same_bits_as_the_gathered_values(options, k, shape):
    hip = options
    nrows, ncols, mean_len = shape
    rng = np.random.default_rng(1000 * k + nrows)
    ir, jc = power_law_csc(rng, nrows, ncols, mean_len, shuffle_rows=True)
    nnz = ir.size
    A = rng.standard_normal(k * ncols).astype(np.float32)
    v = (1.0 - rng.random(nnz)).astype(np.float32)
    v[0] = np.float32(np.inf)                    # the value at position 0 must reach its own nonzero only
    c0 = int(np.searchsorted(jc, 0, side="right")) - 1          # the column of the nonzero at position 0
    A[k * c0:k * (c0 + 1)] = 0.5
    d = Dev(ir=ir, jc=jc, A=A, v=v)
    d.zeros("G1", k * nrows); d.zeros("G0", k * nrows)
    hip_abi.check(hip.bidmat_set_option(b"heavy_min", 2))       # rows cut by panels and rows in one piece
    hip_abi.check(hip.bidmat_set_option(b"seglen", 64 if k % 2 else 512))
    plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
    with_scalar = product(hip, plan, k, d, d.G1, 1)
    gathered = product(hip, plan, k, d, d.G0, 0)
    assert np.array_equal(with_scalar.view(np.uint32), gathered.view(np.uint32)), "the two ways to fetch a value differ"
    r0 = int(ir[0])
    rows = with_scalar.reshape(nrows, k)
    assert np.all(np.isinf(rows[r0])), "the infinite value belongs to row %d" % r0
    others = np.ones(nrows, bool); others[r0] = False
    assert np.all(np.isfinite(rows[others])), "a slot past the end of a segment took the value at position 0"
    v[0] = 1.0
    d.v.upload(v)
    got = product(hip, plan, k, d, d.G1, 1)
    ref64, sa = oracle.fsmultT_f64(A, k, nrows, v, ir, jc, nthreads=8)
    ok, worst = oracle.within_tolerance(got, ref64, sa, 1e-4)
    assert ok, "A *^ S with scalar loads differs from the oracle: %.3e" % worst
    twice = product(hip, plan, k, d, d.G1, 1, beta=1)
    ok2, worst2 = oracle.within_tolerance(twice, 2 * ref64, 2 * sa, 1e-4)
    assert ok2, worst2
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


def test_with_the_dense_block(options):
    """The dense rows' segments are skipped by the kernel that fetches its values by scalar loads too."""
    hip = options
    nrows, ncols, k = 2000, 3000, 256
    rng = np.random.default_rng(77)
    ir, jc = power_law_csc(rng, nrows, ncols, 120, shuffle_rows=True)
    nnz = ir.size
    A = rng.standard_normal(k * ncols).astype(np.float32)
    v = (1.0 - rng.random(nnz)).astype(np.float32)
    d = Dev(ir=ir, jc=jc, A=A, v=v)
    d.zeros("G1", k * nrows); d.zeros("G0", k * nrows)
    before = hip.bidmat_get_option(b"dense_min_nnz")
    hip_abi.check(hip.bidmat_set_option(b"dense_min_nnz", 0))
    try:
        plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
        assert int(hip.bidmat_plan_info(plan, b"dense_rows")) >= 32
        a = product(hip, plan, k, d, d.G1, 1)
        b = product(hip, plan, k, d, d.G0, 0)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        ref64, sa = oracle.fsmultT_f64(A, k, nrows, v, ir, jc, nthreads=8)
        ok, worst = oracle.within_tolerance(a, ref64, sa, 1e-4)
        assert ok, worst
        hip_abi.check(hip.bidmat_plan_destroy(plan))
    finally:
        hip_abi.check(hip.bidmat_set_option(b"dense_min_nnz", before))
    d.free()


def test_values_written_by_the_launch_before_in_a_replayed_graph(options):
    """Q = V ./ DDS(A, B, S) and G = B *^ Q recorded into one HIP graph: the scalar loads of the second product must
    see what the first wrote in the same replay (the scalar cache holds nothing over from the replay before)."""
    import ctypes as C
    hip = options
    nrows, ncols, k = 1500, 2500, 256
    rng = np.random.default_rng(31)
    ir, jc = power_law_csc(rng, nrows, ncols, 60, shuffle_rows=True)
    nnz = ir.size
    A = (0.01 + rng.random(k * nrows)).astype(np.float32)
    B = (0.01 + rng.random(k * ncols)).astype(np.float32)
    v = rng.gamma(1.0, 1.0, size=nnz).astype(np.float32)
    d = Dev(ir=ir, jc=jc, A=A, B=B, v=v)
    d.zeros("Q", nnz); d.zeros("G", k * nrows); d.zeros("Q2", nnz); d.zeros("G2", k * nrows)
    plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
    st = C.c_void_p()
    hip_abi.check(hip.bidmat_stream_create(C.byref(st)))

    def chain(q, g, stream):
        hip_abi.check(hip.bidmat_dds_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.v.ptr, 3, q.ptr, 0, stream))
        hip_abi.check(hip.bidmat_dsmultT_plan(plan, k, d.B.ptr, q.ptr, g.ptr, 0, stream))

    chain(d.Q, d.G, st)                                   # sizes the stream's scratch
    hip_abi.check(hip.bidmat_stream_synchronize(st))
    hip_abi.check(hip.bidmat_graph_begin_capture(st))
    chain(d.Q, d.G, st)
    gx = C.c_void_p()
    hip_abi.check(hip.bidmat_graph_end_capture(st, C.byref(gx)))
    for rep in range(4):
        newv = rng.gamma(1.0, 1.0, size=nnz).astype(np.float32)
        d.v.upload(newv)
        hip_abi.check(hip.bidmat_memset(d.G.ptr, 0xFF, d.G.nbytes))
        hip_abi.check(hip.bidmat_graph_launch(gx, st))
        hip_abi.check(hip.bidmat_stream_synchronize(st))
        hip_abi.check(hip.bidmat_set_option(b"scalar_values", 0))
        chain(d.Q2, d.G2, None)
        hip_abi.check(hip.bidmat_synchronize())
        hip_abi.check(hip.bidmat_set_option(b"scalar_values", 1))
        assert np.array_equal(d.Q.numpy().view(np.int32), d.Q2.numpy().view(np.int32)), "replay %d, Q" % rep
        assert np.array_equal(d.G.numpy().view(np.int32), d.G2.numpy().view(np.int32)), "replay %d, G" % rep
    hip_abi.check(hip.bidmat_graph_destroy(gx))
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    hip_abi.check(hip.bidmat_stream_destroy(st))
    d.free()
