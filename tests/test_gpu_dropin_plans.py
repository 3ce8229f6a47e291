"""What unchanged call sites get on a pattern they use again: the reference-shaped bidmat_dds /
bidmat_dsmult (CUMAT.java:143,211) find the pattern in the fingerprint cache and run through the
column side of a cached plan from their second call on; the operator mirror (GMat.GSMult / madd,
GSMat.DDS: GMat.scala:1041-1074, GSMat.scala:649-667) does the same with the plan of the GSMat, and
a DDS result points at the index arrays of its third operand instead of copying them. Every form must
give what the plain kernels give: DDS bit for bit, A*S within the tolerance of the path (the class
order adds a column's terms in another, fixed, order).
"""
import ctypes as C
import threading

import numpy as np
import pytest

import oracle
from bidmat_amd import hip_abi
from bidmat_amd.device import DeviceArray
from bidmat_amd.mats import DDS, GMat, GSMat
from util import Dev, expand_cols, make_plan, random_csc

pytestmark = pytest.mark.gpu
RTOL = 1e-4


def close(x, ref64, sa, what):
    ok, worst = oracle.within_tolerance(x, ref64, sa, RTOL)
    assert ok, "%s: worst error measure %.3e" % (what, worst)


class Options:
    """Sets library options for a block and restores them."""

    def __init__(self, hip, **opts):
        self.hip, self.opts, self.old = hip, opts, {}

    def __enter__(self):
        for k, v in self.opts.items():
            self.old[k] = self.hip.bidmat_get_option(k.encode())
            hip_abi.check(self.hip.bidmat_set_option(k.encode(), v), k)
        return self

    def __exit__(self, *a):
        for k, v in self.old.items():
            hip_abi.check(self.hip.bidmat_set_option(k.encode(), v), k)


def zipf_pattern(rng, nrows, ncols, lo, hi, long_cols=()):
    """Columns of lo..hi nonzeros whose rows favour small indices (so that a class ordering has hot rows)."""
    lengths = rng.integers(lo, hi, size=ncols)
    for c, n in long_cols:
        lengths[c] = n
    jc = np.zeros(ncols + 1, dtype=np.int32)
    jc[1:] = np.cumsum(lengths)
    p = 1.0 / np.arange(1, nrows + 1) ** 1.1
    p /= p.sum()
    ir = rng.choice(nrows, size=int(jc[-1]), p=p).astype(np.int32)        # unsorted, repeats allowed
    data = (1.0 - rng.random(ir.size)).astype(np.float32)
    return data, ir, jc


@pytest.mark.parametrize("k,classes,long_cols", [(256, 1, ()), (64, 1, ((3, 700), (250, 129))), (100, 0, ((17, 900),)), (32, -1, ())])
def test_reference_shaped_dds_and_dsmult_through_the_cached_column_side(hip, k, classes, long_cols):
    """Five calls each of bidmat_dds and bidmat_dsmult on one pattern: the first runs the plain kernel,
    the second builds the column side of the cached plan, the others reuse it. Then the SAME device
    buffers are refilled with another pattern of equal size: no stale plan may be used."""
    rng = np.random.default_rng(100 + k)
    nrows, ncols = 700, 333
    hip_abi.check(hip.bidmat_release_caches())
    with Options(hip, col_classes=classes, seglen=128, cache_cols_after=2):
        data, ir, jc = zipf_pattern(rng, nrows, ncols, 0, 60, long_cols)
        nnz = int(ir.size)
        ic = expand_cols(jc)
        A = rng.standard_normal(k * nrows).astype(np.float32)
        B = rng.standard_normal(k * ncols).astype(np.float32)
        d = Dev(A=A, B=B, data=data, ir=ir, ic=ic, jc=jc)
        plain_P, plain_C = DeviceArray.zeros(nnz), DeviceArray.zeros(k * ncols)
        hip_abi.check(hip.bidmat_dds_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, plain_P.ptr, 0, None))
        hip_abi.check(hip.bidmat_dsmult_csc(k, ncols, nnz, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr, plain_C.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
        want_P = plain_P.numpy()
        ref64, sa = oracle.fsmult_f64(A, k, data, ir, jc)
        Cs = []
        for call in range(5):
            P, Cm = DeviceArray.zeros(nnz), DeviceArray.zeros(k * ncols)
            hip_abi.check(hip.bidmat_dds(k, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.ic.ptr, P.ptr), "dds call %d" % call)
            assert np.array_equal(P.numpy(), want_P), "bidmat_dds call %d differs from the plain kernel" % call
            hip_abi.check(hip.bidmat_dsmult(k, ncols, nnz, d.A.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, Cm.ptr), "dsmult call %d" % call)
            Cs.append(Cm.numpy())
            close(Cs[-1], ref64, sa, "bidmat_dsmult call %d" % call)
            P.free(); Cm.free()
        # (bidmat_dds came first, so the first bidmat_dsmult is already the pattern's second column-side use)
        for c in Cs[1:]:
            assert np.array_equal(Cs[0], c)                    # the plan's order is fixed
        if classes != 1:
            assert np.array_equal(Cs[0], plain_C.numpy())      # no class ordering: the plain kernel's order
        # accumulate semantics through the plan: a second call on the same output doubles it (not to the
        # bit: passes over the row classes and the segments of long columns add their shares one after the other)
        Cm = DeviceArray.zeros(k * ncols)
        for _ in range(2):
            hip_abi.check(hip.bidmat_dsmult(k, ncols, nnz, d.A.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, Cm.ptr))
        close(Cm.numpy(), 2 * ref64, 2 * sa, "bidmat_dsmult twice into one output")
        # the same buffers, another pattern with the same column lengths: a stale plan would give garbage
        ir2 = rng.permutation(ir).astype(np.int32)
        ir2[0] = ir.max()                                      # same largest row: same size key
        hip_abi.check(hip.bidmat_memcpy_h2d(d.ir.ptr, ir2.ctypes.data, ir2.nbytes))
        hip_abi.check(hip.bidmat_dds_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, plain_P.ptr, 0, None))
        hip_abi.check(hip.bidmat_synchronize())
        ref64, sa = oracle.fsmult_f64(A, k, data, ir2, jc)
        for call in range(3):
            P, Cm = DeviceArray.zeros(nnz), DeviceArray.zeros(k * ncols)
            hip_abi.check(hip.bidmat_dds(k, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.ic.ptr, P.ptr))
            assert np.array_equal(P.numpy(), plain_P.numpy()), "refilled buffers, call %d" % call
            hip_abi.check(hip.bidmat_dsmult(k, ncols, nnz, d.A.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, Cm.ptr))
            close(Cm.numpy(), ref64, sa, "bidmat_dsmult on refilled buffers, call %d" % call)
            P.free(); Cm.free()
        # A*^S on the same entry afterwards: the row side is added to the cached plan
        AT = rng.standard_normal(k * ncols).astype(np.float32)
        dAT, G = DeviceArray.from_numpy(AT), DeviceArray.zeros(k * nrows)
        hip_abi.check(hip.bidmat_dsmultT(k, ncols, nnz, dAT.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, G.ptr), "dsmultT")
        r64, rsa = oracle.fsmultT_f64(AT, k, nrows, data, ir2, jc)
        close(G.numpy(), r64, rsa, "bidmat_dsmultT after the column side was cached")
        d.free()
    hip_abi.check(hip.bidmat_release_caches())


def test_reference_shaped_entries_without_the_cache(hip):
    """cache_cols_after = 0: bidmat_dds / bidmat_dsmult never look a plan up (no digest pass)."""
    rng = np.random.default_rng(7)
    k, nrows, ncols = 48, 90, 200
    data, ir, jc = random_csc(rng, nrows, ncols, lengths=rng.integers(0, 9, size=ncols))
    nnz, ic = int(ir.size), expand_cols(jc)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    B = rng.standard_normal(k * ncols).astype(np.float32)
    d = Dev(A=A, B=B, data=data, ir=ir, ic=ic, jc=jc)
    with Options(hip, cache_cols_after=0):
        for _ in range(3):
            P, Cm = DeviceArray.zeros(nnz), DeviceArray.zeros(k * ncols)
            hip_abi.check(hip.bidmat_dds(k, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.ic.ptr, P.ptr))
            hip_abi.check(hip.bidmat_dsmult(k, ncols, nnz, d.A.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, Cm.ptr))
            r64, sa = oracle.dds_f64(A, B, k, ir, jc)
            close(P.numpy(), r64, sa, "dds")
            r64, sa = oracle.fsmult_f64(A, k, data, ir, jc)
            close(Cm.numpy(), r64, sa, "dsmult")
    assert hip.bidmat_set_option(b"cache_cols_after", -1) == 1
    assert hip.bidmat_set_option(b"cache_plans", 0) == 1
    d.free()


def test_fingerprint_pass_also_builds_the_column_pointer(hip):
    """The digest pass derives jc from ic on the way: empty leading / trailing / inner columns."""
    rng = np.random.default_rng(8)
    k, nrows = 16, 40
    for lengths in ([0, 0, 3, 0, 5, 0, 0], [2], [0], [4, 0, 0, 0], [0, 0, 0, 1]):
        ncols = len(lengths)
        data, ir, jc = random_csc(rng, nrows, ncols, lengths=np.array(lengths))
        nnz = int(ir.size)
        if nnz == 0:
            continue
        ic = expand_cols(jc)
        A = rng.standard_normal(k * nrows).astype(np.float32)
        d = Dev(A=A, data=data, ir=ir, ic=ic)
        Cm = DeviceArray.zeros(k * ncols)
        hip_abi.check(hip.bidmat_dsmult(k, ncols, nnz, d.A.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, Cm.ptr))
        r64, sa = oracle.fsmult_f64(A, k, data, ir, jc)
        close(Cm.numpy(), r64, sa, "dsmult lengths=%s" % lengths)
        d.free()
    hip_abi.check(hip.bidmat_release_caches())


def test_operator_mirror_uses_the_plan_from_the_second_product_on(hip):
    """GMat * GSMat and DDS through libbidmathost: no plan after one product, a plan after two; DDS gives
    the same bits either way and its result points at the index arrays of the pattern operand; a matrix
    whose indices are rewritten afterwards takes private arrays and leaves the other one intact."""
    rng = np.random.default_rng(9)
    k, nrows, ncols = 64, 400, 300
    hip_abi.check(hip.bidmat_set_option(b"col_classes", 1))
    try:
        # sorted, distinct rows inside every column (a host SMat is checked on the way in and out)
        cols = [np.sort(rng.choice(nrows, size=int(rng.integers(1, 40)), replace=False)) for _ in range(ncols)]
        ir = np.concatenate(cols).astype(np.int32)
        jc = np.zeros(ncols + 1, dtype=np.int32)
        jc[1:] = np.cumsum([c.size for c in cols])
        data = (1.0 - rng.random(ir.size)).astype(np.float32)
        S = GSMat.from_csc(nrows, ncols, data, ir + 1, jc + 1)
        A = rng.standard_normal((k, nrows)).astype(np.float32)
        B = rng.standard_normal((k, ncols)).astype(np.float32)
        gA, gB = GMat.from_numpy(A), GMat.from_numpy(B)
        Af, Bf = A.ravel(order="F"), B.ravel(order="F")        # column-major, as the oracle takes them
        assert not S.has_plan()
        P1 = DDS(gA, gB, S)
        assert P1.same_pattern(S) and not S.has_plan()
        C1 = gA * S
        assert S.has_plan()                                  # the second product on the pattern built it
        P2 = DDS(gA, gB, S)
        C2 = gA * S
        C3 = gA * S
        v1, v2 = P1.to_csc()[0], P2.to_csc()[0]
        assert np.array_equal(v1, v2)
        r64, sa = oracle.dds_f64(Af, Bf, k, ir, jc)
        close(v1, r64, sa, "mirror DDS")
        r64, sa = oracle.fsmult_f64(Af, k, data, ir, jc)
        for name, Cx in (("first", C1), ("second", C2), ("third", C3)):
            close(Cx.numpy().ravel(order="F"), r64, sa, "mirror A*S, %s call" % name)
        assert np.array_equal(C2.numpy(), C3.numpy())
        # the result of DDS carries the column pointer too
        assert np.array_equal(P2.device_jc(), jc)
        # rewrite P2's indices (transpose of S into it): S must stay what it was
        St = S.t(out=None)
        assert not St.same_pattern(S)
        back = S.to_csc()
        assert np.array_equal(back[1], ir + 1) and np.array_equal(back[2], jc + 1) and np.array_equal(back[0], data)
        Q = P1.colslice(0, ncols)                            # a new matrix: private arrays
        assert not Q.same_pattern(S)
        assert np.array_equal(Q.to_csc()[1], ir + 1)
        # madd accumulates through the plan as well
        out = GMat.from_numpy(C3.numpy().copy())
        gA.madd(S, out)
        np.testing.assert_array_equal(out.numpy(), 2 * C3.numpy())
    finally:
        hip_abi.check(hip.bidmat_set_option(b"col_classes", -1))


def test_fused_step_in_place_and_overlapping_operands(hip):
    """P == V (the in-place update) is allowed while one pass covers k and refused beyond; a V that
    overlaps P at another offset is always refused."""
    rng = np.random.default_rng(11)
    nrows, ncols = 60, 50
    data, ir, jc = random_csc(rng, nrows, ncols, lengths=rng.integers(1, 12, size=ncols))
    nnz = int(ir.size)
    for k, ok in ((128, True), (1024, True), (2052, False), (1100, False)):
        A = rng.random(k * nrows).astype(np.float32) + 0.1
        B = rng.random(k * ncols).astype(np.float32) + 0.1
        V = rng.random(nnz + 8).astype(np.float32) + 0.5
        d = Dev(A=A, B=B, ir=ir, jc=jc, V=V)
        want = DeviceArray.zeros(nnz)
        hip_abi.check(hip.bidmat_dds_csc_op(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.V.ptr, 3, want.ptr, None))
        hip_abi.check(hip.bidmat_synchronize())
        plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
        # partial overlap: P starts 4 floats into V
        assert hip.bidmat_dds_csc_op(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.V.ptr, 3, d.V.ptr + 16, None) == 1
        assert hip.bidmat_dds_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.V.ptr, 3, d.V.ptr + 16, 0, None) == 1
        rc = hip.bidmat_dds_csc_op(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.V.ptr, 3, d.V.ptr, None)
        hip_abi.check(hip.bidmat_synchronize())
        if ok:
            assert rc == 0
            assert np.array_equal(d.V.numpy()[:nnz], want.numpy())
            assert np.array_equal(d.V.numpy()[nnz:], V[nnz:])
        else:
            assert rc == 1
            assert np.array_equal(d.V.numpy(), V)              # refused before anything ran
            assert hip.bidmat_dds_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, d.V.ptr, 3, d.V.ptr, 0, None) == 1
        hip_abi.check(hip.bidmat_plan_destroy(plan))
        d.free()


def test_checked_mode_refuses_a_pattern_that_is_not_the_plans(hip):
    rng = np.random.default_rng(12)
    k, nrows, ncols = 32, 80, 70
    lengths = rng.integers(1, 9, size=ncols)
    data, ir, jc = random_csc(rng, nrows, ncols, lengths=lengths)
    _, ir2, _ = random_csc(rng, nrows, ncols, lengths=lengths)
    nnz = int(ir.size)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    B = rng.standard_normal(k * ncols).astype(np.float32)
    d = Dev(A=A, B=B, data=data, ir=ir, jc=jc, ir2=ir2)
    P, Cm = DeviceArray.zeros(nnz), DeviceArray.zeros(k * ncols)
    with Options(hip, check_plan=1):
        plan = make_plan(hip, nrows, ncols, nnz, d.ir, d.jc, k)
        assert hip.bidmat_dds_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, None, 0, P.ptr, 0, None) == 0
        assert hip.bidmat_dsmult_plan(plan, k, d.A.ptr, d.data.ptr, d.ir.ptr, d.jc.ptr, Cm.ptr, 0, None) == 0
        assert hip.bidmat_dds_plan(plan, k, d.A.ptr, d.B.ptr, d.ir2.ptr, d.jc.ptr, None, 0, P.ptr, 0, None) == 1
        assert hip.bidmat_dsmult_plan(plan, k, d.A.ptr, d.data.ptr, d.ir2.ptr, d.jc.ptr, Cm.ptr, 0, None) == 1
    # unchecked (the default): the caller's duty, as documented
    assert hip.bidmat_dds_plan(plan, k, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, None, 0, P.ptr, 0, None) == 0
    hip_abi.check(hip.bidmat_synchronize())
    hip_abi.check(hip.bidmat_plan_destroy(plan))
    d.free()


def test_plan_with_one_side_only_refuses_the_other(hip):
    """Cached plans are built side by side; a user's plan always has both. Through the cache: A*^S first
    (row side), then DDS twice (column side added), all correct."""
    rng = np.random.default_rng(13)
    k, nrows, ncols = 40, 120, 150
    data, ir, jc = random_csc(rng, nrows, ncols, lengths=rng.integers(0, 15, size=ncols))
    ir[0] = nrows - 1
    nnz, ic = int(ir.size), expand_cols(jc)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    B = rng.standard_normal(k * ncols).astype(np.float32)
    d = Dev(A=A, B=B, data=data, ir=ir, ic=ic)
    hip_abi.check(hip.bidmat_release_caches())
    with Options(hip, col_classes=1):
        G = DeviceArray.zeros(k * nrows)
        hip_abi.check(hip.bidmat_dsmultT(k, ncols, nnz, d.B.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, G.ptr))
        r64, sa = oracle.fsmultT_f64(B, k, nrows, data, ir, jc)
        close(G.numpy(), r64, sa, "dsmultT")
        r64, sa = oracle.dds_f64(A, B, k, ir, jc)
        for _ in range(3):
            P = DeviceArray.zeros(nnz)
            hip_abi.check(hip.bidmat_dds(k, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.ic.ptr, P.ptr))
            close(P.numpy(), r64, sa, "dds")
        G2 = DeviceArray.zeros(k * nrows)
        hip_abi.check(hip.bidmat_dsmultT(k, ncols, nnz, d.B.ptr, d.data.ptr, d.ir.ptr, d.ic.ptr, G2.ptr))
        assert np.array_equal(G.numpy(), G2.numpy())
    hip_abi.check(hip.bidmat_release_caches())
    d.free()


def test_static_dds_from_two_threads_on_one_stream(hip):
    """bidmat_dds_csc_static takes the device lock: two host threads that enqueue on the same stream
    cannot interleave building the table in the shared array and launching the kernel that reads it."""
    rng = np.random.default_rng(14)
    st = C.c_void_p()
    hip_abi.check(hip.bidmat_stream_create(C.byref(st)))
    jobs = []
    with Options(hip, seglen=64):
        for k, nrows, ncols, long_cols in ((64, 200, 3000, ((5, 900), (2999, 300))), (32, 100, 500, ((17, 2000),))):
            lengths = rng.integers(0, 6, size=ncols)
            for c, n in long_cols:
                lengths[c] = n
            _, ir, jc = random_csc(rng, nrows, ncols, lengths=lengths, sort_rows=False, unique=False)
            A = rng.standard_normal(k * nrows).astype(np.float32)
            B = rng.standard_normal(k * ncols).astype(np.float32)
            d = Dev(A=A, B=B, ir=ir, jc=jc)
            nnz = int(ir.size)
            want = DeviceArray.zeros(nnz)
            hip_abi.check(hip.bidmat_dds_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, want.ptr, 0, None))
            hip_abi.check(hip.bidmat_synchronize())
            jobs.append(dict(k=k, ncols=ncols, nnz=nnz, d=d, want=want.numpy(), outs=[DeviceArray.zeros(nnz) for _ in range(20)]))
        errors = []

        def worker(j):
            try:
                hip_abi.check(hip.bidmat_set_device(0))
                d = j["d"]
                for o in j["outs"]:
                    hip_abi.check(hip.bidmat_dds_csc_static(j["k"], j["ncols"], j["nnz"], d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, o.ptr, 0, st))
            except Exception as e:                            # noqa: BLE001
                errors.append(repr(e))

        ts = [threading.Thread(target=worker, args=(j,)) for j in jobs]
        for t in ts:
            t.start()
        for t in ts:
            t.join()
        hip_abi.check(hip.bidmat_stream_synchronize(st))
        assert not errors, errors
        for j in jobs:
            for o in j["outs"]:
                assert np.array_equal(o.numpy(), j["want"])
            j["d"].free()
    hip_abi.check(hip.bidmat_stream_destroy(st))


def test_the_cache_goes_by_the_content_of_the_index_arrays(hip):
    """The same pattern uploaded into other device arrays is the same pattern: the second bidmat_dsmult on it runs
    through the cached plan's class order (other bits than the plain kernel's stored order), whichever arrays hold it."""
    rng = np.random.default_rng(77)
    k, nrows, ncols = 256, 900, 400                             # from k = 256 on A*S takes the class order in passes
    hip_abi.check(hip.bidmat_release_caches())
    with Options(hip, col_classes=1, cache_cols_after=2):
        data, ir, jc = zipf_pattern(rng, nrows, ncols, 20, 80)
        nnz = int(ir.size)
        ic = expand_cols(jc)
        A = rng.standard_normal(k * nrows).astype(np.float32)
        d1 = Dev(A=A, data=data, ir=ir, ic=ic)
        d2 = Dev(ir=ir, ic=ic)                                  # the same pattern at other addresses
        assert d1.ir.ptr != d2.ir.ptr and d1.ic.ptr != d2.ic.ptr
        outs = []
        for which in (d1, d2, d1, d2):
            Cm = DeviceArray.zeros(k * ncols)
            hip_abi.check(hip.bidmat_dsmult(k, ncols, nnz, d1.A.ptr, d1.data.ptr, which.ir.ptr, which.ic.ptr, Cm.ptr))
            outs.append(Cm.numpy())
            Cm.free()
        ref64, sa = oracle.fsmult_f64(A, k, data, ir, jc)
        for o in outs:
            close(o, ref64, sa, "bidmat_dsmult")
        assert not np.array_equal(outs[0], outs[1]), "the second call (other arrays, same pattern) still ran the plain kernel"
        assert np.array_equal(outs[1], outs[2]) and np.array_equal(outs[2], outs[3])
        d1.free(); d2.free()
    hip_abi.check(hip.bidmat_release_caches())
