"""The host-side mirror of BIDMat's GMat / GSMat operator interface, exercised the way the
reference's own tests do (src/test/scala/BIDMat/GSMatTest.scala, GMatTest.scala): random
inputs at nr=10, nc=20, nk=30, results compared with a dense computation at eps 1e-4,
result types checked, SparseMat.check on sparse results. Host arrays are 1-based
(Mat.ioneBased = 1, the reference's default).
"""
import numpy as np
import pytest

import oracle
from bidmat_amd import mats
from bidmat_amd.mats import DDS, GMat, GSMat, Mat
from util import dense_full, random_csc

nr, nc, nk = 10, 20, 30
EPS = 1e-4


def sprand(rng, m, n, density):
    """Host SMat arrays with the reference's default 1-based indices."""
    data, ir, jc = random_csc(rng, m, n, density)
    return data, ir + 1, jc + 1


def full(m, n, data, ir, jc):
    return dense_full(m, n, data, ir - 1, jc - 1)


# ----------------------------------------------------------------------- no GPU needed
def test_sparse_check_messages():
    mats.smat_check(4, 3, np.array([1, 3, 2, 4]), np.array([1, 3, 3, 5]))
    for ir, jc, msg in [
        ([1, 3, 2, 4], [0, 3, 3, 5], "jc(0) should be 1"),
        ([1, 2, 3, 4], [1, 4, 3, 5], "jc(i) out of order"),
        ([3, 1, 2, 4], [1, 3, 3, 5], "ir(j) out of order"),
        ([1, 9, 2, 4], [1, 3, 3, 5], "out of range"),
        ([1, 3, 2, 4], [1, 3, 3, 4], "jc(ncols) should be"),
    ]:
        with pytest.raises(RuntimeError, match=msg.replace("(", r"\(").replace(")", r"\)")):
            mats.smat_check(4, 3, np.array(ir), np.array(jc))


def test_flags_default_to_the_reference_values():
    assert Mat.get("ioneBased") == 1 and Mat.get("recycleGrow") == pytest.approx(1.2)
    assert Mat.get("useGPUcache") == 0
    with pytest.raises(KeyError):
        Mat.set("noSuchFlag", 1)


# ----------------------------------------------------------------------- GPU
gpu = pytest.mark.gpu


@gpu
def test_matrix_multiplication(hip):
    """'A GSMat should support matrix multiplication' (GSMatTest.scala:55-71), GMat * GSMat half."""
    rng = np.random.default_rng(1)
    b = rng.random((nk, nc)).astype(np.float32)
    bt = np.ascontiguousarray(b.T)                                   # nc x nk
    at = sprand(rng, nk, nr, 0.2)
    aat, bbt = GSMat.from_csc(nk, nr, *at), GMat.from_numpy(bt)
    before = Mat.nflops()
    cct = bbt * aat
    assert cct.mytype == "GMat" and cct.shape == (nc, nr)
    assert Mat.nflops() - before == 2 * nc * at[0].size              # Mat.nflops += 2L * nrows * a.nnz
    dt = bt.astype(np.float64) @ full(nk, nr, *at)
    np.testing.assert_allclose(cct.numpy(), dt, rtol=0, atol=EPS)


@gpu
def test_matrix_times_transpose(hip):
    """'support matrix *^' (GSMatTest.scala:74-83)."""
    rng = np.random.default_rng(2)
    a = rng.random((nr, nk)).astype(np.float32)
    b = sprand(rng, nc, nk, 0.2)
    aa, bb = GMat.from_numpy(a), GSMat.from_csc(nc, nk, *b)
    cc = aa.xT(bb)
    assert cc.mytype == "GMat" and cc.shape == (nr, nc)
    np.testing.assert_allclose(cc.numpy(), a.astype(np.float64) @ full(nc, nk, *b).T, rtol=0, atol=EPS)


@gpu
@pytest.mark.parametrize("axis", [1, 2, 0])
def test_sparse_sums(hip, axis):
    """'support 2D column sum' / 'row sum' (GSMatTest.scala:283-316), loops as written there."""
    rng = np.random.default_rng(3 + axis)
    data, ir, jc = sprand(rng, nr, nc, 0.2)
    aa = GSMat.from_csc(nr, nc, data, ir, jc)
    ax = axis if axis else 1
    b = np.zeros(nc if ax == 1 else nr, dtype=np.float32)
    for i in range(nc):
        j0, j1 = jc[i] - 1, jc[i + 1] - 1
        if ax == 1:
            if j1 > j0:
                b[i] = data[j0]
            for j in range(j0 + 1, j1):
                b[i] = b[i] + data[j]
        else:
            for j in range(j0, j1):
                b[ir[j] - 1] = b[ir[j] - 1] + data[j]
    cc = mats.sum(aa, axis)
    assert cc.mytype == "GMat" and cc.shape == ((1, nc) if ax == 1 else (nr, 1))
    np.testing.assert_allclose(cc.numpy().ravel(), b, rtol=0, atol=EPS)


@gpu
@pytest.mark.parametrize("axis", [1, 2])
def test_dense_sums(hip, axis):
    """GMat sum (GMatTest.scala:938-979)."""
    rng = np.random.default_rng(5)
    a = rng.random((nr, nc)).astype(np.float32)
    cc = mats.sum(GMat.from_numpy(a), axis)
    want = a.astype(np.float64).sum(axis=axis - 1)
    assert cc.shape == ((1, nc) if axis == 1 else (nr, 1))
    np.testing.assert_allclose(cc.numpy().ravel(), want, rtol=0, atol=EPS)


@gpu
def test_dds_keeps_the_pattern(hip):
    """DDS has no test in the reference; pinned by its closed form and by the pattern rule:
    the result's ir / jc equal the input's bit for bit (DDShelper copies them)."""
    rng = np.random.default_rng(6)
    a = rng.random((nk, nr)).astype(np.float32)       # k x nrows(S)
    b = rng.random((nk, nc)).astype(np.float32)       # k x ncols(S)
    data, ir, jc = sprand(rng, nr, nc, 0.3)
    cs = GSMat.from_csc(nr, nc, data, ir, jc)
    before = Mat.nflops()
    p = DDS(GMat.from_numpy(a), GMat.from_numpy(b), cs)
    assert p.mytype == "GSMat" and p.dims == (nr, nc, data.size)
    assert Mat.nflops() - before == 2 * data.size * nk
    vals, pir, pjc = p.to_csc()                        # runs SparseMat.check as well
    assert np.array_equal(pir, ir) and np.array_equal(pjc, jc)
    assert np.array_equal(p.device_jc(), jc - 1)       # the device column pointer travels too
    cols = np.repeat(np.arange(nc), np.diff(jc))
    want = np.einsum("kn,kn->n", a.astype(np.float64)[:, ir - 1], b.astype(np.float64)[:, cols])
    np.testing.assert_allclose(vals, want, rtol=0, atol=EPS)
    ref, _, _ = oracle.dds(a.ravel(order="F"), b.ravel(order="F"), nk, ir, jc, ioff=1)
    np.testing.assert_allclose(vals, ref, rtol=1e-5, atol=1e-6)


@gpu
def test_output_reuse_and_accumulate(hip):
    """`c ~ a * b` reuses c; madd / maddT accumulate into it (GMat.scala:1051-1096)."""
    rng = np.random.default_rng(7)
    a = rng.random((nr, nk)).astype(np.float32)
    s = sprand(rng, nk, nc, 0.2)
    aa, ss = GMat.from_numpy(a), GSMat.from_csc(nk, nc, *s)
    c = GMat.zeros(nr, nc)
    c2 = aa.GSMult(ss, c)
    assert c2.same(c)
    once = c.numpy().copy()
    aa.madd(ss, c)
    np.testing.assert_allclose(c.numpy(), 2 * once, rtol=1e-6)
    bb = GMat.from_numpy(rng.random((nr, nc)).astype(np.float32))
    g = GMat.zeros(nr, nk)
    assert bb.GSMultT(ss, g).same(g)
    once = g.numpy().copy()
    bb.maddT(ss, g)
    np.testing.assert_allclose(g.numpy(), 2 * once, rtol=1e-6)


@gpu
def test_gpu_cache_returns_the_same_output_for_the_same_operands(hip):
    rng = np.random.default_rng(8)
    aa = GMat.from_numpy(rng.random((nr, nk)).astype(np.float32))
    ss = GSMat.from_csc(nk, nc, *sprand(rng, nk, nc, 0.2))
    Mat.set("useGPUcache", 1)
    try:
        c1 = aa * ss
        c2 = aa * ss
        assert c1.same(c2)
        Mat.set("useGPUcache", 0)
        assert not (aa * ss).same(c1)
    finally:
        Mat.set("useGPUcache", 0)
        Mat.clear_caches()


@gpu
def test_dimension_mismatch_messages(hip):
    rng = np.random.default_rng(9)
    aa = GMat.from_numpy(rng.random((nr, nk)).astype(np.float32))
    bad = GSMat.from_csc(nk + 1, nc, *sprand(rng, nk + 1, nc, 0.2))
    with pytest.raises(RuntimeError, match=r"GSMult dimensions mismatch \(10 30\) \(31 20\)"):
        aa * bad
    with pytest.raises(RuntimeError, match=r"GSMult dimensions mismatch"):
        aa.xT(bad)
    with pytest.raises(RuntimeError, match=r"GSMadd dimensions mismatch"):
        aa.madd(GSMat.from_csc(nk, nc, *sprand(rng, nk, nc, 0.2)), GMat.zeros(nr, nc + 1))
    with pytest.raises(RuntimeError, match=r"dimensions mismatch 10,30  10,20  31,20"):
        DDS(aa, GMat.from_numpy(rng.random((nr, nc)).astype(np.float32)), bad)
    with pytest.raises(RuntimeError, match="dimension must be 1 or 2"):
        aa.reduceOp(3, 0.0, 0)


@gpu
def test_index_base_zero_host_matrices(hip):
    rng = np.random.default_rng(10)
    data, ir, jc = random_csc(rng, nk, nc, 0.2)      # 0-based
    Mat.set("ioneBased", 0)
    try:
        ss = GSMat.from_csc(nk, nc, data, ir, jc)
        d2, ir2, jc2 = ss.to_csc()
        assert np.array_equal(ir2, ir) and np.array_equal(jc2, jc) and np.array_equal(d2, data)
    finally:
        Mat.set("ioneBased", 1)
    ss1 = GSMat.from_csc(nk, nc, data, ir + 1, jc + 1)
    d3, ir3, jc3 = ss1.to_csc()
    assert np.array_equal(ir3, ir + 1) and np.array_equal(jc3, jc + 1)


@gpu
def test_nmf_multiplicative_update_chain(hip):
    """The NMF update chain (benchmark configuration 5) at a small size: R = DDS(W,H,V); Q = V ./ R on the
    nonzeros; G = W *^ Q; rs = sum(H, 2)."""
    rng = np.random.default_rng(11)
    k, m, n = 16, 40, 60
    W = (rng.random((k, m)) * 0.99 + 0.01).astype(np.float32)
    H = (rng.random((k, n)) * 0.99 + 0.01).astype(np.float32)
    data, ir, jc = sprand(rng, m, n, 0.15)
    data = rng.exponential(size=data.size).astype(np.float32)
    V = GSMat.from_csc(m, n, data, ir, jc)
    gW, gH = GMat.from_numpy(W), GMat.from_numpy(H)
    R = DDS(gW, gH, V)
    # `R.contents ~ V.contents / R.contents`: the quotient overwrites R's values in place
    V.contents().gOp(R.contents(), 3, out=R.contents())
    Q = R
    Q2 = V.with_values(V.contents() / DDS(gW, gH, V).contents())       # the copying form
    assert np.array_equal(Q2.to_csc()[0], Q.to_csc()[0])
    G = gH.xT(Q)                                   # k x m : sum_c H[:,c] * Q[r,c]
    rs = mats.sum(gH, 2)
    cols = np.repeat(np.arange(n), np.diff(jc))
    r64 = np.einsum("kn,kn->n", W.astype(np.float64)[:, ir - 1], H.astype(np.float64)[:, cols])
    q64 = data.astype(np.float64) / r64
    g64 = np.zeros((k, m))
    np.add.at(g64.T, ir - 1, (H.astype(np.float64)[:, cols] * q64).T)
    np.testing.assert_allclose(Q.to_csc()[0], q64, rtol=1e-4)
    np.testing.assert_allclose(G.numpy(), g64, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(rs.numpy().ravel(), H.astype(np.float64).sum(axis=1), rtol=1e-5)


@gpu
def test_flip_gflop_accounting(hip):
    rng = np.random.default_rng(12)
    aa = GMat.from_numpy(rng.random((64, 200)).astype(np.float32))
    s = sprand(rng, 200, 300, 0.1)
    ss = GSMat.from_csc(200, 300, *s)
    mats.flip()
    aa * ss
    g, secs = mats.gflop()
    assert secs > 0 and g == pytest.approx(2 * 64 * s[0].size / secs / 1e9, rel=0.2)


@gpu
def test_tile_mult_and_messages(hip):
    """GMat.tileMult / tileMultNT (GMat.scala:961-997): windows, argument checks, messages."""
    rng = np.random.default_rng(13)
    a = rng.random((12, 40)).astype(np.float32)
    s = sprand(rng, 35, 30, 0.3)
    c0 = rng.random((15, 33)).astype(np.float32)
    aa, ss = GMat.from_numpy(a), GSMat.from_csc(35, 30, *s)
    S = full(35, 30, *s)
    cc = GMat.from_numpy(c0)
    out = aa.tileMult(7, 9, 11, 3, 5, ss, 6, 4, cc, 2, 8)
    assert out.same(cc)
    want = c0.astype(np.float64).copy()
    want[2:9, 8:17] += a.astype(np.float64)[3:10, 5:16] @ S[6:17, 4:13]
    np.testing.assert_allclose(cc.numpy(), want, rtol=0, atol=EPS)
    cc = GMat.from_numpy(c0)
    aa.tileMultNT(6, 10, 8, 1, 7, ss, 5, 9, cc, 4, 3)
    want = c0.astype(np.float64).copy()
    want[4:10, 3:13] += a.astype(np.float64)[1:7, 7:15] @ S[5:15, 9:17].T
    np.testing.assert_allclose(cc.numpy(), want, rtol=0, atol=EPS)
    with pytest.raises(RuntimeError, match="tileMult: cant have negative offsets or dimensions"):
        aa.tileMult(7, 9, 11, -1, 5, ss, 6, 4, cc, 2, 8)
    with pytest.raises(RuntimeError, match="tileMult: tile strays outside matrix dimensions"):
        aa.tileMult(7, 9, 11, 3, 5, ss, 30, 4, cc, 2, 8)
    with pytest.raises(RuntimeError, match="tileMultNT: tile strays outside matrix dimensions"):
        aa.tileMultNT(6, 10, 8, 1, 7, ss, 5, 25, cc, 4, 3)


@gpu
def test_sparse_times_dense_both_orders(hip):
    """'support matrix multiplication' GSMat * GMat half (GSMatTest.scala:55-63) and
    'support matrix ^*' (GSMatTest.scala:85-94)."""
    rng = np.random.default_rng(14)
    a = sprand(rng, nr, nk, 0.2)
    b = rng.random((nk, nc)).astype(np.float32)
    aa, bb = GSMat.from_csc(nr, nk, *a), GMat.from_numpy(b)
    before = Mat.nflops()
    cc = aa * bb
    assert cc.mytype == "GMat" and cc.shape == (nr, nc)
    assert Mat.nflops() - before == 2 * a[0].size * nc
    np.testing.assert_allclose(cc.numpy(), full(nr, nk, *a) @ b.astype(np.float64), rtol=0, atol=EPS)
    a2 = sprand(rng, nk, nr, 0.2)
    cc = GSMat.from_csc(nk, nr, *a2).Tx(bb)
    assert cc.mytype == "GMat" and cc.shape == (nr, nc)
    np.testing.assert_allclose(cc.numpy(), full(nk, nr, *a2).T @ b.astype(np.float64), rtol=0, atol=EPS)
    with pytest.raises(RuntimeError, match="SDMult dimensions mismatch"):
        aa * GMat.from_numpy(rng.random((nk + 1, nc)).astype(np.float32))
    with pytest.raises(RuntimeError, match="SDTMult dimensions mismatch"):
        aa.Tx(bb)


@gpu
@pytest.mark.parametrize("op,fn", [(0, np.add), (1, np.subtract), (2, np.multiply), (3, np.divide), (10, np.maximum), (11, np.minimum)])
def test_sparse_op_edge_vector(hip, op, fn):
    """GSMat op GMat for row vectors, column vectors and scalars (GSMat.GSDop; the reference's
    testEwise family, GSMatTest.scala:96-280): the op touches the stored values only."""
    rng = np.random.default_rng(15 + op)
    data, ir, jc = sprand(rng, nr, nc, 0.3)
    aa = GSMat.from_csc(nr, nc, data, ir, jc)
    cols = np.repeat(np.arange(nc), np.diff(jc))
    row = (rng.random((1, nc)) + 0.5).astype(np.float32)
    col = (rng.random((nr, 1)) + 0.5).astype(np.float32)
    val = (rng.random((1, 1)) + 0.5).astype(np.float32)
    for b, pick in ((row, row[0, cols]), (col, col[ir - 1, 0]), (val, np.full(data.size, val[0, 0], np.float32))):
        before = Mat.nflops()
        out = aa.GSDop(GMat.from_numpy(b), op)
        assert out.mytype == "GSMat" and Mat.nflops() - before == data.size
        vals, oir, ojc = out.to_csc()
        assert np.array_equal(oir, ir) and np.array_equal(ojc, jc)
        assert np.array_equal(vals, fn(data, pick).astype(np.float32))
    assert np.array_equal(aa.to_csc()[0], data)          # the operand itself is not modified
    with pytest.raises(RuntimeError, match="only edge operators supported"):
        aa.GSDop(GMat.from_numpy(rng.random((nr, nc)).astype(np.float32)), op)
    with pytest.raises(RuntimeError, match="dimensions mismatch"):
        aa.GSDop(GMat.from_numpy(rng.random((1, nc + 1)).astype(np.float32)), op)


@gpu
def test_colslice(hip):
    """GSMat.colslice (GSMat.scala:77-104): the slice is a matrix of its own (pattern bit-exact,
    column pointer rebased), usable by every product; empty and full ranges; bad ranges throw."""
    rng = np.random.default_rng(12)
    m, n, kk = 40, 300, 16
    s = sprand(rng, m, n, 0.15)
    ss = GSMat.from_csc(m, n, *s)
    data, ir, jc = s
    a = rng.random((kk, m)).astype(np.float32)
    b = rng.random((kk, 57)).astype(np.float32)
    aa = GMat.from_numpy(a)
    for c1, c2 in [(0, n), (17, 74), (0, 1), (n - 1, n), (50, 50)]:
        sl = ss.colslice(c1, c2)
        assert sl.mytype == "GSMat" and sl.dims == (m, c2 - c1, int(jc[c2] - jc[c1]))
        d2, ir2, jc2 = sl.to_csc()
        lo, hi = jc[c1] - 1, jc[c2] - 1                           # host arrays are 1-based
        assert np.array_equal(ir2, ir[lo:hi]) and np.array_equal(d2, data[lo:hi])
        assert np.array_equal(jc2, jc[c1:c2 + 1] - jc[c1] + 1)
        assert np.array_equal(sl.device_jc(), jc[c1:c2 + 1] - jc[c1])
        if c2 > c1:
            want = a.astype(np.float64) @ full(m, n, *s)[:, c1:c2]
            np.testing.assert_allclose((aa * sl).numpy(), want, rtol=0, atol=EPS)
    sl = ss.colslice(17, 74)
    bb = GMat.from_numpy(b)                                       # kk x 57
    want = b.astype(np.float64) @ full(m, n, *s)[:, 17:74].T      # kk x m
    np.testing.assert_allclose(bb.xT(sl).numpy(), want, rtol=0, atol=EPS)
    np.testing.assert_allclose(sl.sum(2).numpy().ravel(), full(m, n, *s)[:, 17:74].sum(axis=1), rtol=0, atol=EPS)
    for bad in [(-1, 3), (5, 4), (0, n + 1)]:
        with pytest.raises(RuntimeError, match="colslice"):
            ss.colslice(*bad)


@gpu
def test_onehot_and_nhot(hip):
    """GSMat.oneHot / nHot (GSMat.scala:686-720): patterns with unsorted, repeated rows built on the
    device; A * oneHot(c) is a pure gather (bit-exact), nHot sums the chosen columns."""
    rng = np.random.default_rng(13)
    kk, ncats, n = 24, 37, 500
    a = rng.standard_normal((kk, ncats)).astype(np.float32)
    aa = GMat.from_numpy(a)
    c = rng.integers(0, ncats, size=n).astype(np.int32)
    c[7] = ncats - 1
    s1 = GSMat.oneHot(c)                                          # ncats from the largest category
    assert s1.mytype == "GSMat" and s1.dims == (ncats, n, n)
    assert np.array_equal(s1.device_jc(), np.arange(n + 1))
    assert np.array_equal((aa * s1).numpy(), a[:, c])             # 1.0f * x added to 0: exact
    d, ir, jc = s1.to_csc()
    assert np.array_equal(ir, c + 1) and np.array_equal(d, np.ones(n, np.float32))
    s1b = GSMat.oneHot(c, 50)
    assert s1b.dims == (50, n, n)
    with pytest.raises(RuntimeError, match="category outside"):
        GSMat.oneHot(c, ncats - 1)
    # n-hot with rows in arbitrary order and repeats inside a column
    cats = rng.integers(0, ncats, size=(3, 200)).astype(np.int32)
    cats[:, 5] = 4
    s3 = GSMat.nHot(cats, ncats)
    assert s3.dims == (ncats, 200, 600) and np.array_equal(s3.device_jc(), 3 * np.arange(201))
    want = sum(a.astype(np.float64)[:, cats[i]] for i in range(3))
    np.testing.assert_allclose((aa * s3).numpy(), want, rtol=0, atol=EPS)
    b = rng.standard_normal((kk, 200)).astype(np.float32)
    wantT = np.zeros((kk, ncats))
    for i in range(3):
        np.add.at(wantT.T, cats[i], b.astype(np.float64).T)
    np.testing.assert_allclose(GMat.from_numpy(b).xT(s3).numpy(), wantT, rtol=0, atol=EPS)
    np.testing.assert_allclose(s3.sum(2).numpy().ravel(), np.bincount(cats.ravel(), minlength=ncats), rtol=0, atol=EPS)


@gpu
def test_matrix_transpose_and_full(hip):
    """'A GSMat should support matrix transpose' (GSMatTest.scala:46-53), computed on the device
    here; full() is the dense image (GSMat.scala:206-216)."""
    rng = np.random.default_rng(14)
    for m, n, dens in [(nr, nc, 0.2), (200, 3000, 0.05), (1, 50, 0.5), (50, 1, 0.5), (30, 40, 0.0)]:
        a = sprand(rng, m, n, dens)
        aa = GSMat.from_csc(m, n, *a)
        dense = full(m, n, *a)
        ff = aa.full()
        assert ff.mytype == "GMat" and ff.shape == (m, n)
        assert np.array_equal(ff.numpy(), dense.astype(np.float32))
        bb = aa.t()
        assert bb.mytype == "GSMat" and bb.dims == (n, m, a[0].size)
        d2, ir2, jc2 = bb.to_csc()                                # SparseMat.check passes: rows sorted
        assert np.array_equal(full(n, m, d2, ir2, jc2), dense.T)
        assert np.array_equal(bb.full().numpy(), dense.T.astype(np.float32))
        if a[0].size:
            x = rng.random((7, n)).astype(np.float32)             # x * a^T through the transposed matrix
            np.testing.assert_allclose((GMat.from_numpy(x) * bb).numpy(), x.astype(np.float64) @ dense.T, rtol=0, atol=EPS)
            assert np.array_equal(bb.t().to_csc()[1], a[1])       # transpose twice: the pattern is back
