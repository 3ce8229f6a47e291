"""Random shapes x random settings of every tunable, through the plan-taking forms: DDS through a plan equals the plain
entry bit for bit (also with the elementwise step fused in), A*S / A*^S / sparse row sums through a plan stay within the
tolerance of the fp64 result, and the values stored in a plan give the same bits as the values passed in. Shapes include
k that is not a multiple of 4, empty columns, columns longer than a wave segment, unsorted and repeated rows."""
import ctypes as C

import numpy as np
import pytest

from bidmat_amd import hip_abi
from bidmat_amd.device import DeviceArray
from util import dense_full, random_csc

pytestmark = pytest.mark.gpu
TUNABLES = ("seglen", "panel_kb", "heavy_min", "col_classes", "class_hot", "class_threads", "class_strip", "class_phases",
            "dense_rows", "dense_min_pct", "dense_min_nnz", "dense_cb", "scalar_values")


@pytest.mark.parametrize("seed0", [11, 12])
def test_plan_forms_under_random_shapes_and_settings(hip, seed0):
    lib = hip
    niter = 60

    def opt(n, v):
        hip_abi.check(lib.bidmat_set_option(n.encode(), v), "set_option " + n)

    defaults = {n: lib.bidmat_get_option(n.encode()) for n in TUNABLES}
    try:
        for it in range(niter):
            seed = seed0 * 100000 + it
            rng = np.random.default_rng(seed)
            k = int(rng.choice([1, 3, 4, 7, 8, 16, 20, 32, 33, 64, 100, 128, 132, 200, 256, 260, 384, 512, 1024, 1100, 2052]))
            nrows = int(rng.integers(1, 400)); ncols = int(rng.integers(1, 600))
            mode = rng.integers(0, 4)
            if mode == 0: lengths = rng.integers(0, min(nrows, 40) + 1, size=ncols)
            elif mode == 1: lengths = np.minimum(nrows, (rng.pareto(1.2, size=ncols) * 3).astype(np.int64))
            elif mode == 2: lengths = np.where(rng.random(ncols) < 0.7, 0, rng.integers(0, nrows + 1, size=ncols))
            else: lengths = np.full(ncols, min(nrows, int(rng.integers(1, 300))))
            unique = bool(rng.integers(0, 2)); sort_rows = bool(rng.integers(0, 2))
            if not unique and mode == 3: lengths = rng.integers(0, 500, size=ncols)     # duplicates allow more than nrows
            data, ir, jc = random_csc(rng, nrows, ncols, lengths=lengths, unique=unique, sort_rows=sort_rows)
            # skewed rows now and then
            nnz = int(ir.size)
            o = dict(seglen=int(rng.choice([64, 100, 256, 1024])), panel_kb=int(rng.choice([16, 64, 3072])), heavy_min=int(rng.choice([1, 2, 8])),
                     col_classes=int(rng.choice([-1, 0, 1, 1])), class_hot=int(rng.choice([-1, 0, 1, 3, 16])), class_threads=int(rng.choice([256, 512, 1024])),
                     class_strip=int(rng.choice([1, 3, 16, 64])), class_phases=int(rng.choice([0, 1, 2, 4, 8])),
                     dense_rows=int(rng.choice([0, 32, 96, 128])), dense_min_pct=int(rng.choice([2, 15, 60])),
                     dense_min_nnz=int(rng.choice([0, 0, 1 << 22])), dense_cb=int(rng.choice([0, 16, 50])),
                     scalar_values=int(rng.choice([0, 1, 1])))
            for n, v in o.items(): opt(n, v)
            tag = "seed=%d k=%d %dx%d nnz=%d unique=%s sorted=%s %s" % (seed, k, nrows, ncols, nnz, unique, sort_rows, o)
            A = rng.standard_normal(k * nrows).astype(np.float32); B = rng.standard_normal(k * ncols).astype(np.float32)
            V = (rng.random(nnz).astype(np.float32) + 0.5)
            dA, dB, dv, dV = DeviceArray.from_numpy(A), DeviceArray.from_numpy(B), DeviceArray.from_numpy(data), DeviceArray.from_numpy(V)
            dir_, djc = DeviceArray.from_numpy(ir), DeviceArray.from_numpy(jc)
            plan = C.c_void_p()
            hip_abi.check(lib.bidmat_plan_create(nrows, ncols, nnz, dir_.ptr, djc.ptr, k, C.byref(plan)), "plan_create")
            P1, P2, P3 = DeviceArray.zeros(max(nnz, 1)), DeviceArray.zeros(max(nnz, 1)), DeviceArray.zeros(max(nnz, 1))
            C1, C2 = DeviceArray.zeros(k * ncols), DeviceArray.zeros(k * ncols)
            G1, G2 = DeviceArray.zeros(k * nrows), DeviceArray.zeros(k * nrows)
            rs1, rs2 = DeviceArray.zeros(nrows), DeviceArray.zeros(nrows)
            # DDS: plain vs plan (bit-equal), fused op
            hip_abi.check(lib.bidmat_dds_csc(k, ncols, nnz, dA.ptr, dB.ptr, dir_.ptr, djc.ptr, P1.ptr, 0, None), "dds_csc")
            hip_abi.check(lib.bidmat_dds_plan(plan, k, dA.ptr, dB.ptr, dir_.ptr, djc.ptr, None, 0, P2.ptr, 0, None), "dds_plan")
            hip_abi.check(lib.bidmat_dds_plan(plan, k, dA.ptr, dB.ptr, dir_.ptr, djc.ptr, dV.ptr, 3, P3.ptr, 0, None), "dds_plan op")
            hip_abi.check(lib.bidmat_synchronize())
            p1, p2, p3 = P1.numpy()[:nnz], P2.numpy()[:nnz], P3.numpy()[:nnz]
            assert np.array_equal(p1, p2), "dds_plan != dds_csc " + tag
            with np.errstate(divide="ignore", invalid="ignore"):
                assert np.array_equal(p3, (V / p1).astype(np.float32), equal_nan=True), "fused op " + tag
            A2 = A.reshape(nrows, k).astype(np.float64); B2 = B.reshape(ncols, k).astype(np.float64)
            ic = np.repeat(np.arange(ncols), np.diff(jc))
            if nnz:
                ref = np.einsum("ij,ij->i", A2[ir], B2[ic]); sa = np.einsum("ij,ij->i", np.abs(A2[ir]), np.abs(B2[ic]))
                assert np.all(np.abs(p1 - ref) <= 1e-5 * sa + 1e-30), "dds vs fp64 " + tag
            # A*S: plain vs plan (tolerance), vs fp64
            hip_abi.check(lib.bidmat_dsmult_csc(k, ncols, nnz, dA.ptr, dv.ptr, dir_.ptr, djc.ptr, C1.ptr, 0, None), "dsmult_csc")
            hip_abi.check(lib.bidmat_dsmult_plan(plan, k, dA.ptr, dv.ptr, dir_.ptr, djc.ptr, C2.ptr, 0, None), "dsmult_plan")
            hip_abi.check(lib.bidmat_synchronize())
            S = dense_full(nrows, ncols, data, ir, jc)
            refC = (A2.T @ S).T.ravel(); saC = (np.abs(A2).T @ np.abs(S)).T.ravel()
            for nm, x in (("dsmult_csc", C1.numpy()), ("dsmult_plan", C2.numpy())):
                assert np.all(np.abs(x - refC) <= 1e-5 * saC + 1e-30), nm + " vs fp64 " + tag
            # A*^S and row sums through the plan, fresh and stored values
            AT = rng.standard_normal(k * ncols).astype(np.float32); dAT = DeviceArray.from_numpy(AT)
            hip_abi.check(lib.bidmat_dsmultT_plan(plan, k, dAT.ptr, dv.ptr, G1.ptr, 0, None), "dsmultT_plan")
            hip_abi.check(lib.bidmat_spsum_rows_plan(plan, dv.ptr, rs1.ptr, 0, None), "spsum_rows")
            hip_abi.check(lib.bidmat_plan_set_values(plan, dv.ptr, None), "set_values")
            hip_abi.check(lib.bidmat_dsmultT_plan(plan, k, dAT.ptr, None, G2.ptr, 0, None), "dsmultT_plan stored")
            hip_abi.check(lib.bidmat_spsum_rows_plan(plan, None, rs2.ptr, 0, None), "spsum_rows stored")
            hip_abi.check(lib.bidmat_synchronize())
            AT2 = AT.reshape(ncols, k).astype(np.float64)
            refG = (AT2.T @ S.T).T.ravel(); saG = (np.abs(AT2).T @ np.abs(S).T).T.ravel()
            g1, g2 = G1.numpy(), G2.numpy()
            assert np.all(np.abs(g1 - refG) <= 1e-5 * saG + 1e-30), "dsmultT vs fp64 " + tag
            # values passed in take the plan's dense block (if the pattern got one and k fits it), stored values walk the
            # segments of every row: the rows outside the block have the same bits, the others agree within the tolerance
            nd = int(lib.bidmat_plan_info(plan, b"dense_rows"))
            if nd > 0 and 64 < k <= 256 and o["dense_rows"] > 0:
                drow = np.empty(nd, np.int32)
                ptr, cnt = C.c_void_p(), C.c_longlong()
                hip_abi.check(lib.bidmat_plan_array(plan, b"drow", C.byref(ptr), C.byref(cnt)))
                hip_abi.check(lib.bidmat_memcpy_d2h(drow.ctypes.data, ptr, 4 * nd))
                keep = np.ones(nrows, bool); keep[drow] = False
                assert np.array_equal(g1.reshape(nrows, k)[keep], g2.reshape(nrows, k)[keep]), "dsmultT stored != fresh outside the dense block " + tag
                assert np.all(np.abs(g2 - refG) <= 1e-5 * saG + 1e-30), "dsmultT stored vs fp64 " + tag
            else:
                assert np.array_equal(g1, g2), "dsmultT stored != fresh " + tag
            assert np.array_equal(rs1.numpy(), rs2.numpy()), "row sums stored != fresh " + tag
            assert np.allclose(rs1.numpy(), S.sum(axis=1), rtol=1e-5, atol=1e-6), "row sums " + tag
            hip_abi.check(lib.bidmat_plan_destroy(plan))
            for d in (dA, dB, dv, dV, dir_, djc, P1, P2, P3, C1, C2, G1, G2, rs1, rs2, dAT): d.free()
    finally:
        for n, v in defaults.items():
            opt(n, v)
