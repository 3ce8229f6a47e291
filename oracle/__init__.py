"""ctypes front end of the CPU oracle (oracle/bidmat_oracle.c).

TEST INFRASTRUCTURE ONLY: importable from tests/, from __graft_entry__.smoke() and from
bench.py's cpu_baseline leg. The product (bidmat_amd, libbidmathip.so) never imports it.

All matrices are numpy arrays: dense = float32, column-major flattened (k*ncols) or 2-D
Fortran-ordered; sparse = (data float32[nnz], ir int32[nnz], jc int32[ncols+1]) with the
index base `ioff` the reference's host SMat uses (1 by default there, Mat.scala:718).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libbidmat_oracle.so")
_lib = None


def build():
    subprocess.check_call(["make", "-C", _HERE, "--no-print-directory"], stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        vp, i = C.c_void_p, C.c_int
        L.oracle_smcscm.argtypes = [i, i, vp, i, vp, vp, vp, vp, i, i]
        L.oracle_fsmult.argtypes = [i, i, vp, vp, vp, vp, i, vp, i]
        L.oracle_fsmult_f64.argtypes = [i, i, vp, vp, vp, vp, i, vp, vp, i]
        L.oracle_smcsrm.argtypes = [i, i, vp, i, vp, vp, vp, vp, i]
        L.oracle_fsmultT.argtypes = [i, i, vp, vp, vp, vp, i, vp, i]
        L.oracle_fsmultT_f64.argtypes = [i, i, vp, vp, vp, vp, i, vp, vp, i]
        L.oracle_fsmult_tile.argtypes = [i, i, i, vp, i, vp, vp, vp, i, i, i, vp, i, vp, vp, i]
        L.oracle_fsmult_tileT.argtypes = [i, i, i, vp, i, vp, vp, vp, i, i, i, vp, i, vp, vp]
        L.oracle_fsmult_tile.restype = None
        L.oracle_fsmult_tileT.restype = None
        L.oracle_dds.argtypes = [i, i, vp, vp, vp, vp, i, vp, vp, vp, i]
        L.oracle_dds_f64.argtypes = [i, i, vp, vp, vp, vp, i, vp, vp, i]
        L.oracle_spsum.argtypes = [i, i, vp, vp, vp, i, i, vp]
        L.oracle_spsum.restype = i
        L.oracle_spsum_f64.argtypes = [i, i, vp, vp, vp, i, i, vp, vp]
        L.oracle_dsum.argtypes = [i, i, vp, i, vp]
        L.oracle_dsum.restype = i
        L.oracle_dsum_f64.argtypes = [i, i, vp, i, vp]
        L.oracle_applyop.argtypes = [vp, vp, vp, C.c_longlong, i]
        L.oracle_applyop.restype = i
        L.oracle_reduce_tree.argtypes = [i, i, vp, vp, C.c_float, i, i]
        L.oracle_reduce_tree.restype = i
        L.oracle_check.argtypes = [i, i, i, vp, vp, i, vp]
        L.oracle_check.restype = i
        L.oracle_compress_inds.argtypes = [vp, i, vp, i, i]
        L.oracle_uncompress_inds.argtypes = [vp, i, vp, i]
        L.oracle_max_threads.restype = i
        for f in ("oracle_smcscm", "oracle_fsmult", "oracle_fsmult_f64", "oracle_smcsrm", "oracle_fsmultT",
                  "oracle_fsmultT_f64", "oracle_dds", "oracle_dds_f64", "oracle_spsum_f64", "oracle_dsum_f64",
                  "oracle_compress_inds", "oracle_uncompress_inds"):
            getattr(L, f).restype = None
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32).ravel(order="F"))


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def max_threads():
    return lib().oracle_max_threads()


def fsmult(A, k, data, ir, jc, ioff=0, out=None, nthreads=1, native=False):
    """C (+)= A*S. A k x nrowsS. Returns float32[k*ncols]. native=True runs the C-loop restatement
    (smcscm) instead of the Scala-loop one; both give the same bits."""
    A, data, ir, jc = _f32(A), _f32(data), _i32(ir), _i32(jc)
    ncols = jc.size - 1
    out = np.zeros(k * ncols, dtype=np.float32) if out is None else out
    if native:
        lib().oracle_smcscm(k, ncols, A.ctypes.data, k, data.ctypes.data, ir.ctypes.data, jc.ctypes.data,
                            out.ctypes.data, k, nthreads)
    else:
        lib().oracle_fsmult(k, ncols, A.ctypes.data, data.ctypes.data, ir.ctypes.data, jc.ctypes.data, ioff,
                            out.ctypes.data, nthreads)
    return out


def fsmult_f64(A, k, data, ir, jc, ioff=0, nthreads=1):
    A, data, ir, jc = _f32(A), _f32(data), _i32(ir), _i32(jc)
    ncols = jc.size - 1
    ref = np.zeros(k * ncols, dtype=np.float64)
    sa = np.zeros(k * ncols, dtype=np.float64)
    lib().oracle_fsmult_f64(k, ncols, A.ctypes.data, data.ctypes.data, ir.ctypes.data, jc.ctypes.data, ioff,
                            ref.ctypes.data, sa.ctypes.data, nthreads)
    return ref, sa


def fsmultT(A, k, nrowsS, data, ir, jc, ioff=0, out=None, nthreads=1, native=False):
    """C (+)= A*S^T. A k x ncols. Returns float32[k*nrowsS]."""
    A, data, ir, jc = _f32(A), _f32(data), _i32(ir), _i32(jc)
    ncols = jc.size - 1
    out = np.zeros(k * nrowsS, dtype=np.float32) if out is None else out
    if native:
        lib().oracle_smcsrm(k, ncols, A.ctypes.data, k, data.ctypes.data, ir.ctypes.data, jc.ctypes.data,
                            out.ctypes.data, k)
    else:
        lib().oracle_fsmultT(k, ncols, A.ctypes.data, data.ctypes.data, ir.ctypes.data, jc.ctypes.data, ioff,
                             out.ctypes.data, nthreads)
    return out


def fsmultT_f64(A, k, nrowsS, data, ir, jc, ioff=0, nthreads=1):
    A, data, ir, jc = _f32(A), _f32(data), _i32(ir), _i32(jc)
    ncols = jc.size - 1
    ref = np.zeros(k * nrowsS, dtype=np.float64)
    sa = np.zeros(k * nrowsS, dtype=np.float64)
    lib().oracle_fsmultT_f64(k, ncols, A.ctypes.data, data.ctypes.data, ir.ctypes.data, jc.ctypes.data, ioff,
                             ref.ctypes.data, sa.ctypes.data, nthreads)
    return ref, sa


def fsmult_tile(Aparent, anrows, aroff, acoff, nr, nc, kk, data, ir, jc, broff, bcoff, Cparent, cnrows, croff,
                ccoff, ioff=0, transposed=False, nthreads=1):
    """tileMult / tileMultNT on flattened column-major parents. Adds into Cparent (float32, in
    place) and returns (ref64, sumabs) of the product alone as nr x nc column-major arrays."""
    Aparent, data, ir, jc = _f32(Aparent), _f32(data), _i32(ir), _i32(jc)
    assert Cparent.dtype == np.float32 and Cparent.flags.c_contiguous
    ref = np.zeros(nr * nc, dtype=np.float64)
    sa = np.zeros(nr * nc, dtype=np.float64)
    ap = Aparent.ctypes.data + 4 * (aroff + acoff * anrows)
    cp = Cparent.ctypes.data + 4 * (croff + ccoff * cnrows)
    if transposed:
        lib().oracle_fsmult_tileT(nr, nc, kk, ap, anrows, data.ctypes.data, ir.ctypes.data, jc.ctypes.data, ioff,
                                  broff, bcoff, cp, cnrows, ref.ctypes.data, sa.ctypes.data)
    else:
        lib().oracle_fsmult_tile(nr, nc, kk, ap, anrows, data.ctypes.data, ir.ctypes.data, jc.ctypes.data, ioff,
                                 broff, bcoff, cp, cnrows, ref.ctypes.data, sa.ctypes.data, nthreads)
    return ref, sa


def dds(A, B, k, ir, jc, ioff=0, nthreads=1):
    """Returns (data float32[nnz], out_ir, out_jc): the values and the copied pattern."""
    A, B, ir, jc = _f32(A), _f32(B), _i32(ir), _i32(jc)
    ncols = jc.size - 1
    nnz = int(jc[-1]) - ioff
    out = np.zeros(nnz, dtype=np.float32)
    oir = np.zeros(nnz, dtype=np.int32)
    ojc = np.zeros(ncols + 1, dtype=np.int32)
    lib().oracle_dds(k, ncols, A.ctypes.data, B.ctypes.data, ir.ctypes.data, jc.ctypes.data, ioff,
                     out.ctypes.data, oir.ctypes.data, ojc.ctypes.data, nthreads)
    return out, oir, ojc


def dds_f64(A, B, k, ir, jc, ioff=0, nthreads=1):
    A, B, ir, jc = _f32(A), _f32(B), _i32(ir), _i32(jc)
    ncols = jc.size - 1
    nnz = int(jc[-1]) - ioff
    ref = np.zeros(nnz, dtype=np.float64)
    sa = np.zeros(nnz, dtype=np.float64)
    lib().oracle_dds_f64(k, ncols, A.ctypes.data, B.ctypes.data, ir.ctypes.data, jc.ctypes.data, ioff,
                         ref.ctypes.data, sa.ctypes.data, nthreads)
    return ref, sa


def spsum(nrows, data, ir, jc, dim0, ioff=0):
    data, ir, jc = _f32(data), _i32(ir), _i32(jc)
    ncols = jc.size - 1
    out = np.zeros(max(nrows, ncols, 1), dtype=np.float32)
    n = lib().oracle_spsum(nrows, ncols, data.ctypes.data, ir.ctypes.data, jc.ctypes.data, ioff, dim0,
                           out.ctypes.data)
    if n < 0:
        raise RuntimeError("index must 1 or 2")
    return out[:n].copy()


def spsum_f64(nrows, data, ir, jc, dim, ioff=0):
    data, ir, jc = _f32(data), _i32(ir), _i32(jc)
    ncols = jc.size - 1
    n = ncols if dim == 1 else nrows
    ref = np.zeros(n, dtype=np.float64)
    sa = np.zeros(n, dtype=np.float64)
    lib().oracle_spsum_f64(nrows, ncols, data.ctypes.data, ir.ctypes.data, jc.ctypes.data, ioff, dim,
                           ref.ctypes.data, sa.ctypes.data)
    return ref, sa


def dsum(A, nrows, ncols, dim0):
    A = _f32(A)
    out = np.zeros(max(nrows, ncols, 1), dtype=np.float32)
    n = lib().oracle_dsum(nrows, ncols, A.ctypes.data, dim0, out.ctypes.data)
    if n < 0:
        raise RuntimeError("index must 1 or 2")
    return out[:n].copy()


def dsum_f64(A, nrows, ncols, dim):
    A = _f32(A)
    ref = np.zeros(ncols if dim == 1 else nrows, dtype=np.float64)
    lib().oracle_dsum_f64(nrows, ncols, A.ctypes.data, dim, ref.ctypes.data)
    return ref


def applyop(A, B, opn):
    A, B = _f32(A), _f32(B)
    out = np.empty_like(A)
    if lib().oracle_applyop(A.ctypes.data, B.ctypes.data, out.ctypes.data, A.size, opn) != 0:
        raise RuntimeError("unknown op %d" % opn)
    return out


def reduce_tree(A, nrows, ncols, opn, dim, initv=0.0):
    """reduce1op (dim 1: per column) / reduce2op (dim 2: per row) with any of the 15 ops, in the order of the
    reference's device kernels. A: column-major nrows x ncols."""
    A = _f32(A)
    out = np.empty(ncols if dim == 1 else nrows, dtype=np.float32)
    if lib().oracle_reduce_tree(nrows, ncols, A.ctypes.data, out.ctypes.data, initv, opn, dim) != 0:
        raise RuntimeError("unknown op %d or dim %d" % (opn, dim))
    return out


def check(nrows, ncols, nnz, ir, jc, ioff=0):
    """Returns (rule, where): rule 0 = valid, else the failing rule of SparseMat.check."""
    jc = _i32(jc)
    irp = None if ir is None else _i32(ir)
    where = C.c_int(-1)
    rule = lib().oracle_check(nrows, ncols, nnz, None if irp is None else irp.ctypes.data, jc.ctypes.data, ioff,
                              C.byref(where))
    return rule, where.value


def compress_inds(coli, ncols, ioff=0):
    coli = _i32(coli)
    out = np.zeros(ncols + 1, dtype=np.int32)
    lib().oracle_compress_inds(coli.ctypes.data, ncols, out.ctypes.data, coli.size, ioff)
    return out


def uncompress_inds(jc, ioff=0):
    jc = _i32(jc)
    ncols = jc.size - 1
    out = np.zeros(int(jc[-1]) - ioff, dtype=np.int32)
    lib().oracle_uncompress_inds(jc.ctypes.data, ncols, out.ctypes.data, ioff)
    return out


def within_tolerance(x, ref64, sumabs, rtol=1e-4):
    """The path's float tolerance. Per element the error measure is
    min(|x-ref|/|ref|, |x-ref|/sum|terms|): the plain relative error, or, where the terms of
    a sum cancel, the error relative to the magnitude that was summed.
    Returns (ok, worst measure)."""
    x = np.asarray(x, dtype=np.float64)
    err = np.abs(x - ref64)
    with np.errstate(divide="ignore", invalid="ignore"):
        rel = np.where(err == 0, 0.0, err / np.abs(ref64))
        scaled = np.where(err == 0, 0.0, err / np.asarray(sumabs, dtype=np.float64))
    m = np.minimum(rel, scaled)
    m = np.where(np.isnan(m), np.inf, m)
    worst = float(m.max(initial=0.0))
    return worst <= rtol, worst
