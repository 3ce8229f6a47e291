"""Seeded synthetic matrices for the benchmark configurations (ctypes over libbidmatgen.so).

All generators are deterministic functions of their seed; dense matrices are returned as
1-D float32 arrays in column-major order (k*ncols), sparse patterns as 0-based CSC
(ir int32[nnz] sorted inside each column, jc int32[ncols+1]).
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libbidmatgen.so")
_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("libbidmatgen.so is not built; run `make -C bidmat_amd/gen`")
        lib = C.CDLL(LIB_PATH)
        vp, u64, ll = C.c_void_p, C.c_uint64, C.c_longlong
        lib.gen_uniform.argtypes = [vp, ll, u64, C.c_float, C.c_float]
        lib.gen_uniform_open0.argtypes = [vp, ll, u64]
        lib.gen_normal.argtypes = [vp, ll, u64, C.c_float, C.c_float]
        lib.gen_exponential.argtypes = [vp, ll, u64]
        lib.gen_lengths_const.argtypes = [vp, C.c_int, C.c_int]
        lib.gen_lengths_poisson.argtypes = [vp, C.c_int, C.c_double, u64, C.c_int]
        lib.gen_lengths_pareto.argtypes = [vp, C.c_int, C.c_double, C.c_double, C.c_int, C.c_int, u64]
        lib.gen_jc_from_lengths.argtypes = [vp, C.c_int, vp]
        lib.gen_jc_from_lengths.restype = ll
        lib.gen_rows.argtypes = [C.c_int, C.c_int, vp, vp, C.c_int, C.c_double, u64]
        lib.gen_rows.restype = C.c_int
        lib.gen_max_threads.restype = C.c_int
        for f in ("gen_uniform", "gen_uniform_open0", "gen_normal", "gen_exponential",
                  "gen_lengths_const", "gen_lengths_poisson", "gen_lengths_pareto"):
            getattr(lib, f).restype = None
        _lib = lib
    return _lib


def uniform(n, seed, lo=0.0, hi=1.0):
    out = np.empty(int(n), dtype=np.float32)
    _load().gen_uniform(out.ctypes.data, out.size, seed, lo, hi)
    return out


def uniform_open0(n, seed):
    """U(0,1]: never zero."""
    out = np.empty(int(n), dtype=np.float32)
    _load().gen_uniform_open0(out.ctypes.data, out.size, seed)
    return out


def normal(n, seed, mean=0.0, sigma=1.0):
    out = np.empty(int(n), dtype=np.float32)
    _load().gen_normal(out.ctypes.data, out.size, seed, mean, sigma)
    return out


def exponential(n, seed):
    out = np.empty(int(n), dtype=np.float32)
    _load().gen_exponential(out.ctypes.data, out.size, seed)
    return out


def pattern(nrows, ncols, lengths, rows, seed):
    """CSC pattern. lengths: ("const", L) | ("poisson", lam) | ("pareto", xm, alpha, lo, hi);
    rows: ("uniform",) | ("zipf", s). Rows are drawn until each column holds its length in
    DISTINCT rows, then sorted. Returns (ir, jc)."""
    lib = _load()
    ln = np.empty(ncols, dtype=np.int32)
    if lengths[0] == "const":
        lib.gen_lengths_const(ln.ctypes.data, ncols, int(lengths[1]))
    elif lengths[0] == "poisson":
        lib.gen_lengths_poisson(ln.ctypes.data, ncols, float(lengths[1]), seed, nrows)
    elif lengths[0] == "pareto":
        _, xm, alpha, lo, hi = lengths
        lib.gen_lengths_pareto(ln.ctypes.data, ncols, float(xm), float(alpha), int(lo), min(int(hi), nrows), seed)
    else:
        raise ValueError(lengths)
    jc = np.empty(ncols + 1, dtype=np.int32)
    nnz = lib.gen_jc_from_lengths(ln.ctypes.data, ncols, jc.ctypes.data)
    if nnz < 0:
        raise ValueError("pattern does not fit int32 indexing")
    ir = np.empty(int(nnz), dtype=np.int32)
    dist = 1 if rows[0] == "zipf" else 0
    s = float(rows[1]) if dist == 1 else 0.0
    if lib.gen_rows(nrows, ncols, jc.ctypes.data, ir.ctypes.data, dist, s, seed) != 0:
        raise ValueError("a column asks for more distinct rows than the matrix has")
    return ir, jc


# The five benchmark configurations, parameterised by a scale in (0,1] that shrinks the
# number of columns (and for the big ones the number of rows) but keeps k and the per-column
# statistics. scale=1 is the full configuration.
def config(name, scale=1.0):
    sc = lambda x, lo=1: max(lo, int(round(x * scale)))
    if name == "C1":      # A*S on the CPU-runnable case
        k, m, n = 32, 4096, sc(8192, 8)
        ir, jc = pattern(m, n, ("const", 50), ("uniform",), 1)
        return dict(name=name, op="dsmult", k=k, nrows=m, ncols=n, ir=ir, jc=jc,
                    A=normal(k * m, 11), vals=uniform_open0(ir.size, 12))
    if name in ("C2", "C3", "HEAD"):   # the Zipf(1.1) 100000 x 500000 pattern at k=256
        k, m, n = 256, sc(100000, 1000), sc(500000, 64)
        ir, jc = pattern(m, n, ("poisson", 200), ("zipf", 1.1), 2)
        d = dict(name=name, k=k, nrows=m, ncols=n, ir=ir, jc=jc)
        if name in ("C2", "HEAD"):
            d.update(op="dds", A=uniform(k * m, 21), B=uniform(k * n, 22))
        if name in ("C3", "HEAD"):
            d.update(A_T=normal(k * n, 31), vals=uniform_open0(ir.size, 32))
            if name == "C3":
                d.update(op="dsmultT")
        if name == "HEAD":
            d.update(op="all", A_S=d["A"])
        return d
    if name == "C4":      # wide latent dimension, Pareto column lengths
        k, m, n = 1024, sc(200000, 60000), sc(1000000, 64)
        ir, jc = pattern(m, n, ("pareto", 13.3, 1.5, 1, 50000), ("uniform",), 4)
        return dict(name=name, op="dsmult", k=k, nrows=m, ncols=n, ir=ir, jc=jc,
                    A=normal(k * m, 41, 0.0, 0.02), vals=uniform_open0(ir.size, 42))
    if name == "C5":      # fused NMF multiplicative-update step
        k, m, n = 128, sc(1000000, 1000), sc(1000000, 64)
        ir, jc = pattern(m, n, ("poisson", 400), ("zipf", 1.05), 5)
        return dict(name=name, op="nmf", k=k, nrows=m, ncols=n, ir=ir, jc=jc,
                    W=uniform(k * m, 51, 0.01, 1.0), H=uniform(k * n, 52, 0.01, 1.0),
                    vals=exponential(ir.size, 53))
    raise ValueError(name)
