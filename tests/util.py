"""Helpers shared by the tests: random CSC matrices, device wrappers around the C ABI."""
import ctypes as C

import numpy as np

from bidmat_amd import hip_abi
from bidmat_amd.device import DeviceArray


def random_csc(rng, nrows, ncols, density=0.2, sort_rows=True, lengths=None, unique=True):
    """Random 0-based CSC. lengths: optional explicit column lengths."""
    if lengths is None:
        lengths = rng.binomial(nrows, density, size=ncols)
    lengths = np.asarray(lengths, dtype=np.int64)
    jc = np.zeros(ncols + 1, dtype=np.int32)
    jc[1:] = np.cumsum(lengths)
    ir = np.empty(int(jc[-1]), dtype=np.int32)
    for c in range(ncols):
        L = int(lengths[c])
        if unique:
            rows = rng.choice(nrows, size=L, replace=False)
        else:
            rows = rng.integers(0, nrows, size=L)
        if sort_rows:
            rows = np.sort(rows)
        ir[jc[c]:jc[c + 1]] = rows
    data = (1.0 - rng.random(ir.size)).astype(np.float32)     # U(0,1]
    return data, ir, jc


def dense_full(nrows, ncols, data, ir, jc):
    """full(S) as float64 2-D array (duplicates add up)."""
    S = np.zeros((nrows, ncols), dtype=np.float64)
    ic = np.repeat(np.arange(ncols), np.diff(jc))
    np.add.at(S, (ir, ic), data.astype(np.float64))
    return S


class Dev:
    """Uploads a set of numpy arrays and keeps the DeviceArrays alive."""

    def __init__(self, **arrays):
        self.lib = hip_abi.load()
        self._keep = {}
        for k, v in arrays.items():
            self.put(k, v)

    def put(self, name, a):
        d = DeviceArray.from_numpy(a)
        self._keep[name] = d
        setattr(self, name, d)
        return d

    def zeros(self, name, n, dtype=np.float32):
        d = DeviceArray.zeros(n, dtype)
        self._keep[name] = d
        setattr(self, name, d)
        return d

    def free(self):
        for d in self._keep.values():
            d.free()
        self._keep = {}


def make_plan(lib, nrows, ncols, nnz, d_ir, d_jc, k_hint=0):
    p = C.c_void_p()
    hip_abi.check(lib.bidmat_plan_create(nrows, ncols, nnz, d_ir.ptr, d_jc.ptr, k_hint, C.byref(p)), "plan_create")
    return p


def expand_cols(jc):
    return np.repeat(np.arange(jc.size - 1, dtype=np.int32), np.diff(jc)).astype(np.int32)
