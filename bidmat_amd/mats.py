"""Python face of the host-side mirror (libbidmathost.so): GMat / GSMat objects with BIDMat's
operator names, for scripts and tests. All arithmetic happens in the HIP library; this module
only moves handles around.

    a * s            GMat * GSMat            (GMat.scala:1684)
    a.xT(s)          a *^ s                  (GMat.scala:1686, alias xT :1688)
    DDS(a, b, s)     a ^* (b @@ s)           (MatFunctions.scala:1656-1674)
    sum(s, n), sum(a, n)                     (SFunctions.scala:10-15, GFunctions.scala:227)
    a / b            elementwise             (GMat.scala:1681)
    c.madd / c.maddT via out=...             (the `c ~ a * b` output-reuse form)
"""
import ctypes as C
import os

import numpy as np

from . import hip_abi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libbidmathost.so")
_lib = None
vp = C.c_void_p


def _load():
    global _lib
    if _lib is None:
        hip_abi.load()          # raises if the HIP library is missing; RTLD_GLOBAL for the host layer
        if not os.path.exists(LIB_PATH):
            raise ImportError("libbidmathost.so is not built; run `make -C bidmat_amd/host`")
        L = C.CDLL(LIB_PATH)
        for name in ("bmh_gmat_from_host", "bmh_gmat_zeros", "bmh_gsmat_from_host", "bmh_mult", "bmh_madd",
                     "bmh_multT", "bmh_maddT", "bmh_dds", "bmh_sum_sparse", "bmh_sum_dense", "bmh_reduce",
                     "bmh_gop", "bmh_contents", "bmh_with_values", "bmh_tile_mult", "bmh_sdmult", "bmh_gsdop", "bmh_load_gsmat", "bmh_colslice", "bmh_nhot", "bmh_full", "bmh_t"):
            getattr(L, name).restype = vp
        L.bmh_gmat_from_host.argtypes = [C.c_int, C.c_int, vp]
        L.bmh_gmat_zeros.argtypes = [C.c_int, C.c_int]
        L.bmh_gsmat_from_host.argtypes = [C.c_int, C.c_int, C.c_int, vp, vp, vp]
        for name in ("bmh_mult", "bmh_madd", "bmh_multT", "bmh_maddT"):
            getattr(L, name).argtypes = [vp, vp, vp]
        L.bmh_dds.argtypes = [vp, vp, vp, vp]
        L.bmh_sdmult.argtypes = [vp, vp, vp, C.c_int]
        L.bmh_gsdop.argtypes = [vp, vp, vp, C.c_int]
        L.bmh_colslice.argtypes = [vp, C.c_int, C.c_int, vp]
        L.bmh_nhot.argtypes = [vp, C.c_int, C.c_int, C.c_int]
        L.bmh_full.argtypes = [vp, vp]
        L.bmh_t.argtypes = [vp, vp]
        L.bmh_load_gsmat.argtypes = [C.c_char_p]
        ip = C.POINTER(C.c_int)
        L.bmh_save_smat.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_int, vp, vp, vp]
        L.bmh_load_smat.argtypes = [C.c_char_p, ip, ip, ip, vp, vp, vp]
        L.bmh_save_fmat.argtypes = [C.c_char_p, C.c_int, C.c_int, vp]
        L.bmh_load_fmat.argtypes = [C.c_char_p, ip, ip, vp]
        L.bmh_tile_mult.argtypes = [vp] + [C.c_int] * 5 + [vp, C.c_int, C.c_int, vp, C.c_int, C.c_int, C.c_int]
        L.bmh_sum_sparse.argtypes = [vp, C.c_int, vp]
        L.bmh_sum_dense.argtypes = [vp, C.c_int, vp]
        L.bmh_reduce.argtypes = [vp, vp, C.c_int, C.c_float, C.c_int]
        L.bmh_gop.argtypes = [vp, vp, vp, C.c_int]
        L.bmh_contents.argtypes = [vp]
        L.bmh_with_values.argtypes = [vp, vp]
        L.bmh_release.argtypes = [vp]
        L.bmh_release.restype = None
        L.bmh_last_error.restype = C.c_char_p
        L.bmh_type.restype = C.c_char_p
        L.bmh_type.argtypes = [vp]
        L.bmh_guid.restype = C.c_longlong
        L.bmh_guid.argtypes = [vp]
        L.bmh_same_object.argtypes = [vp, vp]
        L.bmh_same_pattern.argtypes = [vp, vp]
        L.bmh_has_plan.argtypes = [vp]
        L.bmh_gmat_dims.argtypes = [vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        L.bmh_gmat_to_host.argtypes = [vp, vp]
        L.bmh_gsmat_dims.argtypes = [vp, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]
        L.bmh_gsmat_to_host.argtypes = [vp, vp, vp, vp]
        L.bmh_gsmat_device_jc.argtypes = [vp, vp]
        L.bmh_nflops.restype = C.c_longlong
        L.bmh_gflop.restype = C.c_double
        L.bmh_gflop.argtypes = [C.POINTER(C.c_float)]
        L.bmh_set_flag.argtypes = [C.c_char_p, C.c_double]
        L.bmh_get_flag.argtypes = [C.c_char_p]
        L.bmh_get_flag.restype = C.c_double
        L.bmh_smat_check.argtypes = [C.c_int, C.c_int, C.c_int, vp, vp]
        _lib = L
    return _lib


def _ok(h):
    if not h:
        raise RuntimeError(_load().bmh_last_error().decode())
    return h


class Mat:
    """Global flags (object Mat in the reference)."""

    @staticmethod
    def set(name, value):
        if _load().bmh_set_flag(name.encode(), float(value)) != 0:
            raise KeyError(name)

    @staticmethod
    def get(name):
        return _load().bmh_get_flag(name.encode())

    @staticmethod
    def nflops():
        return _load().bmh_nflops()

    @staticmethod
    def clear_caches():
        _load().bmh_clear_caches()


def flip():
    _load().bmh_flip()


def gflop():
    secs = C.c_float(0)
    g = _load().bmh_gflop(C.byref(secs))
    return g, secs.value


class _Handle:
    def __init__(self, h):
        self._h = _ok(h)

    def __del__(self):
        try:
            if self._h:
                _load().bmh_release(self._h)
                self._h = None
        except Exception:
            pass

    @property
    def mytype(self):
        return _load().bmh_type(self._h).decode()

    @property
    def GUID(self):
        return _load().bmh_guid(self._h)

    def same(self, other):
        return bool(_load().bmh_same_object(self._h, other._h))


class GMat(_Handle):
    @classmethod
    def from_numpy(cls, a):
        a = np.asfortranarray(a, dtype=np.float32)
        if a.ndim == 1:
            a = a.reshape(-1, 1, order="F")
        flat = np.ascontiguousarray(a.ravel(order="F"))
        return cls(_load().bmh_gmat_from_host(a.shape[0], a.shape[1], flat.ctypes.data))

    @classmethod
    def zeros(cls, nr, nc):
        return cls(_load().bmh_gmat_zeros(nr, nc))

    @property
    def shape(self):
        nr, nc = C.c_int(), C.c_int()
        _load().bmh_gmat_dims(self._h, C.byref(nr), C.byref(nc))
        return nr.value, nc.value

    def numpy(self):
        nr, nc = self.shape
        out = np.empty(nr * nc, dtype=np.float32)
        if _load().bmh_gmat_to_host(self._h, out.ctypes.data) != 0:
            raise RuntimeError(_load().bmh_last_error().decode())
        return out.reshape(nc, nr).T

    def __mul__(self, s):                 # a * s
        return GMat(_load().bmh_mult(self._h, s._h, None))

    def GSMult(self, s, out=None):
        return GMat(_load().bmh_mult(self._h, s._h, out._h if out else None))

    def madd(self, s, out):
        return GMat(_load().bmh_madd(self._h, s._h, out._h))

    def xT(self, s):                      # a *^ s
        return GMat(_load().bmh_multT(self._h, s._h, None))

    def GSMultT(self, s, out=None):
        return GMat(_load().bmh_multT(self._h, s._h, out._h if out else None))

    def maddT(self, s, out):
        return GMat(_load().bmh_maddT(self._h, s._h, out._h))

    def tileMult(self, nr, nc, kk, aroff, acoff, b, broff, bcoff, c, croff, ccoff):
        return GMat(_load().bmh_tile_mult(self._h, nr, nc, kk, aroff, acoff, b._h, broff, bcoff, c._h, croff, ccoff, 0))

    def tileMultNT(self, nr, nc, kk, aroff, acoff, b, broff, bcoff, c, croff, ccoff):
        return GMat(_load().bmh_tile_mult(self._h, nr, nc, kk, aroff, acoff, b._h, broff, bcoff, c._h, croff, ccoff, 1))

    def gOp(self, b, op, out=None):
        return GMat(_load().bmh_gop(self._h, b._h, out._h if out else None, op))

    def __truediv__(self, b):
        return self.gOp(b, 3)

    def reduceOp(self, dir, initv, op, out=None):
        return GMat(_load().bmh_reduce(self._h, out._h if out else None, dir, initv, op))


class GSMat(_Handle):
    @classmethod
    def from_csc(cls, nrows, ncols, data, ir, jc):
        """Host SMat arrays; ir / jc carry the base Mat.get('ioneBased')."""
        data = np.ascontiguousarray(data, dtype=np.float32)
        ir = np.ascontiguousarray(ir, dtype=np.int32)
        jc = np.ascontiguousarray(jc, dtype=np.int32)
        return cls(_load().bmh_gsmat_from_host(nrows, ncols, data.size, data.ctypes.data, ir.ctypes.data, jc.ctypes.data))

    @classmethod
    def nHot(cls, cats, ncats=0):
        """GSMat.nHot / oneHot: cats is an n x ncols (or 1-D = one-hot) array of 0-based categories."""
        cats = np.asarray(cats, dtype=np.int32)
        if cats.ndim == 1:
            cats = cats.reshape(1, -1)
        n, ncols = cats.shape
        flat = np.ascontiguousarray(cats.T).ravel()                  # column-major
        return cls(_load().bmh_nhot(flat.ctypes.data, n, ncols, ncats))

    oneHot = nHot

    @property
    def dims(self):
        nr, nc, nnz = C.c_int(), C.c_int(), C.c_int()
        _load().bmh_gsmat_dims(self._h, C.byref(nr), C.byref(nc), C.byref(nnz))
        return nr.value, nc.value, nnz.value

    def to_csc(self):
        """Back to host SMat arrays (with SparseMat.check applied): (data, ir, jc)."""
        nr, nc, nnz = self.dims
        data = np.empty(nnz, np.float32)
        ir = np.empty(nnz, np.int32)
        jc = np.empty(nc + 1, np.int32)
        if _load().bmh_gsmat_to_host(self._h, data.ctypes.data, ir.ctypes.data, jc.ctypes.data) != 0:
            raise RuntimeError(_load().bmh_last_error().decode())
        return data, ir, jc

    def same_pattern(self, other):
        """True when both matrices point at the same device index arrays."""
        return bool(_load().bmh_same_pattern(self._h, other._h))

    def has_plan(self):
        return bool(_load().bmh_has_plan(self._h))

    def device_jc(self):
        nr, nc, nnz = self.dims
        jc = np.empty(nc + 1, np.int32)
        hip_abi.check(_load().bmh_gsmat_device_jc(self._h, jc.ctypes.data))
        return jc

    def contents(self):
        return GMat(_load().bmh_contents(self._h))

    def t(self, out=None):                        # transpose, computed on the device
        return GSMat(_load().bmh_t(self._h, out._h if out else None))

    def full(self, out=None):                     # dense image as a GMat
        return GMat(_load().bmh_full(self._h, out._h if out else None))

    def colslice(self, col1, col2, out=None):     # columns [col1, col2)
        return GSMat(_load().bmh_colslice(self._h, col1, col2, out._h if out else None))

    def GSDop(self, b, op, out=None):     # s op edge-vector (row vector, column vector or 1x1)
        return GSMat(_load().bmh_gsdop(self._h, b._h, out._h if out else None, op))

    def __mul__(self, a):                 # s * a   (sparse times dense)
        return GMat(_load().bmh_sdmult(self._h, a._h, None, 0))

    def SDMult(self, a, out=None):
        return GMat(_load().bmh_sdmult(self._h, a._h, out._h if out else None, 0))

    def Tx(self, a):                      # s ^* a  (sparse-transpose times dense)
        return GMat(_load().bmh_sdmult(self._h, a._h, None, 1))

    def SDTMult(self, a, out=None):
        return GMat(_load().bmh_sdmult(self._h, a._h, out._h if out else None, 1))

    def with_values(self, vals):
        return GSMat(_load().bmh_with_values(self._h, vals._h))

    def sum(self, n=0, out=None):
        return GMat(_load().bmh_sum_sparse(self._h, n, out._h if out else None))


def DDS(a, b, c, out=None):
    return GSMat(_load().bmh_dds(a._h, b._h, c._h, out._h if out else None))


def sum(a, n=0, out=None):      # noqa: A001  (the reference's name)
    if isinstance(a, GSMat):
        return a.sum(n, out)
    return GMat(_load().bmh_sum_dense(a._h, n, out._h if out else None))


def saveSMat(fname, nrows, ncols, data, ir, jc):
    """HMat.saveSMat: host SMat arrays (base Mat.ioneBased) to a type-231 file (0-based on disk)."""
    data = np.ascontiguousarray(data, dtype=np.float32)
    ir = np.ascontiguousarray(ir, dtype=np.int32)
    jc = np.ascontiguousarray(jc, dtype=np.int32)
    if _load().bmh_save_smat(os.fsencode(fname), nrows, ncols, data.size, data.ctypes.data, ir.ctypes.data, jc.ctypes.data) != 0:
        raise RuntimeError(_load().bmh_last_error().decode())


def loadSMat(fname):
    """HMat.loadSMat: returns (nrows, ncols, data, ir, jc) with indices in base Mat.ioneBased."""
    nr, nc, nnz = C.c_int(), C.c_int(), C.c_int()
    L = _load()
    if L.bmh_load_smat(os.fsencode(fname), C.byref(nr), C.byref(nc), C.byref(nnz), None, None, None) != 0:
        raise RuntimeError(L.bmh_last_error().decode())
    data = np.empty(nnz.value, np.float32)
    ir = np.empty(nnz.value, np.int32)
    jc = np.empty(nc.value + 1, np.int32)
    if L.bmh_load_smat(os.fsencode(fname), C.byref(nr), C.byref(nc), C.byref(nnz), data.ctypes.data, ir.ctypes.data, jc.ctypes.data) != 0:
        raise RuntimeError(L.bmh_last_error().decode())
    return nr.value, nc.value, data, ir, jc


def saveFMat(fname, a):
    a = np.asfortranarray(a, dtype=np.float32)
    flat = np.ascontiguousarray(a.ravel(order="F"))
    if _load().bmh_save_fmat(os.fsencode(fname), a.shape[0], a.shape[1], flat.ctypes.data) != 0:
        raise RuntimeError(_load().bmh_last_error().decode())


def loadFMat(fname):
    nr, nc = C.c_int(), C.c_int()
    L = _load()
    if L.bmh_load_fmat(os.fsencode(fname), C.byref(nr), C.byref(nc), None) != 0:
        raise RuntimeError(L.bmh_last_error().decode())
    out = np.empty(nr.value * nc.value, np.float32)
    if L.bmh_load_fmat(os.fsencode(fname), C.byref(nr), C.byref(nc), out.ctypes.data) != 0:
        raise RuntimeError(L.bmh_last_error().decode())
    return out.reshape(nc.value, nr.value).T


def loadGSMat(fname):
    """A type-231 file straight onto the device (pinned, double-buffered upload)."""
    return GSMat(_load().bmh_load_gsmat(os.fsencode(fname)))


def smat_check(nrows, ncols, ir, jc):
    """SparseMat.check on host arrays; raises RuntimeError with the reference's message."""
    ir = np.ascontiguousarray(ir, dtype=np.int32)
    jc = np.ascontiguousarray(jc, dtype=np.int32)
    if _load().bmh_smat_check(nrows, ncols, ir.size, ir.ctypes.data, jc.ctypes.data) != 0:
        raise RuntimeError(_load().bmh_last_error().decode())
