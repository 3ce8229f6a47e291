"""ctypes binding of libbidmathip.so (the C ABI declared in include/bidmat_hip.h).

The library is the product; this module only loads it and declares the argument types.
There is no fallback: if the shared library has not been built, loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libbidmathip.so")

c_float_p = C.POINTER(C.c_float)
c_int_p = C.POINTER(C.c_int)
vp = C.c_void_p

# name -> (restype, argtypes); mirrors include/bidmat_hip.h declaration by declaration
SIGNATURES = {
    # reference-shaped launchers
    "bidmat_dsmult": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp]),
    "bidmat_dsmultT": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp]),
    "bidmat_dsmultTile": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, vp, C.c_int, vp, vp, vp, C.c_int, C.c_int, vp, C.c_int]),
    "bidmat_dsmultTileT": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, vp, C.c_int, vp, vp, vp, C.c_int, C.c_int, vp, C.c_int]),
    "bidmat_sdoprow": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, C.c_int, C.c_int]),
    "bidmat_sdopcol": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, C.c_int, C.c_int]),
    "bidmat_dds": (C.c_int, [C.c_int, C.c_int, vp, vp, vp, vp, vp]),
    "bidmat_dds0": (C.c_int, [C.c_int, C.c_int, vp, vp, vp, vp, vp]),
    "bidmat_spsum": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, C.c_int]),
    "bidmat_reduce1op": (C.c_int, [C.c_int, C.c_int, vp, vp, C.c_float, C.c_int]),
    "bidmat_reduce2op": (C.c_int, [C.c_int, C.c_int, vp, vp, C.c_float, C.c_int]),
    "bidmat_applyop": (C.c_int, [vp, C.c_int, C.c_int, vp, C.c_int, C.c_int, vp, C.c_int]),
    # native entries
    "bidmat_dsmult_csc": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp, C.c_int, vp]),
    "bidmat_dds_csc": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp, C.c_int, vp]),
    "bidmat_dds_csc_static": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp, C.c_int, vp]),
    "bidmat_dds_static_max_cols": (C.c_int, []),
    "bidmat_dds_csc_op": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp, C.c_int, vp, vp]),
    "bidmat_plan_set_values": (C.c_int, [vp, vp, vp]),
    "bidmat_dsmult_plan": (C.c_int, [vp, C.c_int, vp, vp, vp, vp, vp, C.c_int, vp]),
    "bidmat_dds_plan": (C.c_int, [vp, C.c_int, vp, vp, vp, vp, vp, C.c_int, vp, C.c_int, vp]),
    "bidmat_dds_plan_stored": (C.c_int, [vp, C.c_int, vp, vp, vp, vp, C.c_int, vp, vp]),
    "bidmat_plan_overflow_segments": (C.c_int, [vp]),
    "bidmat_plan_create": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, C.c_int, C.POINTER(vp)]),
    "bidmat_plan_destroy": (C.c_int, [vp]),
    "bidmat_plan_bytes": (C.c_longlong, [vp]),
    "bidmat_plan_segments": (C.c_int, [vp]),
    "bidmat_plan_info": (C.c_longlong, [vp, C.c_char_p]),
    "bidmat_plan_array": (C.c_int, [vp, C.c_char_p, C.POINTER(vp), C.POINTER(C.c_longlong)]),
    "bidmat_dsmultT_plan": (C.c_int, [vp, C.c_int, vp, vp, vp, C.c_int, vp]),
    "bidmat_dsmultT_plan_staged": (C.c_int, [vp, C.c_int, vp, vp, vp, C.c_int, vp, vp]),
    "bidmat_plan_heavy_nnz": (C.c_longlong, [vp]),
    "bidmat_spsum_cols": (C.c_int, [C.c_int, C.c_int, vp, vp, vp, C.c_int, vp]),
    "bidmat_spsum_rows_plan": (C.c_int, [vp, vp, vp, C.c_int, vp]),
    "bidmat_dds_dsmultT_plan": (C.c_int, [vp, C.c_int, vp, vp, vp, C.c_int, vp, vp, C.c_int, vp]),
    "bidmat_dds_dsmult_csc": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp, C.c_int, vp, vp, C.c_int, vp]),
    "bidmat_dds_dsmult_plan": (C.c_int, [vp, C.c_int, vp, vp, vp, vp, vp, C.c_int, vp, vp, C.c_int, vp]),
    "bidmat_spsum_rows_csc": (C.c_int, [C.c_int, C.c_int, vp, vp, vp, C.c_int, vp]),
    "bidmat_csc_expand_cols": (C.c_int, [C.c_int, C.c_int, vp, vp, vp]),
    "bidmat_csc_implicit_rows": (C.c_int, [C.c_int, C.c_int, vp, vp, vp]),
    "bidmat_csc_validate": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, C.POINTER(C.c_int)]),
    "bidmat_csc_colslice_range": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "bidmat_csc_colslice": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp, vp, vp, vp]),
    "bidmat_csc_transpose": (C.c_int, [C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp, vp]),
    "bidmat_full": (C.c_int, [vp, vp, vp, vp, C.c_int, C.c_int, C.c_int]),
    "bidmat_nhot": (C.c_int, [C.c_int, C.c_int, vp, vp, vp, vp, vp, C.POINTER(C.c_int)]),
    "bidmat_index_shift": (C.c_int, [vp, C.c_longlong, C.c_int, vp]),
    "bidmat_coo_compress_cols": (C.c_int, [C.c_int, C.c_int, vp, vp, vp]),
    "bidmat_sdtmult_csc": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, C.c_int, vp, C.c_int, vp]),
    "bidmat_sdmult_plan": (C.c_int, [vp, C.c_int, vp, vp, C.c_int, vp, C.c_int, vp]),
    "bidmat_transpose": (C.c_int, [C.c_int, C.c_int, vp, C.c_int, vp, C.c_int, vp]),
    "bidmat_applyop_flat": (C.c_int, [vp, vp, vp, C.c_longlong, C.c_int, vp]),
    # memory / runtime
    "bidmat_device_count": (C.c_int, [c_int_p]),
    "bidmat_set_device": (C.c_int, [C.c_int]),
    "bidmat_get_device": (C.c_int, [c_int_p]),
    "bidmat_malloc": (C.c_int, [C.POINTER(vp), C.c_longlong]),
    "bidmat_free": (C.c_int, [vp]),
    "bidmat_memcpy_h2d": (C.c_int, [vp, vp, C.c_longlong]),
    "bidmat_memcpy_d2h": (C.c_int, [vp, vp, C.c_longlong]),
    "bidmat_memcpy_d2d": (C.c_int, [vp, vp, C.c_longlong]),
    "bidmat_memcpy_h2d_async": (C.c_int, [vp, vp, C.c_longlong, vp]),
    "bidmat_memcpy_d2h_async": (C.c_int, [vp, vp, C.c_longlong, vp]),
    "bidmat_memset": (C.c_int, [vp, C.c_int, C.c_longlong]),
    "bidmat_mem_info": (C.c_int, [C.POINTER(C.c_longlong), C.POINTER(C.c_longlong)]),
    "bidmat_synchronize": (C.c_int, []),
    "bidmat_host_alloc": (C.c_int, [C.POINTER(vp), C.c_longlong]),
    "bidmat_host_free": (C.c_int, [vp]),
    "bidmat_stream_create": (C.c_int, [C.POINTER(vp)]),
    "bidmat_stream_destroy": (C.c_int, [vp]),
    "bidmat_stream_synchronize": (C.c_int, [vp]),
    "bidmat_graph_begin_capture": (C.c_int, [vp]),
    "bidmat_graph_end_capture": (C.c_int, [vp, C.POINTER(vp)]),
    "bidmat_graph_launch": (C.c_int, [vp, vp]),
    "bidmat_graph_destroy": (C.c_int, [vp]),
    "bidmat_event_create": (C.c_int, [C.POINTER(vp)]),
    "bidmat_event_destroy": (C.c_int, [vp]),
    "bidmat_event_record": (C.c_int, [vp, vp]),
    "bidmat_event_synchronize": (C.c_int, [vp]),
    "bidmat_event_elapsed_ms": (C.c_int, [vp, vp, c_float_p]),
    "bidmat_error_string": (C.c_char_p, [C.c_int]),
    "bidmat_version": (C.c_char_p, []),
    "bidmat_device_info": (C.c_int, [C.c_char_p, C.c_int, c_int_p, C.POINTER(C.c_longlong)]),
    "bidmat_set_option": (C.c_int, [C.c_char_p, C.c_longlong]),
    "bidmat_get_option": (C.c_longlong, [C.c_char_p]),
    "bidmat_release_caches": (C.c_int, []),
}

_lib = None


class BidmatError(RuntimeError):
    """A non-zero return code of the library (the reference throws RuntimeException with
    cudaGetErrorString on a non-zero launcher result, GMat.scala:1071)."""

    def __init__(self, where, code, text):
        super().__init__("%s: HIP error %d (%s)" % (where, code, text))
        self.code = code


def load():
    """Loads the in-tree shared library and returns the ctypes handle."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libbidmathip.so is not built (expected %s). Run `make -C bidmat_amd/csrc` or "
            "`python -c 'import __graft_entry__ as g; g.build()'`. There is no CPU fallback." % LIB_PATH)
    lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code, where="bidmathip"):
    if code != 0:
        text = load().bidmat_error_string(code)
        raise BidmatError(where, code, text.decode() if text else "?")
