"""The C-ABI shared library loads without a GPU and exports every symbol that
include/bidmat_hip.h declares, with the argument counts the ctypes binding uses."""
import ctypes as C
import os
import re
import subprocess

from bidmat_amd import hip_abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "bidmat_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = {}
    for m in re.finditer(r"\b(?:int|long long|const char \*|const char\*)\s*\*?\s*(bidmat_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        name, args = m.group(1), m.group(2).strip()
        nargs = 0 if args in ("", "void") else len([a for a in args.split(",") if a.strip()])
        decls[name] = nargs
    return decls


def test_header_declares_the_path():
    d = declared_functions()
    for fn in ("bidmat_dsmult", "bidmat_dsmultT", "bidmat_dds", "bidmat_spsum", "bidmat_reduce1op",
               "bidmat_reduce2op", "bidmat_applyop", "bidmat_dsmult_csc", "bidmat_dds_csc",
               "bidmat_dsmultT_plan", "bidmat_plan_create", "bidmat_csc_expand_cols"):
        assert fn in d, fn
    assert len(d) >= 45


def test_library_exports_every_declared_symbol():
    lib = hip_abi.load()
    d = declared_functions()
    for name, nargs in d.items():
        assert hasattr(lib, name), "libbidmathip.so does not export %s" % name
        assert name in hip_abi.SIGNATURES, "ctypes binding misses %s" % name
        assert len(hip_abi.SIGNATURES[name][1]) == nargs, "argument count of %s" % name
    # and nothing in the binding that the header does not declare
    assert set(hip_abi.SIGNATURES) == set(d)


def test_reference_shaped_argument_lists_match_the_reference_stubs():
    """CUMAT.java:143,152,211,209,111,119,31: same number and order of arguments."""
    d = declared_functions()
    assert d["bidmat_dsmult"] == 8 and d["bidmat_dsmultT"] == 8
    assert d["bidmat_dds"] == 7 and d["bidmat_spsum"] == 8
    assert d["bidmat_reduce1op"] == 6 and d["bidmat_reduce2op"] == 6 and d["bidmat_applyop"] == 8


def test_no_compute_without_gpu_helpers_work():
    lib = hip_abi.load()
    assert lib.bidmat_version().startswith(b"bidmathip")
    assert lib.bidmat_get_option(b"seglen") >= 64
    assert lib.bidmat_set_option(b"seglen", 1) == 1            # rejected, unchanged
    assert lib.bidmat_set_option(b"nonsense", 5) == 1
    assert lib.bidmat_get_option(b"nonsense") == -2
    # every documented option: default inside its range, a set/get round trip, out-of-range values refused
    for name, good, bad in ((b"seglen", 512, 0), (b"panel_kb", 1024, 1), (b"heavy_min", 4, 0), (b"col_classes", 1, 2),
                            (b"class_hot", 16, 5000), (b"class_threads", 512, 300), (b"class_strip", 8, 65),
                            (b"class_phases", 4, 3), (b"plan_keep_mb", 0, -1), (b"dense_rows", 64, 100),
                            (b"dense_min_pct", 30, 0), (b"dense_min_nnz", 0, -1), (b"dense_cb", 64, -1),
                            (b"scalar_values", 0, 2)):
        old = lib.bidmat_get_option(name)
        assert old != -2, name
        assert lib.bidmat_set_option(name, bad) == 1 and lib.bidmat_get_option(name) == old, name
        assert lib.bidmat_set_option(name, good) == 0 and lib.bidmat_get_option(name) == good, name
        assert lib.bidmat_set_option(name, old) == 0
    assert lib.bidmat_error_string(0)
    # argument validation happens before any device work
    assert lib.bidmat_dsmult(-1, 1, 1, None, None, None, None, None) == 1
    assert lib.bidmat_plan_destroy(None) == 0


def test_library_has_no_oracle_or_torch_dependency():
    out = subprocess.check_output(["ldd", hip_abi.LIB_PATH]).decode()
    assert "oracle" not in out and "torch" not in out
    assert "libamdhip64" in out


def test_product_sources_never_touch_the_oracle():
    pkg = os.path.join(ROOT, "bidmat_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".hpp", ".h")):
                text = open(os.path.join(base, f), errors="ignore").read()
                assert "import oracle" not in text and "bidmat_oracle" not in text, os.path.join(base, f)
