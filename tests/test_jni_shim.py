"""The JNI shim (bidmat_amd/csrc/jni_shim.cpp) on a machine without a JDK: it must parse as C++
against a stand-in <jni.h> (tests/stubs, type names only), define one
Java_edu_berkeley_bid_HIPMAT_<name> per `native` method of the Java stub class that
INTEGRATION.md shows, with the same number of arguments and a matching return type, and call
only functions that include/bidmat_hip.h declares.
"""
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHIM = os.path.join(ROOT, "bidmat_amd", "csrc", "jni_shim.cpp")
STUBS = os.path.join(ROOT, "tests", "stubs")
JTYPES = {"int": "jint", "long": "jlong", "float": "jfloat", "String": "jstring", "int[]": "jintArray",
          "float[]": "jfloatArray"}


def shim_functions():
    """name -> (return type, [argument types]) of every JFN(...) definition."""
    text = open(SHIM).read()
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for m in re.finditer(r"JFN\((\w+),\s*(\w+)\)\(([^)]*)\)", text):
        ret, name, args = m.group(1), m.group(2), [a.strip() for a in m.group(3).split(",")]
        assert args[0].startswith("JNIEnv*") and args[1].startswith("jclass"), name
        out[name] = (ret, [a.split()[0] for a in args[2:]])
    return out


def java_stub_methods():
    """name -> (return type, [argument types]) of the HIPMAT class in INTEGRATION.md."""
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = text[text.index("public final class HIPMAT"):]
    block = block[: block.index("```")]
    block = re.sub(r"//[^\n]*", "", block)
    out = {}
    for m in re.finditer(r"public static native\s+(\w+)\s+(\w+)\s*\(([^)]*)\)\s*;", block, flags=re.S):
        ret, name, args = m.group(1), m.group(2), m.group(3).strip()
        types = []
        for a in (x.strip() for x in args.split(",") if x.strip()):
            t, _ = a.rsplit(None, 1)
            types.append(t.replace(" ", ""))
        out[name] = (ret, types)
    return out


def test_shim_parses_with_the_stand_in_header():
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-I" + STUBS, SHIM], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_shim_defines_exactly_the_java_stub_methods():
    shim, java = shim_functions(), java_stub_methods()
    assert len(java) >= 30
    assert set(shim) == set(java), "only in shim: %s; only in Java stub: %s" % (
        sorted(set(shim) - set(java)), sorted(set(java) - set(shim)))
    for name, (jret, jargs) in java.items():
        sret, sargs = shim[name]
        assert JTYPES[jret] == sret, name
        assert [JTYPES[a] for a in jargs] == sargs, name


def test_shim_symbols_after_preprocessing():
    """The preprocessed shim defines Java_edu_berkeley_bid_HIPMAT_<name> for the reference-shaped path."""
    r = subprocess.run(["g++", "-std=c++17", "-E", "-I" + STUBS, SHIM], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    names = set(re.findall(r"Java_edu_berkeley_bid_HIPMAT_(\w+)", r.stdout))
    for n in ("dsmult", "dsmultT", "dds", "dds0", "spsum", "reduce1op", "reduce2op", "applyop", "dsmultTile",
              "sdoprow", "sdopcol"):
        assert n in names, n


def test_shim_calls_only_declared_functions():
    header = open(os.path.join(ROOT, "include", "bidmat_hip.h")).read()
    declared = set(re.findall(r"\b(bidmat_\w+)\s*\(", header))
    used = set(re.findall(r"\b(bidmat_\w+)\s*\(", open(SHIM).read()))
    assert used <= declared, sorted(used - declared)
