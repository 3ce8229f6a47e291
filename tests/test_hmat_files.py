"""BIDMat matrix files on this path (HMat.scala:1232-1266, 1444-1480 for SMat; 337-399, 876-891
for FMat): little-endian int32 header [type, nrows, ncols, nnz], 0-based indices on disk, host
matrices in base Mat.ioneBased. Files are checked byte for byte against a numpy writer that
follows the format description, in both directions."""
import gzip
import struct

import numpy as np
import pytest

from bidmat_amd import mats
from util import random_csc


def numpy_smat_bytes(nrows, ncols, data, ir0, jc0):
    return (struct.pack("<4i", 231, nrows, ncols, data.size) + jc0.astype("<i4").tobytes()
            + ir0.astype("<i4").tobytes() + data.astype("<f4").tobytes())


def test_smat_file_round_trip_and_layout(tmp_path):
    rng = np.random.default_rng(1)
    nrows, ncols = 17, 23
    data, ir0, jc0 = random_csc(rng, nrows, ncols, 0.2)
    f = tmp_path / "s.smat"
    mats.saveSMat(f, nrows, ncols, data, ir0 + 1, jc0 + 1)               # host arrays are 1-based
    assert f.read_bytes() == numpy_smat_bytes(nrows, ncols, data, ir0, jc0)   # 0-based on disk
    nr, nc, d2, ir2, jc2 = mats.loadSMat(f)
    assert (nr, nc) == (nrows, ncols)
    assert np.array_equal(d2, data) and np.array_equal(ir2, ir0 + 1) and np.array_equal(jc2, jc0 + 1)
    # a file written by another program (numpy here) loads the same way
    g = tmp_path / "other.smat"
    g.write_bytes(numpy_smat_bytes(nrows, ncols, data, ir0, jc0))
    assert np.array_equal(mats.loadSMat(g)[3], ir0 + 1)
    # base 0 host matrices
    mats.Mat.set("ioneBased", 0)
    try:
        mats.saveSMat(f, nrows, ncols, data, ir0, jc0)
        assert f.read_bytes() == numpy_smat_bytes(nrows, ncols, data, ir0, jc0)
        assert np.array_equal(mats.loadSMat(f)[3], ir0)
    finally:
        mats.Mat.set("ioneBased", 1)


def test_smat_gzip_and_errors(tmp_path):
    rng = np.random.default_rng(2)
    data, ir0, jc0 = random_csc(rng, 9, 11, 0.3)
    f = tmp_path / "s.smat.gz"
    mats.saveSMat(f, 9, 11, data, ir0 + 1, jc0 + 1)
    assert gzip.decompress(f.read_bytes()) == numpy_smat_bytes(9, 11, data, ir0, jc0)
    assert np.array_equal(mats.loadSMat(f)[2], data)
    bad = tmp_path / "bad.smat"
    bad.write_bytes(struct.pack("<4i", 130, 2, 2, 0))
    with pytest.raises(RuntimeError, match="loadSMat expected type field 231 or 331 but was 130"):
        mats.loadSMat(bad)
    bad.write_bytes(struct.pack("<4i", 431, 2, 2, 1) + b"\0" * 16)
    with pytest.raises(RuntimeError, match="231 or 331 but was 431"):
        mats.loadSMat(bad)
    bad.write_bytes(numpy_smat_bytes(9, 11, data, ir0, jc0)[:-5])
    with pytest.raises(RuntimeError, match="unexpected end of file"):
        mats.loadSMat(bad)
    with pytest.raises(RuntimeError, match="lz4"):
        mats.loadSMat(tmp_path / "x.smat.lz4")
    with pytest.raises(RuntimeError, match="cannot open"):
        mats.loadSMat(tmp_path / "missing.smat")


def numpy_smat331_bytes(nrows, ncols, data, jc0):
    return struct.pack("<4i", 331, nrows, ncols, data.size) + jc0.astype("<i4").tobytes() + data.astype("<f4").tobytes()


def test_smat_file_without_row_indices(tmp_path):
    """Type 331 (HMat.scala:1246-1258, 1447-1451): no ir on disk; element j of a column sits in row j."""
    rng = np.random.default_rng(5)
    nrows, ncols = 12, 9
    lens = rng.integers(0, nrows + 1, size=ncols)
    lens[3], lens[4] = 0, nrows
    jc0 = np.zeros(ncols + 1, dtype=np.int32)
    jc0[1:] = np.cumsum(lens)
    data = rng.random(int(jc0[-1])).astype(np.float32)
    f = tmp_path / "norows.smat"
    f.write_bytes(numpy_smat331_bytes(nrows, ncols, data, jc0))
    nr, nc, d2, ir2, jc2 = mats.loadSMat(f)
    want_ir0 = np.concatenate([np.arange(n) for n in lens]).astype(np.int32)
    assert (nr, nc) == (nrows, ncols) and np.array_equal(d2, data)
    assert np.array_equal(jc2, jc0 + 1) and np.array_equal(ir2, want_ir0 + 1)      # host base 1
    # a column longer than the matrix is tall cannot be a 331 file
    jcbad = jc0.copy()
    f.write_bytes(numpy_smat331_bytes(3, ncols, data, jcbad))
    with pytest.raises(RuntimeError, match="column longer"):
        mats.loadSMat(f)


def test_malformed_smat_files_are_refused_on_the_host(tmp_path):
    """Column pointers out of order or past nnz, rows outside the matrix: refused before anything is indexed."""
    rng = np.random.default_rng(6)
    data, ir0, jc0 = random_csc(rng, 9, 11, 0.3)
    f = tmp_path / "bad.smat"
    for what, (jcx, irx) in {
            "jc\\(0\\)": (np.concatenate([[1], jc0[1:]]), ir0),
            "out of order": (np.concatenate([jc0[:4], [jc0[4] + 5], jc0[5:]]) if jc0[5] < jc0[4] + 5 else None, ir0),
            "jc\\(ncols\\)": (np.concatenate([jc0[:-1], [jc0[-1] + 3]]), ir0),
            "out of range": (jc0, np.where(np.arange(ir0.size) == 2, 9, ir0))}.items():
        if jcx is None:
            continue
        f.write_bytes(numpy_smat_bytes(9, 11, data, irx.astype(np.int32), jcx.astype(np.int32)))
        with pytest.raises(RuntimeError, match=what):
            mats.loadSMat(f)


def test_fmat_file_round_trip_and_layout(tmp_path):
    rng = np.random.default_rng(3)
    a = rng.standard_normal((7, 5)).astype(np.float32)
    f = tmp_path / "a.fmat"
    mats.saveFMat(f, a)
    assert f.read_bytes() == struct.pack("<4i", 130, 7, 5, 0) + np.asfortranarray(a).ravel(order="F").astype("<f4").tobytes()
    assert np.array_equal(mats.loadFMat(f), a)


@pytest.mark.gpu
def test_load_gsmat_streams_file_to_device(hip, tmp_path):
    """File -> pinned staging -> device: the GSMat equals the one built from the host arrays, and
    multiplies the same."""
    rng = np.random.default_rng(4)
    nrows, ncols = 3000, 5000
    data, ir0, jc0 = random_csc(rng, nrows, ncols, lengths=rng.integers(0, 600, size=ncols))   # ~12 MB of arrays: several chunks
    f = tmp_path / "big.smat"
    mats.saveSMat(f, nrows, ncols, data, ir0 + 1, jc0 + 1)
    g = mats.loadGSMat(f)
    assert g.dims == (nrows, ncols, data.size)
    d2, ir2, jc2 = g.to_csc()
    assert np.array_equal(d2, data) and np.array_equal(ir2, ir0 + 1) and np.array_equal(jc2, jc0 + 1)
    a = mats.GMat.from_numpy(rng.random((8, nrows)).astype(np.float32))
    ref = mats.GSMat.from_csc(nrows, ncols, data, ir0 + 1, jc0 + 1)
    assert np.array_equal((a * g).numpy(), (a * ref).numpy())
    gz = tmp_path / "big.smat.gz"
    mats.saveSMat(gz, nrows, ncols, data, ir0 + 1, jc0 + 1)
    assert np.array_equal(mats.loadGSMat(gz).to_csc()[1], ir0 + 1)


@pytest.mark.gpu
def test_load_gsmat_type_331_and_malformed_files(hip, tmp_path):
    """A file without row indices straight to the device; corrupted column pointers / rows are
    refused by the device-side check before any kernel indexes with them."""
    rng = np.random.default_rng(7)
    nrows, ncols = 40, 300
    lens = rng.integers(0, nrows + 1, size=ncols)
    jc0 = np.zeros(ncols + 1, dtype=np.int32)
    jc0[1:] = np.cumsum(lens)
    data = rng.random(int(jc0[-1])).astype(np.float32)
    f = tmp_path / "norows.smat"
    f.write_bytes(numpy_smat331_bytes(nrows, ncols, data, jc0))
    g = mats.loadGSMat(f)
    d2, ir2, jc2 = g.to_csc()
    want_ir0 = np.concatenate([np.arange(n) for n in lens]).astype(np.int32)
    assert np.array_equal(d2, data) and np.array_equal(ir2, want_ir0 + 1) and np.array_equal(jc2, jc0 + 1)
    a = mats.GMat.from_numpy(rng.random((8, nrows)).astype(np.float32))
    ref = mats.GSMat.from_csc(nrows, ncols, data, want_ir0 + 1, jc0 + 1)
    assert np.array_equal((a * g).numpy(), (a * ref).numpy())
    # corrupted files
    data3, ir3, jc3 = random_csc(rng, 50, 200, lengths=rng.integers(1, 9, size=200))
    cases = {"pointer past nnz": (np.where(np.arange(jc3.size) == 100, jc3[-1] + 1000, jc3), ir3),
             "pointer order": (np.where(np.arange(jc3.size) == 50, jc3[49] - 1, jc3), ir3),
             "first pointer": (np.where(np.arange(jc3.size) == 0, 1, jc3), ir3),
             "row out of range": (jc3, np.where(np.arange(ir3.size) == 7, 50, ir3)),
             "negative row": (jc3, np.where(np.arange(ir3.size) == 9, -4, ir3))}
    for name, (jcx, irx) in cases.items():
        f.write_bytes(numpy_smat_bytes(50, 200, data3, irx.astype(np.int32), jcx.astype(np.int32)))
        with pytest.raises(RuntimeError, match="malformed"):
            mats.loadGSMat(f)
        # the host-array path (GSMat.fromSMat) makes the same check on the device
        with pytest.raises(RuntimeError, match="malformed"):
            mats.GSMat.from_csc(50, 200, data3, irx.astype(np.int32) + 1, jcx.astype(np.int32) + 1)
    # and the library is still healthy afterwards
    ok = mats.GSMat.from_csc(50, 200, data3, ir3 + 1, jc3 + 1)
    assert np.array_equal(ok.to_csc()[1], ir3 + 1)
