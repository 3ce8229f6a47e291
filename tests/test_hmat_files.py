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
    bad.write_bytes(struct.pack("<4i", 331, 2, 2, 1) + b"\0" * 16)
    with pytest.raises(RuntimeError, match="331"):
        mats.loadSMat(bad)
    bad.write_bytes(numpy_smat_bytes(9, 11, data, ir0, jc0)[:-5])
    with pytest.raises(RuntimeError, match="unexpected end of file"):
        mats.loadSMat(bad)
    with pytest.raises(RuntimeError, match="lz4"):
        mats.loadSMat(tmp_path / "x.smat.lz4")
    with pytest.raises(RuntimeError, match="cannot open"):
        mats.loadSMat(tmp_path / "missing.smat")


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
