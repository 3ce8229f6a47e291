"""bidmat_dds_csc_static, the DDS entry point that allocates nothing (its one scratch buffer, the
table of extra wave segments of long columns, is a fixed array inside the library), against
bidmat_dds_csc through the C ABI: bit-identical results on two calls in a row, the second on a
smaller input, so that stale contents of the shared array from the first call would show.
"""
import numpy as np
import pytest

from bidmat_amd import hip_abi
from bidmat_amd.device import DeviceArray
from util import Dev, random_csc

pytestmark = pytest.mark.gpu


def _case(rng, k, nrows, ncols, long_cols):
    lengths = rng.integers(0, 6, size=ncols)
    for c, n in long_cols:
        lengths[c] = n
    _, ir, jc = random_csc(rng, nrows, ncols, lengths=lengths, sort_rows=False, unique=False)
    A = rng.standard_normal(k * nrows).astype(np.float32)
    B = rng.standard_normal(k * ncols).astype(np.float32)
    return dict(k=k, nrows=nrows, ncols=ncols, ir=ir, jc=jc, A=A, B=B)


def _both(hip, c, beta, rng):
    k, ncols, nnz = c["k"], c["ncols"], int(c["ir"].size)
    d = Dev(A=c["A"], B=c["B"], ir=c["ir"], jc=c["jc"])
    P0 = rng.standard_normal(nnz).astype(np.float32)
    want, got = DeviceArray.from_numpy(P0), DeviceArray.from_numpy(P0)
    hip_abi.check(hip.bidmat_dds_csc(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, want.ptr, beta, None), "dds_csc")
    hip_abi.check(hip.bidmat_dds_csc_static(k, ncols, nnz, d.A.ptr, d.B.ptr, d.ir.ptr, d.jc.ptr, got.ptr, beta, None),
                  "dds_csc_static")
    hip_abi.check(hip.bidmat_synchronize())
    w, g = want.numpy(), got.numpy()
    d.free()
    return w, g


def test_static_dds_equals_dds_csc_on_two_calls_the_second_smaller(hip):
    rng = np.random.default_rng(77)
    assert hip.bidmat_dds_static_max_cols() == 1 << 21
    # first call: more than 262 144 columns (the table is built by the three-kernel scan) with long
    # columns (several overflow segments each); second call: a small matrix (two-kernel table) whose
    # long column sits where the first call left other table entries
    big = _case(rng, 64, 2000, 300000, [(5, 5000), (150000, 1025), (299999, 3000)])
    small = _case(rng, 100, 300, 900, [(17, 2500)])
    tiny = _case(rng, 256, 50, 40, [])                       # no column beyond a segment: no table at all
    for c in (big, small, tiny, small):
        for beta in (0, 1):
            w, g = _both(hip, c, beta, rng)
            assert np.array_equal(w, g), "ncols=%d beta=%d" % (c["ncols"], beta)
    # a smaller segment length makes the same small matrix use many more table entries
    old = hip.bidmat_get_option(b"seglen")
    hip_abi.check(hip.bidmat_set_option(b"seglen", 64))
    try:
        for c in (big, small):
            w, g = _both(hip, c, 0, rng)
            assert np.array_equal(w, g)
    finally:
        hip_abi.check(hip.bidmat_set_option(b"seglen", old))


def test_static_dds_rejects_more_columns_than_its_array_holds(hip):
    n = hip.bidmat_dds_static_max_cols()
    x = DeviceArray.zeros(16)
    assert hip.bidmat_dds_csc_static(8, n + 1, 5, x.ptr, x.ptr, x.ptr, x.ptr, x.ptr, 0, None) == 1
    assert hip.bidmat_dds_csc_static(8, 4, 5, x.ptr, x.ptr, x.ptr, x.ptr, x.ptr, 2, None) == 1     # bad beta
    assert hip.bidmat_dds_csc_static(8, 0, 0, None, None, None, None, None, 0, None) == 0          # nothing to do
