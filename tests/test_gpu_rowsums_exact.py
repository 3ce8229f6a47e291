"""Row sums of sparse values straight from (row index, value): bidmat_spsum_rows_csc and the
reference-shaped bidmat_spsum(n = 2) that runs on it.

The kernel's arithmetic is exact once its one scaling is fixed, so the checker restates that
arithmetic with numpy integers (no GPU, no order) and asks for the same bits; the float64 sum of the
oracle bounds how far that result may lie from the reference's float additions (Arith.cu:250-264).
"""
import numpy as np
import pytest

import oracle
from bidmat_amd import hip_abi
from util import Dev

pytestmark = pytest.mark.gpu


def exact_model(nrows, ir, vals, out0=None):
    """The sums the kernel defines: every finite value times 2^sh, rounded to nearest-even once, added
    as integers; sh = 61 - E - cb with E the exponent of the largest finite magnitude (at least -126)
    and cb the bit length of the number of nonzeros."""
    vals = np.asarray(vals, dtype=np.float32)
    nnz = vals.size
    bits = vals.view(np.uint32) & np.uint32(0x7fffffff)
    finite = bits < np.uint32(0x7f800000)
    m = int(bits[finite].max()) if finite.any() else 0
    e = max((m >> 23) - 127, -126)
    cb = int(nnz).bit_length()
    sh = 61 - e - cb
    a = int(sh / 2)
    b = sh - a
    with np.errstate(under="ignore", invalid="ignore", over="ignore"):
        x = (vals * np.float32(2.0 ** a)) * np.float32(2.0 ** b)
        q = np.where(finite, np.rint(x), 0).astype(np.int64)
    acc = np.zeros(nrows, dtype=np.int64)
    np.add.at(acc, ir[finite], q[finite])
    res = np.ldexp(acc.astype(np.float64), -sh).astype(np.float32)
    isnan = np.zeros(nrows, bool)
    pinf = np.zeros(nrows, bool)
    ninf = np.zeros(nrows, bool)
    isnan[ir[np.isnan(vals)]] = True
    pinf[ir[np.isposinf(vals)]] = True
    ninf[ir[np.isneginf(vals)]] = True
    res[pinf] = np.inf
    res[ninf] = -np.inf
    res[isnan | (pinf & ninf)] = np.nan
    if out0 is not None:
        with np.errstate(invalid="ignore"):
            res = (out0.astype(np.float32) + res).astype(np.float32)
    return res


def run(hip, nrows, ir, vals, beta=0, out0=None, offset=0):
    """offset: elements by which both device arrays are shifted off their 16-byte alignment."""
    pad_i = np.concatenate([np.zeros(offset, np.int32), ir.astype(np.int32)])
    pad_v = np.concatenate([np.zeros(offset, np.float32), vals.astype(np.float32)])
    d = Dev(ir=pad_i if pad_i.size else np.zeros(1, np.int32), v=pad_v if pad_v.size else np.zeros(1, np.float32),
            out=(out0 if out0 is not None else np.full(max(nrows, 1), 7.0, np.float32)))
    hip_abi.check(hip.bidmat_spsum_rows_csc(nrows, ir.size, d.ir.ptr + 4 * offset, d.v.ptr + 4 * offset, d.out.ptr,
                                            beta, None), "spsum_rows_csc")
    hip_abi.check(hip.bidmat_synchronize())
    got = d.out.numpy()[:nrows]
    d.free()
    return got


def same_bits(a, b):
    a = np.asarray(a, np.float32)
    b = np.asarray(b, np.float32)
    return np.array_equal(np.isnan(a), np.isnan(b)) and np.array_equal(a[~np.isnan(a)].view(np.uint32),
                                                                       b[~np.isnan(b)].view(np.uint32))


def zipf_rows(rng, nrows, nnz, a=1.1):
    p = 1.0 / np.arange(1, nrows + 1) ** a
    return rng.choice(nrows, size=nnz, p=p / p.sum()).astype(np.int32)


@pytest.fixture(params=[0, 2], ids=["by_row_count", "hashed_tables"])
def form(hip, request):
    """Both kernels behind the entry (see "rowsum_form"): they must give the same bits."""
    hip_abi.check(hip.bidmat_set_option(b"rowsum_form", request.param), "set_option")
    yield request.param
    hip_abi.check(hip.bidmat_set_option(b"rowsum_form", 0), "set_option")


CASES = [
    # nrows, nnz, value kind
    (1, 1, "u01"), (5, 0, "u01"), (7, 3, "normal"), (100, 4097, "normal"), (1000, 300_000, "u01"),
    (20_000, 1_500_000, "normal"), (50_000, 2_000_003, "wide"), (3000, 700_001, "tiny"), (300, 400_000, "huge"),
    # one, two, four, eight and sixteen ranges of rows; more rows than sixteen ranges hold
    (16_384, 200_000, "normal"), (16_385, 200_000, "normal"), (40_000, 300_000, "u01"), (100_000, 3_000_000, "u01"),
    (262_144, 1_000_000, "normal"), (262_145, 1_000_000, "normal"), (700_000, 1_200_000, "wide"),
]


def values(rng, kind, n):
    if kind == "u01":
        return (1.0 - rng.random(n)).astype(np.float32)
    if kind == "normal":
        return rng.standard_normal(n).astype(np.float32)
    if kind == "wide":          # forty binades: most values fall below the common step in part or whole
        return (rng.standard_normal(n) * np.exp2(rng.integers(-30, 10, size=n))).astype(np.float32)
    if kind == "tiny":          # subnormal and near-subnormal magnitudes: the scaling is 2^(+180)
        return (rng.standard_normal(n) * 1e-38).astype(np.float32)
    if kind == "huge":          # near the top of the range: the scaling is negative
        return (rng.standard_normal(n) * 1e34).astype(np.float32)
    raise ValueError(kind)


@pytest.mark.parametrize("nrows,nnz,kind", CASES)
def test_row_sums_have_the_bits_of_the_exact_integer_model(hip, form, nrows, nnz, kind):
    rng = np.random.default_rng(nrows * 31 + nnz)
    ir = zipf_rows(rng, nrows, nnz) if nnz else np.zeros(0, np.int32)
    vals = values(rng, kind, nnz)
    want = exact_model(nrows, ir, vals)
    got = run(hip, nrows, ir, vals)
    assert same_bits(got, want), "nrows %d nnz %d %s: %d rows differ" % (nrows, nnz, kind, int((got != want).sum()))
    if nnz:
        # and the model itself is a good sum: against the float64 sum, far inside the path's tolerance
        ref64 = np.zeros(nrows)
        np.add.at(ref64, ir, vals.astype(np.float64))
        sa = np.zeros(nrows)
        np.add.at(sa, ir, np.abs(vals.astype(np.float64)))
        scale = np.maximum(sa, float(np.abs(vals).max()))
        assert float(np.max(np.abs(got - ref64) / scale)) < 2e-7


def test_row_sums_do_not_depend_on_the_order_or_the_alignment(hip, form):
    rng = np.random.default_rng(5)
    nrows, nnz = 4000, 900_001
    ir = zipf_rows(rng, nrows, nnz)
    vals = values(rng, "wide", nnz)
    first = run(hip, nrows, ir, vals)
    for offset in (0, 1, 3):
        p = rng.permutation(nnz)
        assert same_bits(run(hip, nrows, ir[p], vals[p], offset=offset), first)
    # rows in runs (sorted by row: every lane of a wave adds to the same row)
    p = np.argsort(ir, kind="stable")
    assert same_bits(run(hip, nrows, ir[p], vals[p]), first)


def test_row_sums_add_to_the_output_and_carry_nan_and_infinities(hip, form):
    rng = np.random.default_rng(6)
    nrows, nnz = 64, 50_000
    ir = rng.integers(0, nrows, size=nnz).astype(np.int32)
    vals = rng.standard_normal(nnz).astype(np.float32)
    for row, v in ((3, np.nan), (5, np.inf), (6, -np.inf), (7, np.inf), (7, -np.inf), (9, np.inf), (9, np.inf)):
        j = int(rng.integers(0, nnz))
        ir[j], vals[j] = row, v
    out0 = rng.standard_normal(nrows).astype(np.float32)
    want = exact_model(nrows, ir, vals, out0)
    got = run(hip, nrows, ir, vals, beta=1, out0=out0.copy())
    assert same_bits(got, want)
    assert np.isnan(got[3]) and got[5] == np.inf and got[6] == -np.inf and np.isnan(got[7]) and got[9] == np.inf
    assert np.isfinite(np.delete(got, [3, 5, 6, 7, 9])).all()


def test_a_row_index_outside_the_output_writes_nothing(hip, form):
    rng = np.random.default_rng(8)
    nrows, ncols, nnz = 50, 40, 2000
    ir = rng.integers(0, nrows, size=nnz).astype(np.int32)
    ir[777] = nrows                                  # one past the end
    ic = np.sort(rng.integers(0, ncols, size=nnz)).astype(np.int32)
    vals = rng.random(nnz).astype(np.float32)
    got = run(hip, nrows, ir, vals)                  # stream form: documented to leave the output alone
    assert (got == 7.0).all()
    ir[777] = -1
    assert (run(hip, nrows, ir, vals) == 7.0).all()
    d = Dev(ir=ir, ic=ic, v=vals, out=np.full(nrows, 7.0, np.float32))
    rc = hip.bidmat_spsum(nrows, ncols, nnz, d.ir.ptr, d.ic.ptr, d.v.ptr, d.out.ptr, 2)
    assert rc == 1 and (d.out.numpy() == 7.0).all()  # hipErrorInvalidValue, output untouched
    hip.bidmat_error_string(rc)
    ir[777] = 0
    d.put("ir", ir)
    hip_abi.check(hip.bidmat_spsum(nrows, ncols, nnz, d.ir.ptr, d.ic.ptr, d.v.ptr, d.out.ptr, 2), "spsum")
    assert same_bits(d.out.numpy(), exact_model(nrows, ir, vals, np.full(nrows, 7.0, np.float32)))
    d.free()


def test_row_sums_against_the_oracle_within_the_path_tolerance(hip):
    """The bar every sum of the path is held to: 1e-4 of the sum of magnitudes against the float64 arbiter."""
    rng = np.random.default_rng(9)
    nrows, ncols = 2000, 3000
    lengths = rng.integers(0, 60, size=ncols)
    jc = np.zeros(ncols + 1, np.int32)
    jc[1:] = np.cumsum(lengths)
    nnz = int(jc[-1])
    ir = zipf_rows(rng, nrows, nnz)
    vals = rng.standard_normal(nnz).astype(np.float32)
    ref64, sa = oracle.spsum_f64(nrows, vals, ir, jc, 2)
    got = run(hip, nrows, ir, vals)
    ok, worst = oracle.within_tolerance(got, ref64, sa, 1e-4)
    assert ok, worst
