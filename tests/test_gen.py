"""The seeded input generators: determinism, pattern validity, distribution shape."""
import numpy as np

import oracle
from bidmat_amd import gen


def test_pattern_is_valid_sorted_distinct_and_deterministic():
    ir, jc = gen.pattern(1000, 300, ("poisson", 20), ("zipf", 1.1), 7)
    ir2, jc2 = gen.pattern(1000, 300, ("poisson", 20), ("zipf", 1.1), 7)
    assert np.array_equal(ir, ir2) and np.array_equal(jc, jc2)
    assert oracle.check(1000, 300, ir.size, ir, jc, 0)[0] == 0      # SparseMat.check: sorted, distinct, in range
    ir3, _ = gen.pattern(1000, 300, ("poisson", 20), ("zipf", 1.1), 8)
    assert ir3.size != ir.size or not np.array_equal(ir, ir3)
    assert abs(np.diff(jc).mean() - 20) < 1.5
    counts = np.bincount(ir, minlength=1000)
    assert counts[:10].mean() > 20 * counts[500:].mean()            # Zipf head


def test_config1_shape():
    c = gen.config("C1", 0.01)
    assert c["k"] == 32 and c["nrows"] == 4096
    assert np.all(np.diff(c["jc"]) == 50)
    assert oracle.check(c["nrows"], c["ncols"], c["ir"].size, c["ir"], c["jc"], 0)[0] == 0
    assert c["vals"].min() > 0 and c["vals"].max() <= 1.0
    assert abs(float(c["A"].mean())) < 0.02 and abs(float(c["A"].std()) - 1) < 0.02


def test_pareto_lengths_and_uniform_rows():
    ir, jc = gen.pattern(60000, 5000, ("pareto", 13.3, 1.5, 1, 50000), ("uniform",), 4)
    L = np.diff(jc)
    assert L.min() >= 1 and L.max() <= 50000 and 25 < L.mean() < 60
    assert oracle.check(60000, 5000, ir.size, ir, jc, 0)[0] == 0


def test_dense_generators():
    u = gen.uniform(100000, 3, 0.01, 1.0)
    assert u.min() >= 0.01 and u.max() < 1.0 and abs(u.mean() - 0.505) < 0.01
    e = gen.exponential(100000, 3)
    assert e.min() > 0 and abs(e.mean() - 1) < 0.02
    n = gen.normal(100000, 3, 0.0, 0.02)
    assert abs(n.std() - 0.02) < 0.001
    assert np.array_equal(gen.normal(1000, 3), gen.normal(1000, 3))
