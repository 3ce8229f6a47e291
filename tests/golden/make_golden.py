#!/usr/bin/env python3
"""Writes tests/golden/sparse_dense_golden.npz: small inputs and their expected results for
A*S, A*^S, DDS and the sparse/dense sums, computed WITHOUT the oracle: scipy.sparse / numpy in
float64 on the float32 inputs (the reference holds no golden files for this path, only the
relations its tests assert: A*S == A*full(S), A*^S == A*full(S)^T, sums by explicit loops).

Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import scipy.sparse as sp

HERE = os.path.dirname(os.path.abspath(__file__))


def case(rng, k, nrows, ncols, density, dist):
    S = sp.random(nrows, ncols, density=density, format="csc", random_state=rng,
                  data_rvs=lambda n: 1.0 - rng.random(n)).astype(np.float32)
    S.sort_indices()
    if dist == "normal":
        A = rng.standard_normal((k, nrows)).astype(np.float32)
        B = rng.standard_normal((k, ncols)).astype(np.float32)
    else:
        A = rng.random((k, nrows)).astype(np.float32)
        B = rng.random((k, ncols)).astype(np.float32)
    S64 = S.astype(np.float64)
    A64, B64 = A.astype(np.float64), B.astype(np.float64)
    AS = A64 @ S64.toarray()                      # k x ncols
    BSt = B64 @ S64.toarray().T                   # k x nrows   (B *^ S)
    coo = S.tocoo()
    order = np.lexsort((coo.row, coo.col))        # CSC order
    r, c = coo.row[order], coo.col[order]
    P = np.einsum("kn,kn->n", A64[:, r], B64[:, c])
    return dict(k=k, nrows=nrows, ncols=ncols, data=S.data, ir=S.indices.astype(np.int32),
                jc=S.indptr.astype(np.int32), A=np.asfortranarray(A).ravel(order="F"),
                B=np.asfortranarray(B).ravel(order="F"),
                AS=np.asfortranarray(AS).ravel(order="F"), BSt=np.asfortranarray(BSt).ravel(order="F"),
                P=P, colsum=np.asarray(S64.sum(axis=0)).ravel(), rowsum=np.asarray(S64.sum(axis=1)).ravel(),
                dsum1=A64.sum(axis=0), dsum2=A64.sum(axis=1))


def main():
    rng = np.random.default_rng(20261125)
    out = {}
    # the reference's test sizes (nr=10, nc=20, nk=30; GSMatTest.scala:13-16) and a few k shapes
    specs = [("ref", 10, 30, 20, 0.2, "uniform"), ("k1", 1, 17, 9, 0.3, "normal"),
             ("k33", 33, 40, 25, 0.15, "normal"), ("k256", 256, 64, 48, 0.1, "normal"),
             ("empty_cols", 8, 12, 30, 0.03, "uniform")]
    for name, k, nr, nc, dens, dist in specs:
        for key, v in case(rng, k, nr, nc, dens, dist).items():
            out["%s__%s" % (name, key)] = v
    np.savez_compressed(os.path.join(HERE, "sparse_dense_golden.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
