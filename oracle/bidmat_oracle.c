/*
 * CPU oracle for BIDMat's sparse-dense product path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the
 * smoke check and the benchmark's cpu_baseline leg may load this library; the
 * product path (the HIP library) never links, loads or calls it.
 *
 * Every function restates, loop for loop, the reference's CPU algorithm for
 * one operation of the path and cites the file:line it follows.  All float
 * arithmetic is plain fp32 with no fused multiply-add (the JVM never fuses;
 * compile with -ffp-contract=off) and in the reference's summation order.
 * The *_f64 functions are the arbiters: same traversal, products of the fp32
 * inputs accumulated in double (an fp32*fp32 product is exact in double).
 *
 * Index base: the reference's host SMat is 1-based by default
 * (Mat.scala:718 ioneBased=1) and its native loops take the base from jc[0]
 * (BIDMat_SPBLAS.c:373).  Every function here takes `ioff` explicitly.
 *
 * Parity pinning (what each function is checked against in tests/):
 *   oracle_smcscm / oracle_fsmult     dense GEMM A*full(S) in numpy fp64, scipy csc product,
 *                                     one-hot gather (bit-exact), identity, golden fixtures
 *   oracle_smcsrm / oracle_fsmultT    A*full(S)^T in fp64, np.add.at, transpose identity, fixtures
 *   oracle_fsmult_tile / _tileT       dense products of numpy windows A[a:b,c:d] @ full(S)[e:f,g:h](^T)
 *   oracle_dds                        closed form dot(A[:,r],B[:,c]); dense pattern == A^T B; fixtures
 *   oracle_spsum                      np.bincount / np.add.reduceat; sum of col sums == sum of row sums
 *   oracle_dsum                       numpy sum along axis
 *   oracle_check                      hand-built valid/invalid patterns (every branch)
 *   oracle_compress/uncompress_inds   np.searchsorted / np.repeat
 *   oracle_applyop                    numpy elementwise results
 *   oracle_reduce_tree                a literal lane-by-lane simulation in Python, numpy for the associative ops,
 *                                     closed forms for sub / div (signs follow the parity of the lane's bit count)
 * No function of this file is left "parity unpinned".
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define EXPORT __attribute__((visibility("default")))

/* ------------------------------------------------------------------ A * S */

/* C += A*S, native loop.  Follows BIDMat_SPBLAS.c:373-388 (smcscm): for each
 * column i of S, for each stored nonzero j in CSC order, C[:,i] += B[j]*A[:,ir[j]].
 * OpenMP over columns as in the reference (:375); per-column order is sequential,
 * so the result does not depend on the thread count. */
EXPORT void oracle_smcscm(int M, int N, const float *A, int lda, const float *B,
                          const int *ir, const int *jc, float *C, int ldc, int nthreads)
{
    int ioff = jc[0];
    int i;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (i = 0; i < N; i++) {
        int j, k;
        float *Cp = C + (size_t)i * ldc;
        for (j = jc[i] - ioff; j < jc[i + 1] - ioff; j++) {
            int ir0 = ir[j] - ioff;
            const float *Ap = A + (size_t)ir0 * lda;
            float bv = B[j];
            for (k = 0; k < M; k++) {
                Cp[k] += bv * Ap[k];
            }
        }
    }
}

/* C += A*S, Scala loop.  Follows FMat.scala:1112-1132 (fSMultHelper) driven by
 * FMat.scala:1174-1184 (madd): numThreads column ranges
 * [ithread*ncols/nt, (ithread+1)*ncols/nt), each running the helper. */
EXPORT void oracle_fsmult(int nrows, int ncols, const float *A, const float *data,
                          const int *ir, const int *jc, int ioff, float *out, int nthreads)
{
    int ithread;
    if (nthreads < 1) nthreads = 1;
    /* FMat.scala:1174: threads only when nrows*nnz > 100000 and numThreads > 1 */
    long long nnz = (long long)jc[ncols] - ioff;
    if (!((long long)nrows * nnz > 100000LL && nthreads > 1)) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static, 1)
    for (ithread = 0; ithread < nthreads; ithread++) {
        int istart = (int)(1LL * ithread * ncols / nthreads);
        int iend = (int)(1LL * (ithread + 1) * ncols / nthreads);
        int i, j, k;
        for (i = istart; i < iend; i++) {
            for (j = jc[i] - ioff; j < jc[i + 1] - ioff; j++) {
                float dval = data[j];
                size_t ival = (size_t)(ir[j] - ioff);
                for (k = 0; k < nrows; k++) {
                    out[k + (size_t)i * nrows] += A[k + ival * nrows] * dval;
                }
            }
        }
    }
}

/* fp64 arbiter for A*S: ref[k,i] = sum_j (double)A[k,ir[j]]*(double)v[j] in CSC order,
 * sumabs = sum of |terms| (used by the cancellation-safe tolerance). Either output may be NULL. */
EXPORT void oracle_fsmult_f64(int nrows, int ncols, const float *A, const float *data,
                              const int *ir, const int *jc, int ioff, double *ref, double *sumabs,
                              int nthreads)
{
    int i;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (i = 0; i < ncols; i++) {
        int j, k;
        for (j = jc[i] - ioff; j < jc[i + 1] - ioff; j++) {
            double dval = data[j];
            size_t ival = (size_t)(ir[j] - ioff);
            for (k = 0; k < nrows; k++) {
                double t = (double)A[k + ival * nrows] * dval;
                if (ref) ref[k + (size_t)i * nrows] += t;
                if (sumabs) sumabs[k + (size_t)i * nrows] += fabs(t);
            }
        }
    }
}

/* ----------------------------------------------------------------- A *^ S */

/* C += A*S^T, native loop.  Follows BIDMat_SPBLAS.c:406-420 (smcsrm): sequential
 * over columns i and nonzeros j: C[:,ir[j]] += B[j]*A[:,i]. */
EXPORT void oracle_smcsrm(int M, int N, const float *A, int lda, const float *B,
                          const int *ir, const int *jc, float *C, int ldc)
{
    int ioff = jc[0];
    int i, j, k;
    for (i = 0; i < N; i++) {
        const float *Ap = A + (size_t)i * lda;
        for (j = jc[i] - ioff; j < jc[i + 1] - ioff; j++) {
            int ir0 = ir[j] - ioff;
            float *Cp = C + (size_t)ir0 * ldc;
            float Bj = B[j];
            for (k = 0; k < M; k++) {
                Cp[k] += Bj * Ap[k];
            }
        }
    }
}

/* C += A*S^T, Scala loop.  Follows FMat.scala:1369-1389 (fSMultTHelper2) driven by
 * FMat.scala:1410-1440 (maddT): when nrows >= 64 and numThreads > 1 the k dimension
 * is cut into nt = min(numThreads, nrows/32) ranges and every thread walks the whole
 * sparse structure for its own range of rows of A. */
EXPORT void oracle_fsmultT(int nrows, int ncols, const float *A, const float *data,
                           const int *ir, const int *jc, int ioff, float *out, int nthreads)
{
    int nt = 1, ithread;
    if (nrows >= 64 && nthreads > 1) {
        nt = nthreads < nrows / 32 ? nthreads : nrows / 32;
    }
#pragma omp parallel for num_threads(nt) schedule(static, 1)
    for (ithread = 0; ithread < nt; ithread++) {
        int istart = (int)(1LL * nrows * ithread / nt);
        int iend = (int)(1LL * nrows * (ithread + 1) / nt);
        int i, j, k;
        for (i = 0; i < ncols; i++) {
            for (j = jc[i] - ioff; j < jc[i + 1] - ioff; j++) {
                float dval = data[j];
                size_t ival = (size_t)(ir[j] - ioff);
                for (k = istart; k < iend; k++) {
                    out[k + ival * nrows] += A[k + (size_t)i * nrows] * dval;
                }
            }
        }
    }
}

/* fp64 arbiter for A*^S. Threads split the k dimension (race-free scatter). */
EXPORT void oracle_fsmultT_f64(int nrows, int ncols, const float *A, const float *data,
                               const int *ir, const int *jc, int ioff, double *ref, double *sumabs,
                               int nthreads)
{
    int nt = nthreads < 1 ? 1 : nthreads, ithread;
    if (nt > nrows) nt = nrows > 0 ? nrows : 1;
#pragma omp parallel for num_threads(nt) schedule(static, 1)
    for (ithread = 0; ithread < nt; ithread++) {
        int istart = (int)(1LL * nrows * ithread / nt);
        int iend = (int)(1LL * nrows * (ithread + 1) / nt);
        int i, j, k;
        for (i = 0; i < ncols; i++) {
            for (j = jc[i] - ioff; j < jc[i + 1] - ioff; j++) {
                double dval = data[j];
                size_t ival = (size_t)(ir[j] - ioff);
                for (k = istart; k < iend; k++) {
                    double t = (double)A[k + (size_t)i * nrows] * dval;
                    if (ref) ref[k + ival * nrows] += t;
                    if (sumabs) sumabs[k + ival * nrows] += fabs(t);
                }
            }
        }
    }
}

/* ------------------------------------------------------------ tile variants */

/* C[0:nr,0:nc] += A[0:nr,0:kk] * S[broff:broff+kk, bcoff:bcoff+nc] on windows of larger
 * matrices.  Follows FMat.scala:1200-1223 (fSMultHelperTile): columns bcoff..bcoff+nc of S,
 * nonzeros in stored order, rows outside [broff, broff+kk) skipped, row rebased to broff.
 * A / C point at the first element of their windows; lda / ldc are the parents' row counts.
 * Threads over column ranges as FMat.scala:1260-1270.  ref/sumabs (double, nr x nc with
 * leading dimension nr) are optional fp64 arbiters of the product alone. */
EXPORT void oracle_fsmult_tile(int nr, int nc, int kk, const float *A, int lda, const float *data,
                               const int *ir, const int *jc, int ioff, int broff, int bcoff,
                               float *C, int ldc, double *ref, double *sumabs, int nthreads)
{
    int i;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (i = 0; i < nc; i++) {
        int j, k;
        for (j = jc[i + bcoff] - ioff; j < jc[i + bcoff + 1] - ioff; j++) {
            int irow0 = ir[j] - ioff;
            if (irow0 >= broff && irow0 < broff + kk) {
                size_t irow = (size_t)(irow0 - broff);
                float dval = data[j];
                for (k = 0; k < nr; k++) {
                    if (C) C[k + (size_t)i * ldc] += A[k + irow * lda] * dval;
                    if (ref) {
                        double t = (double)A[k + irow * lda] * (double)dval;
                        ref[k + (size_t)i * nr] += t;
                        if (sumabs) sumabs[k + (size_t)i * nr] += fabs(t);
                    }
                }
            }
        }
    }
}

/* C[0:nr,0:nc] += A[0:nr,0:kk] * S[broff:broff+nc, bcoff:bcoff+kk]^T.  Follows
 * FMat.scala:1225-1248 (fSMultHelperTileT): columns bcoff..bcoff+kk of S, rows outside
 * [broff, broff+nc) skipped, C[:,row-broff] += A[:,i]*v.  Single thread here: the
 * reference's own column-range threading of this scatter (FMat.scala:1286-1296) lets two
 * threads add into the same output column at once. */
EXPORT void oracle_fsmult_tileT(int nr, int nc, int kk, const float *A, int lda, const float *data,
                                const int *ir, const int *jc, int ioff, int broff, int bcoff,
                                float *C, int ldc, double *ref, double *sumabs)
{
    int i, j, k;
    for (i = 0; i < kk; i++) {
        for (j = jc[i + bcoff] - ioff; j < jc[i + bcoff + 1] - ioff; j++) {
            int irow0 = ir[j] - ioff;
            if (irow0 >= broff && irow0 < broff + nc) {
                size_t irow = (size_t)(irow0 - broff);
                float dval = data[j];
                for (k = 0; k < nr; k++) {
                    if (C) C[k + irow * ldc] += A[k + (size_t)i * lda] * dval;
                    if (ref) {
                        double t = (double)A[k + (size_t)i * lda] * (double)dval;
                        ref[k + irow * nr] += t;
                        if (sumabs) sumabs[k + irow * nr] += fabs(t);
                    }
                }
            }
        }
    }
}

/* -------------------------------------------------------------------- DDS */

/* P = DDS(A,B,S): out.data[j] = dot(A[:,ir[j]], B[:,i]) for nonzero j of column i.
 * Follows MatFunctions.scala:1594-1618 (DDShelper): dsum starts at 0.0f, k ascending,
 * and the pattern is copied (out.ir[j] = c.ir[j], out.jc[i+1] = c.jc[i+1]);
 * MatFunctions.scala:1632 sets out.jc[0] = ioff; :1633-1644 threads over column ranges
 * i*ncols/nt when nnz > 100000. out_ir / out_jc may be NULL (values only). */
EXPORT void oracle_dds(int k, int ncols, const float *A, const float *B, const int *ir,
                       const int *jc, int ioff, float *out_data, int *out_ir, int *out_jc,
                       int nthreads)
{
    int ithread;
    long long nnz = (long long)jc[ncols] - ioff;
    if (nthreads < 1) nthreads = 1;
    if (!(nnz > 100000 && nthreads > 1)) nthreads = 1;
    if (out_jc) out_jc[0] = ioff;
#pragma omp parallel for num_threads(nthreads) schedule(static, 1)
    for (ithread = 0; ithread < nthreads; ithread++) {
        int istart = (int)((long long)ithread * ncols / nthreads);
        int iend = (int)((long long)(ithread + 1) * ncols / nthreads);
        int i, j, kk;
        for (i = istart; i < iend; i++) {
            for (j = jc[i] - ioff; j < jc[i + 1] - ioff; j++) {
                float dsum = 0.0f;
                size_t a0 = (size_t)(ir[j] - ioff) * k;
                size_t b0 = (size_t)i * k;
                for (kk = 0; kk < k; kk++) {
                    dsum += A[kk + a0] * B[kk + b0];
                }
                out_data[j] = dsum;
                if (out_ir) out_ir[j] = ir[j];
            }
            if (out_jc) out_jc[i + 1] = jc[i + 1];
        }
    }
}

/* fp64 arbiter for DDS. */
EXPORT void oracle_dds_f64(int k, int ncols, const float *A, const float *B, const int *ir,
                           const int *jc, int ioff, double *ref, double *sumabs, int nthreads)
{
    int i;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (i = 0; i < ncols; i++) {
        int j, kk;
        for (j = jc[i] - ioff; j < jc[i + 1] - ioff; j++) {
            double s = 0.0, sa = 0.0;
            size_t a0 = (size_t)(ir[j] - ioff) * k;
            size_t b0 = (size_t)i * k;
            for (kk = 0; kk < k; kk++) {
                double t = (double)A[kk + a0] * (double)B[kk + b0];
                s += t;
                sa += fabs(t);
            }
            if (ref) ref[j] = s;
            if (sumabs) sumabs[j] = sa;
        }
    }
}

/* ------------------------------------------------------------ sparse sums */

/* sum(S, n).  Follows SparseMat.scala:596-647 (sgReduceOp) with op1 = identity,
 * op2 = +: dim = (nrows==1 && dim0==0) ? 2 : max(1,dim0); the sparse-vector case
 * (dim0==0 and a single row or column) sums all values into one element;
 * dim 1 = per column, accumulator starts at 0, stored order; dim 2 = out cleared,
 * scatter-add over ir in nonzero order.  Returns the number of outputs written,
 * or -1 for an invalid dim ("index must 1 or 2"). Single thread, as the reference. */
EXPORT int oracle_spsum(int nrows, int ncols, const float *data, const int *ir, const int *jc,
                        int ioff, int dim0, float *out)
{
    int nnz = jc[ncols] - ioff;
    int dim = (nrows == 1 && dim0 == 0) ? 2 : (dim0 > 1 ? dim0 : 1);
    int i, j;
    if (dim0 == 0 && (nrows == 1 || ncols == 1)) {
        float acc = 0.0f;
        for (j = 0; j < nnz; j++) acc = acc + data[j];
        out[0] = acc;
        return 1;
    } else if (dim == 1) {
        for (i = 0; i < ncols; i++) {
            float acc = 0.0f;
            for (j = jc[i] - ioff; j < jc[i + 1] - ioff; j++) acc = acc + data[j];
            out[i] = acc;
        }
        return ncols;
    } else if (dim == 2) {
        for (i = 0; i < nrows; i++) out[i] = 0.0f;
        for (j = 0; j < nnz; j++) out[ir[j] - ioff] = out[ir[j] - ioff] + data[j];
        return nrows;
    }
    return -1;
}

/* fp64 arbiter for the sparse sums; dim is 1 or 2 (already resolved). */
EXPORT void oracle_spsum_f64(int nrows, int ncols, const float *data, const int *ir,
                             const int *jc, int ioff, int dim, double *ref, double *sumabs)
{
    int i, j;
    (void)nrows;
    for (i = 0; i < ncols; i++) {
        for (j = jc[i] - ioff; j < jc[i + 1] - ioff; j++) {
            int o = (dim == 1) ? i : ir[j] - ioff;
            if (ref) ref[o] += (double)data[j];
            if (sumabs) sumabs[o] += fabs((double)data[j]);
        }
    }
}

/* ------------------------------------------------------------- dense sums */

/* sum(A, n) for a dense column-major nrows x ncols matrix.  Follows
 * DenseMat.scala:1080-1108 (ggReduceOpv) with FMat.vecAdd (FMat.scala:2756-2762):
 * dim = (nrows==1 && dim0==0) ? 2 : max(1,dim0);
 * dim 1: out[i] = A[0,i], then add A[1..,i] in index order;
 * dim 2: out[:] = A[:,0], then add column 1, 2, ... in order. */
EXPORT int oracle_dsum(int nrows, int ncols, const float *A, int dim0, float *out)
{
    int dim = (nrows == 1 && dim0 == 0) ? 2 : (dim0 > 1 ? dim0 : 1);
    int i, j;
    if (dim == 1) {
        for (i = 0; i < ncols; i++) {
            float acc = A[(size_t)i * nrows];
            for (j = 1; j < nrows; j++) acc = A[(size_t)i * nrows + j] + acc;
            out[i] = acc;
        }
        return ncols;
    } else if (dim == 2) {
        for (j = 0; j < nrows; j++) out[j] = A[j];
        for (i = 1; i < ncols; i++)
            for (j = 0; j < nrows; j++) out[j] = A[(size_t)i * nrows + j] + out[j];
        return nrows;
    }
    return -1;
}

EXPORT void oracle_dsum_f64(int nrows, int ncols, const float *A, int dim, double *ref)
{
    int i, j;
    for (i = 0; i < ncols; i++)
        for (j = 0; j < nrows; j++)
            ref[dim == 1 ? i : j] += (double)A[(size_t)i * nrows + j];
}

/* ---------------------------------------------------- elementwise binops */

/* C[i] = op(A[i], B[i]) with the reference's op numbering (GMat.scala:2245-2261,
 * device table Operators.cu:86-101, functions Operators.cu:27-41). Returns -1 on an
 * unknown op. */
EXPORT int oracle_applyop(const float *A, const float *B, float *C, long long n, int opn)
{
    long long i;
    if (opn < 0 || opn > 14) return -1;
    for (i = 0; i < n; i++) {
        float a = A[i], b = B[i], c;
        switch (opn) {
        case 0: c = a + b; break;
        case 1: c = a - b; break;
        case 2: c = a * b; break;
        case 3: c = a / b; break;
        case 4: c = (a > b) ? 1.0f : 0.0f; break;
        case 5: c = (a < b) ? 1.0f : 0.0f; break;
        case 6: c = (a == b) ? 1.0f : 0.0f; break;
        case 7: c = (a >= b) ? 1.0f : 0.0f; break;
        case 8: c = (a <= b) ? 1.0f : 0.0f; break;
        case 9: c = (a != b) ? 1.0f : 0.0f; break;
        case 10: c = fmaxf(a, b); break;
        case 11: c = fminf(a, b); break;
        case 12: c = atan2f(a, b); break;
        case 13: c = powf(a, b); break;
        default: c = (a > 0) ? b : 0.0f; break;
        }
        C[i] = c;
    }
    return 0;
}

static float oracle_binop(int opn, float a, float b)
{
    float c;
    oracle_applyop(&a, &b, &c, 1, opn);
    return c;
}

/* Dense reduction with any of the 15 binary ops, in the order of the reference's device kernels
 * (there is no CPU counterpart for ops other than sum: DenseMat.ggReduceOpv is only called with
 * add / max / min).  __reduce1op (Operators.cu:650-671): for a column of n = nrows elements, lane t of
 * L = min(n, 32) lanes folds x[t], x[t+32], x[t+64], ... from the left, v = op(v, next); then for
 * i = 1, 2, 4, ... < L every lane t with t + i < L takes v[t] = op(v[t], v[t+i]) (all lanes read the
 * values of the step before); lane 0 holds the result.  __reduce2op (Operators.cu:828-851) does the
 * same along a row with L = min(ncols, 32) lanes striding over the columns.  dim == 1: one result per
 * column (reduce1op), dim == 2: one per row (reduce2op).  n == 0 gives initv.  Returns -1 on an unknown op. */
EXPORT int oracle_reduce_tree(int nrows, int ncols, const float *A, float *out, float initv, int opn, int dim)
{
    int nout = dim == 1 ? ncols : nrows;
    int n = dim == 1 ? nrows : ncols;
    int o, t, i;
    if (opn < 0 || opn > 14 || (dim != 1 && dim != 2)) return -1;
    for (o = 0; o < nout; o++) {
        float v[32], w[32];
        int L = n < 32 ? n : 32;
        if (n == 0) { out[o] = initv; continue; }
        for (t = 0; t < L; t++) {
            int e;
            for (e = t; e < n; e += 32) {
                float x = dim == 1 ? A[(size_t)o * nrows + e] : A[(size_t)e * nrows + o];
                v[t] = e == t ? x : oracle_binop(opn, v[t], x);
            }
        }
        for (i = 1; i < L; i *= 2) {
            for (t = 0; t < L; t++) w[t] = (t + i < L) ? oracle_binop(opn, v[t], v[t + i]) : v[t];
            memcpy(v, w, sizeof(float) * (size_t)L);
        }
        out[o] = v[0];
    }
    return 0;
}

/* ------------------------------------------------------- structure checks */

/* SparseMat.check (SparseMat.scala:710-740). Returns 0 when the pattern is valid, else
 * the number of the first failing rule: 1 jc(0) != ioff; 2 jc out of order;
 * 3 ir not strictly increasing within a column; 4 ir too small; 5 ir out of range;
 * 6 jc(ncols) != nnz+ioff.  *where receives the offending position. */
EXPORT int oracle_check(int nrows, int ncols, int nnz, const int *ir, const int *jc, int ioff,
                        int *where)
{
    int i, j;
    if (jc[0] != ioff) { if (where) *where = 0; return 1; }
    for (i = 0; i < ncols; i++) {
        j = jc[i] - ioff;
        if (jc[i] > jc[i + 1]) { if (where) *where = i; return 2; }
        if (ir) {
            while (j < jc[i + 1] - ioff - 1) {
                if (ir[j + 1] <= ir[j]) { if (where) *where = j; return 3; }
                if (ir[j] < ioff) { if (where) *where = j; return 4; }
                if (ir[j + 1] >= nrows + ioff) { if (where) *where = j + 1; return 5; }
                j++;
            }
        }
    }
    if (jc[ncols] != nnz + ioff) { if (where) *where = ncols; return 6; }
    return 0;
}

/* SparseMat.compressInds (SparseMat.scala:857-868): per-nonzero column index (0-based,
 * non-decreasing) -> column pointer with base ioff. */
EXPORT void oracle_compress_inds(const int *coli, int ncols, int *out, int nnz0, int ioff)
{
    int i = 0, j = 0;
    out[0] = ioff;
    while (i < ncols) {
        while (j < nnz0 && coli[j] <= i) j++;
        out[i + 1] = j + ioff;
        i++;
    }
}

/* SparseMat.uncompressInds (SparseMat.scala:870-883): column pointer -> per-nonzero
 * 0-based column index. */
EXPORT void oracle_uncompress_inds(const int *coli, int ncols, int *out, int ioff)
{
    int i, j;
    for (i = 0; i < ncols; i++)
        for (j = coli[i] - ioff; j < coli[i + 1] - ioff; j++) out[j] = i;
}

/* Number of OpenMP threads available (the benchmark reports the count it used). */
EXPORT int oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
