/*
 * bidmat_hip.h — C ABI of libbidmathip.so, the MI355X (gfx950) native library behind
 * BIDMat's GMat / GSMat sparse-dense product path.
 *
 * Conventions (all entry points):
 *   - plain C types only; every pointer named d_* / documented "device" is a HIP device
 *     pointer on the calling thread's current device; nothing is retained after return
 *     except by plan objects, which say so.
 *   - dense matrices are column-major fp32 with leading dimension == number of rows
 *     (GMat.scala:19); sparse matrices are CSC with 0-based int32 indices on the device
 *     (GSMat.scala:14-15,626-632): ir[nnz] row index, ic[nnz] per-nonzero column index
 *     (non-decreasing), jc[ncols+1] column pointer, data[nnz] values.  Rows inside a
 *     column need not be sorted or unique.
 *   - return value: 0 on success, otherwise a hipError_t value as int
 *     (1 == hipErrorInvalidValue for rejected arguments).  The reference's launchers
 *     return cudaGetLastError() the same way (Arith.cu:57-59).
 *   - entry points WITHOUT a stream argument block until the result is complete, like the
 *     reference's launchers (cudaStreamSynchronize, MatKernel.hpp:15).  Entry points WITH
 *     a `stream` argument (a hipStream_t passed as void*, NULL = default stream) only
 *     enqueue work.  The library's scratch buffers (including the partial sums of the calls that
 *     go through a plan) are kept per (device, stream): calls on different streams may overlap,
 *     also when they use the same plan handle, which holds data of the pattern only.
 *   - results are deterministic: no floating-point atomics anywhere.
 *   - threads: every entry point may be called from any host thread. Calls that take library
 *     scratch or a cached plan (all product, sum and reduction entries) hold a per-device lock
 *     while they look up / build their scratch and enqueue their kernels (the blocking entries:
 *     until their result is complete), so two threads that drive one device through the blocking
 *     entries or share a stream never see each other's scratch. What stays with the caller:
 *     bidmat_plan_set_values and bidmat_plan_destroy must not run while another call uses the same
 *     plan, and option changes (bidmat_set_option) are process-wide.
 */
#ifndef BIDMAT_HIP_H
#define BIDMAT_HIP_H

#ifdef __cplusplus
extern "C" {
#endif

/* Binary op codes, BinOp in GMat.scala:2245-2261 (device table Operators.cu:86-101). */
enum {
    BIDMAT_OP_ADD = 0, BIDMAT_OP_SUB = 1, BIDMAT_OP_MUL = 2, BIDMAT_OP_DIV = 3,
    BIDMAT_OP_GT = 4, BIDMAT_OP_LT = 5, BIDMAT_OP_EQ = 6, BIDMAT_OP_GE = 7,
    BIDMAT_OP_LE = 8, BIDMAT_OP_NE = 9, BIDMAT_OP_MAX = 10, BIDMAT_OP_MIN = 11,
    BIDMAT_OP_ATAN2 = 12, BIDMAT_OP_POW = 13, BIDMAT_OP_IFPOS = 14
};

/* ------------------------------------------------------------------------------------
 * 1. Reference-shaped launchers: same argument lists as the reference's native
 *    launchers, so a JNI wrapper can forward to them unchanged.
 * ------------------------------------------------------------------------------------ */

/* C += A * S.  Replaces `int dsmult(int nrows,int ncols,int nnz,float*A,float*Bdata,int*Bir,
 * int*Bic,float*C)` (jni/include/MatKernel.hpp, jni/src/Arith.cu:46-60; Java stub
 * CUMAT.java:143; caller GMat.scala:1070).  nrows = rows of A and C (k); ncols = columns of
 * S and C.  C holds the addend (callers clear it first, GMat.scala:1047). */
int bidmat_dsmult(int nrows, int ncols, int nnz, const float *A, const float *Bdata,
                  const int *Bir, const int *Bic, float *C);

/* C += A * S^T.  Replaces `int dsmultT(...)` (Arith.cu:234-248; CUMAT.java:152; caller
 * GMat.scala:1093).  nrows = rows of A and C (k); ncols = columns of S and of A.  C has
 * one column per row of S; the row count of S is not an argument of the reference launcher,
 * so rows of C beyond max(Bir) are left untouched, exactly as there. */
int bidmat_dsmultT(int nrows, int ncols, int nnz, const float *A, const float *Bdata,
                   const int *Bir, const int *Bic, float *C);

/* Windowed products used by tiled matrices (TMat).
 * bidmat_dsmultTile:  C[0:nr,0:nc] += A[0:nr,0:kk] * S[broff:broff+kk, bcoff:bcoff+nc]
 * bidmat_dsmultTileT: C[0:nr,0:nc] += A[0:nr,0:kk] * S[broff:broff+nc, bcoff:bcoff+kk]^T
 * A and C are windows of larger matrices: lda / ldc are their column strides.  Replace
 * `int dsmultTile(int nr,int nc,int kk,int nnz,float*A,int lda,float*Bdata,int*Bir,int*Bic,int broff,
 * int bcoff,float*C,int ldc)` and `dsmultTileT` (Arith.cu:63-189, MatKernel.hpp:142-144; Java stub
 * CUMAT.java:145 with its transpose flag; callers GMat.tileMult / tileMultNT, GMat.scala:961-997). */
int bidmat_dsmultTile(int nr, int nc, int kk, int nnz, const float *A, int lda, const float *Bdata,
                      const int *Bir, const int *Bic, int broff, int bcoff, float *C, int ldc);
int bidmat_dsmultTileT(int nr, int nc, int kk, int nnz, const float *A, int lda, const float *Bdata,
                       const int *Bir, const int *Bic, int broff, int bcoff, float *C, int ldc);

/* Sparse matrix (its nnz stored values A, in place) op edge vector:
 *   bidmat_sdoprow: A[i] = op(A[i], B[Aic[i]])  (B a row vector, one entry per column), or op(A[i], B[0]) if len <= 1
 *   bidmat_sdopcol: A[i] = op(A[i], B[Air[i]])  (B a column vector, one entry per row), same scalar rule.
 * Replace `int sdoprow/sdopcol(int nrows,int ncols,int nnz,float*A,int*Aic|Air,float*B,int len,int opn)`
 * (Operators.cu:585-647; CUMAT.java:135,139; caller GSMat.GSDop, GSMat.scala:315-330). All 15 ops. */
int bidmat_sdoprow(int nrows, int ncols, int nnz, float *A, const int *Aic, const float *B, int len, int opn);
int bidmat_sdopcol(int nrows, int ncols, int nnz, float *A, const int *Air, const float *B, int len, int opn);

/* P[j] += dot(A[:,Cir[j]], B[:,Cic[j]]).  Replaces `int dds(int nrows,int nnz,float*A,float*B,
 * int*Cir,int*Cic,float*P)` (Arith.cu:381-389; CUMAT.java:211; caller GSMat.scala:663).
 * bidmat_dds and bidmat_dsmult recognise a pattern they have met before (same device arrays, same
 * contents: one pass over Cir / Cic per call checks it) and run it through a cached plan from the second
 * call on; see "cache_cols_after".  DDS results are the same bits either way. */
int bidmat_dds(int nrows, int nnz, const float *A, const float *B, const int *Cir,
               const int *Cic, float *P);

/* P[j] = dot(A[:,Cir[j]], B[:,c]) for every nonzero j of column c, with the column POINTER Cjc
 * (ncols+1 entries) instead of the per-nonzero column array; overwrites P.  Replaces `int dds0(int nrows,
 * int ncols,float*A,float*B,int*Cir,int*Cjc,float*P)` (MatKernel.hpp:156, Arith.cu:312-347,391-397;
 * CUMAT.java:213; caller GSMat.DDS0, GSMat.scala:669-684).  The reference kernel assumes nrows == 1024
 * (Arith.cu:316-324); any nrows works here.  Blocking. */
int bidmat_dds0(int nrows, int ncols, const float *A, const float *B, const int *Cir, const int *Cjc,
                float *P);

/* Sparse sums: n == 1: B[Aic[i]] += P[i] (column sums, B has ncols entries); otherwise
 * B[Air[i]] += P[i] (row sums, B has nrows entries).  Replaces `int spsum(...)`
 * (Arith.cu:266-277; CUMAT.java:209; caller GSMat.scala:255). */
int bidmat_spsum(int nrows, int ncols, int nnz, const int *Air, const int *Aic, const float *P,
                 float *B, int n);

/* Dense column reduce B[c] = op_r A[r,c] (B has ncols entries).  Replaces
 * `int reduce1op(int nrows,int ncols,float*A,float*B,float initv,int opn)`
 * (Operators.cu:735-748; CUMAT.java:111; caller GMat.scala:1186).  All 15 op codes.  ADD, MUL, MAX, MIN
 * (the ones BIDMat's sum/prod/maxi/mini issue, GFunctions.scala:225-228) run bandwidth-bound kernels whose
 * order of operations is fixed but not the reference's (they agree with it to rounding).  For every other
 * code the order IS the result (a - b, a / b, a > b ... are not associative), so those follow the reference's
 * kernel step by step (Operators.cu:650-671): 32 lanes per column, lane t folds rows t, t+32, ... from the
 * left, then lanes combine pairwise at distances 1, 2, 4, ...; also for one-column inputs, where the
 * reference's launcher (thrust, Operators.cu:718-731) handles only ADD / MAX / MIN and leaves B untouched
 * for the rest.  nrows == 0 fills B with initv. */
int bidmat_reduce1op(int nrows, int ncols, const float *A, float *B, float initv, int opn);

/* Dense row reduce B[r] = op_c A[r,c] (B has nrows entries).  Replaces `int reduce2op(...)`
 * (Operators.cu:853-866; CUMAT.java:119; caller GMat.scala:1193).  Same op set and the same rules, along the
 * row (Operators.cu:828-851). */
int bidmat_reduce2op(int nrows, int ncols, const float *A, float *B, float initv, int opn);

/* Elementwise C = op(A, B) with BIDMat's broadcasting (equal shapes, row/column vector on
 * either side, scalar on either side).  Replaces `int apply_binop(float*A,int Anrows,int Ancols,
 * float*B,int Bnrows,int Bncols,float*C,int opn)` (Operators.cu:529-553; CUMAT.java:31 applyop;
 * caller GMat.scala:1125).  All 15 op codes. */
int bidmat_applyop(const float *A, int Anrows, int Ancols, const float *B, int Bnrows,
                   int Bncols, float *C, int opn);

/* ------------------------------------------------------------------------------------
 * 2. Native entry points: take the column pointer jc (GSMat.pjc, which the reference
 *    keeps on the device but never passes to its kernels), an overwrite/accumulate flag
 *    and a stream.  beta == 0: the output is overwritten (no clear needed);
 *    beta == 1: the output holds the addend.  They only enqueue work on `stream`.
 * ------------------------------------------------------------------------------------ */

/* C = beta*C + A*S.   A k x nrowsS, S nrowsS x ncols (CSC), C k x ncols. */
int bidmat_dsmult_csc(int k, int ncols, int nnz, const float *A, const float *Sdata,
                      const int *Sir, const int *Sjc, float *C, int beta, void *stream);

/* P = beta*P + DDS(A,B,pattern).  A k x nrowsS, B k x ncols, P one value per nonzero. */
int bidmat_dds_csc(int k, int ncols, int nnz, const float *A, const float *B, const int *Sir,
                   const int *Sjc, float *P, int beta, void *stream);

/* bidmat_dds_csc for callers that must not allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments and results, bit for bit, as bidmat_dds_csc; the one scratch buffer that call
 * takes from the library's workspace (the table of extra wave segments of long columns) lives here
 * in a fixed 16 MiB array inside the library, one copy per device, which limits
 * ncols <= bidmat_dds_static_max_cols() (2 097 152); more columns return hipErrorInvalidValue.
 * No hipMalloc / hipFree or allocating routine is called.  Every call on a device uses that
 * device's one array: calls that overlap on a device (two streams, two threads) race on it. */
int bidmat_dds_csc_static(int k, int ncols, int nnz, const float *A, const float *B, const int *Sir,
                          const int *Sjc, float *P, int beta, void *stream);
int bidmat_dds_static_max_cols(void);

/* DDS with the elementwise step that follows it in an NMF / LDA update fused into the kernel:
 * P[j] = op(V[j], dot_j) with a BinOp code opn (3 = V ./ DDS).  One launch instead of
 * GSMat.DDS + GMat.gOp on the value arrays (GSMat.scala:649-667, GMat.scala:1119-1128,
 * Operators.cu:455-461); bit-identical to bidmat_dds_csc followed by bidmat_applyop_flat.
 * P == V (the update in place) is allowed while one pass covers k (k <= 1024 with 16-byte aligned A, B and
 * k % 4 == 0, otherwise k <= 256); beyond that, and for any other overlap of V and P, the call returns
 * hipErrorInvalidValue (wide k is walked in several passes that keep their running sums in P). */
int bidmat_dds_csc_op(int k, int ncols, int nnz, const float *A, const float *B, const int *Sir,
                      const int *Sjc, const float *V, int opn, float *P, void *stream);

/* Row-binned execution plan of one sparsity pattern, needed by A*^S and by sparse row sums.
 * The plan keeps its own device copies of what it needs; the pattern arrays may be freed
 * afterwards.  The values array is NOT captured: pass the current values to each call.
 * k_hint: the dense leading dimension the plan will mostly be used with (sizes the column
 * panels so that one panel of A stays in an XCD's L2); 0 = 256.
 * Blocking (device synchronisation inside).  Returns 0 and a handle in *plan. */
typedef struct bidmat_plan bidmat_plan;
int bidmat_plan_create(int nrows, int ncols, int nnz, const int *Sir, const int *Sjc, int k_hint,
                       bidmat_plan **plan);
int bidmat_plan_destroy(bidmat_plan *plan);
/* Device bytes held by the plan: index arrays and, after bidmat_plan_set_values, the stored values.
 * (The nseg*k partial sums of a call through the plan are scratch of the stream it runs on.) */
long long bidmat_plan_bytes(const bidmat_plan *plan);
/* Number of row segments of the plan (each yields one k-vector partial sum). */
int bidmat_plan_segments(const bidmat_plan *plan);
/* Inspection (tests, tools; no counterpart in the reference).  bidmat_plan_info: a scalar of the plan by name
 * ("nrows", "ncols", "nnz", "sides" (1 row side | 2 column side), "nseg", "nheavy", "npanels", "panel_cols",
 * "seglen", "col_classes", "class_hot", "longest_column", "xcd_start0" .. "xcd_start8", "dense_rows",
 * "dense_blocks", "dense_block_cols", "dense_segments"); -1 for an unknown name.
 * bidmat_plan_array: device address and element count (int32 each) of one of the plan's index arrays
 * ("pc", "perm", "segstart", "segrow", "rowseg", "rowptr", "cir", "cperm", "cptr", "ovf", "drow", "drank", "dpos";
 * count 0 when the plan does not hold it).  The arrays stay the plan's. */
long long bidmat_plan_info(const bidmat_plan *plan, const char *name);
int bidmat_plan_array(const bidmat_plan *plan, const char *name, const void **dptr, long long *count);

/* C = beta*C + A*S^T through a plan.  A k x ncols, C k x nrows(S).  Sdata: the nnz values
 * in the original CSC order.  With beta == 0 every column of C is written (zeros for empty
 * rows of S).
 * Dense block: when the pattern has rows with a nonzero in a large share of the columns (options "dense_rows",
 * "dense_min_pct", "dense_min_nnz" below; plan info "dense_rows"), the plan ranks up to 128 of them at build time and,
 * for 64 < k <= 256 (values passed in Sdata, or stored by bidmat_plan_set_values), their columns of C are computed as a dense product on the matrix
 * cores (the columns of A streamed once per 32 rows, absent entries as zeros) instead of one gather per nonzero.
 * Only the order in which those rows' terms are added changes (fixed by the pattern: same bits from run to run,
 * within the 1e-4 tolerance of the path); every other row keeps its bits.  A value of A that is not finite makes the
 * call compute those rows from their segments after all (decided on the device, also inside a replayed graph), so
 * an absent entry's zero never meets an infinity. */
int bidmat_dsmultT_plan(bidmat_plan *plan, int k, const float *A, const float *Sdata, float *C,
                        int beta, void *stream);

/* bidmat_dsmultT_plan for harnesses that time its two stages apart: event_between (a hipEvent_t passed as
 * void*, nullable) is recorded on the stream after stage 1 (the gathers into per-segment partial sums) and
 * before stage 2 (the addition of every row's partial sums).  No counterpart in the reference. */
int bidmat_dsmultT_plan_staged(bidmat_plan *plan, int k, const float *A, const float *Sdata, float *C,
                               int beta, void *stream, void *event_between);
/* Nonzeros that belong to rows cut by column panels ("heavy" rows, whose gathers reuse a panel of A that
 * stays in L2); the remaining nnz - heavy nonzeros are gathered once each with no reuse.  Blocking. */
long long bidmat_plan_heavy_nnz(const bidmat_plan *plan);

/* The values of the pattern in plan order, stored in the plan (nnz floats; on a plan with a dense block also the
 * dense rows' values in the layout of the block, ncols x dense rows floats): afterwards
 * bidmat_dsmultT_plan, bidmat_sdmult_plan and bidmat_spsum_rows_plan accept Sdata == NULL and stream
 * the stored values instead of fetching every value through the plan's permutation; so does
 * bidmat_dsmult_plan when the plan carries a row-class ordering of its columns and no column is longer
 * than 8192 nonzeros (otherwise it needs Sdata: hipErrorInvalidValue without).  For callers whose values stay the same over several calls (a data minibatch); call it
 * again when they change. */
int bidmat_plan_set_values(bidmat_plan *plan, const float *Sdata, void *stream);

/* A*S and DDS through a plan: the plan holds what is a function of the pattern alone (whether any
 * column is longer than a wave segment, and the table of the extra segments if so), so a call is
 * one launch when no column is long, and never builds or allocates per call.  bidmat_dds_plan gives
 * the same results, bit for bit, as bidmat_dds_csc / bidmat_dds_csc_op, whichever kernel the plan
 * selects; so does bidmat_dsmult_plan unless the plan carries a row-class ordering of its columns
 * (see "col_classes" below): then the nonzeros of a column are added class by class instead of in
 * stored order - a fixed order that depends on the pattern alone, so results repeat bit for bit
 * from run to run, and stay within the 1e-4 tolerance of the path.  Sir / Sjc: the pattern the plan
 * was made from.  bidmat_dds_plan: V == NULL gives P = beta*P + DDS, otherwise P = op(V, DDS). */
int bidmat_dsmult_plan(bidmat_plan *plan, int k, const float *A, const float *Sdata, const int *Sir,
                       const int *Sjc, float *C, int beta, void *stream);
int bidmat_dds_plan(bidmat_plan *plan, int k, const float *A, const float *B, const int *Sir,
                    const int *Sjc, const float *V, int opn, float *P, int beta, void *stream);
/* P = op(v, DDS) where v are the values stored in the plan by bidmat_plan_set_values (the data
 * matrix of an NMF / LDA update stays the same over all iterations): like bidmat_dds_plan with V, but
 * the kernel streams its copy of the values in the order it walks the nonzeros.
 * hipErrorInvalidValue when no values are stored. */
int bidmat_dds_plan_stored(bidmat_plan *plan, int k, const float *A, const float *B, const int *Sir,
                           const int *Sjc, int opn, float *P, void *stream);
/* One walk over the plan's rows for the chain Q = op(V, DDS(A, B, S)), G = beta*G + B *^ Q (the update of one
 * factor in NMF / LDA: DDS, Arith.cu:349-389; the elementwise step, Operators.cu:86-101; A *^ S, Arith.cu:206-248;
 * callers GSMat.scala:649-667 and GMat.scala:1082-1096).  A is k x nrows, B is k x ncols, G is k x nrows.  For
 * every nonzero the column of B is gathered once and serves the dot product and the accumulation; Q is only
 * written when Q != NULL (nnz values in the stored CSC order).  V == NULL: the values stored in the plan.  The
 * results are those of bidmat_dds_plan[_stored] followed by bidmat_dsmultT_plan, bit for bit (of bidmat_dsmultT_plan
 * walking the segments of every row, i.e. with option "dense_rows" = 0: its dense block adds the most frequent rows'
 * terms in another order).  k must fit one pass
 * (k <= 1024 with 16-byte aligned operands and k % 4 == 0, else k <= 256): otherwise hipErrorInvalidValue, and
 * the two calls remain.  Needs the row side of the plan. */
int bidmat_dds_dsmultT_plan(bidmat_plan *plan, int k, const float *A, const float *B, const float *V, int opn,
                            float *Q, float *G, int beta, void *stream);
/* The same chain by columns, Q = op(V, DDS(A, B, S)) and C = beta*C + A * Q (the E-step of an LDA / NMF update, where the
 * matrix that is dotted against is also the one that is multiplied: DDS, Arith.cu:349-389; the elementwise step,
 * Operators.cu:86-101; A * S, Arith.cu:16-60; callers GSMat.scala:649-667 and GMat.scala:1041-1074).  A is k x nrows,
 * B and C are k x ncols.  Every nonzero's column of A is gathered once for the dot product and the accumulation; Q (nnz
 * values in stored order) is only written when Q != NULL and may be V itself.  The results are those of
 * bidmat_dds_csc_op followed by bidmat_dsmult_csc, bit for bit.  k must fit one pass (k <= 1024 with 16-byte aligned
 * operands and k % 4 == 0, else k <= 256): otherwise hipErrorInvalidValue, and the two calls remain. */
/* The same chain through a plan (column side): with a row-class ordering of the columns (and no column longer than 8192
 * nonzeros) it runs in the passes of bidmat_dsmult_plan ("class_phases"), each pass computing the products and adding the
 * share of its row classes, so that the L2s hold more of the rows that matter; Q has the bits of bidmat_dds_plan with
 * the op, C those of bidmat_dsmult_plan fed with that Q (a fixed order that depends on the pattern alone).  Without a class
 * ordering it is bidmat_dds_dsmult_csc with the plan's table of long columns.  No counterpart in the reference. */
int bidmat_dds_dsmult_plan(bidmat_plan *plan, int k, const float *A, const float *B, const int *Sir, const int *Sjc,
                           const float *V, int opn, float *Q, float *C, int beta, void *stream);
int bidmat_dds_dsmult_csc(int k, int ncols, int nnz, const float *A, const float *B, const int *Sir, const int *Sjc,
                          const float *V, int opn, float *Q, float *C, int beta, void *stream);
/* Number of extra wave segments of the plan's long columns (0: every column fits one segment). */
int bidmat_plan_overflow_segments(const bidmat_plan *plan);

/* Sparse sums: out = beta*out + sums.  Column sums need only jc.  Row sums come in two forms:
 * through a plan (the values stored in the plan, Sdata == NULL, are summed in the plan's row order
 * at streaming speed; values passed in are gathered through the plan's permutation), or, for
 * values that were just produced, straight from the row indices (bidmat_spsum_rows_csc: one
 * pass over Sir and Sdata in any order, no plan, no jc).  The reference adds with float atomics in
 * arrival order (Arith.cu:250-264), so its row sums vary from run to run; bidmat_spsum_rows_csc
 * rounds every value once to a common step of 2^-(61 - bits of nnz) of the largest magnitude's
 * binade and adds 64-bit integers: the same bits whatever the order, and closer to the exact sum
 * than a float running sum.  Rows with NaN, or infinities of both signs, give NaN.  A row index
 * outside [0, nrows) leaves `out` untouched (bidmat_spsum reports it as hipErrorInvalidValue). */
int bidmat_spsum_cols(int ncols, int nnz, const float *Sdata, const int *Sjc, float *out,
                      int beta, void *stream);
int bidmat_spsum_rows_plan(bidmat_plan *plan, const float *Sdata, float *out, int beta,
                           void *stream);
int bidmat_spsum_rows_csc(int nrows, int nnz, const int *Sir, const float *Sdata, float *out,
                          int beta, void *stream);

/* jc[ncols+1] -> ic[nnz] (per-nonzero column index).  Replaces cusparseXcsr2coo at
 * GSMat.scala:639.  Enqueues on stream. */
int bidmat_csc_expand_cols(int ncols, int nnz, const int *Sjc, int *Sic, void *stream);
/* ir[j] = j - jc[c] for every nonzero j of column c: the row indices a sparse matrix stored
 * WITHOUT row indices implies (BIDMat file type 331, HMat.scala:1246-1258; SparseMat.explicitInds,
 * SparseMat.scala:79-93).  Enqueues on stream. */
int bidmat_csc_implicit_rows(int ncols, int nnz, const int *Sjc, int *Sir, void *stream);
/* Checks a device CSC pattern before kernels trust it: *rule = 0 when it is sound, otherwise the
 * first violated rule, numbered like the branches of SparseMat.check (SparseMat.scala:710-740):
 * 1 jc[0] != 0, 2 jc decreasing or outside [0, nnz], 5 a row index outside [0, nrows),
 * 6 jc[ncols] != nnz.  Rows need not be sorted or unique.  Sir may be NULL.  Blocking. */
int bidmat_csc_validate(int nrows, int ncols, int nnz, const int *Sir, const int *Sjc, int *rule);
/* Transpose of a device CSC matrix (nrows x ncols, nnz nonzeros) without leaving the device:
 * out_jc (nrows+1), out_ir (nnz: the original columns, ascending inside every output column),
 * out_data (nnz).  The reference's GSMat.t downloads, transposes on the host and uploads
 * (GSMat.scala:218-223).  Row indices outside the matrix are rejected.  Blocking. */
int bidmat_csc_transpose(int nrows, int ncols, int nnz, const float *Sdata, const int *Sir,
                         const int *Sjc, float *out_data, int *out_ir, int *out_jc);

/* Dense image of a sparse matrix, od[ir[j] + ic[j]*nrows] = data[j]; the caller clears od first
 * (GSMat.full, GSMat.scala:206-214).  Replaces full (CopyFill.cu:1456-1475,
 * CUMAT.java full).  Where a column stores one row twice, one of the values stays, as in the
 * reference.  Indices outside the matrix are skipped.  Blocking. */
int bidmat_full(const int *ir, const int *ic, const float *data, float *od, int nrows, int ncols, int nnz);

/* One-hot / n-hot pattern (GSMat.oneHot / GSMat.nHot, GSMat.scala:686-720): cats is an
 * n x ncols device int matrix of categories; column j of the result holds rows cats[:, j] in
 * the given order (not sorted, repeats allowed) with value 1.  Outputs: out_ir, out_ic,
 * out_data (n*ncols each), out_jc (ncols+1).  *maxcat (host, nullable) receives the largest
 * category (-1 when empty), which the reference uses as nrows-1 when ncats is not given.
 * Replaces a D2D copy, setval, initSeq and cusparseXcoo2csr.  Blocking. */
int bidmat_nhot(int n, int ncols, const int *cats, int *out_ir, int *out_ic, int *out_jc,
                float *out_data, int *maxcat);

/* Columns [col1, col2) of a device CSC matrix as a matrix of its own; replaces the four copies
 * and two index subtractions of GSMat.colslice (GSMat.scala:77-104).  First ask for the range
 * (blocking: reads Sjc[col1] and Sjc[col2]), allocate the outputs, then slice (enqueue only):
 * out_jc[0..col2-col1] rebased to 0, out_ir / out_data the nnz nonzeros from position start,
 * out_ic (nullable) the rebased column of every nonzero.
 * The product entries do not need a copy for a column range: pass Sjc + col1 with
 * ncols = col2 - col1 and the unsliced Sir / Sdata (column pointers are absolute positions). */
int bidmat_csc_colslice_range(int ncols, int col1, int col2, const int *Sjc, int *start, int *nnz);
int bidmat_csc_colslice(int col1, int col2, int start, int nnz, const int *Sjc, const int *Sir,
                        const float *Sdata, int *out_jc, int *out_ir, int *out_ic, float *out_data,
                        void *stream);

/* p[i] += delta on a device int array: the index-base conversion of GSMat.fromSMat / toSMat
 * (host SMat indices are 1-based by default, GSMat.scala:123-125,626-632) done on the device
 * instead of in a host loop.  Enqueues on stream. */
int bidmat_index_shift(int *p, long long n, int delta, void *stream);

/* non-decreasing ic[nnz] -> jc[ncols+1].  Replaces cusparseXcoo2csr at GSMat.scala:698,716
 * and SparseMat.compressInds (SparseMat.scala:857-868). Enqueues on stream. */
int bidmat_coo_compress_cols(int ncols, int nnz, const int *Sic, int *Sjc, void *stream);

/* Sparse times dense, the other operand order (GSMat.SDMult / SDTMult, GSMat.scala:265-313, which
 * call cusparseScsrmm with alpha = 1, beta = 0):
 *   bidmat_sdtmult_csc:  C (ncols x p) = S^T * A,  A is nrows x p   (S ^* A)
 *   bidmat_sdmult_plan:  C (nrows x p) = S * A,    A is ncols x p   (S * A), needs the row plan
 * A and C are column-major with leading dimensions lda / ldc.  Implemented on the gather
 * kernels through dense transposes ((S^T A)^T = A^T S, (S A)^T = A^T S^T) in library workspace. */
int bidmat_sdtmult_csc(int nrows, int ncols, int nnz, int p, const float *Sdata, const int *Sir,
                       const int *Sjc, const float *A, int lda, float *C, int ldc, void *stream);
int bidmat_sdmult_plan(bidmat_plan *plan, int p, const float *Sdata, const float *A, int lda, float *C,
                       int ldc, void *stream);
/* out (ncols x nrows, leading dimension ldo) = transpose of in (nrows x ncols, leading dim ldi). */
int bidmat_transpose(int nrows, int ncols, const float *in, int ldi, float *out, int ldo, void *stream);

/* Elementwise on flat arrays with a stream (the V./R step on GSMat.contents). */
int bidmat_applyop_flat(const float *A, const float *B, float *C, long long n, int opn,
                        void *stream);

/* ------------------------------------------------------------------------------------
 * 3. Device memory and runtime helpers (what the reference does through JCuda:
 *    cublasAlloc/cublasFree GSMat.scala:519-522,225-232; cudaMemcpy GSMat.scala:625-633;
 *    cudaMemset GMat.scala:562-566; cudaMemGetInfo GFunctions.scala:208-213).
 * ------------------------------------------------------------------------------------ */
int bidmat_device_count(int *count);
int bidmat_set_device(int dev);
int bidmat_get_device(int *dev);
int bidmat_malloc(void **dptr, long long bytes);
int bidmat_free(void *dptr);
int bidmat_memcpy_h2d(void *dst, const void *src, long long bytes);
int bidmat_memcpy_d2h(void *dst, const void *src, long long bytes);
int bidmat_memcpy_d2d(void *dst, const void *src, long long bytes);
int bidmat_memset(void *dptr, int value, long long bytes);
int bidmat_mem_info(long long *free_bytes, long long *total_bytes);
int bidmat_synchronize(void);
/* Asynchronous copies between PINNED host memory (bidmat_host_alloc) and the device on a stream. */
int bidmat_memcpy_h2d_async(void *dst, const void *src_pinned, long long bytes, void *stream);
int bidmat_memcpy_d2h_async(void *dst_pinned, const void *src, long long bytes, void *stream);
/* Pinned host staging buffers (allocated, never registered). */
int bidmat_host_alloc(void **hptr, long long bytes);
int bidmat_host_free(void *hptr);
/* HIP graphs (no counterpart in the reference, whose launchers block): record the stream-taking
 * calls issued on `stream` between begin and end, then replay them with one launch per step.
 * Only kernels are recorded (the library clears memory with fill kernels, never memset nodes).
 * Nothing may allocate while recording: run the same calls once on the same stream beforehand,
 * so that the stream's scratch buffers (partial sums of plan calls included) have their size.  The
 * recorded pointers and sizes are fixed; the data they point to may change between replays.
 * A recording also holds the addresses of the stream's scratch buffers and of any plan it used:
 * destroy it (and record again) before a larger problem is run on that stream (scratch grows by
 * reallocation), before the plan is destroyed and before bidmat_release_caches. */
int bidmat_graph_begin_capture(void *stream);
int bidmat_graph_end_capture(void *stream, void **graph_exec);
int bidmat_graph_launch(void *graph_exec, void *stream);
int bidmat_graph_destroy(void *graph_exec);

/* Streams and events for callers that time or overlap work (benchmark harness). */
int bidmat_stream_create(void **stream);
int bidmat_stream_destroy(void *stream);
int bidmat_stream_synchronize(void *stream);
int bidmat_event_create(void **event);
int bidmat_event_destroy(void *event);
int bidmat_event_record(void *event, void *stream);
int bidmat_event_synchronize(void *event);
int bidmat_event_elapsed_ms(void *start, void *stop, float *ms);
/* Text for a return code (cudaGetErrorString in the reference's exceptions, GMat.scala:1071). */
const char *bidmat_error_string(int err);
/* Library / device description: "bidmathip <version> gfx950 ..." */
const char *bidmat_version(void);
/* Name of the compiled-for architecture of the current device ("gfx950"), CU count. */
int bidmat_device_info(char *arch, int arch_len, int *compute_units, long long *total_mem);

/* Tunables (process-wide, read at call time):
 *   "seglen"   nonzeros per wavefront segment when a long column / row is split (default 1024)
 *   "panel_kb" target size in KiB of one column panel of A in a plan (default 4096: what one L2 holds)
 *   "heavy_min" a row is cut by column panels when it averages at least this many nonzeros
 *              per panel (default 8)
 *   "col_classes" row-class ordering of the columns inside a plan, used by bidmat_dds_plan so that the
 *              eight L2s of the device cache disjoint rows: -1 = decide from the pattern and k_hint
 *              (default), 0 = never, 1 = always
 *   "class_hot" most frequent rows per class that the class-ordered DDS kernel keeps in LDS: -1 = as
 *              many as 128 KiB hold when the plan's k_hint is below 256, none from 256 on (default),
 *              0 = none, otherwise the number
 *   "class_threads" workgroup size of that kernel when it keeps rows in LDS (256, 512 or 1024; default 1024)
 *   "class_phases" passes of bidmat_dsmult_plan over a class-ordered pattern, each pass gathering a
 *              disjoint share of the row classes so that the L2s hold more of the rows that matter
 *              (1, 2, 4 or 8; default 2; 0 = always the plain one-pass kernel)
 *   "class_strip" columns per wavefront in the class-ordered DDS kernel (default 16, 1..64)
 *   "cache_cols_after" the reference-shaped bidmat_dsmult / bidmat_dds (which receive no plan handle) find
 *              their pattern in a fingerprint cache; from this many calls on a pattern they build the column
 *              side of a plan for it and run through it (default 2; 0 = never look, always the plain kernels)
 *   "cache_plans" patterns the fingerprint cache keeps, least recently used dropped first (default 4; a
 *              cached plan of a 100 M-nonzero pattern holds 0.8 GB per side)
 *   "check_plan" 1 = plans made from now on keep a digest of their pattern and bidmat_dsmult_plan /
 *              bidmat_dds_plan[_stored] return hipErrorInvalidValue for any other Sir / Sjc (one extra pass
 *              over the index arrays per call; default 0: passing the plan's own pattern is the caller's duty)
 *   "plan_builder" how the row side of a plan is put in order: 0 = stable counting sorts per column panel and by
 *              row, written for this layout (default), 1 = one library radix sort of (key, position) pairs (also
 *              taken by itself when more than 24 575 rows are cut by panels); both give the same plan, bit for bit
 *   "rowsum_form" which kernel bidmat_spsum_rows_csc / bidmat_spsum(n = 2) take: 0 = by the number of rows (up to
 *              262 144 rows: every workgroup owns a range of rows with all accumulators in LDS; more: hashed
 *              tables in LDS in front of accumulators in global memory), 2 = always the latter; the same bits
 *   "plan_pool_mb" device memory of destroyed (or evicted) plans kept for the next plans, MiB per device (default
 *              4096; 0 = give every block back at once): a caller that meets a new pattern with every minibatch
 *              would otherwise pay hipMalloc + hipFree for the same sizes on every call; bidmat_release_caches frees it
 *   "plan_keep_mb" temporaries of a plan build up to this many MiB stay allocated on the device for the
 *              next build (default 4096: a 100 M-nonzero pattern needs 3.7 GB; 0 = always give them
 *              back); bidmat_release_caches frees them
 *   "dense_rows" how many of a pattern's most frequent rows a plan may treat as a dense block of A *^ S (see
 *              bidmat_dsmultT_plan; a multiple of 32 up to 128, default 128; 0 = none: plans made while it is 0 get no
 *              dense block, and calls made while it is 0 walk the segments of every row whatever the plan holds)
 *   "dense_min_pct" a row belongs to the dense block when it has a nonzero in at least this percentage of the
 *              columns (default 15; below about 9 % a gather per nonzero is cheaper than multiplying zeros)
 *   "dense_min_nnz" patterns with fewer nonzeros get no dense block (default 4 194 304)
 *   "dense_cb" columns per block of the dense product, each block giving one partial sum per dense row
 *              (default 0 = chosen from the column count so that the blocks fill the device evenly, about 330 to 400)
 *   "scalar_values" 1 (default): A *^ S over a plan, with the values in the caller's order and k > 128 (k > 32 when
 *              k is no multiple of 4 or an operand is not 16-byte aligned), fetches each nonzero's value by a scalar
 *              load from its position; 0: by one gather per lane and chunk of 64 nonzeros. Same bits either way.
 * Returns 0, or hipErrorInvalidValue for an unknown name / bad value; bidmat_get_option returns -2
 * for an unknown name. */
int bidmat_set_option(const char *name, long long value);
long long bidmat_get_option(const char *name);

/* Drops every cached plan and workspace buffer of the current device. */
int bidmat_release_caches(void);

#ifdef __cplusplus
}
#endif
#endif /* BIDMAT_HIP_H */
