// Host-side launchers of the gfx950 kernels (internal to the library; the C ABI in
// capi.cpp validates arguments and calls these).
#pragma once
#include <hip/hip_runtime.h>

namespace bm {

// ---- tunables (capi.cpp owns the storage)
int opt_seglen();      // nonzeros per wave segment for long columns / rows
int opt_panel_kb();    // KiB of A per column panel in a plan
int opt_heavy_min();   // a row is cut by panels when it averages at least this many nonzeros per panel
int opt_class_threads(); // workgroup size of the class-ordered DDS kernel when it keeps hot rows in LDS (256, 512, 1024)
int opt_class_phases(); // passes of A*S over a class-ordered pattern (1, 2, 4, 8), 0 = plain kernel
int opt_class_strip(); // columns per wave in the class-ordered DDS kernel (1..64)
int opt_plan_keep_mb(); // plan-build temporaries up to this many MiB stay allocated for the next build
int opt_class_hot();   // hot rows per class kept in LDS by the class-ordered DDS kernel: -1 = by k_hint (default), 0 = none
int opt_plan_pool_mb(); // MiB of freed plan blocks kept per device for the next plans
int opt_class_shift();  // class ordering: class of row r = (r >> shift) & 7; -1 = chosen from k
int opt_rowsum_form();  // bidmat_spsum_rows_csc: 0 = by the row count (default), 2 = always the hashed tables with global accumulators
int opt_plan_builder(); // row side of a plan: 0 = per-panel counting sorts (default), 1 = one library radix sort
int opt_check_plan();  // 1: plans keep a digest of their pattern and the plan-taking calls compare it
int opt_col_classes(); // row-class ordering of the columns in a plan: -1 decide from the pattern, 0 never, 1 always
int opt_dense_rows();  // rows a plan may treat as a dense block of A *^ S (0 = none, at most 128)
int opt_dense_min_pct(); // a row counts as dense when it has a nonzero in at least this percentage of the columns
int opt_dense_min_nnz(); // patterns with fewer nonzeros get no dense block
int opt_dense_cb();    // columns per block of the dense product (0 = chosen from the column count)
int opt_scalar_values();   // A *^ S over a plan fetches the caller's values by scalar loads (1) or by a gather per lane (0)

// ---- CSC utilities (csc_util.hip)
hipError_t csc_expand_cols(int ncols, int nnz, const int* jc, int* ic, hipStream_t s);
hipError_t coo_compress_cols(int ncols, int nnz, const int* ic, int* jc, hipStream_t s);
// jc[c] = number of entries of the sorted ic[0..nnz) below c, c = 0..ncols, by a binary search per c
hipError_t sorted_lower_bounds(int ncols, int nnz, const int* ic, int* jc, hipStream_t s);
// ir[j] = j - jc[c]: the implied rows of a sparse matrix stored without row indices
hipError_t csc_implicit_rows(int ncols, int nnz, const int* jc, int* ir, hipStream_t s);
// *d_flags (device int) = bit set of violated rules: 1 jc[0] != 0, 2 jc decreasing or outside
// [0, nnz], 5 a row index outside [0, nrows), 6 jc[ncols] != nnz. ir may be nullptr (rows not checked).
hipError_t csc_validate(int nrows, int ncols, int nnz, const int* ir, const int* jc, int* d_flags, hipStream_t s);
// columns [col1, col1+nc) with n nonzeros starting at position `start`: out_jc (nc+1, rebased),
// out_ir / out_data (n), out_ic (n, nullable)
hipError_t csc_colslice(int nc, int start, int n, const int* jc_at_col1, const int* ir, const float* data,
                        int* out_jc, int* out_ir, int* out_ic, float* out_data, hipStream_t s);
// n-hot pattern from an n x ncols category matrix; *d_maxcat (device int) receives the largest category
hipError_t nhot(int n, int ncols, const int* cats, int* ir, int* ic, int* jc, float* data, int* d_maxcat,
                hipStream_t s);
// transpose of a CSC matrix (csc_transpose.hip): out_jc has nrows+1 entries, out_ir holds the
// original columns in ascending order inside every output column. Blocks until done.
hipError_t csc_transpose(int nrows, int ncols, int nnz, const float* data, const int* ir, const int* jc,
                         float* out_data, int* out_ir, int* out_jc, hipStream_t s);
// od[ir[j] + ic[j]*ld] = data[j] for every nonzero (od cleared by the caller)
hipError_t full_from_coo(int nrows, int ncols, int nnz, const int* ir, const int* ic, const float* data, float* od,
                         int ld, hipStream_t s);
// p[i] += delta
hipError_t index_shift(int* p, long long n, int delta, hipStream_t s);
// out[i] = v for i < n (a kernel, so that callers may record it into a HIP graph)
hipError_t fill_f32(float* out, long long n, float v, hipStream_t s);
hipError_t fill_i32(int* out, long long n, int v, hipStream_t s);
// One pass over the two index arrays of a pattern (device result, 4 x uint64): [0], [1] two 64-bit digests
// of the sequence of (ic, ir) pairs, [2] (as int) the largest entry of ir (-1: empty). d_out must hold
// pattern_digest_words() words (the rest is scratch of the pass).
size_t pattern_digest_words();
// jc != nullptr: also writes the column pointer jc[ncols+1] that ic implies (ic non-decreasing), in the same pass.
// z != nullptr (and nnz > 0): d_out[3] = 0 exactly when every word of z[0..nz) is +0.0f.
hipError_t pattern_digest(const int* ir, const int* ic, long long nnz, unsigned long long* d_out, hipStream_t s,
                          int ncols = 0, int* jc = nullptr, const float* z = nullptr, long long nz = 0);

// ---- overflow-segment table shared by dsmult and dds (spmm.hip)
// Returns in *d_ovf a device table int[ncols+1] (exclusive scan of the number of extra
// seglen-sized segments of each column), or nullptr when no column can exceed seglen.
hipError_t build_overflow_table(int ncols, int nnz, const int* jc, int seglen, int** d_ovf,
                                hipStream_t s);
// The same into caller-provided memory of overflow_table_ints(ncols) ints (no allocation).
size_t overflow_table_ints(int ncols);
hipError_t build_overflow_table_in(int ncols, int nnz, const int* jc, int seglen, int* buf, int** d_ovf,
                                   hipStream_t s);
// A column overflow table that the caller already holds (a plan builds it once per pattern):
// seglen it was built with, table (ncols+1 ints; unused when novf == 0), number of overflow
// segments. (A*S keeps the novf*k partial sums of those segments in the stream's scratch.)
struct ColTable { int seglen; const int* ovf; long long novf; };

// A window [off, off+len) on the gather index of the nonzeros (tile variants); on == 0: no filter.
struct Window { int on, off, len; };

// ---- A*S (spmm.hip)
hipError_t dsmult_csc(int k, int ncols, int nnz, const float* A, const float* vals, const int* ir,
                      const int* jc, float* C, int beta, hipStream_t s, const ColTable* tab = nullptr);
// tile form: A and C with their own column strides; only nonzeros with a row inside `rows`
// take part, rebased to rows.off (jc already points at the first column of the tile).
hipError_t dsmult_csc_ex(int k, int lda, int ldc, int ncols, int nnz, const float* A, const float* vals,
                         const int* ir, const int* jc, float* C, int beta, Window rows, hipStream_t s,
                         const ColTable* tab = nullptr);
// A*S on a plan's class-ordered pattern (cir / cperm / cptr with 16 groups per column, no hot-row
// ranks) in nphase passes over disjoint row classes; see spmm.hip.
hipError_t dsmult_phased(int k, int ncols, const float* A, const float* vals, const int* cir, const int* cperm,
                         const int* cptr, int nphase, float* C, int beta, hipStream_t s);
// ---- DDS (dds.hip)
// V != nullptr: P[j] = op(V[j], dot_j) with the BinOp code opn (beta must be 0) - the elementwise
// step that follows DDS in an NMF update, applied before the result leaves the registers.
hipError_t dds_csc(int k, int ncols, int nnz, const float* A, const float* B, const int* ir,
                   const int* jc, float* P, int beta, hipStream_t s, const float* V = nullptr, int opn = 0,
                   const ColTable* tab = nullptr);
// DDS over a row-class ordered pattern (a plan's cir / cperm / cptr); same results, bit for bit.
// hcap / hotrows: the hot rows per class the ordering was built with. v_classed: V is in class order. Fails with hipErrorInvalidValue
// when hcap rows of k floats do not fit the kernel's LDS budget (callers then use dds_csc).
size_t dds_classed_lds_budget();
hipError_t dds_classed(int k, int ncols, const float* A, const float* B, const int* cir, const int* cperm,
                       const int* cptr, int hcap, const int* hotrows, float* P, int beta, hipStream_t s,
                       const float* V = nullptr, int opn = 0, bool v_classed = false);
// The same with no allocation at all: the overflow table lives in a fixed device array of the
// library (one copy per device). ncols may not exceed dds_static_max_cols().
int dds_static_max_cols();
hipError_t dds_csc_static(int k, int ncols, int nnz, const float* A, const float* B, const int* ir,
                          const int* jc, float* P, int beta, hipStream_t s);

// ---- plan stage kernels (spmm.hip): segment s gathers columns pc[p] of A scaled by
// vals[perm[p]] for p in [segstart[s], segstart[s+1]) into partial[s*k ..].
// xcd_start[9]: segment groups per XCD (see plan.hpp); workgroup b is assumed to run on XCD b % 8.
// skip (nullable): a byte per segment, 1 = leave the segment out. flag (nullable): an int the launch clears.
hipError_t gather_segments(int k, int nseg, const int* xcd_start, const float* A, const float* vals,
                           const int* pc, const int* perm, const int* segstart, float* partial,
                           hipStream_t s, const unsigned char* skip = nullptr, int* flag = nullptr);
// The segments list[0..n) only, and only if *flag != 0 when the launch runs (its waves return at once otherwise).
hipError_t gather_segments_listed(int k, int n, const int* list, const int* flag, const float* A, const float* vals,
                                  const int* pc, const int* perm, const int* segstart, float* partial, hipStream_t s);
// tile form: column stride lda of A; only nonzeros whose column lies in `cols` (rebased), only
// segments whose row (segrow) lies in `rowsel`.
hipError_t gather_segments_ex(int k, int lda, int nseg, const int* xcd_start, const float* A,
                              const float* vals, const int* pc, const int* perm, const int* segstart,
                              float* partial, Window cols, const int* segrow, Window rowsel, hipStream_t s);
// Fused form: q_p = op(vals, dot(R[:, row of the segment], A[:, pc[p]])) and partial[s*k ..] = sum of q_p * A[:, pc[p]]
// (vals through perm, or in plan order when perm == nullptr); qout (nullable) receives q_p at qperm[p] (plan order
// when qperm == nullptr). hipErrorInvalidValue when k does not fit one pass (k > 1024, or > 256 unaligned).
hipError_t fused_segments(int k, int ldr, int lda, int nseg, const int* xcd_start, const int* segrow,
                          const float* R, const float* A, const float* vals, const int* pc, const int* perm,
                          const int* qperm, int opn, const int* segstart, float* partial, float* qout,
                          hipStream_t s);
// The chain by columns: Q[j] = op(vals[j], dot(A[:, ir[j]], B[:, c])) (nullable output) and C[:, c] = beta*C[:, c] + sum of
// Q[j] * A[:, ir[j]]; segments and order of additions of dsmult_csc. hipErrorInvalidValue when k does not fit one pass.
hipError_t fused_columns(int k, int ncols, int nnz, const float* A, const float* B, const float* vals, const int* ir,
                         const int* jc, int opn, float* Q, float* C, int beta, hipStream_t s, const ColTable* tab = nullptr);
// The same over a plan's class-ordered pattern (no hot-row ranks) in nphase passes over disjoint row classes, like
// dsmult_phased: q as above (bit for bit), C's additions pass by pass and class by class.
hipError_t fused_columns_phased(int k, int ncols, const float* A, const float* B, const float* vals, const int* cir,
                                const int* cperm, const int* cptr, int nphase, int opn, float* Q, float* C, int beta,
                                hipStream_t s);
// C[:,r] = beta*C[:,r] + sum over q in [rowptr[r], rowptr[r+1]) of partial[rowseg[q]*k ..]
// rowptr2 / rowseg2 / flag (nullable): the table to use instead while *flag == 0.
hipError_t reduce_segments(int k, int nrows, const int* rowptr, const int* rowseg,
                           const float* partial, float* C, int beta, hipStream_t s, const int* rowptr2 = nullptr,
                           const int* rowseg2 = nullptr, const int* flag = nullptr);
// tile form: rows [row0, row0+nrows) of the plan go to columns 0.. of C (stride ldc)
hipError_t reduce_segments_ex(int k, int ldc, int row0, int nrows, const int* rowptr, const int* rowseg,
                              const float* partial, float* C, int beta, hipStream_t s, const int* rowptr2 = nullptr,
                              const int* rowseg2 = nullptr, const int* flag = nullptr);

// ---- sums (sums.hip)
hipError_t spsum_cols(int ncols, int nnz, const float* vals, const int* jc, float* out, int beta,
                      hipStream_t s);
hipError_t spsum_segments(int nseg, const int* xcd_start, const float* vals, const int* perm, const int* segstart,
                          float* partial, hipStream_t s);
// out[r] (+)= sum of vals[j] over ir[j] == r, from the unordered (row, value) list itself: exact
// 64-bit integer accumulation after one common scaling, so the result does not depend on the order
// in which nonzeros arrive. If a row index lies outside [0, nrows) nothing is written; `bad_rows`
// (optional) makes the call wait for the stream and reports that.
hipError_t spsum_rows_exact(int nrows, long long nnz, const int* ir, const float* vals, float* out, int beta,
                            int* bad_rows, hipStream_t s);
hipError_t reduce1op(int nrows, int ncols, const float* A, float* B, float initv, int opn,
                     hipStream_t s);
hipError_t reduce2op(int nrows, int ncols, const float* A, float* B, float initv, int opn,
                     hipStream_t s);

// ---- elementwise (applyop.hip)
hipError_t applyop(const float* A, int Anr, int Anc, const float* B, int Bnr, int Bnc, float* C,
                   int opn, hipStream_t s);

// A[i] = op(A[i], len > 1 ? B[idx[i]] : B[0]) over the nnz stored values (in place)
hipError_t sdop(long long nnz, float* A, const int* idx, const float* B, int len, int opn, hipStream_t s);
// out (ncols x nrows, leading dimension ldo) = transpose of in (nrows x ncols, leading dimension ldi)
hipError_t transpose(int nrows, int ncols, const float* in, int ldi, float* out, int ldo, hipStream_t s);

}  // namespace bm
