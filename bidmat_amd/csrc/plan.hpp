// Row-binned execution plan of one CSC sparsity pattern (internal definition of the
// opaque bidmat_plan of the C ABI).
//
// The nonzeros are reordered so that all nonzeros of one row that fall into one column panel
// are contiguous ("segments"); a segment never exceeds seglen nonzeros. Rows with many
// nonzeros ("heavy" rows) are cut by column panels, sized so that a panel of the dense operand
// (panel columns x k floats) stays in L2 while every heavy row's segment of that panel is
// processed; all other rows form one run over the whole column range. Stage 1 gathers each
// segment into a k-vector partial sum, stage 2 adds a row's partial sums in a fixed order.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

// A plan has two independent halves. The row side (PLAN_ROWS) serves A*^S, S*A and sparse row sums;
// the column side (PLAN_COLS) serves A*S and DDS. Either can be built alone and the other added later.
namespace bm { enum { PLAN_ROWS = 1, PLAN_COLS = 2 }; }

struct bidmat_plan {
    int device = 0;
    int nrows = 0, ncols = 0, nnz = 0;
    int sides = 0;           // PLAN_ROWS | PLAN_COLS: which halves have been built
    int k_hint = 0;          // dense leading dimension the plan was sized for
    // 64-bit digests of the ir and jc arrays the plan was built from, taken when option "check_plan" is on:
    // the plan-taking calls then refuse a pattern that is not the plan's
    bool has_digest = false;
    unsigned long long digest[2] = {0, 0};
    int nseg = 0;            // number of segments
    int nheavy = 0;          // rows cut by column panels
    int npanels = 0;
    int panel_cols = 0;
    int seglen = 0;
    // Segments are stored heavy first, grouped by the XCD that is to process them: group x
    // (panels x, x+8, x+16, ... in ascending order) is [xcd_start[x], xcd_start[x+1]); the
    // light-row segments follow from xcd_start[8] and are dealt round-robin to the XCDs.
    int xcd_start[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
    int* pc = nullptr;       // [nnz]    column of the p-th nonzero in plan order
    int* perm = nullptr;     // [nnz]    its position in the original CSC order
    int* segstart = nullptr; // [nseg+1] segment boundaries in plan order
    int* segrow = nullptr;   // [nseg]   row of each segment
    int* rowptr = nullptr;   // [nrows+1] range of a row's segments in rowseg
    int* rowseg = nullptr;   // [nseg]   segment ids grouped by row, ascending within a row
    void* block_nnz = nullptr;   // owns pc, perm, rowptr
    void* block_seg = nullptr;   // owns segstart, segrow, rowseg
    // The densest rows as a dense block of A *^ S (dense_rows.hip; optional, ndense == 0: none). The segments of
    // these rows stay in the arrays above (row sums and the other walks over the plan use them); A *^ S leaves
    // them out (dskip) and multiplies the rows on the matrix cores instead, one partial sum per dense row and
    // block of dcb columns, which the second row table (rowptr2 / rowseg2) lists in place of the segments.
    int ndense = 0;              // dense rows, a multiple of 32
    int dcb = 0;                 // columns per block of the dense product
    int ndblocks = 0;            // blocks of columns
    int ndseg = 0;               // segments of the dense rows
    int* drank = nullptr;        // [nrows]  rank of a dense row (by count, descending), -1 for every other row
    int* drow = nullptr;         // [ndense] row of every rank
    int* dpos = nullptr;         // [ncols*ndense] position (stored order) of column c's nonzero in dense row d, or -1
    float* dvals = nullptr;      // [ncols*ndense] the stored values at those positions, 0 where there is none (optional:
                                 // bidmat_plan_set_values on a plan with a dense block)
    unsigned char* dskip = nullptr;  // [nseg] 1: segment of a dense row
    int* dseglist = nullptr;     // [ndseg] those segments
    int* rowptr2 = nullptr;      // [nrows+1] like rowptr / rowseg, a dense row's entries being the partial sums
    int* rowseg2 = nullptr;      //           nseg + (ndblocks + ch)*ndense + d of the chunks ch of blocks of columns
    void* block_dense = nullptr; // owns drank, drow, dskip, dseglist, rowptr2, rowseg2
    size_t dense_bytes = 0;      // device bytes of the dense block's arrays (counted in row_bytes)
    // (the nseg*k partial sums of a call live in the scratch of the stream it runs on, not here)
    size_t row_bytes = 0;        // device bytes of the row side's index arrays
    size_t col_bytes = 0;        // device bytes of the column side's index arrays
    // Column side (A*S and DDS through the plan): the overflow-segment table of the columns is a
    // function of jc and seglen only, so it is built once here instead of on every call.
    int col_seglen = 0;          // seglen in force when the plan was built
    int novf = 0;                // overflow segments of all columns (0: no column is longer than col_seglen)
    int* ovf = nullptr;          // [ncols+1] exclusive scan of extra segments per column (only when novf > 0)
    // Row-class ordering of every column (DDS through the plan). The eight XCDs have one L2 each;
    // when each of them gathers from the whole dense operand, all eight L2s end up holding the same
    // popular rows. Rows are dealt to eight classes (row & 7) and the nonzeros of every column are
    // grouped by the class of their row (stored order kept inside a group); a workgroup that runs
    // on XCD x only touches class-x nonzeros, so every L2 caches one eighth of the rows.
    // Built when the pattern promises a gain (plan.hip: wants_classes) or when the option says so.
    int ncls = 0;                // 0: no class ordering; otherwise 8
    int cshift = 0;              // class of row r = (r >> cshift) & 7
    int maxlen = 0;              // longest column
    int* cir = nullptr;          // [nnz]         row of the p-th nonzero in class order
    int* cperm = nullptr;        // [nnz]         its position in the original CSC order
    int* cptr = nullptr;         // [16*ncols + 1] column c, class x: hot-row nonzeros from cptr[16*c + 2*x],
                                 //               the others from cptr[16*c + 2*x + 1]
    // The most frequent rows of every class ("hot": at most hcap per class) are kept in LDS by the DDS
    // kernel. For their nonzeros cir holds the row's rank among its class's hot rows, not the row.
    int hcap = 0;                // hot rows per class the ordering was built for (0: none)
    int* hotrows = nullptr;      // [8*hcap] row of rank h of class x at hotrows[x*hcap + h], -1 = unused
    // Values in plan order (optional, bidmat_plan_set_values): pvals[p] = data[perm[p]], so that
    // A*^S and row sums stream their values instead of fetching each one through perm.
    float* pvals = nullptr;
    float* cvals = nullptr;      // the same in class order (with a class ordering): cvals[p] = data[cperm[p]]
    float* svals = nullptr;      // the same in stored (CSC) order (without a class ordering): a plain copy
};

namespace bm {
// sides: which halves to build now (PLAN_ROWS, PLAN_COLS or both).
hipError_t plan_build(int nrows, int ncols, int nnz, const int* ir, const int* jc, int k_hint,
                      bidmat_plan** out, int sides = PLAN_ROWS | PLAN_COLS);
// Builds the halves named in `sides` that the plan does not hold yet, from the pattern the plan was
// made from. On failure the plan keeps the halves it had.
hipError_t plan_extend(bidmat_plan* p, const int* ir, const int* jc, int sides);
hipError_t plan_free(bidmat_plan* p);
// Row side by per-panel counting sorts (plan_rows.hip): fills pc, perm, rowptr (allocated by the caller) and
// allocates and fills the segment tables. hcode[r]: heavy rank of row r or -1; hrow: row of every rank.
// At most rows_binned_max_heavy() heavy rows.
int rows_binned_max_heavy();
// *unfit = 1 (with hipSuccess, nothing allocated in the plan) when the pattern does not fit this builder.
hipError_t build_rows_binned(bidmat_plan* plan, const int* ir, const int* jc, const int* hcode, const int* hrow,
                             int nheavy, int p8, int* bad, int* unfit, hipStream_t s);
// d[0], d[1] = digests of ir[nnz] and jc[ncols+1] (blocking; default stream)
hipError_t plan_digest(int nnz, int ncols, const int* ir, const int* jc, unsigned long long d[2]);
// pvals[p] = data[perm[p]] (allocates pvals on first use).
hipError_t plan_set_values(bidmat_plan* p, const float* data, hipStream_t s);
// The dense block of the row side (dense_rows.hip). cnt[r]: about (nonzeros of row r) / sample.
hipError_t build_dense_rows(bidmat_plan* plan, const int* ir, const int* jc, const int* cnt, int sample, hipStream_t s);
hipError_t drop_dense(bidmat_plan* p);
bool dense_rows_fit(int k);      // the dense product is written for 64 < k <= 256
int dense_rows_max();
int dense_rows_fold(int ndblocks);   // partial sums per dense row that reach the row reduction
// vals == nullptr: the values come from dvals (the plan's copy in the layout of dpos) instead of vals[dpos[..]]
hipError_t dense_rows_stage(int k, int ncols, int nd, int cb, int ndblocks, const float* A, const float* vals,
                            const int* dpos, const float* dvals, float* part, int* flag, hipStream_t s);
// dvals[i] = dpos[i] >= 0 ? data[dpos[i]] : 0 for the ncols*nd slots of a plan's dense block (allocates dvals on first use;
// without memory for it the plan keeps none and calls with stored values walk the segments of every row)
hipError_t dense_rows_set_values(bidmat_plan* plan, const float* data, hipStream_t s);
}  // namespace bm
