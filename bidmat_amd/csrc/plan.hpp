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

struct bidmat_plan {
    int device = 0;
    int nrows = 0, ncols = 0, nnz = 0;
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
    float* partial = nullptr;
    size_t partial_floats = 0;
    size_t index_bytes = 0;
};

namespace bm {
hipError_t plan_build(int nrows, int ncols, int nnz, const int* ir, const int* jc, int k_hint,
                      bidmat_plan** out);
hipError_t plan_free(bidmat_plan* p);
// Makes sure the plan's partial buffer holds nseg*k floats.
hipError_t plan_reserve_partial(bidmat_plan* p, int k);
}  // namespace bm
