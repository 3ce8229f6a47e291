// Elementwise binary operators with BIDMat's broadcasting rules. Streaming kernels: 12 bytes
// per element; the equal-shape case uses 128-bit accesses.
#include "common.hpp"
#include "kernels.hpp"
#include "ops.hpp"
#include <math.h>

namespace bm {
namespace {

// Index modes: how element i (column-major, nrows x ncols) picks its operand.
enum Mode { FULL = 0, COL = 1, ROW = 2, VAL = 3 };

template <int MODE>
__device__ __forceinline__ long long pick(long long i, int nrows) {
    if constexpr (MODE == FULL) return i;
    else if constexpr (MODE == COL) return i % nrows;      // column vector: one entry per row
    else if constexpr (MODE == ROW) return i / nrows;      // row vector: one entry per column
    else return 0;
}

template <int OP, int MA, int MB>
__global__ __launch_bounds__(BM_BLOCK) void k_apply(const float* __restrict__ A, const float* __restrict__ B,
                                                    float* __restrict__ C, long long n, int nrows) {
    long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    for (; i < n; i += stride) C[i] = binop<OP>(A[pick<MA>(i, nrows)], B[pick<MB>(i, nrows)]);
}

template <int OP>
__global__ __launch_bounds__(BM_BLOCK) void k_apply_full4(const float4* __restrict__ A, const float4* __restrict__ B,
                                                          float4* __restrict__ C, long long n4) {
    // a workgroup walks tiles of 4 x 256 vectors: four independent 128-bit loads per operand in
    // flight per thread, neighbouring in memory
    constexpr int UN = 4;
    long long i = (long long)blockIdx.x * (UN * BM_BLOCK) + threadIdx.x;
    const long long stride = (long long)gridDim.x * (UN * BM_BLOCK);
    for (; i + (UN - 1) * BM_BLOCK < n4; i += stride) {
        float4 a[UN], b[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) { a[u] = A[i + u * BM_BLOCK]; b[u] = B[i + u * BM_BLOCK]; }
#pragma unroll
        for (int u = 0; u < UN; ++u)
            C[i + u * BM_BLOCK] = make_float4(binop<OP>(a[u].x, b[u].x), binop<OP>(a[u].y, b[u].y),
                                              binop<OP>(a[u].z, b[u].z), binop<OP>(a[u].w, b[u].w));
    }
    // the last, partial tile
#pragma unroll
    for (int u = 0; u < UN; ++u) {
        const long long j = i + u * BM_BLOCK;
        if (j < n4) {
            const float4 a = A[j], b = B[j];
            C[j] = make_float4(binop<OP>(a.x, b.x), binop<OP>(a.y, b.y), binop<OP>(a.z, b.z), binop<OP>(a.w, b.w));
        }
    }
}

// Sparse values op edge vector, in place: A[i] = op(A[i], B[idx[i]]) (GATHER) or op(A[i], B[0]).
template <int OP, bool GATHER>
__global__ __launch_bounds__(BM_BLOCK) void k_sdop(long long nnz, float* __restrict__ A, const int* __restrict__ idx,
                                                   const float* __restrict__ B) {
    // tiles of 4 x 256 values per workgroup: four loads (and four dependent gathers) in flight
    constexpr int UN = 4;
    long long i = (long long)blockIdx.x * (UN * BM_BLOCK) + threadIdx.x;
    const long long stride = (long long)gridDim.x * (UN * BM_BLOCK);
    const float bval = GATHER ? 0.f : B[0];
    for (; i < nnz; i += stride) {
        float a[UN], b[UN];
        int ix[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const long long j = i + u * BM_BLOCK;
            const bool ok = j < nnz;
            a[u] = ok ? A[j] : 0.f;
            ix[u] = (GATHER && ok) ? idx[j] : 0;
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) b[u] = GATHER ? B[ix[u]] : bval;
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const long long j = i + u * BM_BLOCK;
            if (j < nnz) A[j] = binop<OP>(a[u], b[u]);
        }
    }
}

// Dense transpose through a padded LDS tile: in is nrows x ncols (column-major, leading dimension
// ldi), out is ncols x nrows (leading dimension ldo). Reads and writes are both coalesced.
constexpr int TT = 32;
__global__ __launch_bounds__(BM_BLOCK) void k_transpose(int nrows, int ncols, const float* __restrict__ in, int ldi,
                                                        float* __restrict__ out, int ldo) {
    __shared__ float tile[TT][TT + 1];
    const int tx = threadIdx.x & (TT - 1), ty = threadIdx.x / TT;     // 32 x 8 threads
    const long long r0 = (long long)blockIdx.x * TT, c0 = (long long)blockIdx.y * TT;
#pragma unroll
    for (int j = ty; j < TT; j += BM_BLOCK / TT) {
        const long long r = r0 + tx, c = c0 + j;
        if (r < nrows && c < ncols) tile[j][tx] = in[(size_t)c * ldi + r];
    }
    __syncthreads();
#pragma unroll
    for (int j = ty; j < TT; j += BM_BLOCK / TT) {
        const long long c = c0 + tx, r = r0 + j;                      // out[c, r] = in[r, c]
        if (r < nrows && c < ncols) out[(size_t)r * ldo + c] = tile[tx][j];
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

inline unsigned grid_for(long long n) {
    long long b = (n + BM_BLOCK - 1) / BM_BLOCK;
    if (b < 1) b = 1;
    if (b > 16384) b = 16384;
    return (unsigned)b;
}

template <int OP>
hipError_t apply_impl(const float* A, int ma, const float* B, int mb, float* C, long long n, int nrows,
                      hipStream_t s) {
    if (n <= 0) return hipSuccess;
    if (ma == FULL && mb == FULL) {
        long long n4 = 0;
        if (aligned16(A) && aligned16(B) && aligned16(C)) {
            n4 = n / 4;
            if (n4 > 0) hipLaunchKernelGGL(k_apply_full4<OP>, dim3(grid_for((n4 + 3) / 4)), dim3(BM_BLOCK), 0, s,
                                           (const float4*)A, (const float4*)B, (float4*)C, n4);
        }
        long long done = n4 * 4;
        if (done < n) hipLaunchKernelGGL((k_apply<OP, FULL, FULL>), dim3(grid_for(n - done)), dim3(BM_BLOCK), 0, s,
                                         A + done, B + done, C + done, n - done, nrows);
        return hipGetLastError();
    }
    dim3 grid(grid_for(n)), block(BM_BLOCK);
#define BM_M(MA_, MB_)                                                                        \
    if (ma == MA_ && mb == MB_) {                                                             \
        hipLaunchKernelGGL((k_apply<OP, MA_, MB_>), grid, block, 0, s, A, B, C, n, nrows);    \
        return hipGetLastError();                                                             \
    }
    BM_M(FULL, COL) BM_M(FULL, ROW) BM_M(COL, FULL) BM_M(ROW, FULL) BM_M(FULL, VAL) BM_M(VAL, FULL)
#undef BM_M
    return hipErrorInvalidValue;
}

}  // namespace

hipError_t sdop(long long nnz, float* A, const int* idx, const float* B, int len, int opn, hipStream_t s) {
    if (nnz <= 0) return hipSuccess;
    dim3 grid(grid_for((nnz + 3) / 4)), block(BM_BLOCK);
    switch (opn) {
#define BM_OP(N_)                                                                                          \
    case N_:                                                                                               \
        if (len > 1) hipLaunchKernelGGL((k_sdop<N_, true>), grid, block, 0, s, nnz, A, idx, B);            \
        else hipLaunchKernelGGL((k_sdop<N_, false>), grid, block, 0, s, nnz, A, idx, B);                   \
        return hipGetLastError();
    BM_OP(0) BM_OP(1) BM_OP(2) BM_OP(3) BM_OP(4) BM_OP(5) BM_OP(6) BM_OP(7)
    BM_OP(8) BM_OP(9) BM_OP(10) BM_OP(11) BM_OP(12) BM_OP(13) BM_OP(14)
#undef BM_OP
    default: return hipErrorInvalidValue;
    }
}

hipError_t transpose(int nrows, int ncols, const float* in, int ldi, float* out, int ldo, hipStream_t s) {
    if (nrows <= 0 || ncols <= 0) return hipSuccess;
    const long long bx = ((long long)nrows + TT - 1) / TT, by = ((long long)ncols + TT - 1) / TT;
    if (by > 65535) {
        // very wide inputs: walk the columns in slabs the grid's y dimension can hold
        const int slab = 65535 * TT;
        for (long long c = 0; c < ncols; c += slab) {
            const int nc = (int)((ncols - c) < slab ? (ncols - c) : slab);
            hipError_t e = transpose(nrows, nc, in + (size_t)c * ldi, ldi, out + c, ldo, s);
            if (e != hipSuccess) return e;
        }
        return hipSuccess;
    }
    hipLaunchKernelGGL(k_transpose, dim3((unsigned)bx, (unsigned)by), dim3(BM_BLOCK), 0, s, nrows, ncols, in, ldi, out, ldo);
    return hipGetLastError();
}

// Same case analysis, in the same order, as apply_binop (Operators.cu:529-553).
hipError_t applyop(const float* A, int Anr, int Anc, const float* B, int Bnr, int Bnc, float* C,
                   int opn, hipStream_t s) {
    const int nr = Anr > Bnr ? Anr : Bnr;
    const int nc = Anc > Bnc ? Anc : Bnc;
    const long long n = (long long)nr * nc;
    int ma, mb;
    if (Anr == Bnr && Anc == Bnc) { ma = FULL; mb = FULL; }
    else if (Anr == Bnr && Bnc == 1) { ma = FULL; mb = COL; }
    else if (Anc == Bnc && Bnr == 1) { ma = FULL; mb = ROW; }
    else if (Anr == Bnr && Anc == 1) { ma = COL; mb = FULL; }
    else if (Anc == Bnc && Anr == 1) { ma = ROW; mb = FULL; }
    else if (Bnr == 1 && Bnc == 1) { ma = FULL; mb = VAL; }
    else if (Anr == 1 && Anc == 1) { ma = VAL; mb = FULL; }
    else return hipErrorInvalidValue;      // the reference launches nothing for incompatible shapes
    switch (opn) {
#define BM_OP(N_) case N_: return apply_impl<N_>(A, ma, B, mb, C, n, nr, s);
    BM_OP(0) BM_OP(1) BM_OP(2) BM_OP(3) BM_OP(4) BM_OP(5) BM_OP(6) BM_OP(7)
    BM_OP(8) BM_OP(9) BM_OP(10) BM_OP(11) BM_OP(12) BM_OP(13) BM_OP(14)
#undef BM_OP
    default: return hipErrorInvalidValue;
    }
}

}  // namespace bm
