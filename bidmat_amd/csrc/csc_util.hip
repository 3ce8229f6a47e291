// Integer utilities around the CSC container: column pointer <-> per-nonzero column index,
// fills, an int maximum and a pattern fingerprint. All integer work, bandwidth-bound.
#include "common.hpp"
#include "kernels.hpp"

namespace bm {
namespace {

// 16 lanes per column: lane l writes ic[jc[c] + l], + 16, ... Positions outside [0, nnz) are never
// written, whatever a malformed jc says. ROWS: instead of the column index, the position inside the
// column (the implied row of a sparse matrix stored without row indices).
template <bool ROWS>
__global__ __launch_bounds__(BM_BLOCK) void k_expand_cols(int ncols, int nnz, const int* __restrict__ jc,
                                                          int* __restrict__ out) {
    const long long t = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long c = t >> 4;
    const int l = (int)(t & 15);
    if (c >= ncols) return;
    int s = jc[c], e = jc[c + 1];
    if (s < 0) s = 0;
    if (e > nnz) e = nnz;
    for (long long j = (long long)s + l; j < e; j += 16) out[j] = ROWS ? (int)(j - s) : (int)c;
}

// What the kernels rely on: jc[0] == 0, jc non-decreasing inside [0, nnz], jc[ncols] == nnz,
// 0 <= ir < nrows. Sets bit r of *flags for every violated rule r (numbered like the branches of
// SparseMat.check: 1 first pointer, 2 pointer order, 5 row out of range, 6 last pointer).
__global__ __launch_bounds__(BM_BLOCK) void k_csc_validate(int nrows, int ncols, int nnz, const int* __restrict__ ir,
                                                           const int* __restrict__ jc, int* __restrict__ flags) {
    long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    const long long lim = nnz > ncols + 1 ? nnz : (long long)ncols + 1;
    int bad = 0;
    for (; i < lim; i += stride) {
        if (i <= ncols) {
            const int v = jc[i];
            if (i == 0 && v != 0) bad |= 1 << 1;
            if (v < 0 || v > nnz || (i < ncols && v > jc[i + 1])) bad |= 1 << 2;
            if (i == ncols && v != nnz) bad |= 1 << 6;
        }
        if (i < nnz && ir != nullptr) {
            if ((unsigned)ir[i] >= (unsigned)nrows) bad |= 1 << 5;
        }
    }
    if (bad) atomicOr(flags, bad);
}

// Thread j fills jc for every column that starts at position j:
// columns ic[j-1]+1 .. ic[j] (with ic[-1] = -1 and ic[nnz] = ncols).
__global__ __launch_bounds__(BM_BLOCK) void k_compress_cols(int ncols, int nnz, const int* __restrict__ ic,
                                                            int* __restrict__ jc) {
    const long long j = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (j > nnz) return;
    int prev = (j == 0) ? -1 : ic[j - 1];
    int cur = (j == nnz) ? ncols : ic[j];
    if (prev >= ncols) prev = ncols - 1;      // malformed input: stay inside jc
    if (prev < -1) prev = -1;
    if (cur > ncols) cur = ncols;
    for (int c = prev + 1; c <= cur; ++c) jc[c] = (int)j;
}

template <typename T>
__global__ __launch_bounds__(BM_BLOCK) void k_fill(T* __restrict__ out, long long n, T v) {
    long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    for (; i < n; i += stride) out[i] = v;
}

// 64-bit finaliser (splitmix64): every input bit reaches every output bit.
__device__ __forceinline__ unsigned long long mix64(unsigned long long x) {
    x ^= x >> 30; x *= 0xBF58476D1CE4E5B9ULL;
    x ^= x >> 27; x *= 0x94D049BB133111EBULL;
    x ^= x >> 31;
    return x;
}
// Contribution of (position i, value v) to a digest: a non-linear 64-bit hash of the pair, so that
// neither moving a value to another position nor trading amounts between two positions cancels out.
__device__ __forceinline__ unsigned long long digest_term(unsigned long long i, unsigned v, unsigned long long salt) {
    return mix64(((i + 1ULL) << 32 | (unsigned long long)v) ^ salt);
}

// One pass over both index arrays of a pattern: digests sum_i hash64(i, value_i) of ir and of ic
// (64-bit integer sums: position-sensitive, independent of the order in which threads contribute)
// and the largest row index. A workgroup walks tiles of 4 x 256 positions with four
// loads per array in flight per thread. out: [0] digest of ir, [1] digest of ic, [2] (int) max.
// jc != nullptr: the column pointer of the pattern is written in the same pass (what k_compress_cols
// does): position j closes the columns ic[j-1]+1 .. ic[j], the last position also those behind ic[n-1].
__global__ __launch_bounds__(BM_BLOCK) void k_pattern_digest(const int* __restrict__ ir, const int* __restrict__ ic,
                                                             long long n, unsigned long long* out, int ncols,
                                                             int* __restrict__ jc) {
    constexpr int UN = 4;
    long long i = (long long)blockIdx.x * (UN * BM_BLOCK) + threadIdx.x;
    const long long stride = (long long)gridDim.x * (UN * BM_BLOCK);
    unsigned long long ha = 0, hb = 0;
    int m = -1;
    for (; i < n; i += stride) {
        int r[UN], c[UN], cp[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const long long j = i + u * BM_BLOCK;
            r[u] = j < n ? ir[j] : -1;
            c[u] = j < n ? ic[j] : -1;
            cp[u] = (jc != nullptr && j > 0 && j < n) ? ic[j - 1] : -1;      // the neighbour's line: a cache hit
        }
        if (jc != nullptr) {
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const long long j = i + u * BM_BLOCK;
                if (j < n) {
                    // malformed input: stay inside jc
                    int prev = cp[u] < -1 ? -1 : (cp[u] >= ncols ? ncols - 1 : cp[u]);
                    int cur = c[u] > ncols ? ncols : c[u];
                    for (int q = prev + 1; q <= cur; ++q) jc[q] = (int)j;
                    if (j == n - 1) {
                        prev = cur < -1 ? -1 : (cur >= ncols ? ncols - 1 : cur);
                        for (int q = prev + 1; q <= ncols; ++q) jc[q] = (int)n;
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const long long j = i + u * BM_BLOCK;
            if (j < n) {
                ha += digest_term((unsigned long long)j, (unsigned)r[u], 0x7F4A7C159E3779B9ULL);
                hb += digest_term((unsigned long long)j, (unsigned)c[u], 0x2545F4914F6CDD1DULL);
                m = max(m, r[u]);
            }
        }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        ha += __shfl_xor(ha, d, 64);
        hb += __shfl_xor(hb, d, 64);
        m = max(m, __shfl_xor(m, d, 64));
    }
    // one set of atomics per workgroup: thousands of them on three addresses would serialise
    __shared__ unsigned long long sa[BM_WAVES_PER_BLOCK], sb[BM_WAVES_PER_BLOCK];
    __shared__ int sm[BM_WAVES_PER_BLOCK];
    if ((threadIdx.x & 63) == 0) { sa[threadIdx.x >> 6] = ha; sb[threadIdx.x >> 6] = hb; sm[threadIdx.x >> 6] = m; }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < BM_WAVES_PER_BLOCK; ++w) { ha += sa[w]; hb += sb[w]; m = max(m, sm[w]); }
        atomicAdd(out, ha);
        atomicAdd(out + 1, hb);
        if (m >= 0) atomicMax(reinterpret_cast<int*>(out + 2), m);
    }
}

// out[0..1] = 0, (int)out[2] = -1
__global__ void k_digest_init(unsigned long long* out) {
    if (threadIdx.x < 2) out[threadIdx.x] = 0;
    if (threadIdx.x == 2) { out[2] = 0; *reinterpret_cast<int*>(out + 2) = -1; }
}

// Columns [col1, col1+nc) of a CSC matrix as a matrix of its own: nonzero range copied, column
// pointer rebased to 0, per-nonzero column rebuilt afterwards by k_expand_cols.
__global__ __launch_bounds__(BM_BLOCK) void k_colslice(int nc, int start, int n, const int* __restrict__ jc_at_col1,
                                                       const int* __restrict__ ir, const float* __restrict__ data,
                                                       int* __restrict__ out_jc, int* __restrict__ out_ir,
                                                       float* __restrict__ out_data) {
    long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    const long long lim = n > nc + 1 ? n : nc + 1;
    for (; i < lim; i += stride) {
        if (i < n) {
            out_ir[i] = ir[(long long)start + i];
            out_data[i] = data[(long long)start + i];
        }
        if (i <= nc) out_jc[i] = jc_at_col1[i] - start;
    }
}

// n-hot pattern: column j holds the n row indices cats[j*n .. j*n+n) with value 1 (rows in the
// given order, repeats allowed); also the largest category, for callers that size the matrix by it.
__global__ __launch_bounds__(BM_BLOCK) void k_nhot(int n, int ncols, const int* __restrict__ cats,
                                                   int* __restrict__ ir, int* __restrict__ ic, int* __restrict__ jc,
                                                   float* __restrict__ data, int* __restrict__ maxcat) {
    long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    const long long total = (long long)n * ncols;
    int m = -1;
    for (; i < total || i <= ncols; i += stride) {
        if (i < total) {
            const int r = cats[i];
            ir[i] = r;
            ic[i] = (int)(i / n);
            data[i] = 1.0f;
            m = max(m, r);
        }
        if (i <= ncols) jc[i] = (int)(i * n);
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) m = max(m, __shfl_xor(m, d, 64));
    if ((threadIdx.x & 63) == 0 && m >= 0) atomicMax(maxcat, m);
}

// Dense image of a sparse matrix: od[row + col*ld] = value for every stored nonzero (the output is
// cleared by the caller; where a column stores a row twice, one of the values stays).
__global__ __launch_bounds__(BM_BLOCK) void k_full(long long nnz, const int* __restrict__ ir, const int* __restrict__ ic,
                                                   const float* __restrict__ data, float* __restrict__ od,
                                                   int nrows, int ncols, long long ld) {
    long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    for (; i < nnz; i += stride) {
        const int r = ir[i], c = ic[i];
        if ((unsigned)r < (unsigned)nrows && (unsigned)c < (unsigned)ncols) od[r + c * ld] = data[i];
    }
}

// p[i] += delta (index-base conversion of uploaded / downloaded index arrays)
__global__ __launch_bounds__(BM_BLOCK) void k_index_shift(int* __restrict__ p, long long n, int delta) {
    long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    for (; i < n; i += stride) p[i] += delta;
}

inline unsigned grid_for(long long n, int maxblocks = 8192) {
    long long b = (n + BM_BLOCK - 1) / BM_BLOCK;
    if (b < 1) b = 1;
    if (b > maxblocks) b = maxblocks;
    return (unsigned)b;
}

}  // namespace

hipError_t csc_expand_cols(int ncols, int nnz, const int* jc, int* ic, hipStream_t s) {
    if (ncols <= 0 || nnz <= 0) return hipSuccess;
    long long threads = (long long)ncols * 16;
    long long nblk = (threads + BM_BLOCK - 1) / BM_BLOCK;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(k_expand_cols<false>, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, ncols, nnz, jc, ic);
    return hipGetLastError();
}

hipError_t csc_implicit_rows(int ncols, int nnz, const int* jc, int* ir, hipStream_t s) {
    if (ncols <= 0 || nnz <= 0) return hipSuccess;
    long long nblk = ((long long)ncols * 16 + BM_BLOCK - 1) / BM_BLOCK;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(k_expand_cols<true>, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, ncols, nnz, jc, ir);
    return hipGetLastError();
}

hipError_t csc_validate(int nrows, int ncols, int nnz, const int* ir, const int* jc, int* d_flags, hipStream_t s) {
    hipError_t e = fill_i32(d_flags, 1, 0, s);
    if (e != hipSuccess) return e;
    const long long lim = nnz > ncols + 1 ? nnz : (long long)ncols + 1;
    hipLaunchKernelGGL(k_csc_validate, dim3(grid_for(lim, 4096)), dim3(BM_BLOCK), 0, s, nrows, ncols, nnz, ir, jc, d_flags);
    return hipGetLastError();
}

hipError_t coo_compress_cols(int ncols, int nnz, const int* ic, int* jc, hipStream_t s) {
    if (ncols < 0 || nnz < 0) return hipErrorInvalidValue;
    long long nblk = ((long long)nnz + 1 + BM_BLOCK - 1) / BM_BLOCK;
    hipLaunchKernelGGL(k_compress_cols, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, ncols, nnz, ic, jc);
    return hipGetLastError();
}

hipError_t fill_f32(float* out, long long n, float v, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_fill<float>, dim3(grid_for(n)), dim3(BM_BLOCK), 0, s, out, n, v);
    return hipGetLastError();
}

hipError_t fill_i32(int* out, long long n, int v, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_fill<int>, dim3(grid_for(n)), dim3(BM_BLOCK), 0, s, out, n, v);
    return hipGetLastError();
}

hipError_t csc_colslice(int nc, int start, int n, const int* jc_at_col1, const int* ir, const float* data,
                        int* out_jc, int* out_ir, int* out_ic, float* out_data, hipStream_t s) {
    const long long lim = n > nc + 1 ? n : (long long)nc + 1;
    hipLaunchKernelGGL(k_colslice, dim3(grid_for(lim, 16384)), dim3(BM_BLOCK), 0, s, nc, start, n, jc_at_col1, ir, data,
                       out_jc, out_ir, out_data);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess && out_ic != nullptr) e = csc_expand_cols(nc, n, out_jc, out_ic, s);
    return e;
}

hipError_t nhot(int n, int ncols, const int* cats, int* ir, int* ic, int* jc, float* data, int* d_maxcat,
                hipStream_t s) {
    hipError_t e = fill_i32(d_maxcat, 1, -1, s);
    if (e != hipSuccess) return e;
    const long long total = (long long)n * ncols;
    const long long lim = total > (long long)ncols + 1 ? total : (long long)ncols + 1;
    hipLaunchKernelGGL(k_nhot, dim3(grid_for(lim)), dim3(BM_BLOCK), 0, s, n, ncols, cats, ir, ic, jc, data, d_maxcat);
    return hipGetLastError();
}

hipError_t full_from_coo(int nrows, int ncols, int nnz, const int* ir, const int* ic, const float* data, float* od,
                         int ld, hipStream_t s) {
    if (nnz <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_full, dim3(grid_for(nnz, 16384)), dim3(BM_BLOCK), 0, s, (long long)nnz, ir, ic, data, od,
                       nrows, ncols, (long long)ld);
    return hipGetLastError();
}

hipError_t index_shift(int* p, long long n, int delta, hipStream_t s) {
    if (n <= 0 || delta == 0) return hipSuccess;
    hipLaunchKernelGGL(k_index_shift, dim3(grid_for(n, 16384)), dim3(BM_BLOCK), 0, s, p, n, delta);
    return hipGetLastError();
}

hipError_t pattern_digest(const int* ir, const int* ic, long long nnz, unsigned long long* d_out, hipStream_t s,
                          int ncols, int* jc) {
    hipLaunchKernelGGL(k_digest_init, dim3(1), dim3(64), 0, s, d_out);
    if (nnz > 0)
        hipLaunchKernelGGL(k_pattern_digest, dim3(grid_for((nnz + 3) / 4, 2048)), dim3(BM_BLOCK), 0, s, ir, ic, nnz, d_out,
                           ncols, jc);
    else if (jc != nullptr)
        return fill_i32(jc, (long long)ncols + 1, 0, s);
    return hipGetLastError();
}

}  // namespace bm
