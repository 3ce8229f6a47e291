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

// rowptr[r] = number of entries of the sorted array a[0..n) that are smaller than r, for r = 0..nrows: one thread per r
// and a binary search. (Closing the columns from the positions where a column starts, as k_compress_cols does, leaves a
// run of absent columns to one thread: among the light rows of a plan the panel-cut rows are absent, with row indices ordered
// by frequency the first several thousand, closed one store after the other in 0.2 ms.)
__global__ __launch_bounds__(BM_BLOCK) void k_lower_bounds(int n, int nrows, const int* __restrict__ a, int* __restrict__ rowptr) {
    const long long r = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (r > nrows) return;
    int lo = 0, hi = n;                  // first position whose row is >= r
    while (lo < hi) {
        const int mid = (int)(((long long)lo + hi) >> 1);
        if (a[mid] < (int)r) lo = mid + 1; else hi = mid;
    }
    rowptr[r] = lo;
}

// Position j closes the columns ic[j-1]+1 .. ic[j] (with ic[-1] = -1 and ic[nnz] = ncols): jc[c] = j for
// each of them. A thread takes four consecutive positions (one 128-bit load when ic is 16-byte aligned).
__global__ __launch_bounds__(BM_BLOCK) void k_compress_cols(int ncols, int nnz, const int* __restrict__ ic,
                                                            int* __restrict__ jc) {
    const long long j0 = 4 * ((long long)blockIdx.x * BM_BLOCK + threadIdx.x);
    if (j0 > nnz) return;
    int v[5];
    v[0] = (j0 == 0) ? -1 : ic[j0 - 1];
    if (j0 + 4 <= nnz && (reinterpret_cast<uintptr_t>(ic) & 15) == 0) {
        const int4 q = *reinterpret_cast<const int4*>(ic + j0);
        v[1] = q.x; v[2] = q.y; v[3] = q.z; v[4] = q.w;
    } else {
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u + 1] = j0 + u < nnz ? ic[j0 + u] : ncols;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const long long j = j0 + u;
        if (j > nnz) break;
        int prev = v[u], cur = (j == nnz) ? ncols : v[u + 1];
        if (prev >= ncols) prev = ncols - 1;      // malformed input: stay inside jc
        if (prev < -1) prev = -1;
        if (cur > ncols) cur = ncols;
        for (int c = prev + 1; c <= cur; ++c) jc[c] = (int)j;
    }
}

template <typename T>
__global__ __launch_bounds__(BM_BLOCK) void k_fill(T* __restrict__ out, long long n, T v) {
    long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    for (; i < n; i += stride) out[i] = v;
}

constexpr int DIGEST_MAX_BLOCKS = 4096;

// One pass over both index arrays of a pattern. With p_j = (j+1) * 0x9E3779B9 (32 bits), position j adds
//   out[0] += fold32((ir[j] ^ p_j) * 0x85EBCA6B) << 32 | fold32(((ir[j] + 0x27D4EB2F * ic[j]) ^ ~p_j) * 0xC2B2AE35)
//             with fold32(h) = h ^ (h >> 15): two different non-linear 32-bit hashes of (position, row, column)
//             side by side (xor before the multiplication, fold after it), so that neither moving an entry to
//             another position nor trading amounts between positions cancels out;
//   out[1] += ic[j] << 32 | ir[j]       the plain sum of the pairs.
// Both are 64-bit integer sums, independent of the order in which threads add.
// out[2] (as int) = the largest entry of ir. Every thread takes four consecutive positions at a time
// (one 128-bit load per array when both are 16-byte aligned; the position word advances by addition).
// jc != nullptr: the column pointer of the pattern is written in the same pass (what k_compress_cols
// does): position j closes the columns ic[j-1]+1 .. ic[j], the last position also those behind ic[n-1].
// z != nullptr: the fourth word counts the workgroups that met a word of z[0..nz) other than +0.0f (callers
// that accumulate into an output they have just cleared can then overwrite it instead of reading it).
// Workgroup b leaves its four words at out[4*(b+1) ..]; k_digest_final combines them into out[0..3].
template <bool VEC>
__global__ __launch_bounds__(BM_BLOCK) void k_pattern_digest(const int* __restrict__ ir, const int* __restrict__ ic,
                                                             long long n, unsigned long long* out, int ncols,
                                                             int* __restrict__ jc, const unsigned* __restrict__ z,
                                                             long long nz) {
    constexpr unsigned G = 0x9E3779B9u;
    constexpr int T = 2;                                  // tiles of four positions per thread and trip: 4 T loads in flight
    const long long first = 4 * ((long long)blockIdx.x * BM_BLOCK + threadIdx.x);
    const long long tile = 4LL * gridDim.x * BM_BLOCK;    // positions one sweep of the grid covers
    unsigned long long ha = 0, hb = 0;
    int m = -1;
    unsigned any = 0;
    for (long long i0 = first; i0 < n; i0 += T * tile) {
        int r[T][4], c[T][4], before[T];
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const long long i = i0 + t * tile;
            if (VEC && i + 4 <= n) {
                const int4 rv = *reinterpret_cast<const int4*>(ir + i);
                const int4 cv = *reinterpret_cast<const int4*>(ic + i);
                r[t][0] = rv.x; r[t][1] = rv.y; r[t][2] = rv.z; r[t][3] = rv.w;
                c[t][0] = cv.x; c[t][1] = cv.y; c[t][2] = cv.z; c[t][3] = cv.w;
            } else {
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    r[t][u] = i + u < n ? ir[i + u] : -1;
                    c[t][u] = i + u < n ? ic[i + u] : -1;
                }
            }
            before[t] = (jc != nullptr && i > 0 && i < n) ? ic[i - 1] : -1;      // the neighbour's line: a cache hit
        }
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const long long i = i0 + t * tile;
            unsigned pos = (unsigned)(i + 1) * G;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const long long j = i + u;
                if (j < n) {
                    unsigned h1 = ((unsigned)r[t][u] ^ pos) * 0x85EBCA6Bu;
                    unsigned h2 = (((unsigned)r[t][u] + 0x27D4EB2Fu * (unsigned)c[t][u]) ^ ~pos) * 0xC2B2AE35u;
                    h1 ^= h1 >> 15;
                    h2 ^= h2 >> 15;
                    ha += ((unsigned long long)h1 << 32) | h2;
                    hb += ((unsigned long long)(unsigned)c[t][u] << 32) | (unsigned)r[t][u];
                    m = max(m, r[t][u]);
                    if (jc != nullptr && c[t][u] != before[t]) {
                        // malformed input: stay inside jc
                        const int prev = before[t] < -1 ? -1 : (before[t] >= ncols ? ncols - 1 : before[t]);
                        const int cur = c[t][u] > ncols ? ncols : c[t][u];
                        for (int q = prev + 1; q <= cur; ++q) jc[q] = (int)j;
                        before[t] = c[t][u];
                    }
                    if (jc != nullptr && j == n - 1) {
                        const int last = c[t][u] < -1 ? -1 : (c[t][u] >= ncols ? ncols - 1 : c[t][u]);
                        for (int q = last + 1; q <= ncols; ++q) jc[q] = (int)n;
                    }
                }
                pos += G;
            }
        }
    }
    if (z != nullptr) {
        const bool zvec = (reinterpret_cast<uintptr_t>(z) & 15) == 0;
        constexpr int TZ = 4;
        for (long long t0 = first; t0 < nz; t0 += TZ * tile) {
#pragma unroll
            for (int t = 0; t < TZ; ++t) {
                const long long p = t0 + t * tile;
                if (zvec && p + 4 <= nz) {
                    const uint4 v = *reinterpret_cast<const uint4*>(z + p);
                    any |= v.x | v.y | v.z | v.w;
                } else {
                    for (int u = 0; u < 4 && p + u < nz; ++u) any |= z[p + u];
                }
            }
        }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        ha += __shfl_xor(ha, d, 64);
        hb += __shfl_xor(hb, d, 64);
        m = max(m, __shfl_xor(m, d, 64));
    }
    const bool wave_any = __ballot(any != 0) != 0ULL;
    // one line of four words per workgroup, summed up by k_digest_final (thousands of atomics on
    // three addresses would serialise and cost more than the pass itself)
    __shared__ unsigned long long sa[BM_WAVES_PER_BLOCK], sb[BM_WAVES_PER_BLOCK];
    __shared__ int sm[BM_WAVES_PER_BLOCK], sz[BM_WAVES_PER_BLOCK];
    if ((threadIdx.x & 63) == 0) {
        sa[threadIdx.x >> 6] = ha; sb[threadIdx.x >> 6] = hb; sm[threadIdx.x >> 6] = m; sz[threadIdx.x >> 6] = wave_any ? 1 : 0;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int zany = sz[0];
#pragma unroll
        for (int w = 1; w < BM_WAVES_PER_BLOCK; ++w) { ha += sa[w]; hb += sb[w]; m = max(m, sm[w]); zany |= sz[w]; }
        unsigned long long* mine = out + 4 * (size_t)(blockIdx.x + 1);
        mine[0] = ha;
        mine[1] = hb;
        mine[2] = (unsigned long long)(long long)m;
        mine[3] = (unsigned long long)zany;
    }
}

// out[0..3] = the workgroups' lines out[4*(b+1) ..] combined: two sums, the maximum (as int in out[2]),
// the count of workgroups that met a nonzero word. One workgroup.
__global__ __launch_bounds__(BM_BLOCK) void k_digest_final(int nblocks, unsigned long long* out) {
    unsigned long long ha = 0, hb = 0, nz = 0;
    int m = -1;
    for (int b = threadIdx.x; b < nblocks; b += BM_BLOCK) {
        const unsigned long long* p = out + 4 * (size_t)(b + 1);
        ha += p[0]; hb += p[1]; m = max(m, (int)(long long)p[2]); nz += p[3];
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        ha += __shfl_xor(ha, d, 64);
        hb += __shfl_xor(hb, d, 64);
        nz += __shfl_xor(nz, d, 64);
        m = max(m, __shfl_xor(m, d, 64));
    }
    __shared__ unsigned long long sa[BM_WAVES_PER_BLOCK], sb[BM_WAVES_PER_BLOCK], sn[BM_WAVES_PER_BLOCK];
    __shared__ int sm[BM_WAVES_PER_BLOCK];
    if ((threadIdx.x & 63) == 0) { sa[threadIdx.x >> 6] = ha; sb[threadIdx.x >> 6] = hb; sn[threadIdx.x >> 6] = nz; sm[threadIdx.x >> 6] = m; }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < BM_WAVES_PER_BLOCK; ++w) { ha += sa[w]; hb += sb[w]; nz += sn[w]; m = max(m, sm[w]); }
        out[0] = ha;
        out[1] = hb;
        out[2] = 0;
        *reinterpret_cast<int*>(out + 2) = m;
        out[3] = nz;
    }
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

hipError_t sorted_lower_bounds(int ncols, int nnz, const int* ic, int* jc, hipStream_t s) {
    if (ncols < 0 || nnz < 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(k_lower_bounds, dim3((unsigned)(((long long)ncols + 1 + BM_BLOCK - 1) / BM_BLOCK)), dim3(BM_BLOCK), 0, s, nnz, ncols, ic, jc);
    return hipGetLastError();
}

hipError_t coo_compress_cols(int ncols, int nnz, const int* ic, int* jc, hipStream_t s) {
    if (ncols < 0 || nnz < 0) return hipErrorInvalidValue;
    // few columns for the entries: a search per column costs no more than a pass over the entries, and a long run of
    // empty columns is not left to one thread
    if ((long long)ncols * 128 < (long long)nnz) return sorted_lower_bounds(ncols, nnz, ic, jc, s);
    long long nblk = ((long long)nnz / 4 + 1 + BM_BLOCK - 1) / BM_BLOCK;
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

size_t pattern_digest_words() { return 4 * (size_t)(DIGEST_MAX_BLOCKS + 1); }

hipError_t pattern_digest(const int* ir, const int* ic, long long nnz, unsigned long long* d_out, hipStream_t s,
                          int ncols, int* jc, const float* z, long long nz) {
    int nblocks = 0;
    if (nnz > 0) {
        const bool vec = ((reinterpret_cast<uintptr_t>(ir) | reinterpret_cast<uintptr_t>(ic)) & 15) == 0;
        nblocks = (int)grid_for((nnz + 3) / 4, DIGEST_MAX_BLOCKS);
        const dim3 grid((unsigned)nblocks), block(BM_BLOCK);
        const unsigned* zw = reinterpret_cast<const unsigned*>(z);
        if (vec) hipLaunchKernelGGL(k_pattern_digest<true>, grid, block, 0, s, ir, ic, nnz, d_out, ncols, jc, zw, nz);
        else hipLaunchKernelGGL(k_pattern_digest<false>, grid, block, 0, s, ir, ic, nnz, d_out, ncols, jc, zw, nz);
    } else if (jc != nullptr) {
        hipError_t e = fill_i32(jc, (long long)ncols + 1, 0, s);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(k_digest_final, dim3(1), dim3(BM_BLOCK), 0, s, nblocks, d_out);
    return hipGetLastError();
}

}  // namespace bm
