// Integer utilities around the CSC container: column pointer <-> per-nonzero column index,
// fills, an int maximum and a pattern fingerprint. All integer work, bandwidth-bound.
#include "common.hpp"
#include "kernels.hpp"

namespace bm {
namespace {

// 16 lanes per column: lane l writes ic[jc[c] + l], + 16, ...
__global__ __launch_bounds__(BM_BLOCK) void k_expand_cols(int ncols, const int* __restrict__ jc,
                                                          int* __restrict__ ic) {
    const long long t = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long c = t >> 4;
    const int l = (int)(t & 15);
    if (c >= ncols) return;
    const int s = jc[c], e = jc[c + 1];
    for (int j = s + l; j < e; j += 16) ic[j] = (int)c;
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

__global__ __launch_bounds__(BM_BLOCK) void k_int_max(const int* __restrict__ in, long long n, int* out) {
    long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    int m = -1;
    for (; i < n; i += stride) m = max(m, in[i]);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) m = max(m, __shfl_xor(m, d, 64));
    if ((threadIdx.x & 63) == 0 && m >= 0) atomicMax(out, m);
}

__device__ __forceinline__ unsigned long long mix64(unsigned long long x) {
    x ^= x >> 33; x *= 0xff51afd7ed558ccdULL;
    x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ULL;
    x ^= x >> 33;
    return x;
}

// Sum over positions of mix(position, value): position-sensitive, and the integer sum does
// not depend on the order in which threads contribute.
__global__ __launch_bounds__(BM_BLOCK) void k_fingerprint(const int* __restrict__ in, long long n,
                                                          unsigned long long* out) {
    long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    unsigned long long h = 0;
    for (; i < n; i += stride)
        h += mix64(((unsigned long long)i << 32) ^ (unsigned long long)(unsigned)in[i] ^ 0x9e3779b97f4a7c15ULL);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) h += __shfl_xor(h, d, 64);
    if ((threadIdx.x & 63) == 0) atomicAdd(out, h);
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
    hipLaunchKernelGGL(k_expand_cols, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, ncols, jc, ic);
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

hipError_t int_max(const int* d_in, long long n, int* d_out, hipStream_t s) {
    hipError_t e = fill_i32(d_out, 1, -1, s);
    if (e != hipSuccess || n <= 0) return e;
    hipLaunchKernelGGL(k_int_max, dim3(grid_for(n, 2048)), dim3(BM_BLOCK), 0, s, d_in, n, d_out);
    return hipGetLastError();
}

hipError_t fingerprint(const int* a, long long na, const int* b, long long nb,
                       unsigned long long* d_out, hipStream_t s) {
    hipError_t e = fill_i32(reinterpret_cast<int*>(d_out), 4, 0, s);
    if (e != hipSuccess) return e;
    if (na > 0) hipLaunchKernelGGL(k_fingerprint, dim3(grid_for(na, 2048)), dim3(BM_BLOCK), 0, s, a, na, d_out);
    if (nb > 0) hipLaunchKernelGGL(k_fingerprint, dim3(grid_for(nb, 2048)), dim3(BM_BLOCK), 0, s, b, nb, d_out + 1);
    return hipGetLastError();
}

}  // namespace bm
