// Transpose of a CSC matrix on the device: one stable radix sort of the nonzeros by row, each
// carrying its (column, position); the result has its rows in ascending order inside every column,
// like the host transpose the reference goes through (GSMat.t, GSMat.scala:218-223).
#include "common.hpp"
#include "kernels.hpp"
#include "workspace.hpp"
#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>

namespace bm {
namespace {

// 16 lanes per column: (column, position) of every nonzero; rows outside the matrix raise *bad.
__global__ __launch_bounds__(BM_BLOCK) void k_colpos(int ncols, int nrows, const int* __restrict__ jc,
                                                     const int* __restrict__ ir,
                                                     unsigned long long* __restrict__ colpos, int* __restrict__ bad) {
    const long long t = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long c = t >> 4;
    const int l = (int)(t & 15);
    if (c >= ncols) return;
    const int s = jc[c], e = jc[c + 1];
    for (int j = s + l; j < e; j += 16) {
        if ((unsigned)ir[j] >= (unsigned)nrows) *bad = 1;
        colpos[j] = ((unsigned long long)(unsigned)c << 32) | (unsigned)j;
    }
}

__global__ __launch_bounds__(BM_BLOCK) void k_scatter_t(long long nnz, const unsigned long long* __restrict__ colpos,
                                                        const float* __restrict__ data, int* __restrict__ out_ir,
                                                        float* __restrict__ out_data) {
    long long p = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    for (; p < nnz; p += stride) {
        const unsigned long long cp = colpos[p];
        out_ir[p] = (int)(cp >> 32);
        out_data[p] = data[cp & 0xffffffffULL];
    }
}

inline int bits_for(unsigned long long maxval) {
    int b = 1;
    while (b < 32 && (maxval >> b) != 0) ++b;
    return b;
}

inline size_t round256(size_t b) { return (b + 255) & ~size_t(255); }

}  // namespace

hipError_t csc_transpose(int nrows, int ncols, int nnz, const float* data, const int* ir, const int* jc,
                         float* out_data, int* out_ir, int* out_jc, hipStream_t s) {
    hipError_t err;
    if (nnz <= 0) return fill_i32(out_jc, (long long)nrows + 1, 0, s);
    const int rbits = bits_for((unsigned long long)(nrows > 0 ? nrows - 1 : 0));
    size_t sort_bytes = 0;
    err = rocprim::radix_sort_pairs(nullptr, sort_bytes, (const unsigned*)nullptr, (unsigned*)nullptr,
                                    (unsigned long long*)nullptr, (unsigned long long*)nullptr, (size_t)nnz, 0, rbits, s);
    if (err != hipSuccess) return err;
    const size_t n = (size_t)nnz;
    const size_t off_keys = 0, off_in = off_keys + round256(4 * n), off_out = off_in + round256(8 * n),
                 off_sort = off_out + round256(8 * n), off_bad = off_sort + round256(sort_bytes),
                 total = off_bad + 256;
    char* base = static_cast<char*>(ws_get(WS_TRANSPOSE, total, &err, s));
    if (!base) return err;
    unsigned* keys_out = reinterpret_cast<unsigned*>(base + off_keys);
    unsigned long long* cp_in = reinterpret_cast<unsigned long long*>(base + off_in);
    unsigned long long* cp_out = reinterpret_cast<unsigned long long*>(base + off_out);
    int* bad = reinterpret_cast<int*>(base + off_bad);
    if ((err = fill_i32(bad, 1, 0, s)) != hipSuccess) return err;
    {
        const long long nblk = ((long long)ncols * 16 + BM_BLOCK - 1) / BM_BLOCK;
        if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
        hipLaunchKernelGGL(k_colpos, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, ncols, nrows, jc, ir, cp_in, bad);
    }
    err = rocprim::radix_sort_pairs(base + off_sort, sort_bytes, reinterpret_cast<const unsigned*>(ir), keys_out, cp_in,
                                    cp_out, n, 0, rbits, s);
    if (err != hipSuccess) return err;
    long long nb = ((long long)nnz + BM_BLOCK - 1) / BM_BLOCK;
    if (nb > 16384) nb = 16384;
    hipLaunchKernelGGL(k_scatter_t, dim3((unsigned)nb), dim3(BM_BLOCK), 0, s, (long long)nnz, cp_out, data, out_ir, out_data);
    if ((err = coo_compress_cols(nrows, nnz, reinterpret_cast<const int*>(keys_out), out_jc, s)) != hipSuccess) return err;
    int h_bad = 0;
    if ((err = hipMemcpyAsync(&h_bad, bad, sizeof(int), hipMemcpyDeviceToHost, s)) != hipSuccess) return err;
    if ((err = hipStreamSynchronize(s)) != hipSuccess) return err;
    return h_bad ? hipErrorInvalidValue : hipGetLastError();
}

}  // namespace bm
