#include "scan.hpp"
#include "common.hpp"

namespace bm {

namespace {
constexpr int SCAN_ITEMS = 8;
constexpr int SCAN_TILE = BM_BLOCK * SCAN_ITEMS;   // 2048 elements per block

__global__ __launch_bounds__(BM_BLOCK) void k_scan_blocksums(const int* __restrict__ in, long long n,
                                                              int* __restrict__ bsum) {
    __shared__ int smem[8];
    long long base = (long long)blockIdx.x * SCAN_TILE + (long long)threadIdx.x * SCAN_ITEMS;
    int s = 0;
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i) {
        long long p = base + i;
        if (p < n) s += in[p];
    }
    int total;
    (void)block_exclusive_scan_256(s, total, smem);
    if (threadIdx.x == 0) bsum[blockIdx.x] = total;
}

// One block scans the nb block sums in place (exclusive) and writes the grand total.
__global__ __launch_bounds__(BM_BLOCK) void k_scan_top(int* __restrict__ bsum, long long nb,
                                                        int* __restrict__ total_out) {
    __shared__ int smem[8];
    int carry = 0;
    for (long long base = 0; base < nb; base += BM_BLOCK) {
        long long p = base + threadIdx.x;
        int v = (p < nb) ? bsum[p] : 0;
        int total;
        int ex = block_exclusive_scan_256(v, total, smem);
        if (p < nb) bsum[p] = carry + ex;
        carry += total;
    }
    if (threadIdx.x == 0) *total_out = carry;
}

__global__ __launch_bounds__(BM_BLOCK) void k_scan_final(const int* __restrict__ in, long long n,
                                                          const int* __restrict__ bsum,
                                                          int* __restrict__ out) {
    __shared__ int smem[8];
    long long base = (long long)blockIdx.x * SCAN_TILE + (long long)threadIdx.x * SCAN_ITEMS;
    int v[SCAN_ITEMS];
    int s = 0;
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i) {
        long long p = base + i;
        v[i] = (p < n) ? in[p] : 0;
        s += v[i];
    }
    int total;
    int ex = block_exclusive_scan_256(s, total, smem) + bsum[blockIdx.x];
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i) {
        long long p = base + i;
        if (p < n) out[p] = ex;
        ex += v[i];
    }
}
}  // namespace

size_t scan_tmp_ints(long long n) {
    long long nb = (n + SCAN_TILE - 1) / SCAN_TILE;
    return (size_t)(nb < 1 ? 1 : nb);
}

hipError_t scan_exclusive_i32(const int* in, int* out, long long n, int* tmp, hipStream_t stream) {
    if (n < 0) return hipErrorInvalidValue;
    long long nb = (n + SCAN_TILE - 1) / SCAN_TILE;
    if (nb > 0x7fffffffLL) return hipErrorInvalidValue;
    if (nb > 0) {
        hipLaunchKernelGGL(k_scan_blocksums, dim3((unsigned)nb), dim3(BM_BLOCK), 0, stream, in, n, tmp);
    }
    hipLaunchKernelGGL(k_scan_top, dim3(1), dim3(BM_BLOCK), 0, stream, tmp, nb, out + n);
    if (nb > 0) {
        hipLaunchKernelGGL(k_scan_final, dim3((unsigned)nb), dim3(BM_BLOCK), 0, stream, in, n, tmp, out);
    }
    return hipGetLastError();
}

}  // namespace bm
