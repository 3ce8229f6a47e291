// Device-wide exclusive prefix sum of int32 (three launches, no host synchronisation).
#pragma once
#include <hip/hip_runtime.h>

namespace bm {

// out[i] = sum_{j<i} in[j] for i in [0, n]; out has n+1 entries (out[n] = total).
// `tmp` must hold scan_tmp_ints(n) ints. in and out may not alias.
size_t scan_tmp_ints(long long n);
hipError_t scan_exclusive_i32(const int* in, int* out, long long n, int* tmp, hipStream_t stream);

// Block-wide exclusive scan for BM_BLOCK (256) threads; returns the exclusive prefix of v and
// the block total in `total`. `smem` must hold 8 ints. All threads must call it.
__device__ __forceinline__ int block_exclusive_scan_256(int v, int& total, int* smem) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int inc = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        int t = __shfl_up(inc, d, 64);
        if (lane >= d) inc += t;
    }
    if (lane == 63) smem[wave] = inc;
    __syncthreads();
    int woff = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        int s = smem[w];
        if (w < wave) woff += s;
        tot += s;
    }
    __syncthreads();
    total = tot;
    return woff + inc - v;
}

}  // namespace bm
