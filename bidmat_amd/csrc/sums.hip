// Column / row reductions of sparse values and of dense matrices. All are streaming,
// bandwidth-bound kernels; every sum has a fixed order (two-stage, no atomics).
#include "common.hpp"
#include "kernels.hpp"
#include "ops.hpp"
#include "workspace.hpp"
#include <math.h>

namespace bm {
namespace {

// ------------------------------------------------------------------ sparse
// 16 lanes per column: strided partial sums (four loads in flight per lane, combined in a fixed
// order), DPP butterfly inside the 16-lane row.
__global__ __launch_bounds__(BM_BLOCK) void k_spsum_ranges(int nranges, const float* __restrict__ vals,
                                                           const int* __restrict__ ptr,
                                                           float* __restrict__ out, int beta) {
    const long long t = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long c = t >> 4;
    const int l = (int)(t & 15);
    float acc = 0.f;
    if (c < nranges) {
        const int s = ptr[c], e = ptr[c + 1];
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        int j = s + l;
        for (; j + 48 < e; j += 64) {
            const float v0 = vals[j], v1 = vals[j + 16], v2 = vals[j + 32], v3 = vals[j + 48];
            a0 += v0; a1 += v1; a2 += v2; a3 += v3;
        }
        for (; j < e; j += 16) a0 += vals[j];
        acc = (a0 + a1) + (a2 + a3);
    }
    acc = group_allsum<16>(acc);
    if (c < nranges && l == 0) out[c] = beta ? out[c] + acc : acc;
}

// Sums of the plan's segments, walked in the plan's XCD order (workgroup b runs on XCD b % 8 and
// takes that XCD's group of heavy segments, panel after panel, then every 8th light segment): the
// values a panel's segments pick through `perm` lie in that panel's columns, a few MiB that stay
// in the XCD's L2 while all heavy rows of the panel are summed.
struct XcdStarts { int v[9]; };
__global__ __launch_bounds__(BM_BLOCK) void k_spsum_plan(int nseg, XcdStarts xs, const float* __restrict__ vals,
                                                         const int* __restrict__ perm,
                                                         const int* __restrict__ segstart,
                                                         float* __restrict__ out) {
    const int xcd = blockIdx.x & 7;
    const long long wi = (long long)(blockIdx.x >> 3) * (BM_BLOCK / 16) + (threadIdx.x >> 4);
    const int l = threadIdx.x & 15;
    const int hstart = xs.v[xcd], hcount = xs.v[xcd + 1] - hstart;
    const long long seg = wi < hcount ? hstart + wi : xs.v[8] + (wi - hcount) * 8 + xcd;
    float acc = 0.f;
    if (seg < nseg) {
        const int s = segstart[seg], e = segstart[seg + 1];
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        int j = s + l;
        if (perm != nullptr) {
            for (; j + 48 < e; j += 64) {
                const int p0 = perm[j], p1 = perm[j + 16], p2 = perm[j + 32], p3 = perm[j + 48];
                a0 += vals[p0]; a1 += vals[p1]; a2 += vals[p2]; a3 += vals[p3];
            }
            for (; j < e; j += 16) a0 += vals[perm[j]];
        } else {                                        // values already in plan order
            for (; j + 48 < e; j += 64) {
                const float v0 = vals[j], v1 = vals[j + 16], v2 = vals[j + 32], v3 = vals[j + 48];
                a0 += v0; a1 += v1; a2 += v2; a3 += v3;
            }
            for (; j < e; j += 16) a0 += vals[j];
        }
        acc = (a0 + a1) + (a2 + a3);
    }
    acc = group_allsum<16>(acc);
    if (seg < nseg && l == 0) out[seg] = acc;
}

// ------------------------------------------------------------------ dense
template <int OP> __device__ __forceinline__ float op2(float a, float b);
template <> __device__ __forceinline__ float op2<0>(float a, float b) { return a + b; }
template <> __device__ __forceinline__ float op2<2>(float a, float b) { return a * b; }
template <> __device__ __forceinline__ float op2<10>(float a, float b) { return fmaxf(a, b); }
template <> __device__ __forceinline__ float op2<11>(float a, float b) { return fminf(a, b); }
template <int OP> __device__ __forceinline__ float op_identity();
template <> __device__ __forceinline__ float op_identity<0>() { return 0.f; }
template <> __device__ __forceinline__ float op_identity<2>() { return 1.f; }
template <> __device__ __forceinline__ float op_identity<10>() { return -INFINITY; }
template <> __device__ __forceinline__ float op_identity<11>() { return INFINITY; }

// Column reduce. lpc lanes (power of two <= 64) per column, W consecutive rows per lane and step
// (W = 4: 128-bit loads); rows [r0, r1) of chunk blockIdx.y. out[chunk*ncols + c].
template <int OP, int W>
__global__ __launch_bounds__(BM_BLOCK) void k_reduce_cols(int nrows, int ncols, int lpc, int rows_per_chunk,
                                                          const float* __restrict__ A,
                                                          float* __restrict__ out) {
    const long long t = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long c = t / lpc;
    const int l = (int)(t % lpc);
    const long long r0 = (long long)blockIdx.y * rows_per_chunk;
    long long r1 = r0 + rows_per_chunk;
    if (r1 > nrows) r1 = nrows;
    float acc = op_identity<OP>();
    if (c < ncols) {
        const float* col = A + (size_t)c * nrows;
        for (long long r = r0 + (long long)l * W; r < r1; r += (long long)lpc * W) {
            const Vec<W> v = Vec<W>::load(col + r);
            const float* f = reinterpret_cast<const float*>(&v);
#pragma unroll
            for (int i = 0; i < W; ++i) acc = op2<OP>(acc, f[i]);
        }
    }
    for (int d = 1; d < lpc; d <<= 1) acc = op2<OP>(acc, __shfl_xor(acc, d, 64));
    if (c < ncols && l == 0) out[(size_t)blockIdx.y * ncols + c] = acc;
}

// Row reduce, stage 1. A block is rb row-lanes x cl column-lanes (rb*cl == 256); every lane owns W
// consecutive rows (W = 4: 128-bit loads); blockIdx.x = row tile, blockIdx.y = column chunk.
// Four independent accumulators per lane keep four loads in flight. out[chunk*nrows + r].
template <int OP, int W>
__global__ __launch_bounds__(BM_BLOCK) void k_reduce_rows(int nrows, int ncols, int rb, int cols_per_chunk,
                                                          const float* __restrict__ A,
                                                          float* __restrict__ out) {
    __shared__ float sm[BM_BLOCK * W];
    const int cl = BM_BLOCK / rb;
    const int tr = threadIdx.x % rb;
    const int tc = threadIdx.x / rb;
    const long long r = ((long long)blockIdx.x * rb + tr) * W;
    const long long c0 = (long long)blockIdx.y * cols_per_chunk;
    long long c1 = c0 + cols_per_chunk;
    if (c1 > ncols) c1 = ncols;
    float acc[4][W];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int i = 0; i < W; ++i) acc[u][i] = op_identity<OP>();
    if (r < nrows) {
        long long c = c0 + tc;
        for (; c + 3LL * cl < c1; c += 4LL * cl) {
            Vec<W> v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = Vec<W>::load(A + (size_t)(c + (long long)u * cl) * nrows + r);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const float* f = reinterpret_cast<const float*>(&v[u]);
#pragma unroll
                for (int i = 0; i < W; ++i) acc[u][i] = op2<OP>(acc[u][i], f[i]);
            }
        }
        for (; c < c1; c += cl) {
            Vec<W> v = Vec<W>::load(A + (size_t)c * nrows + r);
            const float* f = reinterpret_cast<const float*>(&v);
#pragma unroll
            for (int i = 0; i < W; ++i) acc[0][i] = op2<OP>(acc[0][i], f[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < W; ++i)
        sm[threadIdx.x * W + i] = op2<OP>(op2<OP>(acc[0][i], acc[1][i]), op2<OP>(acc[2][i], acc[3][i]));
    __syncthreads();
    if (tc == 0 && r < nrows) {
#pragma unroll
        for (int i = 0; i < W; ++i) {
            float a = sm[threadIdx.x * W + i];
            for (int q = 1; q < cl; ++q) a = op2<OP>(a, sm[(q * rb + tr) * W + i]);
            out[(size_t)blockIdx.y * nrows + r + i] = a;
        }
    }
}

// Stage 2 of both reductions: out[i] = op over chunks of part[chunk*n + i], in chunk order.
template <int OP>
__global__ __launch_bounds__(BM_BLOCK) void k_reduce_chunks(int n, int nchunks, const float* __restrict__ part,
                                                            float* __restrict__ out) {
    const long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (i >= n) return;
    float acc = part[i];
    for (int q = 1; q < nchunks; ++q) acc = op2<OP>(acc, part[(size_t)q * n + i]);
    out[i] = acc;
}

template <int OP>
hipError_t reduce1_impl(int nrows, int ncols, const float* A, float* B, hipStream_t s) {
    const bool vec = (nrows % 4 == 0) && ((reinterpret_cast<uintptr_t>(A) & 15) == 0);
    const int W = vec ? 4 : 1;
    const int nv = (nrows + W - 1) / W;
    int lpc = pow2ceil(nv) < 64 ? pow2ceil(nv) : 64;
    // few, very long columns: cut the rows into chunks so the whole chip works
    int nchunks = 1;
    if ((long long)ncols * lpc < 64 * 2048 && nrows > 8192) {
        long long want = (64LL * 4096) / ((long long)ncols * lpc);
        long long maxc = (nrows + 4095) / 4096;
        nchunks = (int)(want < maxc ? want : maxc);
        if (nchunks < 1) nchunks = 1;
        if (nchunks > 4096) nchunks = 4096;
    }
    int rows_per_chunk = (nrows + nchunks - 1) / nchunks;
    rows_per_chunk = (rows_per_chunk + 3) & ~3;            // chunk starts stay 16-byte aligned
    nchunks = (nrows + rows_per_chunk - 1) / rows_per_chunk;
    long long threads = (long long)ncols * lpc;
    long long nblk = (threads + BM_BLOCK - 1) / BM_BLOCK;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    float* dst = B;
    if (nchunks > 1) {
        hipError_t err;
        dst = (float*)ws_get(WS_REDUCE, sizeof(float) * (size_t)nchunks * ncols, &err, s);
        if (!dst) return err;
    }
    if (vec) hipLaunchKernelGGL((k_reduce_cols<OP, 4>), dim3((unsigned)nblk, (unsigned)nchunks), dim3(BM_BLOCK), 0, s,
                                nrows, ncols, lpc, rows_per_chunk, A, dst);
    else hipLaunchKernelGGL((k_reduce_cols<OP, 1>), dim3((unsigned)nblk, (unsigned)nchunks), dim3(BM_BLOCK), 0, s,
                            nrows, ncols, lpc, rows_per_chunk, A, dst);
    if (nchunks > 1) {
        unsigned nb2 = (unsigned)(((long long)ncols + BM_BLOCK - 1) / BM_BLOCK);
        hipLaunchKernelGGL(k_reduce_chunks<OP>, dim3(nb2), dim3(BM_BLOCK), 0, s, ncols, nchunks, dst, B);
    }
    return hipGetLastError();
}

// Row reduce of a column-major nrows x ncols matrix with leading dimension nrows. Stage 1 cuts the
// columns into chunks (one workgroup each); the chunk partials form an nrows x nchunks matrix that
// is reduced the same way again until few enough chunks remain for k_reduce_chunks. `scratch`
// is a workspace of `scratch_floats` floats for the partials (nullptr: take it from the slot).
template <int OP>
hipError_t reduce2_impl(int nrows, int ncols, const float* A, float* B, hipStream_t s,
                        float* scratch = nullptr, size_t scratch_floats = 0) {
    const bool vec = (nrows % 4 == 0) && ((reinterpret_cast<uintptr_t>(A) & 15) == 0);
    const int W = vec ? 4 : 1;
    const int lanes = (nrows + W - 1) / W;                 // row-lanes needed
    int rb = pow2ceil(lanes) < BM_BLOCK ? pow2ceil(lanes) : BM_BLOCK;
    int cl = BM_BLOCK / rb;
    long long rowtiles = ((long long)lanes + rb - 1) / rb;
    // enough column chunks to fill the chip, at least 16 columns per column-lane
    long long nchunks = 4096 / rowtiles;
    long long maxc = ((long long)ncols + (long long)cl * 16 - 1) / ((long long)cl * 16);
    if (nchunks > maxc) nchunks = maxc;
    if (nchunks < 1) nchunks = 1;
    int cols_per_chunk = (int)(((long long)ncols + nchunks - 1) / nchunks);
    nchunks = ((long long)ncols + cols_per_chunk - 1) / cols_per_chunk;
    if (rowtiles > 0x7fffffffLL || nchunks > 65535) return hipErrorInvalidValue;
    float* dst = B;
    if (nchunks > 1) {
        const size_t need = (size_t)nchunks * nrows;
        if (!scratch) {
            // room for this level's partials and, behind them, every deeper level's (each at most
            // 1/16 of the one before)
            hipError_t err;
            scratch_floats = need + need / 8 + 4096;
            scratch = (float*)ws_get(WS_REDUCE, sizeof(float) * scratch_floats, &err, s);
            if (!scratch) return err;
        }
        if (need > scratch_floats) return hipErrorInvalidValue;
        dst = scratch;
    }
    dim3 grid((unsigned)rowtiles, (unsigned)nchunks), block(BM_BLOCK);
    if (vec) hipLaunchKernelGGL((k_reduce_rows<OP, 4>), grid, block, 0, s, nrows, ncols, rb, cols_per_chunk, A, dst);
    else hipLaunchKernelGGL((k_reduce_rows<OP, 1>), grid, block, 0, s, nrows, ncols, rb, cols_per_chunk, A, dst);
    if (nchunks > 32) {
        const size_t used = ((size_t)nchunks * nrows + 3) & ~size_t(3);     // keep 16-byte alignment
        return reduce2_impl<OP>(nrows, (int)nchunks, dst, B, s, scratch + used, scratch_floats - used);
    }
    if (nchunks > 1) {
        unsigned nb2 = (unsigned)(((long long)nrows + BM_BLOCK - 1) / BM_BLOCK);
        hipLaunchKernelGGL(k_reduce_chunks<OP>, dim3(nb2), dim3(BM_BLOCK), 0, s, nrows, (int)nchunks, dst, B);
    }
    return hipGetLastError();
}

// Reduction with ANY of the 15 binary ops (most are neither associative nor commutative, so the order IS the
// result): the order of the reference's kernels (Operators.cu:650-671, 828-851). 32 lanes per output; lane t
// folds elements t, t+32, ... from the left, then for i = 1, 2, 4, ... the lanes t with t + i < L = min(n, 32)
// take op(own, lane t+i's value of the step before). DIM == 1: one output per column (elements are
// contiguous), DIM == 2: one per row (elements nrows apart).
template <int DIM>
__global__ __launch_bounds__(BM_BLOCK) void k_reduce_tree(int nrows, int ncols, const float* __restrict__ A,
                                                          float* __restrict__ out, int opn) {
    const long long o = ((long long)blockIdx.x * BM_BLOCK + threadIdx.x) >> 5;
    const int t = threadIdx.x & 31;
    const int nout = DIM == 1 ? ncols : nrows;
    const int n = DIM == 1 ? nrows : ncols;
    const bool live = o < nout;
    const int L = n < 32 ? n : 32;
    float v = 0.f;
    if (live && t < L) {
        const float* base = DIM == 1 ? A + (size_t)o * nrows : A + o;
        const size_t step = DIM == 1 ? 1 : (size_t)nrows;
        v = base[(size_t)t * step];
        for (long long e = t + 32; e < n; e += 32) v = binop_rt(opn, v, base[(size_t)e * step]);
    }
    for (int i = 1; i < L; i <<= 1) {
        const float other = __shfl_down(v, i, 32);
        if (t + i < L) v = binop_rt(opn, v, other);
    }
    if (live && t == 0) out[o] = v;
}

template <int DIM>
hipError_t reduce_tree(int nrows, int ncols, const float* A, float* B, int opn, hipStream_t s) {
    const long long nout = DIM == 1 ? ncols : nrows;
    const long long nblk = (nout * 32 + BM_BLOCK - 1) / BM_BLOCK;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(k_reduce_tree<DIM>, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, nrows, ncols, A, B, opn);
    return hipGetLastError();
}

}  // namespace

hipError_t spsum_cols(int ncols, int nnz, const float* vals, const int* jc, float* out, int beta, hipStream_t s) {
    (void)nnz;
    if (ncols <= 0) return hipSuccess;
    long long nblk = ((long long)ncols * 16 + BM_BLOCK - 1) / BM_BLOCK;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(k_spsum_ranges, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, ncols, vals, jc, out, beta);
    return hipGetLastError();
}

hipError_t spsum_segments(int nseg, const int* xcd_start, const float* vals, const int* perm, const int* segstart,
                          float* partial, hipStream_t s) {
    if (nseg <= 0) return hipSuccess;
    XcdStarts xs;
    int maxheavy = 0;
    for (int x = 0; x < 9; ++x) xs.v[x] = xcd_start[x];
    for (int x = 0; x < 8; ++x) maxheavy = xs.v[x + 1] - xs.v[x] > maxheavy ? xs.v[x + 1] - xs.v[x] : maxheavy;
    const long long nlight = (long long)nseg - xs.v[8];
    const long long per_xcd = (long long)maxheavy + (nlight + 7) / 8;          // segments per XCD
    const long long nblk = 8 * ((per_xcd + BM_BLOCK / 16 - 1) / (BM_BLOCK / 16));
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(k_spsum_plan, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, nseg, xs, vals, perm, segstart, partial);
    return hipGetLastError();
}

hipError_t reduce1op(int nrows, int ncols, const float* A, float* B, float initv, int opn, hipStream_t s) {
    if (ncols <= 0) return hipSuccess;
    if (nrows <= 0) return fill_f32(B, ncols, initv, s);
    switch (opn) {
    case 0: return reduce1_impl<0>(nrows, ncols, A, B, s);
    case 2: return reduce1_impl<2>(nrows, ncols, A, B, s);
    case 10: return reduce1_impl<10>(nrows, ncols, A, B, s);
    case 11: return reduce1_impl<11>(nrows, ncols, A, B, s);
    default: return (opn > 0 && opn <= 14) ? reduce_tree<1>(nrows, ncols, A, B, opn, s) : hipErrorInvalidValue;
    }
}

hipError_t reduce2op(int nrows, int ncols, const float* A, float* B, float initv, int opn, hipStream_t s) {
    if (nrows <= 0) return hipSuccess;
    if (ncols <= 0) return fill_f32(B, nrows, initv, s);
    switch (opn) {
    case 0: return reduce2_impl<0>(nrows, ncols, A, B, s);
    case 2: return reduce2_impl<2>(nrows, ncols, A, B, s);
    case 10: return reduce2_impl<10>(nrows, ncols, A, B, s);
    case 11: return reduce2_impl<11>(nrows, ncols, A, B, s);
    default: return (opn > 0 && opn <= 14) ? reduce_tree<2>(nrows, ncols, A, B, opn, s) : hipErrorInvalidValue;
    }
}

}  // namespace bm
