// The densest rows of a pattern as a dense block of A *^ S.
//
// In a power-law pattern a few rows hold a nonzero in a large share of all columns (the 128 most frequent of
// 100 000 Zipf(1.1) rows: 30 % of the nonzeros, each in 20 % to 100 % of the columns). For such rows
// C[:, r] = sum over columns c of A[:, c] * S[r, c] is a dense matrix product in all but name: gathering the
// column of A once per nonzero re-reads every column of A up to 128 times out of L2. Here the columns of A are
// streamed once per group of 32 dense rows and multiplied on the matrix cores (fp32 MFMA 32x32x2: a k-slice of
// 32 elements x 2 columns of A times 2 columns x 32 dense rows of S), absent entries entering as zeros.
//
// What a plan holds for it (row side, built after the segments): the dense rows ranked by count (drank), for
// every column the position in the stored arrays of its nonzero in each dense row (dpos, -1 = none), a byte per
// segment that tells stage 1 of A *^ S to leave the dense rows' segments out (dskip), the list of those
// segments (dseglist), and a second row -> partial-sum table (rowptr2 / rowseg2) in which a dense row's partial
// sums are the ones this file's kernel writes, one per block of columns.
//
// 0 * inf: a zero that stands for an absent entry must not turn a non-finite element of A into a NaN of a row
// that has no nonzero in that column. The kernel therefore watches the elements of A it streams and raises a
// flag when one is not finite; stage 1 is then run for the dense rows' segments after all (a launch whose waves
// return at once while the flag is down), and the row reduction picks the table that matches the flag.
#include <algorithm>
#include "plan.hpp"
#include "common.hpp"
#include "kernels.hpp"
#include "scan.hpp"
#include "workspace.hpp"
#include <initializer_list>

namespace bm {
namespace {

constexpr int DR_MAX = 128;        // dense rows at most (four groups of 32)
constexpr int DR_CAND = 1024;      // rows ranked at most
constexpr int DR_LEVELS = 16;      // thresholds thr, 2 thr, 4 thr, ... tried to get at most DR_CAND candidates

// Carves 256-byte aligned pieces out of one allocation (base == nullptr: only adds up the sizes).
struct Arena {
    char* base = nullptr;
    size_t used = 0;
    template <typename T> T* take(size_t count) {
        T* p = base ? reinterpret_cast<T*>(base + used) : nullptr;
        used += (sizeof(T) * (count ? count : 1) + 255) & ~size_t(255);
        return p;
    }
};

inline unsigned blocks_for(long long n) {
    long long b = (n + BM_BLOCK - 1) / BM_BLOCK;
    return (unsigned)(b < 1 ? 1 : b);
}

// counts[i] = rows with cnt >= thr << i
__global__ __launch_bounds__(BM_BLOCK) void k_dense_levels(int nrows, const int* __restrict__ cnt, long long thr,
                                                           int* __restrict__ counts) {
    __shared__ int loc[DR_LEVELS];
    if (threadIdx.x < DR_LEVELS) loc[threadIdx.x] = 0;
    __syncthreads();
    const long long r = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (r < nrows) {
        const long long c = cnt[r];
        for (int i = 0; i < DR_LEVELS && c >= (thr << i); ++i) atomicAdd(&loc[i], 1);
    }
    __syncthreads();
    if (threadIdx.x < DR_LEVELS && loc[threadIdx.x]) atomicAdd(&counts[threadIdx.x], loc[threadIdx.x]);
}

__device__ __forceinline__ int dense_level(const int* counts) {
    int lev = 0;
    while (lev < DR_LEVELS && counts[lev] > DR_CAND) ++lev;
    return lev;                    // DR_LEVELS: even the highest threshold leaves too many rows
}

// The rows at or above the lowest threshold that leaves at most DR_CAND of them: cand[2i] = row, cand[2i+1] = count.
// (Their order here depends on the scheduling; k_dense_rank orders them.)
__global__ __launch_bounds__(BM_BLOCK) void k_dense_collect(int nrows, const int* __restrict__ cnt, long long thr,
                                                            const int* __restrict__ counts, int* __restrict__ cand,
                                                            int* __restrict__ ncand) {
    const int lev = dense_level(counts);
    if (lev >= DR_LEVELS) return;
    const long long r = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (r < nrows && (long long)cnt[r] >= (thr << lev)) {
        const int at = atomicAdd(ncand, 1);
        if (at < DR_CAND) { cand[2 * at] = (int)r; cand[2 * at + 1] = cnt[r]; }
    }
}

// One workgroup: rank of every candidate by (count descending, row ascending); the first nd = min(cap, n)
// rounded down to whole groups of 32 become the dense rows. out[0] = nd.
__global__ __launch_bounds__(DR_CAND) void k_dense_rank(const int* __restrict__ cand, const int* __restrict__ ncand,
                                                        int cap, int* __restrict__ drow, int* __restrict__ drank,
                                                        int* __restrict__ out) {
    __shared__ int srow[DR_CAND], scnt[DR_CAND];
    int n = *ncand;
    if (n > DR_CAND) n = DR_CAND;
    const int i = threadIdx.x;
    if (i < n) { srow[i] = cand[2 * i]; scnt[i] = cand[2 * i + 1]; }
    __syncthreads();
    const int nd = (n < cap ? n : cap) & ~31;
    if (i == 0) out[0] = nd;
    if (i >= n) return;
    const int r = srow[i], c = scnt[i];
    int rank = 0;
    for (int j = 0; j < n; ++j) rank += (scnt[j] > c || (scnt[j] == c && srow[j] < r)) ? 1 : 0;
    if (rank < nd) { drow[rank] = r; drank[r] = rank; }
}

// One wave per column: dpos[c*nd + d] = position of the column's nonzero in dense row d, or -1. Two nonzeros of
// one column in the same dense row (a pattern with repeated entries) raise *dup: such a pattern gets no dense block.
__global__ __launch_bounds__(BM_BLOCK) void k_dense_positions(int ncols, int nrows, int nd, const int* __restrict__ ir,
                                                              const int* __restrict__ jc, const int* __restrict__ drank,
                                                              int* __restrict__ dpos, int* __restrict__ dup) {
    __shared__ int slot[BM_WAVES_PER_BLOCK][DR_MAX];
    const int lane = threadIdx.x & 63, wave = wave_uniform(threadIdx.x >> 6);
    const long long c = (long long)blockIdx.x * BM_WAVES_PER_BLOCK + wave;
    if (c >= ncols) return;
    int* mine = slot[wave];
    for (int i = lane; i < nd; i += 64) mine[i] = -1;
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    const int s = jc[c], e = jc[c + 1];
    for (int j0 = s; j0 < e; j0 += 4 * 64) {
        int r[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) { const int j = j0 + u * 64 + lane; r[u] = j < e ? ir[j] : -1; }
        int d[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) d[u] = (unsigned)r[u] < (unsigned)nrows ? drank[r[u]] : -1;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (d[u] >= 0) {
                const int old = atomicExch(&mine[d[u]], j0 + u * 64 + lane);
                if (old != -1) *dup = 1;
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    int* out = dpos + (size_t)c * nd;
    for (int i = lane; i < nd; i += 64) out[i] = mine[i];
}

__global__ __launch_bounds__(BM_BLOCK) void k_dense_skip(int nseg, const int* __restrict__ segrow, const int* __restrict__ drank,
                                                         unsigned char* __restrict__ dskip) {
    const long long q = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (q < nseg) dskip[q] = drank[segrow[q]] >= 0 ? 1 : 0;
}

// partial sums per row in the second table: a dense row has one per chunk of blocks of columns
__global__ __launch_bounds__(BM_BLOCK) void k_dense_rowcount(int nrows, const int* __restrict__ rowptr, const int* __restrict__ drank,
                                                             int nfold, int* __restrict__ cnt2) {
    const long long r = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (r < nrows) cnt2[r] = drank[r] >= 0 ? nfold : rowptr[r + 1] - rowptr[r];
}

// One wave per row. The partial sum of (chunk ch of the blocks of columns, dense row d) is partial slot first + ch*nd + d.
__global__ __launch_bounds__(BM_BLOCK) void k_dense_rowseg(int nrows, int first, int nd, int nfold, const int* __restrict__ rowptr,
                                                           const int* __restrict__ rowseg, const int* __restrict__ drank,
                                                           const int* __restrict__ rowptr2, int* __restrict__ rowseg2) {
    const long long r = ((long long)blockIdx.x * BM_BLOCK + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (r >= nrows) return;
    const int d = drank[r], o = rowptr2[r];
    if (d >= 0) {
        for (int j = lane; j < nfold; j += 64) rowseg2[o + j] = first + j * nd + d;
    } else {
        const int s = rowptr[r], n = rowptr[r + 1] - s;
        for (int i = lane; i < n; i += 64) rowseg2[o + i] = rowseg[s + i];
    }
}

// One workgroup per dense row: its segments go to the list behind those of the rows ranked before it.
// out[0] = number of all of them.
__global__ __launch_bounds__(BM_BLOCK) void k_dense_seglist(int nd, const int* __restrict__ drow, const int* __restrict__ rowptr,
                                                            const int* __restrict__ rowseg, int* __restrict__ list,
                                                            int* __restrict__ out) {
    __shared__ int before[BM_BLOCK];
    const int d = blockIdx.x;
    int mine = 0;                                  // segments of the rows ranked before d (thread t: rank t, t < DR_MAX)
    if ((int)threadIdx.x < (d < nd ? d : nd)) mine = rowptr[drow[threadIdx.x] + 1] - rowptr[drow[threadIdx.x]];
    before[threadIdx.x] = mine;
    __syncthreads();
    for (int o = BM_BLOCK / 2; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) before[threadIdx.x] += before[threadIdx.x + o];
        __syncthreads();
    }
    const int off = before[0];
    if (d == nd) {                                 // the extra workgroup: the total
        if (threadIdx.x == 0) out[0] = off;
        return;
    }
    const int s = rowptr[drow[d]], n = rowptr[drow[d] + 1] - s;
    for (int i = threadIdx.x; i < n; i += BM_BLOCK) list[off + i] = rowseg[s + i];
}

// ---- the product. One wave per (block of columns, group of 32 dense rows); the waves of a block of columns
// sit on one XCD (workgroup b runs on XCD b % 8) and share the block's columns of A in its L2. Per step two
// columns: lane l supplies A[32 s + l % 32, c + l / 32] for each k-slice s and S[c + l / 32, row 32 g + l % 32]
// (the stored value at dpos, or 0). DEPTH steps are in flight. The 32 x 32 result of slice s: lane l holds dense
// row l % 32 and, in register v, element 32 s + 8 (v / 4) + 4 (l / 32) + v % 4.
typedef float f16v __attribute__((ext_vector_type(16)));

// DIRECT: `dpos` holds the values themselves (the plan's copy in the layout of dpos, 0 where a column has no nonzero
// in the row) instead of positions into vals.
template <int NSW, int DEPTH, bool DIRECT>
__device__ __forceinline__ void dense_mfma_body(int k, int ncols, int nd, int cb, const float* __restrict__ A,
                                                const float* __restrict__ vals, const int* __restrict__ dpos,
                                                float* __restrict__ part, int* __restrict__ flag) {
    const int lane = threadIdx.x;
    const int G = nd >> 5;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int g = idx % G, j = (idx / G) * 8 + xcd;
    const long long c0 = (long long)j * cb;
    if (c0 >= ncols) return;
    const int c1 = (int)(c0 + cb < ncols ? c0 + cb : ncols);
    const int half = lane >> 5, n = lane & 31;
    f16v acc[NSW];
#pragma unroll
    for (int s = 0; s < NSW; ++s)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[s][v] = 0.f;
    bool ev[NSW];
#pragma unroll
    for (int s = 0; s < NSW; ++s) ev[s] = s * 32 + n < k;
    unsigned worst = 0;              // largest magnitude bits of A met: not finite from 0x7f800000 on
    // Every load is issued unconditionally, from a clamped address, and its result is masked only where it is consumed,
    // DEPTH steps later: a branch around a load (or a select right behind it) makes the compiler wait for every load
    // in flight before each step's matrix instructions, which takes the steps meant to be under way out of flight.
    const int clast = c1 - 1;
    auto rawpos = [&](int c) -> int { const int cc = c + half; return dpos[(size_t)(cc < c1 ? cc : clast) * nd + g * 32 + n]; };
    auto rawval = [&](int p) -> float { return DIRECT ? __int_as_float(p) : vals[p >= 0 ? p : 0]; };
    constexpr int NONE = DIRECT ? 0 : -1;        // what stands for "no nonzero": the bits of +0.0f / no position
    int eoff[NSW];
#pragma unroll
    for (int s = 0; s < NSW; ++s) eoff[s] = ev[s] ? s * 32 : -n;          // an element past k: the column's first instead
    auto rawA = [&](int c, float (&x)[NSW]) {
        const int cc = c + half;
        const float* p = A + (size_t)(cc < c1 ? cc : clast) * (size_t)k + n;
#pragma unroll
        for (int s = 0; s < NSW; ++s) x[s] = p[eoff[s]];
    };
    float a[DEPTH][NSW], bv[DEPTH];
    int bp[DEPTH];                   // the position each bv was fetched from (-1: no nonzero there)
    // the positions run two steps ahead of the values fetched through them: a wait for the load issued last would
    // be a wait for every load in flight
    int pos[DEPTH + 2];
#pragma unroll
    for (int d = 0; d < DEPTH + 2; ++d) pos[d] = rawpos((int)c0 + 2 * d);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        bp[d] = ((int)c0 + 2 * d + half < c1) ? pos[d] : NONE;
        bv[d] = rawval(bp[d]);
        rawA((int)c0 + 2 * d, a[d]);
    }
    for (int c = (int)c0; c < c1; c += 2 * DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            // take slot d (columns c + 2d and c + 2d + 1), refill it for the columns 2 DEPTH further on
            const bool in = c + 2 * d + half < c1;
            float ax[NSW];
#pragma unroll
            for (int s = 0; s < NSW; ++s) ax[s] = (ev[s] && in) ? a[d][s] : 0.f;
            const float bx = (DIRECT || bp[d] >= 0) ? bv[d] : 0.f;
            const int cn = c + 2 * (d + DEPTH);
            const int pnext = (cn + half < c1) ? pos[DEPTH] : NONE;
#pragma unroll
            for (int q = 0; q < DEPTH + 1; ++q) pos[q] = pos[q + 1];
            pos[DEPTH + 1] = rawpos(cn + 4);
            bp[d] = pnext;
            bv[d] = rawval(pnext);
            rawA(cn, a[d]);
            __builtin_amdgcn_sched_barrier(0);       // the refill is on its way before the matrix instructions start
#pragma unroll
            for (int s = 0; s < NSW; ++s) {
                const unsigned m = __float_as_uint(ax[s]) & 0x7fffffffu;
                worst = m > worst ? m : worst;
                acc[s] = __builtin_amdgcn_mfma_f32_32x32x2f32(ax[s], bx, acc[s], 0, 0, 0);
            }
        }
    }
    if (worst >= 0x7f800000u) *flag = 1;
    float* out = part + ((size_t)j * nd + g * 32 + n) * (size_t)k;
    const bool vec = (k & 3) == 0 && (reinterpret_cast<uintptr_t>(part) & 15) == 0;
#pragma unroll
    for (int s = 0; s < NSW; ++s)
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {
            const int el = s * 32 + 8 * v4 + 4 * half;
            if (vec) {
                if (el < k) *reinterpret_cast<float4*>(out + el) = make_float4(acc[s][4 * v4], acc[s][4 * v4 + 1], acc[s][4 * v4 + 2], acc[s][4 * v4 + 3]);
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (el + t < k) out[el + t] = acc[s][4 * v4 + t];
            }
        }
}

template <int NSW, int DEPTH>
__global__ __launch_bounds__(64) void k_dense_mfma(int k, int ncols, int nd, int cb, const float* __restrict__ A,
                                                   const float* __restrict__ vals, const int* __restrict__ dpos,
                                                   float* __restrict__ part, int* __restrict__ flag) {
    dense_mfma_body<NSW, DEPTH, false>(k, ncols, nd, cb, A, vals, dpos, part, flag);
}
// the same with the values stored in the plan (dvals, in the layout of dpos)
template <int NSW, int DEPTH>
__global__ __launch_bounds__(64) void k_dense_mfma_stored(int k, int ncols, int nd, int cb, const float* __restrict__ A,
                                                          const float* __restrict__ dvals, float* __restrict__ part,
                                                          int* __restrict__ flag) {
    dense_mfma_body<NSW, DEPTH, true>(k, ncols, nd, cb, A, nullptr, reinterpret_cast<const int*>(dvals), part, flag);
}

// The partial sums of `per` consecutive blocks of columns added up, block after block: one wave per (chunk of
// blocks, dense row), a quarter of k per lane and step. A dense row then has a few partial sums for the row
// reduction to add instead of one per block (the wave that owns the row there adds them one after the other).
__global__ __launch_bounds__(64) void k_dense_fold(int k, int nd, int ndblocks, int per, const float* __restrict__ part,
                                                   float* __restrict__ fold) {
    const int d = blockIdx.x % nd, ch = blockIdx.x / nd;
    const int j0 = ch * per, j1 = j0 + per < ndblocks ? j0 + per : ndblocks;
    const bool vec = (k & 3) == 0 && ((reinterpret_cast<uintptr_t>(part) | reinterpret_cast<uintptr_t>(fold)) & 15) == 0;
    float* out = fold + ((size_t)ch * nd + d) * (size_t)k;
    if (vec) {
        for (int el = 4 * threadIdx.x; el < k; el += 256) {
            Vec<4> acc = Vec<4>::zero();
            int j = j0;
            for (; j + 8 <= j1; j += 8) {
                Vec<4> p[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) p[u] = Vec<4>::load(part + ((size_t)(j + u) * nd + d) * (size_t)k + el);
#pragma unroll
                for (int u = 0; u < 8; ++u) acc.add(p[u]);
            }
            for (; j < j1; ++j) acc.add(Vec<4>::load(part + ((size_t)j * nd + d) * (size_t)k + el));
            acc.store(out + el);
        }
    } else {
        for (int el = threadIdx.x; el < k; el += 64) {
            float acc = 0.f;
            for (int j = j0; j < j1; ++j) acc += part[((size_t)j * nd + d) * (size_t)k + el];
            out[el] = acc;
        }
    }
}

}  // namespace

int dense_rows_max() { return DR_MAX; }
int dense_rows_fold(int ndblocks) { return ndblocks < 16 ? ndblocks : 16; }

hipError_t drop_dense(bidmat_plan* p) {
    hipError_t e = hipSuccess;
    for (void** b : {&p->block_dense, (void**)&p->dpos, (void**)&p->dvals}) {
        if (*b) {
            hipError_t f = pool_free(*b);
            if (f != hipSuccess) e = f;
            *b = nullptr;
        }
    }
    p->row_bytes -= p->dense_bytes;
    p->dense_bytes = 0;
    p->ndense = p->ndblocks = p->dcb = p->ndseg = 0;
    p->drank = p->drow = p->rowptr2 = p->rowseg2 = p->dseglist = nullptr;
    p->dskip = nullptr;
    return e;
}

#define DR_CHECK(expr)                                          \
    do {                                                        \
        hipError_t _e = (expr);                                 \
        if (_e != hipSuccess) return _e;                        \
    } while (0)

// cnt[r]: about (nonzeros of row r) / sample. Leaves the plan without a dense block (ndense == 0) when no row is
// dense enough, when too many are, or when a column holds the same dense row twice. Blocks (two small read-backs).
hipError_t build_dense_rows(bidmat_plan* plan, const int* ir, const int* jc, const int* cnt, int sample, hipStream_t s) {
    const int nrows = plan->nrows, ncols = plan->ncols, nseg = plan->nseg;
    int cap = opt_dense_rows();
    if (cap > DR_MAX) cap = DR_MAX;
    cap &= ~31;
    if (cap <= 0 || nseg <= 0 || ncols < 64) return hipSuccess;
    long long thr = ((long long)ncols * opt_dense_min_pct() + 100LL * sample - 1) / (100LL * sample);
    if (thr < 1) thr = 1;

    hipError_t werr;
    Arena tmp;
    int *small = nullptr, *cand = nullptr, *cnt2 = nullptr, *scantmp = nullptr;
    for (int pass = 0; pass < 2; ++pass) {
        tmp.used = 0;
        small = tmp.take<int>(DR_LEVELS + 8);      // level counts, then: number of candidates, nd, dup, ndseg
        cand = tmp.take<int>(2 * DR_CAND);
        cnt2 = tmp.take<int>((size_t)nrows + 1);
        scantmp = tmp.take<int>(scan_tmp_ints((long long)nrows + 1));
        if (pass == 0) {
            tmp.base = static_cast<char*>(ws_get(WS_PLAN_ROWS_B, tmp.used, &werr, s));
            if (!tmp.base) return werr;
        }
    }
    int* const counts = small;
    int* const ncand = small + DR_LEVELS;
    int* const ndout = small + DR_LEVELS + 1;
    int* const dup = small + DR_LEVELS + 2;
    int* const nlist = small + DR_LEVELS + 3;

    // what the plan keeps, part 1 (sizes known now; the segment list and the second table are sized by their bounds)
    const long long dcb_opt = opt_dense_cb();
    long long cb = dcb_opt;
    if (cb <= 0) {
        // blocks of columns: a multiple of 512 waves' worth per group, about 330 to 400 columns each
        const long long rounds = (ncols + 512LL * 400 - 1) / (512LL * 400);
        cb = (ncols + 512 * rounds - 1) / (512 * rounds);
    }
    if (cb < 16) cb = 16;
    cb = (cb + 1) & ~1LL;                          // two columns per step
    const int ndblocks = (int)((ncols + cb - 1) / cb);
    Arena own;
    int *drank = nullptr, *drow = nullptr, *rowptr2 = nullptr, *rowseg2 = nullptr, *dseglist = nullptr;
    unsigned char* dskip = nullptr;
    void* block = nullptr;
    for (int pass = 0; pass < 2; ++pass) {
        own.used = 0;
        drank = own.take<int>((size_t)nrows);
        drow = own.take<int>(DR_MAX);
        rowptr2 = own.take<int>((size_t)nrows + 1);
        rowseg2 = own.take<int>((size_t)nseg + (size_t)cap * 16);
        dseglist = own.take<int>((size_t)nseg);
        dskip = own.take<unsigned char>((size_t)nseg);
        if (pass == 0) {
            block = pool_alloc(own.used, &werr);
            if (!block) return werr;
            own.base = static_cast<char*>(block);
        }
    }
    auto give_up = [&](hipError_t e) {
        (void)hipStreamSynchronize(s);
        (void)pool_free(block);
        return e;
    };

    // ---- which rows
    hipError_t e;
    if ((e = fill_i32(small, DR_LEVELS + 8, 0, s)) != hipSuccess) return give_up(e);
    if ((e = fill_i32(drank, nrows, -1, s)) != hipSuccess) return give_up(e);
    hipLaunchKernelGGL(k_dense_levels, dim3(blocks_for(nrows)), dim3(BM_BLOCK), 0, s, nrows, cnt, thr, counts);
    hipLaunchKernelGGL(k_dense_collect, dim3(blocks_for(nrows)), dim3(BM_BLOCK), 0, s, nrows, cnt, thr, counts, cand, ncand);
    hipLaunchKernelGGL(k_dense_rank, dim3(1), dim3(DR_CAND), 0, s, cand, ncand, cap, drow, drank, ndout);
    if ((e = hipGetLastError()) != hipSuccess) return give_up(e);
    int nd = 0;
    if ((e = hipMemcpyAsync(&nd, ndout, sizeof(int), hipMemcpyDeviceToHost, s)) != hipSuccess) return give_up(e);
    if ((e = hipStreamSynchronize(s)) != hipSuccess) return give_up(e);
    if (nd <= 0) return give_up(hipSuccess);

    // ---- positions per column, segments to leave out, the second table, the list of left-out segments
    int* dpos = static_cast<int*>(pool_alloc(sizeof(int) * (size_t)ncols * (size_t)nd, &werr));
    if (!dpos) return give_up(werr);
    auto give_up2 = [&](hipError_t err) {
        (void)hipStreamSynchronize(s);
        (void)pool_free(dpos);
        (void)pool_free(block);
        return err;
    };
    hipLaunchKernelGGL(k_dense_positions, dim3((unsigned)(((long long)ncols + BM_WAVES_PER_BLOCK - 1) / BM_WAVES_PER_BLOCK)), dim3(BM_BLOCK), 0, s,
                       ncols, nrows, nd, ir, jc, drank, dpos, dup);
    hipLaunchKernelGGL(k_dense_skip, dim3(blocks_for(nseg)), dim3(BM_BLOCK), 0, s, nseg, plan->segrow, drank, dskip);
    const int nfold = dense_rows_fold(ndblocks);
    hipLaunchKernelGGL(k_dense_rowcount, dim3(blocks_for(nrows)), dim3(BM_BLOCK), 0, s, nrows, plan->rowptr, drank, nfold, cnt2);
    if ((e = scan_exclusive_i32(cnt2, rowptr2, nrows, scantmp, s)) != hipSuccess) return give_up2(e);
    hipLaunchKernelGGL(k_dense_rowseg, dim3(blocks_for(64LL * nrows)), dim3(BM_BLOCK), 0, s, nrows, nseg + ndblocks * nd, nd, nfold, plan->rowptr,
                       plan->rowseg, drank, rowptr2, rowseg2);
    hipLaunchKernelGGL(k_dense_seglist, dim3((unsigned)nd + 1), dim3(BM_BLOCK), 0, s, nd, drow, plan->rowptr, plan->rowseg, dseglist, nlist);
    if ((e = hipGetLastError()) != hipSuccess) return give_up2(e);
    int back[2] = {0, 0};                          // dup, ndseg
    if ((e = hipMemcpyAsync(back, dup, sizeof(back), hipMemcpyDeviceToHost, s)) != hipSuccess) return give_up2(e);
    if ((e = hipStreamSynchronize(s)) != hipSuccess) return give_up2(e);
    if (back[0]) return give_up2(hipSuccess);

    plan->ndense = nd; plan->dcb = (int)cb; plan->ndblocks = ndblocks; plan->ndseg = back[1];
    plan->drank = drank; plan->drow = drow; plan->rowptr2 = rowptr2; plan->rowseg2 = rowseg2;
    plan->dseglist = dseglist; plan->dskip = dskip; plan->dpos = dpos; plan->block_dense = block;
    plan->dense_bytes = own.used + sizeof(int) * (size_t)ncols * (size_t)nd;
    plan->row_bytes += plan->dense_bytes;
    return hipSuccess;
}

bool dense_rows_fit(int k) { return k > 64 && k <= 256; }

// part: (ndblocks + dense_rows_fold(ndblocks)) * nd partial sums of k floats, the folded ones last. *flag (cleared by the caller's stage 1) is raised when A holds a
// value that is not finite.
namespace {
__global__ __launch_bounds__(BM_BLOCK) void k_dense_values(long long n, const int* __restrict__ dpos, const float* __restrict__ data,
                                                           float* __restrict__ dvals) {
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    for (long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x; i < n; i += stride) {
        const int p = dpos[i];
        dvals[i] = p >= 0 ? data[p] : 0.f;
    }
}
}  // namespace

hipError_t dense_rows_set_values(bidmat_plan* plan, const float* data, hipStream_t s) {
    if (plan->ndense <= 0 || plan->dpos == nullptr) return hipSuccess;
    const size_t n = (size_t)plan->ncols * (size_t)plan->ndense;
    if (plan->dvals == nullptr) {
        hipError_t e;
        plan->dvals = static_cast<float*>(pool_alloc(sizeof(float) * n, &e));
        if (plan->dvals == nullptr) {
            (void)hipGetLastError();
            return e == hipErrorOutOfMemory ? hipSuccess : e;       // no room: stored values go without the dense block
        }
        plan->dense_bytes += sizeof(float) * n;
        plan->row_bytes += sizeof(float) * n;
    }
    hipLaunchKernelGGL(k_dense_values, dim3((unsigned)std::min<long long>(16384, ((long long)n + BM_BLOCK - 1) / BM_BLOCK)), dim3(BM_BLOCK), 0, s, (long long)n, plan->dpos, data, plan->dvals);
    return hipGetLastError();
}

hipError_t dense_rows_stage(int k, int ncols, int nd, int cb, int ndblocks, const float* A, const float* vals,
                            const int* dpos, const float* dvals, float* part, int* flag, hipStream_t s) {
    if (nd <= 0 || ndblocks <= 0) return hipSuccess;
    const int G = nd >> 5;
    const long long nblk = (long long)((ndblocks + 7) / 8) * 8 * G;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    if (vals == nullptr) {
        if (dvals == nullptr) return hipErrorInvalidValue;
        if (k > 128)
            hipLaunchKernelGGL((k_dense_mfma_stored<8, 4>), dim3((unsigned)nblk), dim3(64), 0, s, k, ncols, nd, cb, A, dvals, part, flag);
        else
            hipLaunchKernelGGL((k_dense_mfma_stored<4, 4>), dim3((unsigned)nblk), dim3(64), 0, s, k, ncols, nd, cb, A, dvals, part, flag);
    } else if (k > 128) {
        hipLaunchKernelGGL((k_dense_mfma<8, 4>), dim3((unsigned)nblk), dim3(64), 0, s, k, ncols, nd, cb, A, vals, dpos, part, flag);
    } else {
        hipLaunchKernelGGL((k_dense_mfma<4, 4>), dim3((unsigned)nblk), dim3(64), 0, s, k, ncols, nd, cb, A, vals, dpos, part, flag);
    }
    const int nfold = dense_rows_fold(ndblocks);
    hipLaunchKernelGGL(k_dense_fold, dim3((unsigned)(nfold * nd)), dim3(64), 0, s, k, nd, ndblocks, (ndblocks + nfold - 1) / nfold, part,
                       part + (size_t)ndblocks * (size_t)nd * (size_t)k);
    return hipGetLastError();
}

}  // namespace bm
