// Builds the row-binned plan on the device: row histogram, heavy-row ranking, one stable
// radix sort of (panel,row) keys, segment boundaries by scan. Integer work only; the build is
// paid once per sparsity pattern and reused by every A*^S / row-sum call on it.
#include "plan.hpp"
#include "common.hpp"
#include "kernels.hpp"
#include "scan.hpp"
#include "workspace.hpp"
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>
#include <rocprim/iterator/counting_iterator.hpp>
#include <rocprim/iterator/transform_iterator.hpp>
#include <mutex>
#include <initializer_list>
#include <new>
#include <vector>

namespace bm {
namespace {

// Carves 256-byte aligned pieces out of one allocation.
struct Arena {
    char* base = nullptr;
    size_t used = 0;
    static size_t round(size_t b) { return (b + 255) & ~size_t(255); }
    template <typename T> T* take(size_t count) {
        T* p = base ? reinterpret_cast<T*>(base + used) : nullptr;
        used += round(sizeof(T) * (count ? count : 1));
        return p;
    }
};

// Build temporaries up to option "plan_keep_mb" (4096 MiB: what a 100 M-nonzero pattern needs) stay in the
// library's workspace for the next build - a caller that meets a new pattern with every minibatch builds a plan
// per call, and allocating and freeing 3.7 GB each time costs 0.9 of its 6.5 ms; larger ones are given back at
// once. bidmat_release_caches frees the kept area.

// Row histogram. The first HIST_LDS_ROWS rows are counted in a per-workgroup LDS copy that is
// flushed once at the end (popular rows tend to carry small indices in count-sorted vocabularies,
// and even when they do not this only costs the flush); all other rows go straight to global
// integer atomics. The counts do not depend on the order of the increments.
// The counts only steer choices that do not change any result (which rows are cut by panels, whether
// the columns get a class ordering, which rows count as hot), so large patterns are counted on a
// fixed pseudo-random eighth of their 256-nonzero chunks: sample = 8 keeps chunk ch when the top three
// bits of ch * 0x9E3779B1 are zero, and every count is then about an eighth of the true one.
// Row indices are checked here only as far as they are seen; k_make_keys checks every one.
constexpr int HIST_LDS_ROWS = 16384;
constexpr int HIST_SAMPLE = 8;
constexpr long long HIST_SAMPLE_FROM = 16LL << 20;        // nonzeros from which the histogram is sampled
__global__ __launch_bounds__(BM_BLOCK) void k_row_hist(int nnz, int nrows, int sample, const int* __restrict__ ir,
                                                       int* __restrict__ cnt, int* __restrict__ bad) {
    __shared__ int local[HIST_LDS_ROWS];
    for (int i = threadIdx.x; i < HIST_LDS_ROWS; i += BM_BLOCK) local[i] = 0;
    __syncthreads();
    const long long nchunks = ((long long)nnz + BM_BLOCK - 1) / BM_BLOCK;
    for (long long ch = blockIdx.x; ch < nchunks; ch += gridDim.x) {
        if (sample > 1 && (((unsigned)ch * 0x9E3779B1u) >> 29) != 0u) continue;
        const long long j = ch * BM_BLOCK + threadIdx.x;
        if (j >= nnz) continue;
        const int r = ir[j];
        if (r < 0 || r >= nrows) *bad = 1;
        else if (r < HIST_LDS_ROWS) atomicAdd(&local[r], 1);
        else atomicAdd(&cnt[r], 1);
    }
    __syncthreads();
    const int lim = nrows < HIST_LDS_ROWS ? nrows : HIST_LDS_ROWS;
    for (int i = threadIdx.x; i < lim; i += BM_BLOCK) {
        const int v = local[i];
        if (v) atomicAdd(&cnt[i], v);
    }
}

__global__ __launch_bounds__(BM_BLOCK) void k_heavy_flag(int nrows, const int* __restrict__ cnt, int thresh,
                                                         int* __restrict__ flag) {
    const long long r = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (r < nrows) flag[r] = cnt[r] >= thresh ? 1 : 0;
}

// hrow[hrank[r]] = r for heavy rows; flag[r] becomes the row's code for the key kernel: its
// heavy rank, or -1 for a light row (one lookup per nonzero instead of two).
__global__ __launch_bounds__(BM_BLOCK) void k_heavy_rows(int nrows, int* __restrict__ flag,
                                                         const int* __restrict__ hrank, int* __restrict__ hrow) {
    const long long r = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (r >= nrows) return;
    if (flag[r]) {
        const int h = hrank[r];
        hrow[h] = (int)r;
        flag[r] = h;
    } else {
        flag[r] = -1;
    }
}

// 16 lanes per column: key of every nonzero, and its (column, original position) as the value
// that is sorted along with it.
__global__ __launch_bounds__(BM_BLOCK) void k_make_keys(int ncols, int nrows, const int* __restrict__ jc,
                                                        const int* __restrict__ ir, const int* __restrict__ hcode,
                                                        int nheavy, int npanels,
                                                        int panel_cols, int p8, unsigned* __restrict__ keys,
                                                        unsigned long long* __restrict__ colpos, int* __restrict__ bad) {
    const long long t = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long c = t >> 4;
    const int l = (int)(t & 15);
    if (c >= ncols) return;
    const int s = jc[c], e = jc[c + 1];
    // panels are ordered by the XCD that will own them: panel p -> slot (p % 8) * p8 + p / 8
    const unsigned praw = (unsigned)(c / panel_cols);
    const unsigned panel = (praw & 7u) * (unsigned)p8 + (praw >> 3);
    const unsigned light_base = 8u * (unsigned)p8 * (unsigned)nheavy;
    (void)npanels;
    // four nonzeros per lane and step: the row loads, then the dependent code lookups, then the stores
    constexpr int UN = 4;
    for (int j0 = s + l; j0 < e; j0 += 16 * UN) {
        int r[UN], h[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int j = j0 + 16 * u;
            r[u] = j < e ? ir[j] : 0;
            if ((unsigned)r[u] >= (unsigned)nrows) { *bad = 1; r[u] = 0; }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) h[u] = hcode[r[u]];             // heavy rank, or -1
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int j = j0 + 16 * u;
            if (j < e) {
                keys[j] = h[u] >= 0 ? panel * (unsigned)nheavy + (unsigned)h[u] : light_base + (unsigned)r[u];
                colpos[j] = ((unsigned long long)(unsigned)c << 32) | (unsigned)j;   // travels with the key
            }
        }
    }
}

// 1 where a segment starts in the sorted key sequence: at a new key and every seglen positions.
// Position n (one past the end) counts as 0, so an exclusive scan over n+1 positions ends with the
// number of segments.
struct SegmentStart {
    const unsigned* keys;
    unsigned n;
    unsigned seglen;
    __device__ __forceinline__ bool at(unsigned p) const {
        return p == 0 || keys[p] != keys[p - 1] || (p % seglen) == 0;
    }
    __device__ __forceinline__ int operator()(unsigned p) const { return (p < n && at(p)) ? 1 : 0; }
};

// Column and original position of every nonzero in plan order; segment tables at the flagged
// positions.
__global__ __launch_bounds__(BM_BLOCK) void k_emit(int nnz, const unsigned* __restrict__ keys,
                                                   const unsigned long long* __restrict__ colpos,
                                                   SegmentStart starts, const int* __restrict__ segidx,
                                                   const int* __restrict__ hrow, int nheavy, int p8,
                                                   int* __restrict__ pc, int* __restrict__ perm,
                                                   int* __restrict__ segstart,
                                                   unsigned* __restrict__ segrow, int* __restrict__ segid,
                                                   unsigned char* __restrict__ segclass) {
    long long p = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    const unsigned per_xcd = (unsigned)p8 * (unsigned)nheavy;     // keys per XCD group
    const unsigned light_base = 8u * per_xcd;
    for (; p < nnz; p += stride) {
        const unsigned long long cp = colpos[p];
        pc[p] = (int)(cp >> 32);
        perm[p] = (int)(cp & 0xffffffffULL);
        if (starts.at((unsigned)p)) {
            const int sidx = segidx[p];
            const unsigned key = keys[p];
            segstart[sidx] = (int)p;
            segrow[sidx] = key >= light_base ? key - light_base : (unsigned)hrow[key % (unsigned)nheavy];
            segid[sidx] = sidx;
            segclass[sidx] = (unsigned char)(key >= light_base ? 8 : (int)(key / per_xcd));
        }
    }
}

// Segments are sorted by key, so their XCD class is non-decreasing: class c starts at the first
// segment whose class is >= c. start[0..8] must be preset to nseg.
__global__ __launch_bounds__(BM_BLOCK) void k_class_bounds(int nseg, const unsigned char* __restrict__ segclass,
                                                           int* __restrict__ start) {
    const long long s = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (s >= nseg) return;
    const int cls = segclass[s];
    const int prev = s == 0 ? -1 : (int)segclass[s - 1];
    for (int c = prev + 1; c <= cls; ++c) start[c] = (int)s;
}

// One wavefront per column: counts the column's nonzeros per bucket, bucket = 2 * (row & 7) + (0 if the
// row is one of its class's hot rows, else 1), then writes them out bucket by bucket, keeping the
// stored order inside a bucket. cptr[16*c + b] = start of bucket b of column c; the last entry closes
// the last column. For a hot row cir holds its rank among the hot rows of its class, otherwise the row.
// HOT == false: no hot rows, the even buckets stay empty and only the eight classes are counted.
template <bool HOT>
__global__ __launch_bounds__(BM_BLOCK) void k_class_partition(int ncols, int nrows, const int* __restrict__ ir,
                                                              const int* __restrict__ jc,
                                                              const int* __restrict__ hotrank, int cshift,
                                                              int* __restrict__ cir,
                                                              int* __restrict__ cperm, int* __restrict__ cptr,
                                                              int* __restrict__ maxlen, int* __restrict__ bad) {
    constexpr int NB = HOT ? 16 : 8;
    const int lane = threadIdx.x & 63;
    const long long c = (long long)blockIdx.x * BM_WAVES_PER_BLOCK + wave_uniform(threadIdx.x >> 6);
    if (c >= ncols) return;
    const int s = jc[c], e = jc[c + 1];
    const unsigned long long below = (1ULL << lane) - 1ULL;
    if (e - s <= 4 * 64) {
        // The usual column: all its row indices are requested at once and stay in registers, so the wave waits
        // for memory once (twice with hot rows) instead of once per 64 nonzeros and per pass.
        int r[4], hr[4], bucket[4];
        bool valid[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int j = s + u * 64 + lane;
            valid[u] = j < e;
            r[u] = valid[u] ? ir[j] : 0;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if ((unsigned)r[u] >= (unsigned)nrows) *bad = 1;
            hr[u] = (HOT && valid[u] && (unsigned)r[u] < (unsigned)nrows) ? hotrank[r[u]] : -1;
        }
        // Bucket numbers are NBITS bits wide: one ballot per bit and chunk; every bucket's lanes then follow from
        // the ballots by scalar mask arithmetic (counts), and a lane finds the lanes before it in its own bucket
        // by selecting each ballot or its complement.
        constexpr int NBITS = HOT ? 4 : 3;
        unsigned long long vm[4], bm[4][NBITS];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int cls = (r[u] >> cshift) & 7;
            bucket[u] = HOT ? 2 * cls + (hr[u] < 0 ? 1 : 0) : cls;
            vm[u] = __ballot(valid[u]);
#pragma unroll
            for (int b = 0; b < NBITS; ++b) bm[u][b] = __ballot(valid[u] && ((bucket[u] >> b) & 1));
        }
        int cntx[4][NB];                               // lanes of chunk u in bucket x (wave-uniform)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
#pragma unroll
            for (int x = 0; x < NB; ++x) {
                unsigned long long m = vm[u];
#pragma unroll
                for (int b = 0; b < NBITS; ++b) m &= ((x >> b) & 1) ? bm[u][b] : ~bm[u][b];
                cntx[u][x] = __popcll(m);
            }
        }
        int base[NB], run = 0;
#pragma unroll
        for (int x = 0; x < NB; ++x) {
            base[x] = run;
#pragma unroll
            for (int u = 0; u < 4; ++u) run += cntx[u][x];
        }
        if (lane < 16) {
            const int which = HOT ? lane : lane >> 1;
            int bb = 0;
#pragma unroll
            for (int x = 0; x < NB; ++x) bb = (which == x) ? base[x] : bb;
            cptr[c * 16 + lane] = s + bb;
        }
        if (c == ncols - 1 && lane == 0) cptr[(long long)ncols * 16] = e;
        if (lane == 0 && e - s > __hip_atomic_load(maxlen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(maxlen, e - s);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            unsigned long long peers = vm[u];
            int mybase = 0;
#pragma unroll
            for (int b = 0; b < NBITS; ++b) peers &= ((bucket[u] >> b) & 1) ? bm[u][b] : ~bm[u][b];
#pragma unroll
            for (int x = 0; x < NB; ++x) mybase = (bucket[u] == x) ? base[x] : mybase;
            if (valid[u]) {
                const int dest = s + mybase + __popcll(peers & below);
                cir[dest] = hr[u] < 0 ? r[u] : hr[u];
                cperm[dest] = s + u * 64 + lane;
            }
#pragma unroll
            for (int x = 0; x < NB; ++x) base[x] += cntx[u][x];
        }
        return;
    }
    int cnt[NB];
#pragma unroll
    for (int x = 0; x < NB; ++x) cnt[x] = 0;
    for (int j0 = s; j0 < e; j0 += 64) {
        const int j = j0 + lane;
        const bool valid = j < e;
        const int r = valid ? ir[j] : 0;
        if ((unsigned)r >= (unsigned)nrows) *bad = 1;           // a row outside the matrix: the build fails
        const int hr = (HOT && valid && (unsigned)r < (unsigned)nrows) ? hotrank[r] : -1;
        const int cls = (r >> cshift) & 7;
        const int bucket = HOT ? 2 * cls + (hr < 0 ? 1 : 0) : cls;
#pragma unroll
        for (int x = 0; x < NB; ++x) cnt[x] += __popcll(__ballot(valid && bucket == x));
    }
    int base[NB], run = 0;
#pragma unroll
    for (int x = 0; x < NB; ++x) { base[x] = run; run += cnt[x]; }
    if (lane < 16) {
        // table entry `lane` = start of bucket `lane` of the 16; without hot rows bucket 2x is empty and starts
        // where bucket 2x+1 (class x) does
        const int which = HOT ? lane : lane >> 1;
        int bb = 0;
#pragma unroll
        for (int x = 0; x < NB; ++x) bb = (which == x) ? base[x] : bb;
        cptr[c * 16 + lane] = s + bb;
    }
    if (c == ncols - 1 && lane == 0) cptr[(long long)ncols * 16] = e;
    // every column would hit the same address: only columns longer than the longest seen so far do
    // (the plain read may be stale, which only costs a redundant atomic)
    if (lane == 0 && e - s > __hip_atomic_load(maxlen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(maxlen, e - s);
    for (int j0 = s; j0 < e; j0 += 64) {
        const int j = j0 + lane;
        const bool valid = j < e;
        const int r = valid ? ir[j] : 0;
        const int hr = (HOT && valid && (unsigned)r < (unsigned)nrows) ? hotrank[r] : -1;
        const int cls = (r >> cshift) & 7;
        const int bucket = HOT ? 2 * cls + (hr < 0 ? 1 : 0) : cls;
        int dest = -1;
#pragma unroll
        for (int x = 0; x < NB; ++x) {
            const bool mine = valid && bucket == x;
            const unsigned long long m = __ballot(mine);
            if (mine) dest = s + base[x] + __popcll(m & below);
            base[x] += __popcll(m);
        }
        if (valid) { cir[dest] = hr < 0 ? r : hr; cperm[dest] = j; }
    }
}

__global__ __launch_bounds__(BM_BLOCK) void k_iota(int n, int* __restrict__ out) {
    const long long i = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (i < n) out[i] = (int)i;
}

// hotrank[rows[i]] = ranks[i]
__global__ __launch_bounds__(BM_BLOCK) void k_scatter_rank(int n, const int* __restrict__ rows,
                                                           const int* __restrict__ ranks, int* __restrict__ hotrank) {
    const int i = blockIdx.x * BM_BLOCK + threadIdx.x;
    if (i < n) hotrank[rows[i]] = ranks[i];
}

// out[0] = number of nonzeros in the n1 most frequent rows, out[1] = in the n8 most frequent rows;
// sorted = row counts in descending order. One workgroup, integer sums.
__global__ __launch_bounds__(BM_BLOCK) void k_top_coverage(int nrows, const int* __restrict__ sorted, int n1, int n8,
                                                           unsigned long long* __restrict__ out) {
    __shared__ unsigned long long s1[BM_BLOCK], s8[BM_BLOCK];
    unsigned long long a = 0, b = 0;
    for (int i = threadIdx.x; i < nrows && i < n8; i += BM_BLOCK) {
        const unsigned long long v = (unsigned long long)sorted[i];
        if (i < n1) a += v;
        b += v;
    }
    s1[threadIdx.x] = a; s8[threadIdx.x] = b;
    __syncthreads();
    for (int d = BM_BLOCK / 2; d > 0; d >>= 1) {
        if ((int)threadIdx.x < d) { s1[threadIdx.x] += s1[threadIdx.x + d]; s8[threadIdx.x] += s8[threadIdx.x + d]; }
        __syncthreads();
    }
    if (threadIdx.x == 0) { out[0] = s1[0]; out[1] = s8[0]; }
}

// Nonzeros in the N most frequent rows without sorting the counts: rows are binned by count (exactly below
// 2048, above that by the exponent and six more bits: under 2 % wide), per bin the rows and the sum of their
// counts. k_top_from_bins then walks the bins from the top until N rows are in. The result steers a yes/no
// choice that changes no product, so the small error of the wide bins is of no account.
constexpr int TOPBINS = 2048 + 21 * 64;
__device__ __forceinline__ int count_bin(unsigned c) {
    if (c < 2048u) return (int)c;
    const int e = 31 - __clz((int)c);                       // >= 11
    return 2048 + (e - 11) * 64 + (int)((c >> (e - 6)) & 63u);
}
__global__ __launch_bounds__(BM_BLOCK) void k_count_bins(int nrows, const int* __restrict__ cnt, int* __restrict__ brows,
                                                         unsigned long long* __restrict__ bsum) {
    __shared__ int lr[TOPBINS];
    __shared__ unsigned long long ls[TOPBINS];
    for (int i = threadIdx.x; i < TOPBINS; i += BM_BLOCK) { lr[i] = 0; ls[i] = 0; }
    __syncthreads();
    for (long long r = (long long)blockIdx.x * BM_BLOCK + threadIdx.x; r < nrows; r += (long long)gridDim.x * BM_BLOCK) {
        const unsigned c = (unsigned)cnt[r];
        if (c == 0) continue;
        const int b = count_bin(c);
        atomicAdd(&lr[b], 1);
        atomicAdd(&ls[b], (unsigned long long)c);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < TOPBINS; i += BM_BLOCK) {
        if (lr[i]) { atomicAdd(&brows[i], lr[i]); atomicAdd(&bsum[i], ls[i]); }
    }
}
// out[0], out[1] = nonzeros in the n1 / n8 most frequent rows. One workgroup: every thread takes a run of
// bins (from the top), the runs are scanned, and the thread whose run crosses n1 (n8) rows interpolates inside
// the bin that crosses.
__global__ __launch_bounds__(BM_BLOCK) void k_top_from_bins(const int* __restrict__ brows,
                                                            const unsigned long long* __restrict__ bsum, int n1, int n8,
                                                            unsigned long long* __restrict__ out) {
    constexpr int PER = (TOPBINS + BM_BLOCK - 1) / BM_BLOCK;
    __shared__ long long srows[BM_BLOCK + 1];
    __shared__ unsigned long long ssum[BM_BLOCK + 1];
    const int t = threadIdx.x;
    long long nr[PER];
    unsigned long long sb[PER];
    long long r = 0;
    unsigned long long sm = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int b = TOPBINS - 1 - (t * PER + j);
        nr[j] = b >= 0 ? brows[b] : 0;
        sb[j] = b >= 0 ? bsum[b] : 0ull;
        r += nr[j];
        sm += sb[j];
    }
    srows[t] = r;
    ssum[t] = sm;
    if (t == 0) { out[0] = 0ull; out[1] = 0ull; }
    __syncthreads();
    if (t == 0) {                                   // exclusive scan of 256 pairs in LDS
        long long ar = 0;
        unsigned long long as = 0;
        for (int i = 0; i < BM_BLOCK; ++i) {
            const long long xr = srows[i];
            const unsigned long long xs = ssum[i];
            srows[i] = ar; ssum[i] = as;
            ar += xr; as += xs;
        }
        srows[BM_BLOCK] = ar; ssum[BM_BLOCK] = as;
    }
    __syncthreads();
    long long rows = srows[t];
    unsigned long long sum = ssum[t];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        if (nr[j] > 0) {
#pragma unroll
            for (int which = 0; which < 2; ++which) {
                const long long want = which == 0 ? n1 : n8;
                if (rows < want && rows + nr[j] >= want)
                    out[which] = sum + (unsigned long long)((double)sb[j] * (double)(want - rows) / (double)nr[j]);
            }
        }
        rows += nr[j];
        sum += sb[j];
    }
    if (t == 0) {                                   // fewer rows than asked for: all of them
        if (srows[BM_BLOCK] < n1) out[0] = ssum[BM_BLOCK];
        if (srows[BM_BLOCK] < n8) out[1] = ssum[BM_BLOCK];
    }
}

inline unsigned grid_for(long long n, int maxblocks = 16384) {
    long long b = (n + BM_BLOCK - 1) / BM_BLOCK;
    if (b < 1) b = 1;
    if (b > maxblocks) b = maxblocks;
    return (unsigned)b;
}

inline int bits_for(unsigned long long maxval) {
    int b = 1;
    while (b < 32 && (maxval >> b) != 0) ++b;
    return b;
}

}  // namespace

namespace {
// The plan's memory goes back to the pool of plan blocks (idle by then: plan_free and the failure paths of
// a build synchronise first).
void free_all(std::initializer_list<void**> bufs, hipError_t* e) {
    for (void** b : bufs) {
        if (*b) {
            hipError_t f = pool_free(*b);
            if (f != hipSuccess) *e = f;
            *b = nullptr;
        }
    }
}
template <typename T>
hipError_t plan_alloc(T** p, size_t bytes) {
    hipError_t e;
    *p = static_cast<T*>(pool_alloc(bytes, &e));
    return e;
}
// Frees one half of a plan and marks it absent.
hipError_t drop_rows(bidmat_plan* p) {
    hipError_t e = drop_dense(p);
    free_all({&p->block_nnz, &p->block_seg, (void**)&p->pvals}, &e);
    p->pc = p->perm = p->rowptr = p->segstart = p->segrow = p->rowseg = nullptr;
    p->nseg = p->nheavy = 0;
    for (int& x : p->xcd_start) x = 0;
    p->row_bytes = 0;
    p->sides &= ~PLAN_ROWS;
    return e;
}
hipError_t drop_cols(bidmat_plan* p) {
    hipError_t e = hipSuccess;
    free_all({(void**)&p->ovf, (void**)&p->cir, (void**)&p->cperm, (void**)&p->cptr, (void**)&p->hotrows,
              (void**)&p->cvals, (void**)&p->svals}, &e);
    p->novf = p->ncls = p->hcap = p->maxlen = 0;
    p->col_bytes = 0;
    p->sides &= ~PLAN_COLS;
    return e;
}
}  // namespace

hipError_t plan_free(bidmat_plan* p) {
    if (!p) return hipSuccess;
    (void)hipDeviceSynchronize();            // kernels that still read the plan finish before its blocks can be reused
    hipError_t e = drop_rows(p), f = drop_cols(p);
    delete p;
    return e != hipSuccess ? e : f;
}

namespace {
__global__ __launch_bounds__(BM_BLOCK) void k_permute_values(long long n, const float* __restrict__ data,
                                                             const int* __restrict__ perm, float* __restrict__ out) {
    // tiles of 4 x 256 positions per workgroup: four dependent gathers in flight per thread
    constexpr int UN = 4;
    long long i = (long long)blockIdx.x * (UN * BM_BLOCK) + threadIdx.x;
    const long long stride = (long long)gridDim.x * (UN * BM_BLOCK);
    for (; i < n; i += stride) {
        int ix[UN];
        float v[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) { const long long j = i + u * BM_BLOCK; ix[u] = j < n ? perm[j] : 0; }
#pragma unroll
        for (int u = 0; u < UN; ++u) v[u] = data[ix[u]];
#pragma unroll
        for (int u = 0; u < UN; ++u) { const long long j = i + u * BM_BLOCK; if (j < n) out[j] = v[u]; }
    }
}

hipError_t value_buffer(float** buf, int nnz) {
    if (*buf) return hipSuccess;
    hipError_t e = plan_alloc(buf, sizeof(float) * (size_t)nnz);
    if (e != hipSuccess) { (void)hipGetLastError(); *buf = nullptr; }
    return e;
}
}  // namespace

// Stores the values in the orders the built halves walk: plan order (row side), class order or stored
// order (column side with / without a class ordering).
hipError_t plan_set_values(bidmat_plan* p, const float* data, hipStream_t s) {
    if (p->nnz <= 0) return hipSuccess;
    hipError_t e;
    const dim3 grid(grid_for(((long long)p->nnz + 3) / 4, 8192)), block(BM_BLOCK);
    if (p->sides & PLAN_ROWS) {
        if ((e = value_buffer(&p->pvals, p->nnz)) != hipSuccess) return e;
        hipLaunchKernelGGL(k_permute_values, grid, block, 0, s, (long long)p->nnz, data, p->perm, p->pvals);
        // the dense block of A *^ S reads its values in the layout of its position table
        if ((e = dense_rows_set_values(p, data, s)) != hipSuccess) return e;
    }
    if ((p->sides & PLAN_COLS) && p->ncls == 8) {
        // A*S in passes over row classes and the fused step of DDS read their values in class order
        if ((e = value_buffer(&p->cvals, p->nnz)) != hipSuccess) return e;
        hipLaunchKernelGGL(k_permute_values, grid, block, 0, s, (long long)p->nnz, data, p->cperm, p->cvals);
    } else if (p->sides & PLAN_COLS) {
        // without a class ordering the fused step of DDS reads them in stored order: a plain copy
        if ((e = value_buffer(&p->svals, p->nnz)) != hipSuccess) return e;
        if ((e = hipMemcpyAsync(p->svals, data, sizeof(float) * (size_t)p->nnz, hipMemcpyDeviceToDevice, s)) != hipSuccess) return e;
    }
    return hipGetLastError();
}

namespace {

// Builds the row-class ordering of the columns (see plan.hpp). `bad` is set when a row index lies
// outside the matrix.
hipError_t plan_build_classes(bidmat_plan* plan, const int* ir, const int* jc, const int* hotrank, int* bad, hipStream_t s) {
    const int ncols = plan->ncols, nnz = plan->nnz;
    if (ncols <= 0 || nnz <= 0 || (long long)ncols * 16 + 1 > 0x7fffffffLL) return hipSuccess;
    hipError_t e;
    const size_t nsub = (size_t)ncols * 16 + 1;
    if ((e = plan_alloc(&plan->cptr, sizeof(int) * (nsub + 1))) != hipSuccess) return e;
    if ((e = plan_alloc(&plan->cir, sizeof(int) * (size_t)nnz)) != hipSuccess) return e;
    if ((e = plan_alloc(&plan->cperm, sizeof(int) * (size_t)nnz)) != hipSuccess) return e;
    int* d_maxlen = plan->cptr + nsub;                   // one spare int behind the table
    if ((e = fill_i32(d_maxlen, 1, 0, s)) != hipSuccess) return e;
    const long long nblk = ((long long)ncols + BM_WAVES_PER_BLOCK - 1) / BM_WAVES_PER_BLOCK;
    if (hotrank != nullptr)
        hipLaunchKernelGGL(k_class_partition<true>, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, ncols, plan->nrows, ir, jc, hotrank, plan->cshift,
                           plan->cir, plan->cperm, plan->cptr, d_maxlen, bad);
    else
        hipLaunchKernelGGL(k_class_partition<false>, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, ncols, plan->nrows, ir, jc, hotrank, plan->cshift,
                           plan->cir, plan->cperm, plan->cptr, d_maxlen, bad);
    if ((e = hipGetLastError()) != hipSuccess) return e;
    if ((e = hipMemcpy(&plan->maxlen, d_maxlen, sizeof(int), hipMemcpyDeviceToHost)) != hipSuccess) return e;
    plan->ncls = 8;
    plan->col_bytes += sizeof(int) * (nsub + 1 + 2 * (size_t)nnz);
    return hipSuccess;
}

#define PB_CHECK(expr)                                          \
    do {                                                        \
        hipError_t _e = (expr);                                 \
        if (_e != hipSuccess) return _e;                        \
    } while (0)

// Temporaries of one build, carved out of the library's workspace.
struct BuildTmp {
    int *cnt = nullptr, *hflag = nullptr, *hrank = nullptr, *hrow = nullptr, *crank = nullptr, *scantmp = nullptr, *bad = nullptr;
    unsigned *keys_in = nullptr, *keys_out = nullptr;
    unsigned long long *colpos_in = nullptr, *colpos_out = nullptr;
    char* sorttmp = nullptr;
    size_t sort_bytes = 0, arena_bytes = 0;
    int sample = 1;
};

// Column side: the overflow-segment table of the columns (kept only when a column is longer than
// seglen) and, where the pattern promises a gain, the row-class ordering. cnt: the row histogram.
hipError_t build_cols(bidmat_plan* plan, const int* ir, const int* jc, const BuildTmp& t, hipStream_t s) {
    const int nrows = plan->nrows, ncols = plan->ncols, nnz = plan->nnz;
    const int k_hint = plan->k_hint;
    plan->cshift = opt_class_shift() >= 0 ? opt_class_shift() : 0;
    plan->col_seglen = opt_seglen();
    {
        int* tbl = nullptr;
        PB_CHECK(build_overflow_table(ncols, nnz, jc, plan->col_seglen, &tbl, s));
        if (tbl) {
            int n = 0;
            PB_CHECK(hipMemcpy(&n, tbl + ncols, sizeof(int), hipMemcpyDeviceToHost));
            if (n > 0) {
                PB_CHECK(plan_alloc(&plan->ovf, sizeof(int) * ((size_t)ncols + 1)));
                PB_CHECK(hipMemcpy(plan->ovf, tbl, sizeof(int) * ((size_t)ncols + 1), hipMemcpyDeviceToDevice));
                plan->novf = n;
                plan->col_bytes += sizeof(int) * ((size_t)ncols + 1);
            }
        }
    }
    // Column classes for DDS and A*S: worth it when one L2 (4 MiB) holds clearly fewer of the gathered
    // rows' nonzeros than eight L2s with disjoint rows would. The rows are sorted by count (descending)
    // and the nonzeros of the top n1 and top 8*n1 rows compared, n1 = rows of the operand per L2. The
    // same ranking names every class's hot rows, the ones the DDS kernel keeps in LDS.
    const int mode = opt_col_classes();       // -1 auto, 0 never, 1 always
    bool want = mode == 1;
    // Measured: 100 M nonzeros, Zipf(1.1) rows, k = 256: 5.53 -> 4.78 ms. With rows of 512 bytes
    // (k = 128, 400 M nonzeros, Zipf(1.05)) the class-ordered kernel alone is bound by its
    // instruction stream and loses (14.8 -> 16.1 ms), but wins with each class's most frequent rows
    // in LDS (13.75 ms): below k = 256 the hot rows are switched on with the classes.
    const bool candidate = mode == 1 || (mode < 0 && ncols > 0 && nnz / ncols >= 64 &&
                                         (long long)nrows * 4 * k_hint > (8LL << 20));
    int* hotrank = nullptr;
    // hot rows per class kept in LDS. -1 (default): what the LDS budget holds when k_hint < 256, none
    // from k = 256 on, where they were measured to change nothing (4.78 ms without, 4.85 ms with
    // 128 rows per class: the 1024-thread persistent workgroups that share the LDS rows cost
    // what the rows save).
    long long hcap = opt_class_hot();
    if (hcap < 0) hcap = k_hint < 256 ? (long long)(dds_classed_lds_budget() / (4 * (size_t)k_hint)) : 0;
    if (hcap > 1024) hcap = 1024;
    const long long n1 = (4LL << 20) / (4LL * k_hint);
    if (candidate && (size_t)nrows <= (size_t)nnz && hcap == 0) {
        // no list of hot rows to make: the coverage of the top rows comes from a histogram of the counts
        int* brows = reinterpret_cast<int*>(t.colpos_in);
        unsigned long long* bsum = t.colpos_out + 8;
        unsigned long long* cov = t.colpos_out;
        PB_CHECK(fill_i32(brows, TOPBINS, 0, s));
        PB_CHECK(fill_i32(reinterpret_cast<int*>(bsum), 2 * TOPBINS, 0, s));
        hipLaunchKernelGGL(k_count_bins, dim3(grid_for(nrows, 256)), dim3(BM_BLOCK), 0, s, nrows, t.cnt, brows, bsum);
        hipLaunchKernelGGL(k_top_from_bins, dim3(1), dim3(BM_BLOCK), 0, s, brows, bsum, (int)(n1 < nrows ? n1 : nrows),
                           (int)(8 * n1 < nrows ? 8 * n1 : nrows), cov);
        unsigned long long h[2] = {0, 0};
        PB_CHECK(hipMemcpy(h, cov, sizeof(h), hipMemcpyDeviceToHost));
        // at least a tenth of all gathers must move from "misses L2" to "hits L2"
        if (mode < 0) want = (double)(h[1] - h[0]) * t.sample >= 0.10 * (double)nnz;
    } else if (candidate && (size_t)nrows <= (size_t)nnz) {
        int* iota = reinterpret_cast<int*>(t.keys_in);
        unsigned* cnt_sorted = t.keys_out;
        int* rows_sorted = reinterpret_cast<int*>(t.colpos_in);
        unsigned long long* cov = reinterpret_cast<unsigned long long*>(t.colpos_out);
        size_t tb = 0;
        PB_CHECK(rocprim::radix_sort_pairs_desc(nullptr, tb, reinterpret_cast<unsigned*>(t.cnt), cnt_sorted, iota, rows_sorted,
                                                (size_t)nrows, 0, 32, s));
        if (tb <= t.sort_bytes) {
            hipLaunchKernelGGL(k_iota, dim3(grid_for(nrows, 1 << 30)), dim3(BM_BLOCK), 0, s, nrows, iota);
            PB_CHECK(rocprim::radix_sort_pairs_desc(t.sorttmp, tb, reinterpret_cast<unsigned*>(t.cnt), cnt_sorted, iota, rows_sorted,
                                                    (size_t)nrows, 0, 32, s));
            hipLaunchKernelGGL(k_top_coverage, dim3(1), dim3(BM_BLOCK), 0, s, nrows, reinterpret_cast<const int*>(cnt_sorted),
                               (int)(n1 < nrows ? n1 : nrows), (int)(8 * n1 < nrows ? 8 * n1 : nrows), cov);
            unsigned long long h[2] = {0, 0};
            PB_CHECK(hipMemcpy(h, cov, sizeof(h), hipMemcpyDeviceToHost));
            // at least a tenth of all gathers must move from "misses L2" to "hits L2"
            if (mode < 0) want = (double)(h[1] - h[0]) * t.sample >= 0.10 * (double)nnz;
            if (want) {
                const int ntop = (int)(8 * hcap < nrows ? 8 * hcap : nrows);
                std::vector<int> top((size_t)ntop), cnts((size_t)ntop);
                PB_CHECK(hipMemcpy(top.data(), rows_sorted, sizeof(int) * (size_t)ntop, hipMemcpyDeviceToHost));
                PB_CHECK(hipMemcpy(cnts.data(), cnt_sorted, sizeof(int) * (size_t)ntop, hipMemcpyDeviceToHost));
                std::vector<int> hotrows((size_t)(8 * hcap), -1), rows, ranks;
                int filled[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (int i = 0; i < ntop; ++i) {
                    const int r = top[i], x = (r >> plan->cshift) & 7;
                    if (cnts[i] < 2 || filled[x] >= hcap) continue;      // a row used once gains nothing
                    hotrows[(size_t)x * hcap + filled[x]] = r;
                    rows.push_back(r);
                    ranks.push_back(filled[x]++);
                }
                if (!rows.empty()) {
                    PB_CHECK(plan_alloc(&plan->hotrows, sizeof(int) * hotrows.size()));
                    PB_CHECK(hipMemcpy(plan->hotrows, hotrows.data(), sizeof(int) * hotrows.size(), hipMemcpyHostToDevice));
                    plan->hcap = (int)hcap;
                    plan->col_bytes += sizeof(int) * hotrows.size();
                    hotrank = t.crank;
                    PB_CHECK(fill_i32(hotrank, nrows, -1, s));
                    // the two small lists ride in the (still free) coverage area
                    int* d_rows = reinterpret_cast<int*>(t.colpos_out);
                    int* d_ranks = d_rows + rows.size();
                    PB_CHECK(hipMemcpy(d_rows, rows.data(), sizeof(int) * rows.size(), hipMemcpyHostToDevice));
                    PB_CHECK(hipMemcpy(d_ranks, ranks.data(), sizeof(int) * ranks.size(), hipMemcpyHostToDevice));
                    hipLaunchKernelGGL(k_scatter_rank, dim3(grid_for((long long)rows.size(), 1 << 30)), dim3(BM_BLOCK), 0, s,
                                       (int)rows.size(), d_rows, d_ranks, hotrank);
                }
            }
        }
    }
    if (want) PB_CHECK(plan_build_classes(plan, ir, jc, hotrank, t.bad, s));
    return hipGetLastError();
}

// Ranks the heavy rows (those the row side cuts by column panels): t.hflag becomes every row's code (heavy
// rank, or -1), t.hrow the row of every rank. Returns their number in *nheavy_out.
hipError_t detect_heavy(bidmat_plan* plan, const BuildTmp& t, int p8, int* nheavy_out, hipStream_t s) {
    const int nrows = plan->nrows;
    int nheavy = 0;
    int h2[2] = {0, 0};                                  // {number of heavy rows, bad-index flag}
    if (plan->npanels >= 2) {
        long long thresh = (long long)plan->npanels * opt_heavy_min();
        if (thresh > 0x7fffffffLL) thresh = 0x7fffffffLL;
        thresh = (thresh + t.sample - 1) / t.sample;
        hipLaunchKernelGGL(k_heavy_flag, dim3(grid_for(nrows, 1 << 30)), dim3(BM_BLOCK), 0, s, nrows, t.cnt, (int)thresh, t.hflag);
        // the scan writes hrank[0..nrows]; the bad-index flag sits behind it
        PB_CHECK(scan_exclusive_i32(t.hflag, t.hrank, nrows, t.scantmp, s));
    }
    PB_CHECK(hipMemcpy(h2, t.hrank + nrows, sizeof(h2), hipMemcpyDeviceToHost));
    if (h2[1]) return hipErrorInvalidValue;
    if (plan->npanels >= 2) {
        nheavy = h2[0];
        // keys must fit 32 bits
        if (8ULL * (unsigned long long)p8 * (unsigned long long)nheavy + (unsigned long long)nrows > 0xffffffffULL) nheavy = 0;
    }
    if (nheavy == 0) {
        PB_CHECK(fill_i32(t.hflag, nrows, -1, s));        // every row is light
    } else {
        hipLaunchKernelGGL(k_heavy_rows, dim3(grid_for(nrows, 1 << 30)), dim3(BM_BLOCK), 0, s, nrows, t.hflag, t.hrank, t.hrow);
    }
    *nheavy_out = nheavy;
    return hipGetLastError();
}

// Row side through one stable radix sort (rocPRIM) of (panel,row) keys: the reference the binned builder
// (plan_rows.hip) is tested against, and the way out when there are more heavy rows than its LDS bins hold.
hipError_t build_rows_sorted(bidmat_plan* plan, const int* ir, const int* jc, const BuildTmp& t, int nheavy, int p8, hipStream_t s) {
    const int nrows = plan->nrows, ncols = plan->ncols, nnz = plan->nnz;
    const int rbits = bits_for((unsigned long long)nrows);
    // temporaries sized by the nonzeros
    unsigned *keys_in = nullptr, *keys_out = nullptr;
    unsigned long long *colpos_in = nullptr, *colpos_out = nullptr;
    int *segidx = nullptr, *class_count = nullptr;
    unsigned char* segclass = nullptr;
    char* sorttmp = nullptr;
    size_t sort_bytes = 0;
    {
        const unsigned long long maxkey_bound = 8ULL * (unsigned long long)p8 * (unsigned long long)nrows + (unsigned long long)nrows;
        size_t b1 = 0, b2 = 0, b3 = 0;
        PB_CHECK(rocprim::radix_sort_pairs(nullptr, b1, (unsigned*)nullptr, (unsigned*)nullptr, (unsigned long long*)nullptr,
                                           (unsigned long long*)nullptr, (size_t)nnz, 0, bits_for(maxkey_bound > 0xffffffffULL ? 0xffffffffULL : maxkey_bound), s));
        PB_CHECK(rocprim::radix_sort_pairs(nullptr, b2, (unsigned*)nullptr, (unsigned*)nullptr, (int*)nullptr,
                                           (int*)nullptr, (size_t)nnz, 0, rbits, s));
        auto in = rocprim::make_transform_iterator(rocprim::make_counting_iterator<unsigned>(0u),
                                                   SegmentStart{nullptr, (unsigned)nnz, 1u});
        PB_CHECK(rocprim::exclusive_scan(nullptr, b3, in, (int*)nullptr, 0, (size_t)nnz + 1, rocprim::plus<int>(), s));
        sort_bytes = b1 > b2 ? b1 : b2;
        if (b3 > sort_bytes) sort_bytes = b3;
    }
    Arena tmp;
    for (int pass = 0; pass < 2; ++pass) {
        tmp.used = 0;
        class_count = tmp.take<int>(9);
        keys_in = tmp.take<unsigned>((size_t)nnz);               // later: ids of the segments
        keys_out = tmp.take<unsigned>((size_t)nnz);
        colpos_in = tmp.take<unsigned long long>((size_t)nnz);   // later: segment rows in sorted order
        colpos_out = tmp.take<unsigned long long>((size_t)nnz);
        segidx = tmp.take<int>((size_t)nnz + 1);
        segclass = tmp.take<unsigned char>((size_t)nnz);
        sorttmp = tmp.take<char>(sort_bytes);
        if (pass == 0) {
            hipError_t werr;
            tmp.base = static_cast<char*>(ws_get(WS_PLAN_ROWS_A, tmp.used, &werr, s));
            if (!tmp.base) return werr;
        }
    }

    // keys + stable radix sort
    {
        long long nblk = ((long long)ncols * 16 + BM_BLOCK - 1) / BM_BLOCK;
        hipLaunchKernelGGL(k_make_keys, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, ncols, nrows, jc, ir,
                           t.hflag, nheavy, plan->npanels, plan->panel_cols, p8, keys_in, colpos_in, t.bad);
    }
    const unsigned long long maxkey = 8ULL * (unsigned long long)p8 * nheavy + (unsigned long long)nrows;
    const int end_bit = bits_for(maxkey);
    {
        size_t tmp_bytes = 0;
        PB_CHECK(rocprim::radix_sort_pairs(nullptr, tmp_bytes, keys_in, keys_out, colpos_in, colpos_out, (size_t)nnz, 0, end_bit, s));
        if (tmp_bytes > sort_bytes) return hipErrorOutOfMemory;
        PB_CHECK(rocprim::radix_sort_pairs(sorttmp, tmp_bytes, keys_in, keys_out, colpos_in, colpos_out, (size_t)nnz, 0, end_bit, s));
    }

    // segment boundaries
    const SegmentStart starts{keys_out, (unsigned)nnz, (unsigned)plan->seglen};
    {
        auto in = rocprim::make_transform_iterator(rocprim::make_counting_iterator<unsigned>(0u), starts);
        size_t tmp_bytes = 0;
        PB_CHECK(rocprim::exclusive_scan(nullptr, tmp_bytes, in, segidx, 0, (size_t)nnz + 1, rocprim::plus<int>(), s));
        if (tmp_bytes > sort_bytes) return hipErrorOutOfMemory;
        PB_CHECK(rocprim::exclusive_scan(sorttmp, tmp_bytes, in, segidx, 0, (size_t)nnz + 1, rocprim::plus<int>(), s));
    }
    int nseg = 0;
    PB_CHECK(hipMemcpy(&nseg, segidx + nnz, sizeof(int), hipMemcpyDeviceToHost));
    {
        int badv = 0;                                    // k_make_keys has seen every row index by now
        PB_CHECK(hipMemcpy(&badv, t.bad, sizeof(int), hipMemcpyDeviceToHost));
        if (badv) return hipErrorInvalidValue;
    }
    plan->nseg = nseg;

    // memory the plan keeps, part 2: the segment tables
    {
        Arena own;
        for (int pass = 0; pass < 2; ++pass) {
            own.used = 0;
            plan->segstart = own.take<int>((size_t)nseg + 1);
            plan->segrow = own.take<int>((size_t)nseg);
            plan->rowseg = own.take<int>((size_t)nseg);
            if (pass == 0) {
                PB_CHECK(plan_alloc(&plan->block_seg, own.used));
                own.base = static_cast<char*>(plan->block_seg);
                plan->row_bytes += own.used;
            }
        }
    }
    // the sort's inputs are dead by now: their space holds the segment ids and the sorted rows
    int* const segid = reinterpret_cast<int*>(keys_in);
    unsigned* const segrow_sorted = reinterpret_cast<unsigned*>(colpos_in);
    unsigned* const segrow_u = reinterpret_cast<unsigned*>(plan->segrow);
    PB_CHECK(fill_i32(class_count, 9, nseg, s));
    hipLaunchKernelGGL(k_emit, dim3(grid_for(nnz)), dim3(BM_BLOCK), 0, s, nnz, keys_out, colpos_out,
                       starts, segidx, t.hrow, nheavy > 0 ? nheavy : 1,
                       nheavy > 0 ? p8 : 0, plan->pc, plan->perm, plan->segstart, segrow_u, segid, segclass);
    PB_CHECK(fill_i32(plan->segstart + nseg, 1, nnz, s));
    hipLaunchKernelGGL(k_class_bounds, dim3(grid_for(nseg, 1 << 30)), dim3(BM_BLOCK), 0, s, nseg, segclass, class_count);
    PB_CHECK(hipMemcpy(plan->xcd_start, class_count, sizeof(int) * 9, hipMemcpyDeviceToHost));

    // a row's segments, in ascending segment order (stable sort by row)
    {
        size_t tmp_bytes = 0;
        PB_CHECK(rocprim::radix_sort_pairs(nullptr, tmp_bytes, segrow_u, segrow_sorted, segid, plan->rowseg, (size_t)nseg, 0, rbits, s));
        if (tmp_bytes > sort_bytes) return hipErrorOutOfMemory;
        PB_CHECK(rocprim::radix_sort_pairs(sorttmp, tmp_bytes, segrow_u, segrow_sorted, segid, plan->rowseg, (size_t)nseg, 0, rbits, s));
        PB_CHECK(coo_compress_cols(nrows, nseg, reinterpret_cast<const int*>(segrow_sorted), plan->rowptr, s));
        PB_CHECK(hipStreamSynchronize(s));
    }
    if (tmp.used > ((size_t)opt_plan_keep_mb() << 20)) PB_CHECK(ws_drop(WS_PLAN_ROWS_A, s));
    return hipGetLastError();
}

// BIDMAT_PLAN_TIMING=1 in the environment: every stage of a build is followed by a device synchronisation and
// its wall-clock time printed (a build then takes longer than without).
struct StageClock {
    bool on;
    std::chrono::steady_clock::time_point t0;
    StageClock() : on(false) {
        const char* e = getenv("BIDMAT_PLAN_TIMING");
        on = e && e[0] == '1';
        t0 = std::chrono::steady_clock::now();
    }
    void mark(const char* what) {
        if (!on) return;
        (void)hipDeviceSynchronize();
        const auto t1 = std::chrono::steady_clock::now();
        fprintf(stderr, "[bidmathip] plan build: %-28s %8.3f ms\n", what, std::chrono::duration<double, std::milli>(t1 - t0).count());
        t0 = t1;
    }
};

// Builds the halves named in `sides` into `plan` (whose sizes and k_hint are set). On failure the
// caller drops what was begun.
hipError_t build_sides(bidmat_plan* plan, const int* ir, const int* jc, int sides) {
    StageClock clock;
    const bool rows = (sides & PLAN_ROWS) != 0, cols = (sides & PLAN_COLS) != 0;
    const int nrows = plan->nrows, ncols = plan->ncols, nnz = plan->nnz;
    const int k_hint = plan->k_hint;
    hipStream_t s = nullptr;
    int p8 = 0;
    if (rows) {
        plan->seglen = opt_seglen();
        {
            // small patterns: shorter segments, so that the gather stage still has a few waves for
            // every wave slot of the device
            long long want = ((long long)nnz / 32768 / 64) * 64;
            if (want < 64) want = 64;
            if (want < plan->seglen) plan->seglen = (int)want;
        }
        long long pcols = (long long)opt_panel_kb() * 1024 / (4LL * k_hint);
        if (pcols < 64) pcols = 64;
        if (pcols > ncols) pcols = ncols > 0 ? ncols : 1;
        if (ncols >= 8 * 64) {
            // panels are dealt to the 8 XCDs round-robin: a multiple of 8 keeps them all equally busy
            long long np = (ncols + pcols - 1) / pcols;
            np = ((np + 7) / 8) * 8;
            pcols = (ncols + np - 1) / np;
        }
        plan->panel_cols = (int)pcols;
        plan->npanels = ncols > 0 ? (int)(((long long)ncols + pcols - 1) / pcols) : 1;
        p8 = (plan->npanels + 7) / 8;          // panels per XCD group
        // memory the plan keeps, part 1: everything whose size is known now
        Arena own;
        for (int pass = 0; pass < 2; ++pass) {
            own.used = 0;
            plan->rowptr = own.take<int>((size_t)nrows + 1);
            plan->perm = own.take<int>((size_t)nnz);
            plan->pc = own.take<int>((size_t)nnz);
            if (pass == 0) {
                PB_CHECK(plan_alloc(&plan->block_nnz, own.used));
                own.base = static_cast<char*>(plan->block_nnz);
                plan->row_bytes += own.used;
            }
        }
    }
    clock.mark("row-side arrays allocated");
    if (nnz == 0 || nrows == 0 || ncols == 0) {
        if (rows) {
            PB_CHECK(fill_i32(plan->rowptr, (long long)nrows + 1, 0, s));
            PB_CHECK(hipStreamSynchronize(s));
        }
        if (cols) plan->col_seglen = opt_seglen();
        return hipSuccess;
    }

    // temporaries sized by the rows: one arena out of the library's workspace (the row-side builders take
    // what they need per nonzero from slots of their own)
    const size_t nitem = (size_t)(nrows > (1 << 14) ? nrows : (1 << 14));
    BuildTmp t;
    PB_CHECK(rocprim::radix_sort_pairs_desc(nullptr, t.sort_bytes, (unsigned*)nullptr, (unsigned*)nullptr, (int*)nullptr, (int*)nullptr,
                                            (size_t)nrows, 0, 32, s));
    Arena tmp;
    for (int pass = 0; pass < 2; ++pass) {
        tmp.used = 0;
        t.cnt = tmp.take<int>((size_t)nrows);
        t.hflag = tmp.take<int>((size_t)nrows);
        t.hrank = tmp.take<int>((size_t)nrows + 2);        // [nrows] = number of heavy rows, [nrows+1] = bad-index flag
        t.hrow = tmp.take<int>((size_t)nrows);
        t.crank = tmp.take<int>((size_t)nrows);            // rank of a row among its class's hot rows, or -1
        t.scantmp = tmp.take<int>(scan_tmp_ints((long long)nrows));
        t.keys_in = tmp.take<unsigned>(nitem);             // the ranking of the rows by count (column side)
        t.keys_out = tmp.take<unsigned>(nitem);
        t.colpos_in = tmp.take<unsigned long long>(nitem);
        t.colpos_out = tmp.take<unsigned long long>(nitem);
        t.sorttmp = tmp.take<char>(t.sort_bytes);
        if (pass == 0) {
            hipError_t werr;
            tmp.base = static_cast<char*>(ws_get(WS_PLAN, tmp.used, &werr));
            if (!tmp.base) return werr;
        }
    }
    t.arena_bytes = tmp.used;
    t.bad = t.hrank + nrows + 1;

    // row histogram (integer atomics: the counts do not depend on the order)
    PB_CHECK(fill_i32(t.cnt, nrows, 0, s));
    PB_CHECK(fill_i32(t.hrank + nrows, 2, 0, s));
    // few, long-lived workgroups: every one flushes its LDS histogram once at the end
    t.sample = (long long)nnz >= HIST_SAMPLE_FROM ? HIST_SAMPLE : 1;     // cnt[r] ~ (nonzeros of row r) / sample
    hipLaunchKernelGGL(k_row_hist, dim3(grid_for(nnz, 1024)), dim3(BM_BLOCK), 0, s, nnz, nrows, t.sample, ir, t.cnt, t.bad);
    clock.mark("workspace + row histogram");

    if (cols) {
        PB_CHECK(build_cols(plan, ir, jc, t, s));
        clock.mark("column side");
        if (!rows) {
            int badv = 0;                                // set by the histogram (as far as it looked) or the class ordering
            PB_CHECK(hipMemcpy(&badv, t.bad, sizeof(int), hipMemcpyDeviceToHost));
            if (badv) return hipErrorInvalidValue;
        }
    }
    if (rows) {
        int nheavy = 0;
        PB_CHECK(detect_heavy(plan, t, p8, &nheavy, s));
        plan->nheavy = nheavy;
        clock.mark("heavy rows ranked");
        int unfit = 1;
        if (opt_plan_builder() == 0) PB_CHECK(build_rows_binned(plan, ir, jc, t.hflag, t.hrow, nheavy, p8, t.bad, &unfit, s));
        if (unfit) PB_CHECK(build_rows_sorted(plan, ir, jc, t, nheavy, p8, s));
        clock.mark(unfit ? "row side (library sort)" : "row side (counting sorts)");
        if (opt_dense_rows() > 0 && (long long)nnz >= opt_dense_min_nnz() && dense_rows_fit(k_hint)) {
            // the dense block is an extra: a plan that cannot get the memory for it works without
            const hipError_t de = build_dense_rows(plan, ir, jc, t.cnt, t.sample, s);
            if (de == hipErrorOutOfMemory) (void)hipGetLastError();
            else PB_CHECK(de);
            clock.mark("dense rows");
        }
    }
    PB_CHECK(hipGetLastError());
    if (t.arena_bytes > ((size_t)opt_plan_keep_mb() << 20)) PB_CHECK(ws_drop(WS_PLAN));
    return hipSuccess;
}

// builds share the workspace arena of their device: one at a time
std::mutex g_build_mu;

}  // namespace

hipError_t plan_digest(int nnz, int ncols, const int* ir, const int* jc, unsigned long long d[2]) {
    d[0] = d[1] = 0;
    hipError_t e;
    const size_t words = pattern_digest_words();
    unsigned long long* dm = (unsigned long long*)ws_get(WS_MISC, 2 * sizeof(unsigned long long) * words, &e);
    if (!dm) return e;
    if ((e = pattern_digest(ir, ir, nnz, dm, nullptr)) != hipSuccess) return e;
    if ((e = pattern_digest(jc, jc, (long long)ncols + 1, dm + words, nullptr)) != hipSuccess) return e;
    if ((e = hipMemcpy(&d[0], dm, sizeof(unsigned long long), hipMemcpyDeviceToHost)) != hipSuccess) return e;
    return hipMemcpy(&d[1], dm + words, sizeof(unsigned long long), hipMemcpyDeviceToHost);
}

hipError_t plan_build(int nrows, int ncols, int nnz, const int* ir, const int* jc, int k_hint,
                      bidmat_plan** out, int sides) {
    *out = nullptr;
    if ((sides & ~(PLAN_ROWS | PLAN_COLS)) != 0 || sides == 0) return hipErrorInvalidValue;
    std::lock_guard<std::mutex> build_lock(g_build_mu);
    bidmat_plan* plan = new (std::nothrow) bidmat_plan();
    if (!plan) return hipErrorOutOfMemory;
    hipError_t e = hipGetDevice(&plan->device);
    plan->nrows = nrows; plan->ncols = ncols; plan->nnz = nnz;
    plan->k_hint = k_hint > 0 ? k_hint : 256;
    if (e == hipSuccess) e = build_sides(plan, ir, jc, sides);
    if (e == hipSuccess && opt_check_plan() && nnz > 0 && ncols > 0) {
        e = plan_digest(nnz, ncols, ir, jc, plan->digest);
        plan->has_digest = e == hipSuccess;
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        (void)plan_free(plan);
        return e;
    }
    plan->sides = sides;
    *out = plan;
    return hipSuccess;
}

hipError_t plan_extend(bidmat_plan* plan, const int* ir, const int* jc, int sides) {
    if (!plan || (sides & ~(PLAN_ROWS | PLAN_COLS)) != 0) return hipErrorInvalidValue;
    const int missing = sides & ~plan->sides;
    if (missing == 0) return hipSuccess;
    std::lock_guard<std::mutex> build_lock(g_build_mu);
    hipError_t e = build_sides(plan, ir, jc, missing);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        if (missing & PLAN_ROWS) (void)drop_rows(plan);
        if (missing & PLAN_COLS) (void)drop_cols(plan);
        return e;
    }
    plan->sides |= missing;
    return hipSuccess;
}

}  // namespace bm
