// Builds the row-binned plan on the device: row histogram, heavy-row ranking, one stable
// radix sort of (panel,row) keys, segment boundaries by scan. Integer work only; the build is
// paid once per sparsity pattern and reused by every A*^S / row-sum call on it.
#include "plan.hpp"
#include "common.hpp"
#include "kernels.hpp"
#include "scan.hpp"
#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>
#include <new>

namespace bm {
namespace {

struct DevBuf {
    void* p = nullptr;
    hipError_t alloc(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 256); }
    ~DevBuf() { if (p) (void)hipFree(p); }
    template <typename T> T* as() { return static_cast<T*>(p); }
};


// Row histogram. The first HIST_LDS_ROWS rows are counted in a per-workgroup LDS copy that is
// flushed once at the end (popular rows tend to carry small indices in count-sorted vocabularies,
// and even when they do not this only costs the flush); all other rows go straight to global
// integer atomics. The counts do not depend on the order of the increments.
constexpr int HIST_LDS_ROWS = 16384;
__global__ __launch_bounds__(BM_BLOCK) void k_row_hist(int nnz, int nrows, const int* __restrict__ ir,
                                                       int* __restrict__ cnt, int* __restrict__ bad) {
    __shared__ int local[HIST_LDS_ROWS];
    for (int i = threadIdx.x; i < HIST_LDS_ROWS; i += BM_BLOCK) local[i] = 0;
    __syncthreads();
    long long j = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    for (; j < nnz; j += stride) {
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

// hrow[hrank[r]] = r for heavy rows
__global__ __launch_bounds__(BM_BLOCK) void k_heavy_rows(int nrows, const int* __restrict__ flag,
                                                         const int* __restrict__ hrank, int* __restrict__ hrow) {
    const long long r = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (r < nrows && flag[r]) hrow[hrank[r]] = (int)r;
}

// 16 lanes per column: key and original position of every nonzero.
__global__ __launch_bounds__(BM_BLOCK) void k_make_keys(int ncols, int nrows, const int* __restrict__ jc,
                                                        const int* __restrict__ ir, const int* __restrict__ flag,
                                                        const int* __restrict__ hrank, int nheavy, int npanels,
                                                        int panel_cols, int p8, unsigned* __restrict__ keys,
                                                        int* __restrict__ pos) {
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
    for (int j = s + l; j < e; j += 16) {
        int r = ir[j];
        r = r < 0 ? 0 : (r >= nrows ? nrows - 1 : r);
        keys[j] = flag[r] ? panel * (unsigned)nheavy + (unsigned)hrank[r] : light_base + (unsigned)r;
        pos[j] = j;
    }
}

__global__ __launch_bounds__(BM_BLOCK) void k_boundaries(int nnz, int seglen, const unsigned* __restrict__ keys,
                                                         int* __restrict__ flag) {
    long long p = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    for (; p < nnz; p += stride)
        flag[p] = (p == 0 || keys[p] != keys[p - 1] || (p % seglen) == 0) ? 1 : 0;
}

// Column of every nonzero in plan order; segment tables at the flagged positions.
__global__ __launch_bounds__(BM_BLOCK) void k_emit(int nnz, const unsigned* __restrict__ keys,
                                                   const int* __restrict__ perm, const int* __restrict__ ic,
                                                   const int* __restrict__ flag, const int* __restrict__ segidx,
                                                   const int* __restrict__ hrow, int nheavy, int p8,
                                                   int* __restrict__ pc, int* __restrict__ segstart,
                                                   unsigned* __restrict__ segrow, int* __restrict__ segid,
                                                   unsigned char* __restrict__ segclass) {
    long long p = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * BM_BLOCK;
    const unsigned per_xcd = (unsigned)p8 * (unsigned)nheavy;     // keys per XCD group
    const unsigned light_base = 8u * per_xcd;
    for (; p < nnz; p += stride) {
        pc[p] = ic[perm[p]];
        if (flag[p]) {
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

hipError_t plan_free(bidmat_plan* p) {
    if (!p) return hipSuccess;
    hipError_t e = hipSuccess, f;
    void* bufs[] = {p->pc, p->perm, p->segstart, p->segrow, p->rowptr, p->rowseg, p->partial};
    for (void* b : bufs)
        if (b && (f = hipFree(b)) != hipSuccess) e = f;
    delete p;
    return e;
}

hipError_t plan_reserve_partial(bidmat_plan* p, int k) {
    size_t need = (size_t)p->nseg * (size_t)k;
    if (need <= p->partial_floats) return hipSuccess;
    if (p->partial) {
        hipError_t e = hipFree(p->partial);
        p->partial = nullptr; p->partial_floats = 0;
        if (e != hipSuccess) return e;
    }
    hipError_t e = hipMalloc((void**)&p->partial, need * sizeof(float));
    if (e != hipSuccess) return e;
    p->partial_floats = need;
    return hipSuccess;
}

#define PB_CHECK(expr)                                          \
    do {                                                        \
        hipError_t _e = (expr);                                 \
        if (_e != hipSuccess) { (void)plan_free(plan); return _e; }   \
    } while (0)

hipError_t plan_build(int nrows, int ncols, int nnz, const int* ir, const int* jc, int k_hint,
                      bidmat_plan** out) {
    *out = nullptr;
    bidmat_plan* plan = new (std::nothrow) bidmat_plan();
    if (!plan) return hipErrorOutOfMemory;
    hipStream_t s = nullptr;
    PB_CHECK(hipGetDevice(&plan->device));
    plan->nrows = nrows; plan->ncols = ncols; plan->nnz = nnz;
    plan->seglen = opt_seglen();
    if (k_hint <= 0) k_hint = 256;
    long long pcols = (long long)opt_panel_kb() * 1024 / (4LL * k_hint);
    if (pcols < 64) pcols = 64;
    if (pcols > ncols) pcols = ncols > 0 ? ncols : 1;
    plan->panel_cols = (int)pcols;
    plan->npanels = ncols > 0 ? (int)(((long long)ncols + pcols - 1) / pcols) : 1;
    const int p8 = (plan->npanels + 7) / 8;          // panels per XCD group

    PB_CHECK(hipMalloc((void**)&plan->rowptr, sizeof(int) * ((size_t)nrows + 1)));
    plan->index_bytes += sizeof(int) * ((size_t)nrows + 1);
    if (nnz == 0 || nrows == 0 || ncols == 0) {
        PB_CHECK(fill_i32(plan->rowptr, (long long)nrows + 1, 0, s));
        PB_CHECK(hipStreamSynchronize(s));
        *out = plan;
        return hipSuccess;
    }

    DevBuf cnt, hflag, hrank, hrow, scantmp, bad, keys_in, keys_out, pos_in, ic, flag, segidx;
    PB_CHECK(cnt.alloc(sizeof(int) * (size_t)nrows));
    PB_CHECK(hflag.alloc(sizeof(int) * (size_t)nrows));
    PB_CHECK(hrank.alloc(sizeof(int) * ((size_t)nrows + 1)));
    PB_CHECK(hrow.alloc(sizeof(int) * (size_t)nrows));
    size_t scan_n = (size_t)(nnz > nrows ? nnz : nrows);
    PB_CHECK(scantmp.alloc(sizeof(int) * scan_tmp_ints((long long)scan_n)));
    PB_CHECK(bad.alloc(sizeof(int)));

    // 1. row histogram (integer atomics: the counts do not depend on the order)
    PB_CHECK(fill_i32(cnt.as<int>(), nrows, 0, s));
    PB_CHECK(fill_i32(bad.as<int>(), 1, 0, s));
    // few, long-lived workgroups: every one flushes its LDS histogram once at the end
    hipLaunchKernelGGL(k_row_hist, dim3(grid_for(nnz, 1024)), dim3(BM_BLOCK), 0, s, nnz, nrows, ir, cnt.as<int>(), bad.as<int>());
    int h_bad = 0;
    PB_CHECK(hipMemcpy(&h_bad, bad.p, sizeof(int), hipMemcpyDeviceToHost));
    if (h_bad) { (void)plan_free(plan); return hipErrorInvalidValue; }

    // 2. heavy rows and their ranks
    int nheavy = 0;
    if (plan->npanels >= 2) {
        long long thresh = (long long)plan->npanels * opt_heavy_min();
        if (thresh > 0x7fffffffLL) thresh = 0x7fffffffLL;
        hipLaunchKernelGGL(k_heavy_flag, dim3(grid_for(nrows, 1 << 30)), dim3(BM_BLOCK), 0, s, nrows, cnt.as<int>(), (int)thresh, hflag.as<int>());
        PB_CHECK(scan_exclusive_i32(hflag.as<int>(), hrank.as<int>(), nrows, scantmp.as<int>(), s));
        PB_CHECK(hipMemcpy(&nheavy, hrank.as<int>() + nrows, sizeof(int), hipMemcpyDeviceToHost));
        // keys must fit 32 bits
        if (8ULL * (unsigned long long)p8 * (unsigned long long)nheavy + (unsigned long long)nrows > 0xffffffffULL) nheavy = 0;
    }
    if (nheavy == 0) {
        PB_CHECK(fill_i32(hflag.as<int>(), nrows, 0, s));
        PB_CHECK(fill_i32(hrank.as<int>(), (long long)nrows + 1, 0, s));
    } else {
        hipLaunchKernelGGL(k_heavy_rows, dim3(grid_for(nrows, 1 << 30)), dim3(BM_BLOCK), 0, s, nrows, hflag.as<int>(), hrank.as<int>(), hrow.as<int>());
    }
    plan->nheavy = nheavy;

    // 3. keys + stable radix sort
    PB_CHECK(keys_in.alloc(sizeof(unsigned) * (size_t)nnz));
    PB_CHECK(keys_out.alloc(sizeof(unsigned) * (size_t)nnz));
    PB_CHECK(pos_in.alloc(sizeof(int) * (size_t)nnz));
    PB_CHECK(hipMalloc((void**)&plan->perm, sizeof(int) * (size_t)nnz));
    PB_CHECK(hipMalloc((void**)&plan->pc, sizeof(int) * (size_t)nnz));
    plan->index_bytes += 2 * sizeof(int) * (size_t)nnz;
    {
        long long nblk = ((long long)ncols * 16 + BM_BLOCK - 1) / BM_BLOCK;
        hipLaunchKernelGGL(k_make_keys, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, ncols, nrows, jc, ir,
                           hflag.as<int>(), hrank.as<int>(), nheavy, plan->npanels, plan->panel_cols, p8,
                           keys_in.as<unsigned>(), pos_in.as<int>());
    }
    const unsigned long long maxkey = 8ULL * (unsigned long long)p8 * nheavy + (unsigned long long)nrows;
    const int end_bit = bits_for(maxkey);
    {
        size_t tmp_bytes = 0;
        PB_CHECK(rocprim::radix_sort_pairs(nullptr, tmp_bytes, keys_in.as<unsigned>(), keys_out.as<unsigned>(),
                                           pos_in.as<int>(), plan->perm, (size_t)nnz, 0, end_bit, s));
        DevBuf sorttmp;
        PB_CHECK(sorttmp.alloc(tmp_bytes));
        PB_CHECK(rocprim::radix_sort_pairs(sorttmp.p, tmp_bytes, keys_in.as<unsigned>(), keys_out.as<unsigned>(),
                                           pos_in.as<int>(), plan->perm, (size_t)nnz, 0, end_bit, s));
        PB_CHECK(hipStreamSynchronize(s));
    }

    // 4. segment boundaries
    PB_CHECK(ic.alloc(sizeof(int) * (size_t)nnz));
    PB_CHECK(csc_expand_cols(ncols, nnz, jc, ic.as<int>(), s));
    PB_CHECK(flag.alloc(sizeof(int) * (size_t)nnz));
    PB_CHECK(segidx.alloc(sizeof(int) * ((size_t)nnz + 1)));
    hipLaunchKernelGGL(k_boundaries, dim3(grid_for(nnz)), dim3(BM_BLOCK), 0, s, nnz, plan->seglen, keys_out.as<unsigned>(), flag.as<int>());
    PB_CHECK(scan_exclusive_i32(flag.as<int>(), segidx.as<int>(), nnz, scantmp.as<int>(), s));
    int nseg = 0;
    PB_CHECK(hipMemcpy(&nseg, segidx.as<int>() + nnz, sizeof(int), hipMemcpyDeviceToHost));
    plan->nseg = nseg;

    DevBuf segid, segrow_sorted, class_count;
    DevBuf segclass;
    PB_CHECK(class_count.alloc(sizeof(int) * 9));
    PB_CHECK(fill_i32(class_count.as<int>(), 9, nseg, s));
    PB_CHECK(segclass.alloc((size_t)(nseg > 0 ? nseg : 1)));
    PB_CHECK(hipMalloc((void**)&plan->segrow, sizeof(int) * (size_t)(nseg > 0 ? nseg : 1)));
    unsigned* const segrow_u = reinterpret_cast<unsigned*>(plan->segrow);
    PB_CHECK(segid.alloc(sizeof(int) * (size_t)nseg));
    PB_CHECK(segrow_sorted.alloc(sizeof(unsigned) * (size_t)nseg));
    PB_CHECK(hipMalloc((void**)&plan->segstart, sizeof(int) * ((size_t)nseg + 1)));
    PB_CHECK(hipMalloc((void**)&plan->rowseg, sizeof(int) * (size_t)nseg));
    plan->index_bytes += sizeof(int) * (3 * (size_t)nseg + 1);
    hipLaunchKernelGGL(k_emit, dim3(grid_for(nnz)), dim3(BM_BLOCK), 0, s, nnz, keys_out.as<unsigned>(), plan->perm,
                       ic.as<int>(), flag.as<int>(), segidx.as<int>(), hrow.as<int>(), nheavy > 0 ? nheavy : 1,
                       nheavy > 0 ? p8 : 0, plan->pc, plan->segstart, segrow_u, segid.as<int>(),
                       segclass.as<unsigned char>());
    PB_CHECK(fill_i32(plan->segstart + nseg, 1, nnz, s));
    hipLaunchKernelGGL(k_class_bounds, dim3(grid_for(nseg, 1 << 30)), dim3(BM_BLOCK), 0, s, nseg,
                       segclass.as<unsigned char>(), class_count.as<int>());
    PB_CHECK(hipMemcpy(plan->xcd_start, class_count.p, sizeof(int) * 9, hipMemcpyDeviceToHost));

    // 5. a row's segments, in ascending segment order (stable sort by row)
    {
        const int rbits = bits_for((unsigned long long)nrows);
        size_t tmp_bytes = 0;
        PB_CHECK(rocprim::radix_sort_pairs(nullptr, tmp_bytes, segrow_u, segrow_sorted.as<unsigned>(),
                                           segid.as<int>(), plan->rowseg, (size_t)nseg, 0, rbits, s));
        DevBuf sorttmp;
        PB_CHECK(sorttmp.alloc(tmp_bytes));
        PB_CHECK(rocprim::radix_sort_pairs(sorttmp.p, tmp_bytes, segrow_u, segrow_sorted.as<unsigned>(),
                                           segid.as<int>(), plan->rowseg, (size_t)nseg, 0, rbits, s));
        PB_CHECK(coo_compress_cols(nrows, nseg, reinterpret_cast<const int*>(segrow_sorted.as<unsigned>()), plan->rowptr, s));
        PB_CHECK(hipStreamSynchronize(s));
    }
    PB_CHECK(hipGetLastError());
    *out = plan;
    return hipSuccess;
}

}  // namespace bm
