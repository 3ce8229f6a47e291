// Sampled dense-dense products on a sparse pattern: P[j] = dot(A[:,ir[j]], B[:,c]) for every
// stored nonzero j of column c.
//
// One wavefront owns a column (long columns: seglen-sized segments, extra waves take the
// overflow segments; no reduction is needed between segments). The column of B stays in
// registers for the whole segment. A group of LPN lanes covers one column of A, so a wave
// gathers 64/LPN columns of A per load instruction; the dot product is finished with a
// butterfly inside the group (DPP inside 16-lane rows) and each lane keeps the result of
// "its" nonzero, so a chunk of 64 results is written with one coalesced store.
#include "common.hpp"
#include "kernels.hpp"
#include "ops.hpp"
#include "workspace.hpp"
#include <mutex>

namespace bm {
namespace {

struct DdsArgs {
    int k;
    int ncols;
    int seglen;
    int beta;
    const float* A;
    const float* B;
    const int* ir;
    const int* jc;
    const int* ovf;
    float* P;
    const float* V;      // epilogue operand (nullable): P[j] = op(V[j], dot_j)
    int opn;
};

template <int V, int LPN>
struct Unroll { static constexpr int raw = 8 / V; static constexpr int U = raw < 1 ? 1 : (raw > LPN ? LPN : raw); };

// One round of a chunk: U nonzeros per group gathered back to back, dotted against the column of B
// and reduced together; returns the running per-lane result (lane l keeps the l-th nonzero of the
// chunk). PRED: the round may reach past the end of the segment; slots there issue no load at all
// (so a short segment costs the memory pipeline nothing for its unused slots) and contribute zeros.
// LDSROWS: myrow holds ranks of hot rows, which sit in the workgroup's LDS (hot_lds) instead of A.
extern __shared__ __align__(16) float hot_lds[];

template <int W, int V, int LPN, bool EXACT, bool PRED, bool LDSROWS = false>
__device__ __forceinline__ float dds_round(const float* __restrict__ A, int k, int myrow, int it0, int rem, int g, int l,
                                           int label, const int (&eld)[V], const bool (&ev)[V], const Vec<W> (&b)[V],
                                           float res) {
    constexpr int NG = 64 / LPN;
    constexpr int U = Unroll<V, LPN>::U;
    constexpr bool MULTI = (LPN >= 8) && (U >= 2);       // U dot products reduced together
    Vec<W> av[U][V];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        // slot u of the round belongs to the nonzero kept by lane it0 + slot_offset(u)
        const int it = it0 + (MULTI ? slot_offset<U>(u, it0) : u);
        int r;
        if constexpr (LPN == 64) r = __builtin_amdgcn_readlane(myrow, it);
        else r = lane_read(myrow, g * LPN + it);
        if (!PRED || (it * NG + g) < rem) {
            if constexpr (LDSROWS) {
                const float* hp = hot_lds + __mul24(r, k);      // a rank times k: below the LDS size, a full-rate multiply
#pragma unroll
                for (int i = 0; i < V; ++i) av[u][i] = Vec<W>::load(hp + eld[i]);
            } else {
                const float* ap = A + (size_t)r * (size_t)k;
#pragma unroll
                for (int i = 0; i < V; ++i) av[u][i] = Vec<W>::load(ap + eld[i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) av[u][i] = Vec<W>::zero();
        }
    }
    float sums[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < V; ++i) {
            Vec<W> x = av[u][i];
            if (!EXACT) x = ev[i] ? x : Vec<W>::zero();   // lanes past k contribute nothing
            s = x.dotacc(b[i], s);
        }
        sums[u] = s;
    }
    if constexpr (MULTI) {
        const float red = group_multisum<LPN, U>(sums, label);
        res = (l / U == it0 / U) ? red : res;
    } else {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float s = group_allsum<LPN>(sums[u]);
            res = (l == it0 + u) ? s : res;
        }
    }
    return res;
}

template <int W, int V, int LPN, bool EXACT, bool FULL, bool LDSROWS = false>
__device__ __forceinline__ void dds_chunk(const float* __restrict__ A, int k, int myrow, float* o, int rem, int g,
                                          int l, const int (&eld)[V], const bool (&ev)[V],
                                          const Vec<W> (&b)[V], float oldp, bool apply, float vval, int opn) {
    constexpr int NG = 64 / LPN;
    constexpr int U = Unroll<V, LPN>::U;
    const int q = l * NG + g;            // the nonzero of this chunk whose result this lane keeps
    float res = 0.f;
    const int label = slot_label(l);
    if (FULL) {
#pragma unroll 1
        for (int it0 = 0; it0 < LPN; it0 += U)
            res = dds_round<W, V, LPN, EXACT, false, LDSROWS>(A, k, myrow, it0, rem, g, l, label, eld, ev, b, res);
    } else {
        const int niter = (rem + NG - 1) / NG;
        const int nwhole = (rem / (NG * U)) * U;         // rounds whose every slot lies inside the segment
        int it0 = 0;
#pragma unroll 1
        for (; it0 < nwhole; it0 += U)
            res = dds_round<W, V, LPN, EXACT, false, LDSROWS>(A, k, myrow, it0, rem, g, l, label, eld, ev, b, res);
#pragma unroll 1
        for (; it0 < niter; it0 += U)
            res = dds_round<W, V, LPN, EXACT, true, LDSROWS>(A, k, myrow, it0, rem, g, l, label, eld, ev, b, res);
    }
    if (FULL || q < rem) {                                        // o: where this lane's nonzero goes
        res += oldp;                                              // the addend (0 when the output is overwritten)
        if (apply) res = binop_rt(opn, vval, res);               // only on the last pass over k
        *o = res;
    }
}

template <int W, int V, int LPN, bool EXACT>
__global__ __launch_bounds__(BM_BLOCK) void k_dds(DdsArgs a) {
    constexpr int KT = W * V * LPN;
    const int lane = threadIdx.x & 63;
    const long long w = (long long)blockIdx.x * BM_WAVES_PER_BLOCK + wave_uniform(threadIdx.x >> 6);
    const int g = lane / LPN, l = lane % LPN;

    int c, jstart, jend;
    if (w < a.ncols) {
        c = (int)w;
        const int s = a.jc[c], e = a.jc[c + 1];
        jstart = s;
        jend = (e - s > a.seglen) ? s + a.seglen : e;
    } else {
        if (a.ovf == nullptr) return;
        const long long x = w - a.ncols;
        if (x >= a.ovf[a.ncols]) return;
        int lo = 0, hi = a.ncols;        // ovf[lo] <= x < ovf[hi]
        while (hi - lo > 1) {
            const int mid = (int)(((long long)lo + hi) >> 1);
            if (a.ovf[mid] <= x) lo = mid; else hi = mid;
        }
        c = lo;
        const long long qseg = x - a.ovf[lo] + 1;
        const long long s = (long long)a.jc[lo] + qseg * a.seglen;
        const long long e = a.jc[lo + 1];
        jstart = (int)s;
        jend = (int)((e - s > a.seglen) ? s + a.seglen : e);
    }
    if (jstart >= jend) return;

    const float* bp = a.B + (size_t)c * (size_t)a.k;
    for (int k0 = 0; k0 < a.k; k0 += KT) {
        int eld[V];
        bool ev[V];
        Vec<W> b[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            const int e = k0 + (i * LPN + l) * W;
            ev[i] = e < a.k;
            eld[i] = ev[i] ? e : 0;
            b[i] = ev[i] ? Vec<W>::load(bp + e) : Vec<W>::zero();
        }
        const bool accumulate = (a.beta != 0) || (k0 > 0);
        // The next chunk's row indices are requested before the current chunk's gathers.
        const int q = l * (64 / LPN) + g;
        int j0 = jstart, rem = jend - jstart;
        int crow = (q < rem) ? a.ir[j0 + q] : 0;
        while (rem > 0) {
            const int nrow = (q < rem - 64) ? a.ir[j0 + 64 + q] : 0;
            float* o = a.P + j0 + q;
            // the epilogue's operand is requested before the gathers, so that it is there when they are done
            const bool apply = a.V != nullptr && k0 + KT >= a.k;
            const float vval = (apply && q < rem) ? a.V[j0 + q] : 0.f;
            // so is the addend of an accumulating call (and the running sum of an earlier pass over k)
            const float oldp = (accumulate && q < rem) ? *o : 0.f;
            if (rem >= 64) dds_chunk<W, V, LPN, EXACT, true>(a.A, a.k, crow, o, 64, g, l, eld, ev, b, oldp, apply, vval, a.opn);
            else dds_chunk<W, V, LPN, EXACT, false>(a.A, a.k, crow, o, rem, g, l, eld, ev, b, oldp, apply, vval, a.opn);
            crow = nrow;
            j0 += 64;
            rem -= 64;
        }
    }
}

// ---- DDS over a row-class ordered pattern (plan.hpp): workgroup b runs on XCD b % 8 and only
// touches the nonzeros whose row belongs to class b % 8, so the eight L2s cache disjoint rows, and
// the class's most frequent rows sit in the workgroup's LDS (filled once; workgroups are persistent
// and walk strips of consecutive columns). For each column a wave loads the column of B once, runs
// the class's hot-row nonzeros against LDS and the others against global memory, through the same
// chunk code as k_dds. Results go to their CSC positions through cperm: bit-identical to k_dds.
constexpr int CL_MAX_THREADS = 1024;
constexpr size_t CL_LDS_MAX = size_t(128) << 10;         // most LDS one workgroup may ask for
constexpr size_t CL_LDS_PER_CU = size_t(160) << 10;

struct DdsClassedArgs {
    int k;
    int ncols;
    int strip;           // columns per wave and step (<= 64)
    int beta;
    int opn;
    int hcap;            // hot rows per class
    const float* A;
    const float* B;
    const float* V;
    int v_classed;       // V is in class order (indexed like cir), not in stored order (indexed through cperm)
    const int* cir;
    const int* cperm;
    const int* cptr;
    const int* hotrows;
    float* P;
};

// One run of nonzeros [jstart, jend) of the current column. (crow, cpos): row / output position of
// this lane's nonzero of the run's first chunk, loaded by the caller ahead of time.
template <int W, int V, int LPN, bool EXACT, bool LDSROWS>
__device__ __forceinline__ void dds_classed_run(const DdsClassedArgs& a, int jstart, int jend, int crow, int cpos, int q,
                                                int g, int l, const int (&eld)[V], const bool (&ev)[V],
                                                const Vec<W> (&b)[V], bool accumulate, bool last) {
    int j0 = jstart, rem = jend - jstart;
    while (rem > 0) {
        int nrow = 0, npos = 0;
        if (q < rem - 64) { nrow = a.cir[j0 + 64 + q]; npos = a.cperm[j0 + 64 + q]; }
        float* o = a.P + cpos;
        const bool apply = a.V != nullptr && last;
        const float vval = (apply && q < rem) ? (a.v_classed ? a.V[j0 + q] : a.V[cpos]) : 0.f;     // requested before the gathers
        const float oldp = (accumulate && q < rem) ? *o : 0.f;                                     // likewise
        if (rem >= 64) dds_chunk<W, V, LPN, EXACT, true, LDSROWS>(a.A, a.k, crow, o, 64, g, l, eld, ev, b, oldp, apply, vval, a.opn);
        else dds_chunk<W, V, LPN, EXACT, false, LDSROWS>(a.A, a.k, crow, o, rem, g, l, eld, ev, b, oldp, apply, vval, a.opn);
        crow = nrow; cpos = npos;
        j0 += 64;
        rem -= 64;
    }
}

// What a wave loads ahead for one column: bounds of its two runs, this lane's nonzero of each run's
// first chunk, and the first pass of the column of B.
template <int W, int V>
struct ColumnAhead {
    int js, jm, je;
    int hrow, hpos, trow, tpos;
    Vec<W> b[V];
};

template <int W, int V, int LPN, bool HOTLDS>
__device__ __forceinline__ void load_column_ahead(const DdsClassedArgs& a, long long c, int js, int jm, int je, int q,
                                                  int l, ColumnAhead<W, V>& n) {
    n.js = js; n.jm = jm; n.je = je;
    n.hrow = n.hpos = n.trow = n.tpos = 0;
    if (HOTLDS && q < jm - js) { n.hrow = a.cir[js + q]; n.hpos = a.cperm[js + q]; }
    if (q < je - jm) { n.trow = a.cir[jm + q]; n.tpos = a.cperm[jm + q]; }
    const float* bp = a.B + (size_t)c * (size_t)a.k;
#pragma unroll
    for (int i = 0; i < V; ++i) {
        const int e = (i * LPN + l) * W;
        n.b[i] = (e < a.k && js < je) ? Vec<W>::load(bp + e) : Vec<W>::zero();
    }
}

// HOTLDS == false: no hot rows (hcap == 0): no LDS, no hot-row runs, workgroups of BM_BLOCK threads, and the
// registers this saves buy occupancy (the kernel waits on L2 misses: the more waves, the more gathers in flight).
template <int W, int V, int LPN, bool EXACT, bool HOTLDS>
__device__ __forceinline__ void dds_classed_body(const DdsClassedArgs& a) {
    constexpr int KT = W * V * LPN;
    const int lane = threadIdx.x & 63;
    const int wave = wave_uniform(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int x = blockIdx.x & 7;
    // ---- this class's hot rows into LDS, row h at hot_lds[h*k ..]
    if (HOTLDS && a.hcap > 0) {
        const int vpr = (a.k + W - 1) / W;                // vectors per row (W == 4 implies k % 4 == 0)
        const int total = a.hcap * vpr;
        for (int i = threadIdx.x; i < total; i += blockDim.x) {
            const int h = i / vpr, e = (i - h * vpr) * W;
            const int row = a.hotrows[x * a.hcap + h];
            const Vec<W> v = row >= 0 ? Vec<W>::load(a.A + (size_t)row * (size_t)a.k + e) : Vec<W>::zero();
            v.store(hot_lds + h * a.k + e);
        }
        __syncthreads();
    }
    const int g = lane / LPN, l = lane % LPN;
    const int q = l * (64 / LPN) + g;
    const long long nstrips = ((long long)a.ncols + a.strip - 1) / a.strip;
    const long long wstride = (long long)(gridDim.x >> 3) * nwaves;
    for (long long strip = (long long)(blockIdx.x >> 3) * nwaves + wave; strip < nstrips; strip += wstride) {
        const long long c0 = strip * a.strip;
        const int nc = (int)((a.ncols - c0) < a.strip ? (a.ncols - c0) : a.strip);
        // lane i holds the bounds of class x in column c0 + i: hot-row nonzeros [ps, pm), the others [pm, pe)
        int ps = 0, pm = 0, pe = 0;
        if (lane < nc) {
            const long long sc = (c0 + lane) * 16 + 2 * x;
            ps = a.cptr[sc];
            pm = a.cptr[sc + 1];
            pe = a.cptr[sc + 2];
        }
        ColumnAhead<W, V> nx;
        load_column_ahead<W, V, LPN, HOTLDS>(a, c0, __builtin_amdgcn_readlane(ps, 0), __builtin_amdgcn_readlane(pm, 0),
                                     __builtin_amdgcn_readlane(pe, 0), q, l, nx);
        for (int ci = 0; ci < nc; ++ci) {
            const ColumnAhead<W, V> cur = nx;
            // the next column's index chunks and its column of B are requested before this column's gathers
            if (ci + 1 < nc)
                load_column_ahead<W, V, LPN, HOTLDS>(a, c0 + ci + 1, __builtin_amdgcn_readlane(ps, ci + 1),
                                             __builtin_amdgcn_readlane(pm, ci + 1), __builtin_amdgcn_readlane(pe, ci + 1), q, l, nx);
            if (cur.js >= cur.je) continue;
            const float* bp = a.B + (size_t)(c0 + ci) * (size_t)a.k;
            for (int k0 = 0; k0 < a.k; k0 += KT) {
                int eld[V];
                bool ev[V];
                Vec<W> b[V];
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    const int e = k0 + (i * LPN + l) * W;
                    ev[i] = e < a.k;
                    eld[i] = ev[i] ? e : 0;
                    if (k0 == 0) b[i] = cur.b[i];
                    else b[i] = ev[i] ? Vec<W>::load(bp + e) : Vec<W>::zero();
                }
                const bool accumulate = (a.beta != 0) || (k0 > 0);
                const bool last = k0 + KT >= a.k;
                if constexpr (HOTLDS)
                    dds_classed_run<W, V, LPN, EXACT, true>(a, cur.js, cur.jm, cur.hrow, cur.hpos, q, g, l, eld, ev, b, accumulate, last);
                dds_classed_run<W, V, LPN, EXACT, false>(a, cur.jm, cur.je, cur.trow, cur.tpos, q, g, l, eld, ev, b, accumulate, last);
            }
        }
    }
}

template <int W, int V, int LPN, bool EXACT>
__global__ __launch_bounds__(CL_MAX_THREADS) void k_dds_classed(DdsClassedArgs a) {
    dds_classed_body<W, V, LPN, EXACT, true>(a);
}
template <int W, int V, int LPN, bool EXACT>
__global__ __launch_bounds__(BM_BLOCK) void k_dds_classed_nolds(DdsClassedArgs a) {
    dds_classed_body<W, V, LPN, EXACT, false>(a);
}
// The shape of k in (128, 256] fits six waves per SIMD (80 registers) without spilling, one more than the
// compiler settles on by itself (4.78 against 4.84 ms at the headline); asked for seven or eight it spills inside
// the gather loop and loses a fifth (5.85 ms), and the other shapes spill already at six.
template <bool EXACT>
__global__ __launch_bounds__(BM_BLOCK) __attribute__((amdgpu_waves_per_eu(6, 6)))
void k_dds_classed_nolds_k256(DdsClassedArgs a) {
    dds_classed_body<4, 1, 64, EXACT, false>(a);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

hipError_t launch_dds(const Shape& sh, bool exact, const DdsArgs& a, long long nwaves, hipStream_t s) {
    if (nwaves <= 0) return hipSuccess;
    long long nblk = (nwaves + BM_WAVES_PER_BLOCK - 1) / BM_WAVES_PER_BLOCK;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    dim3 grid((unsigned)nblk), block(BM_BLOCK);
#define BM_CASE(W_, V_, L_, E_)                                                          \
    if (sh.W == W_ && sh.V == V_ && sh.LPN == L_ && exact == E_) {                       \
        hipLaunchKernelGGL((k_dds<W_, V_, L_, E_>), grid, block, 0, s, a);               \
        return hipGetLastError();                                                        \
    }
#define BM_CASES(W_, E_)                                                                 \
    BM_CASE(W_, 1, 1, E_) BM_CASE(W_, 1, 2, E_) BM_CASE(W_, 1, 4, E_) BM_CASE(W_, 1, 8, E_) \
    BM_CASE(W_, 1, 16, E_) BM_CASE(W_, 1, 32, E_) BM_CASE(W_, 1, 64, E_) BM_CASE(W_, 2, 64, E_) \
    BM_CASE(W_, 4, 64, E_)
    BM_CASES(1, false)
    BM_CASES(4, false)
    BM_CASES(4, true)
#undef BM_CASES
#undef BM_CASE
    return hipErrorInvalidValue;
}

hipError_t launch_dds_classed(const Shape& sh, bool exact, const DdsClassedArgs& a, size_t lds_bytes, hipStream_t s) {
    int dev = 0, cus = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    const long long nstrips = ((long long)a.ncols + a.strip - 1) / a.strip;
    int threads = (int)opt_class_threads();
    long long nblk;
    if (lds_bytes == 0) {
        // nothing to keep per workgroup: one strip per wave, small workgroups
        threads = BM_BLOCK;
        nblk = 8 * ((nstrips + BM_WAVES_PER_BLOCK - 1) / BM_WAVES_PER_BLOCK);
    } else {
        // persistent workgroups (each fills its LDS once): as many per CU as LDS and wave slots allow,
        // a multiple of 8 so that every XCD gets the same number
        const int waves = threads / 64;
        long long per_cu = (long long)(CL_LDS_PER_CU / lds_bytes);
        if (per_cu > 32 / waves) per_cu = 32 / waves;
        if (per_cu < 1) per_cu = 1;
        long long per_xcd = per_cu * (cus / 8 > 0 ? cus / 8 : 1);
        const long long need = ((nstrips + 7) / 8 + waves - 1) / waves;    // workgroups per XCD that still find a strip
        if (need < per_xcd) per_xcd = need > 0 ? need : 1;
        nblk = 8 * per_xcd;
    }
    if (nblk <= 0) return hipSuccess;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    dim3 grid((unsigned)nblk), block((unsigned)threads);
#define BM_CASE(W_, V_, L_, E_)                                                          \
    if (sh.W == W_ && sh.V == V_ && sh.LPN == L_ && exact == E_) {                       \
        if (lds_bytes == 0) {                                                            \
            if (W_ == 4 && V_ == 1 && L_ == 64)                                          \
                hipLaunchKernelGGL((k_dds_classed_nolds_k256<E_>), grid, block, 0, s, a); \
            else                                                                         \
                hipLaunchKernelGGL((k_dds_classed_nolds<W_, V_, L_, E_>), grid, block, 0, s, a); \
            return hipGetLastError();                                                    \
        }                                                                                \
        auto kern = k_dds_classed<W_, V_, L_, E_>;                                       \
        if (lds_bytes > (48u << 10)) {                                                   \
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes); \
            if (e != hipSuccess) return e;                                               \
        }                                                                                \
        hipLaunchKernelGGL(kern, grid, block, lds_bytes, s, a);                          \
        return hipGetLastError();                                                        \
    }
#define BM_CASES(W_, E_)                                                                 \
    BM_CASE(W_, 1, 1, E_) BM_CASE(W_, 1, 2, E_) BM_CASE(W_, 1, 4, E_) BM_CASE(W_, 1, 8, E_) \
    BM_CASE(W_, 1, 16, E_) BM_CASE(W_, 1, 32, E_) BM_CASE(W_, 1, 64, E_) BM_CASE(W_, 2, 64, E_) \
    BM_CASE(W_, 4, 64, E_)
    BM_CASES(1, false)
    BM_CASES(4, false)
    BM_CASES(4, true)
#undef BM_CASES
#undef BM_CASE
    return hipErrorInvalidValue;
}

}  // namespace

// Most LDS the class-ordered kernel may ask for on the current device: what the device grants one
// workgroup, and never more than CL_LDS_MAX.
size_t dds_classed_lds_budget() {
    static std::mutex mu;
    static size_t per_device[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 48u << 10;
    std::lock_guard<std::mutex> lock(mu);
    if (!per_device[dev]) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess || v <= 0) v = 48 << 10;
        per_device[dev] = (size_t)v < CL_LDS_MAX ? (size_t)v : CL_LDS_MAX;
    }
    return per_device[dev];
}

hipError_t dds_classed(int k, int ncols, const float* A, const float* B, const int* cir, const int* cperm,
                       const int* cptr, int hcap, const int* hotrows, float* P, int beta, hipStream_t s,
                       const float* V, int opn, bool v_classed) {
    if (ncols <= 0 || k <= 0) return hipErrorInvalidValue;          // callers route those cases to dds_csc
    if (V != nullptr && (beta != 0 || opn < 0 || opn > 14)) return hipErrorInvalidValue;
    const size_t lds_bytes = (size_t)hcap * (size_t)k * sizeof(float);
    if (lds_bytes > dds_classed_lds_budget() || (hcap > 0 && !hotrows)) return hipErrorInvalidValue;
    Shape sh = pick_shape(k, aligned16(A) && aligned16(B));
    if (sh.V > 4) sh.V = 4;
    const bool exact = (sh.W == 4) && (k % (sh.W * sh.V * sh.LPN) == 0);
    DdsClassedArgs a;
    a.k = k; a.ncols = ncols; a.beta = beta; a.opn = opn; a.hcap = hcap;
    a.strip = (int)opt_class_strip();
    a.A = A; a.B = B; a.V = V; a.v_classed = v_classed ? 1 : 0; a.cir = cir; a.cperm = cperm; a.cptr = cptr; a.hotrows = hotrows; a.P = P;
    return launch_dds_classed(sh, exact, a, lds_bytes, s);
}

hipError_t dds_csc(int k, int ncols, int nnz, const float* A, const float* B, const int* ir,
                   const int* jc, float* P, int beta, hipStream_t s, const float* V, int opn,
                   const ColTable* tab) {
    if (ncols <= 0 || nnz <= 0) return hipSuccess;
    if (V != nullptr && (beta != 0 || opn < 0 || opn > 14)) return hipErrorInvalidValue;
    if (k <= 0) {
        // empty dot products: P = beta*P + 0, or op(V, 0)
        if (V != nullptr) {
            hipError_t e = fill_f32(P, nnz, 0.f, s);
            return e != hipSuccess ? e : applyop(V, nnz, 1, P, nnz, 1, P, opn, s);
        }
        if (!beta) return fill_f32(P, nnz, 0.f, s);
        return hipSuccess;
    }
    int seglen = opt_seglen();
    int* ovf = nullptr;
    long long novf_max = 0;
    if (tab) {
        seglen = tab->seglen;
        if (tab->novf > 0) { ovf = const_cast<int*>(tab->ovf); novf_max = tab->novf; }
    } else {
        hipError_t err = build_overflow_table(ncols, nnz, jc, seglen, &ovf, s);
        if (err != hipSuccess) return err;
        novf_max = ovf ? nnz / seglen : 0;
    }
    Shape sh = pick_shape(k, aligned16(A) && aligned16(B));
    if (sh.V > 4) sh.V = 4;
    const bool exact = (sh.W == 4) && (k % (sh.W * sh.V * sh.LPN) == 0);
    DdsArgs a;
    a.k = k; a.ncols = ncols; a.seglen = seglen; a.beta = beta;
    a.A = A; a.B = B; a.ir = ir; a.jc = jc; a.ovf = ovf; a.P = P; a.V = V; a.opn = opn;
    return launch_dds(sh, exact, a, (long long)ncols + novf_max, s);
}

// ---------------------------------------------------------------- DDS that allocates nothing
// The only device memory dds_csc needs beyond its arguments is the overflow-segment table of the
// columns. Here it lives in a fixed array inside the library's code object (every device that
// loads the library holds its own copy until the process ends), so the call allocates nothing.
// All calls on one device share the array: calls that overlap on a device race on it.
namespace {
constexpr int STATIC_MAX_COLS = 1 << 21;
// table area (2*ncols + 2 ints, rounded up to 64) + block sums of the scan (one per 2048 columns)
constexpr size_t STATIC_SCRATCH_INTS = (((2 * (size_t)STATIC_MAX_COLS + 2) + 63) & ~size_t(63)) + STATIC_MAX_COLS / 2048 + 64;
static __device__ __align__(256) int scratch[STATIC_SCRATCH_INTS];

constexpr int STATIC_MAX_DEVICES = 64;
std::mutex g_static_mu;
int* g_static_ptr[STATIC_MAX_DEVICES] = {nullptr};

// Device address of this device's copy of `scratch` (the array's name is only a host-side handle).
hipError_t static_scratch(int** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= STATIC_MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_static_mu);
    if (!g_static_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        g_static_ptr[dev] = static_cast<int*>(p);
    }
    *out = g_static_ptr[dev];
    return hipSuccess;
}
}  // namespace

int dds_static_max_cols() { return STATIC_MAX_COLS; }

hipError_t dds_csc_static(int k, int ncols, int nnz, const float* A, const float* B, const int* ir,
                          const int* jc, float* P, int beta, hipStream_t s) {
    if (ncols <= 0 || nnz <= 0) return hipSuccess;
    if (ncols > STATIC_MAX_COLS || overflow_table_ints(ncols) > STATIC_SCRATCH_INTS) return hipErrorInvalidValue;
    if (k <= 0) return beta ? hipSuccess : fill_f32(P, nnz, 0.f, s);
    int* buf = nullptr;
    hipError_t err = static_scratch(&buf);
    if (err != hipSuccess) return err;
    const int seglen = opt_seglen();
    int* ovf = nullptr;
    // every entry of the table that the kernels read is written by this build: nothing to clear
    err = build_overflow_table_in(ncols, nnz, jc, seglen, buf, &ovf, s);
    if (err != hipSuccess) return err;
    const ColTable tab{seglen, ovf, ovf ? (long long)(nnz / seglen) : 0};
    return dds_csc(k, ncols, nnz, A, B, ir, jc, P, beta, s, nullptr, 0, &tab);
}

}  // namespace bm
