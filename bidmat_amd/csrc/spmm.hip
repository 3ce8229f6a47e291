// Gather-accumulate kernels: C = beta*C + A*S over CSC columns (dsmult) and the segment
// stage of the row-binned plan (dsmultT).
//
// Scheduling: one wavefront owns one column (or one plan segment). A column longer than
// `seglen` nonzeros is cut into seglen-sized segments; the first stays with the column's
// wave, the others are "overflow" segments picked up by extra waves that write k-vector
// partial sums, added to C afterwards in a fixed order (no atomics, deterministic).
//
// Data movement: a dense column of k floats is covered by a group of LPN lanes holding V
// vectors of W floats each (W = 4: 128-bit loads). With LPN < 64 a wave works on 64/LPN
// nonzeros per load instruction. Index/value arrays are read 64 at a time, coalesced, and
// handed to the owning group by lane reads; U independent gathers are issued back to back
// before their FMAs to keep the memory pipeline full.
#include "common.hpp"
#include "kernels.hpp"
#include "ops.hpp"
#include "scan.hpp"
#include "workspace.hpp"
#include <algorithm>

namespace bm {
namespace {

struct GatherArgs {
    int k;               // rows of A / of the output that are computed
    int lda;             // column stride of A
    int ldo;             // column stride of the output C (partials always use k)
    int win_on;          // tile mode: only nonzeros whose gather index lies in [win_off, win_off+win_len)
    int win_off;         //   take part, and the index is rebased to win_off
    int win_len;
    const int* segrow;   // tile mode on a plan: row of each segment; segments outside
    int row_off;         //   [row_off, row_off+row_len) are skipped
    int row_len;
    int nfirst;          // columns (CSC mode) or segments (plan mode)
    int seglen;
    int beta;
    const float* A;
    const float* vals;
    const int* idx;      // ir (CSC mode) / pc (plan mode): which column of A to gather
    const int* perm;     // plan mode: position of the value in the original CSC order (nullptr: vals is in plan order)
    const int* ptr;      // jc (CSC mode) / segstart (plan mode)
    const int* ovf;      // CSC mode: overflow table (nullable)
    float* out;          // C (CSC mode) / partial (plan mode)
    float* partial;      // CSC mode: partial sums of overflow segments
    int xcd_start[9];    // plan mode: segment groups per XCD, light segments from xcd_start[8]
    // CSC mode on a class-ordered pattern: the wave of column w takes the nonzeros
    // [ptr[w*pstride + poff], ptr[w*pstride + poff + pspan]) (plain CSC: 1, 0, 1)
    int pstride, poff, pspan;
    // fused DDS + A*^S over a plan (k_fused_rows): the dense matrix whose column `row of the segment` is dotted
    // with every gathered column, the op applied to (value, dot), where the products go (CSC order, nullable)
    const float* R;
    int ldr;
    int opn;
    float* qout;
    const int* qperm;    // position of each product in qout (nullptr: plan order)
    // plan mode, A *^ S with the densest rows multiplied elsewhere (dense_rows.hip)
    const unsigned char* skip;   // a byte per segment, 1 = not this launch's (nullable)
    int* flag;                   // cleared by the launch over all segments; the launch over `seglist` only works when it is set
    const int* seglist;          // the launch takes segments seglist[0 .. nfirst) instead of all (nullable)
};

template <int V, int LPN>
struct Unroll { static constexpr int raw = 8 / V; static constexpr int U = raw < 1 ? 1 : (raw > LPN ? LPN : raw); };

// Loads this lane's nonzero of a chunk: lane (g,l) holds nonzero q = l*NG + g, so group g meets
// its nonzeros q = it*NG + g in lane l == it of its own group. Lanes past `rem` keep (0, 0).
template <bool PLAN, bool SV = false>
__device__ __forceinline__ void load_chunk(const GatherArgs& a, int j0, int ahead, int rem, int q, int& myrow,
                                           float& myval) {
    myrow = 0;
    myval = 0.f;
    if (q < rem) {
        const int p = j0 + ahead + q;
        myrow = a.idx[p];
        if constexpr (SV) myval = __int_as_float(a.perm[p]);          // the position only: gather_chunk fetches the value
        else myval = a.perm != nullptr ? a.vals[a.perm[p]] : a.vals[p];     // perm == nullptr: vals is in the order of idx
    }
}

// SV ("scalar values", for walks whose values sit behind a permutation): a nonzero's value is fetched by a scalar load
// from its position, wave-uniform like the row index, instead of one 4-byte gather per lane and chunk. In plan order a
// lane-wise gather of 64 values touches 64 cache lines, one look-up each in the per-CU vector cache that the row gathers
// already keep busy (an eighth of their line requests at k = 256); the scalar cache is a path of its own to L2.
// Read-only use: the values were written by earlier launches, and nothing here writes through that cache.
typedef const float __attribute__((address_space(4))) scalar_float;

template <int W, int V, int LPN, bool FULL, bool TILE, bool SV = false>
__device__ __forceinline__ void gather_chunk(const GatherArgs& a, int myrow, float myval, int rem, int g, int l,
                                             const int (&eld)[V], Vec<W> (&acc)[V]) {
    constexpr int NG = 64 / LPN;
    constexpr int U = Unroll<V, LPN>::U;
    const int q = l * NG + g;
    unsigned long long inmask = ~0ULL;
    if (TILE) {
        // window filter: nonzeros outside the tile contribute nothing (their lane keeps index 0)
        const int rr = myrow - a.win_off;
        const bool inside = (FULL || q < rem) && (unsigned)rr < (unsigned)a.win_len;
        myrow = inside ? rr : 0;
        myval = inside ? myval : 0.f;
        inmask = __ballot(inside);
    }
    const int niter = FULL ? LPN : (rem + NG - 1) / NG;
    // One round of U gathers at a time: unrolled further, the compiler hoists every load of the
    // chunk and the register count collapses the occupancy (256 VGPRs at LPN = 32).
#pragma unroll 1
    for (int it0 = 0; it0 < niter; it0 += U) {
        Vec<W> av[U][V];
        float vv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int it = it0 + u;
            int r;
            if constexpr (LPN == 64) {
                r = __builtin_amdgcn_readlane(myrow, it);
                if constexpr (SV) {
                    const int pp = __builtin_amdgcn_readlane(__float_as_int(myval), it);
                    const float sv = ((scalar_float*)a.vals)[pp];
                    vv[u] = (FULL || it < rem) ? sv : 0.f;       // a slot past the end holds position 0: not its value
                } else {
                    vv[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(myval), it));
                }
            } else {
                const int src = g * LPN + it;
                r = lane_read(myrow, src);
                if constexpr (SV) {
                    float sv = 0.f;
#pragma unroll
                    for (int gg = 0; gg < NG; ++gg) {
                        const int pp = __builtin_amdgcn_readlane(__float_as_int(myval), gg * LPN + it);
                        const float x = ((scalar_float*)a.vals)[pp];
                        sv = g == gg ? x : sv;
                    }
                    vv[u] = (FULL || (it * NG + g) < rem) ? sv : 0.f;
                } else {
                    vv[u] = lane_read(myval, src);
                }
            }
            const float* ap = a.A + (size_t)r * (size_t)a.lda;
            if (!FULL || TILE) {
                // past the end of the segment (or outside the tile) no load is issued at all: the slot
                // costs the memory pipeline nothing, and a non-finite entry of A's column 0 cannot
                // leak in as 0*inf.
                bool ok = FULL || (it * NG + g) < rem;
                if (TILE) ok = ok && ((inmask >> (LPN == 64 ? it : g * LPN + it)) & 1ULL);
                if (ok) {
#pragma unroll
                    for (int i = 0; i < V; ++i) av[u][i] = Vec<W>::load(ap + eld[i]);
                } else {
#pragma unroll
                    for (int i = 0; i < V; ++i) av[u][i] = Vec<W>::zero();
                }
            } else {
#pragma unroll
                for (int i = 0; i < V; ++i) av[u][i] = Vec<W>::load(ap + eld[i]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i].fma(av[u][i], vv[u]);
        }
    }
}

template <int W>
__device__ __forceinline__ Vec<W> vec_xor_add(Vec<W> x, int m);
template <>
__device__ __forceinline__ Vec<1> vec_xor_add<1>(Vec<1> x, int m) {
    x.x += __shfl_xor(x.x, m, 64);
    return x;
}
template <>
__device__ __forceinline__ Vec<4> vec_xor_add<4>(Vec<4> x, int m) {
    x.v.x += __shfl_xor(x.v.x, m, 64);
    x.v.y += __shfl_xor(x.v.y, m, 64);
    x.v.z += __shfl_xor(x.v.z, m, 64);
    x.v.w += __shfl_xor(x.v.w, m, 64);
    return x;
}

template <int W, int V, int LPN, bool PLAN, bool SV = false>
__device__ __forceinline__ void gather_axpy_body(const GatherArgs& a) {
    constexpr int KT = W * V * LPN;      // elements of a dense column covered per pass
    const int lane = threadIdx.x & 63;
    const long long w = (long long)blockIdx.x * BM_WAVES_PER_BLOCK + wave_uniform(threadIdx.x >> 6);
    const int g = lane / LPN, l = lane % LPN;

    // ---- which segment does this wave own (all wave-uniform)
    int jstart, jend;
    float* outp;
    bool accumulate;
    if (PLAN) {
        // Workgroups are dealt to the 8 XCDs round-robin, so workgroup b runs on XCD b % 8.
        // Each XCD first walks its own group of heavy segments (whole column panels, one after
        // the other, so that the panel of A it is gathering stays in its L2), then its share of
        // the light segments (every 8th one). Interleaving the two kinds, with or without
        // non-temporal loads for the light gathers, was measured slower: the light gathers miss
        // L2 and evict the panel the heavy segments are reusing.
        long long seg;
        if (a.seglist != nullptr) {
            if (*a.flag == 0 || w >= a.nfirst) return;
            seg = a.seglist[w];
        } else {
            if (a.flag != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *a.flag = 0;
            const int xcd = blockIdx.x & 7;
            const long long wi = (long long)(blockIdx.x >> 3) * BM_WAVES_PER_BLOCK + wave_uniform(threadIdx.x >> 6);
            const int hstart = a.xcd_start[xcd];
            const int hcount = a.xcd_start[xcd + 1] - hstart;
            seg = wi < hcount ? hstart + wi : a.xcd_start[8] + (wi - hcount) * 8 + xcd;
            if (seg >= a.nfirst) return;
            if (a.skip != nullptr && a.skip[seg]) return;
        }
        if (a.segrow != nullptr && (unsigned)(a.segrow[seg] - a.row_off) >= (unsigned)a.row_len) return;
        jstart = a.ptr[seg];
        jend = a.ptr[seg + 1];
        outp = a.out + (size_t)seg * (size_t)a.k;
        accumulate = false;
    } else if (w < a.nfirst) {
        const long long pi = w * a.pstride + a.poff;
        const int s = a.ptr[pi], e = a.ptr[pi + a.pspan];
        jstart = s;
        jend = (e - s > a.seglen) ? s + a.seglen : e;
        outp = a.out + (size_t)w * (size_t)a.ldo;
        accumulate = a.beta != 0;
    } else {
        if (a.ovf == nullptr) return;
        const long long x = w - a.nfirst;
        if (x >= a.ovf[a.nfirst]) return;
        int lo = 0, hi = a.nfirst;       // ovf[lo] <= x < ovf[hi]
        while (hi - lo > 1) {
            const int mid = (int)(((long long)lo + hi) >> 1);
            if (a.ovf[mid] <= x) lo = mid; else hi = mid;
        }
        const long long qseg = x - a.ovf[lo] + 1;
        const long long s = (long long)a.ptr[lo] + qseg * a.seglen;
        const long long e = a.ptr[lo + 1];
        jstart = (int)s;
        jend = (int)((e - s > a.seglen) ? s + a.seglen : e);
        outp = a.partial + (size_t)x * (size_t)a.k;
        accumulate = false;
    }

    for (int k0 = 0; k0 < a.k; k0 += KT) {
        int est[V], eld[V];
        bool ev[V];
        Vec<W> acc[V];
#pragma unroll
        for (int i = 0; i < V; ++i) {
            est[i] = k0 + (i * LPN + l) * W;
            ev[i] = est[i] < a.k;
            eld[i] = ev[i] ? est[i] : 0;     // lanes past k re-read element 0; never stored
            acc[i] = Vec<W>::zero();
        }
        // An accumulating call's addend is requested now, so that it is there when the column's gathers are
        // done (with V > 2 the sixteen registers it would hold cost more occupancy than the wait at the end).
        constexpr bool EARLY_ADDEND = !PLAN && V <= 2;
        Vec<W> addend[V];
        if constexpr (EARLY_ADDEND) {
#pragma unroll
            for (int i = 0; i < V; ++i)
                addend[i] = (accumulate && g == 0 && ev[i]) ? Vec<W>::load(outp + est[i]) : Vec<W>::zero();
        }
        // The next chunk's indices and values are requested before the current chunk's gathers,
        // so their latency overlaps the gathers instead of preceding them.
        const int q = l * (64 / LPN) + g;
        int rem = jend - jstart, j0 = jstart;
        int crow;
        float cval;
        load_chunk<PLAN, SV>(a, j0, 0, rem, q, crow, cval);
        while (rem > 0) {
            int nrow;
            float nval;
            load_chunk<PLAN, SV>(a, j0, 64, rem - 64, q, nrow, nval);
            if (!SV && a.win_on) {
                if (rem >= 64) gather_chunk<W, V, LPN, true, true>(a, crow, cval, 64, g, l, eld, acc);
                else gather_chunk<W, V, LPN, false, true>(a, crow, cval, rem, g, l, eld, acc);
            } else {
                if (rem >= 64) gather_chunk<W, V, LPN, true, false, SV>(a, crow, cval, 64, g, l, eld, acc);
                else gather_chunk<W, V, LPN, false, false, SV>(a, crow, cval, rem, g, l, eld, acc);
            }
            crow = nrow;
            cval = nval;
            j0 += 64;
            rem -= 64;
        }

#pragma unroll
        for (int m = LPN; m < 64; m <<= 1) {
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i] = vec_xor_add<W>(acc[i], m);
        }
        if (g == 0) {
#pragma unroll
            for (int i = 0; i < V; ++i) {
                if (ev[i]) {
                    float* o = outp + est[i];
                    Vec<W> r = acc[i];
                    if constexpr (EARLY_ADDEND) r.add(addend[i]);
                    else if (accumulate) r.add(Vec<W>::load(o));
                    r.store(o);
                }
            }
        }
    }
}

template <int W, int V, int LPN, bool PLAN>
__global__ __launch_bounds__(BM_BLOCK) void k_gather_axpy(GatherArgs a) {
    gather_axpy_body<W, V, LPN, PLAN>(a);
}
// The same walk over a list of segments, launched behind the dense block of A *^ S: its waves return at once
// unless the block met a value that is not finite (a kernel of its own so that traces tell the two apart).
template <int W, int V, int LPN>
__global__ __launch_bounds__(BM_BLOCK) void k_gather_listed(GatherArgs a) {
    gather_axpy_body<W, V, LPN, true>(a);
}
// The walks whose values sit behind a permutation - all segments of a plan with the values in the caller's order
// (PLAN), the columns of a class-ordered pattern (A * S in passes over the classes) - with each value fetched by a
// scalar load (SV above).
template <int W, int V, int LPN, bool PLAN>
__global__ __launch_bounds__(BM_BLOCK) void k_gather_axpy_sv(GatherArgs a) {
    gather_axpy_body<W, V, LPN, PLAN, true>(a);
}

// ---- DDS, the elementwise step and A*^S in one walk over a plan's segments (an NMF update's
// G = B *^ op(V, DDS(R, B, V))): the segment's row of R stays in registers, every nonzero's column of B is
// gathered once and serves both the dot product and the accumulation, and the products q never travel through
// memory unless the caller asks for them. The arithmetic is that of the two kernels it replaces, step for
// step: the dot product in the lane layout and reduction tree of the DDS kernels (dotacc over the lane's
// vectors, butterfly over the group), the accumulation in the order of k_gather_axpy.
template <int W, int V, int LPN, bool FULL, bool SV = false>
__device__ __forceinline__ float fused_chunk(const GatherArgs& a, int mycol, float myval, int rem, int g, int l,
                                             const int (&eld)[V], const bool (&ev)[V], const Vec<W> (&rr)[V],
                                             Vec<W> (&acc)[V]) {
    constexpr int NG = 64 / LPN;
    constexpr int U = Unroll<V, LPN>::U > 4 ? 4 : Unroll<V, LPN>::U;   // fewer registers buy a fifth wave per SIMD
    const int niter = FULL ? LPN : (rem + NG - 1) / NG;
    float keep = 0.f;                                   // the product of the nonzero this lane loaded
#pragma unroll 1
    for (int it0 = 0; it0 < niter; it0 += U) {
        Vec<W> bv[U][V];
        float vv[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int it = it0 + u;
            int c;
            if constexpr (LPN == 64) {
                c = __builtin_amdgcn_readlane(mycol, it);
                if constexpr (SV) {
                    // (a slot past the end reads position 0: its product is masked below)
                    vv[u] = ((scalar_float*)a.vals)[__builtin_amdgcn_readlane(__float_as_int(myval), it)];
                } else {
                    vv[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(myval), it));
                }
            } else {
                static_assert(!SV, "scalar values: a nonzero's row takes the whole wave");
                const int src = g * LPN + it;
                c = lane_read(mycol, src);
                vv[u] = lane_read(myval, src);
            }
            ok[u] = FULL || (it * NG + g) < rem;
            const float* bp = a.A + (size_t)c * (size_t)a.lda;
            if (ok[u]) {
#pragma unroll
                for (int i = 0; i < V; ++i) bv[u][i] = Vec<W>::load(bp + eld[i]);
            } else {
#pragma unroll
                for (int i = 0; i < V; ++i) bv[u][i] = Vec<W>::zero();
            }
        }
        float qq[U];
        if constexpr ((LPN >= 8) && (U >= 2)) {
            // The U dot products are reduced together (group_multisum: the additions of group_allsum, shared
            // between the lanes), which leaves the sum of slot slot_label(lane) in every lane; that lane applies
            // the op once for its slot, and the U products are then read back from the lanes that hold them.
            float sums[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float s = 0.f;
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    s = rr[i].dotacc(bv[u][i], s);                     // rr is zero in lanes past k
                }
                sums[u] = s;
            }
            const int label = slot_label(l) & (U - 1);
            const float red = group_multisum<LPN, U>(sums, slot_label(l));
            float vmine = vv[0];
#pragma unroll
            for (int u = 1; u < U; ++u) vmine = (label == u) ? vv[u] : vmine;
            const bool okmine = FULL || ((it0 + label) * NG + g) < rem;
            const float qmine = okmine ? binop_rt(a.opn, vmine, red) : 0.f;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int holder = it0 + slot_offset<U>(u, it0);        // the lane of the group that holds slot u
                if constexpr (LPN == 64) qq[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(qmine), holder));
                else qq[u] = lane_read(qmine, g * LPN + holder);
                keep = (l == it0 + u) ? qq[u] : keep;
            }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float s = 0.f;
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    s = rr[i].dotacc(bv[u][i], s);                     // rr is zero in lanes past k
                }
                s = group_allsum<LPN>(s);
                qq[u] = ok[u] ? binop_rt(a.opn, vv[u], s) : 0.f;
                keep = (l == it0 + u) ? qq[u] : keep;
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i].fma(bv[u][i], qq[u]);
        }
    }
    return keep;
}

template <int W, int V, int LPN, bool SV>
__device__ __forceinline__ void fused_rows_body(const GatherArgs& a) {
    const int lane = threadIdx.x & 63;
    const int g = lane / LPN, l = lane % LPN;
    const int xcd = blockIdx.x & 7;
    const long long wi = (long long)(blockIdx.x >> 3) * BM_WAVES_PER_BLOCK + wave_uniform(threadIdx.x >> 6);
    const int hstart = a.xcd_start[xcd];
    const int hcount = a.xcd_start[xcd + 1] - hstart;
    const long long seg = wi < hcount ? hstart + wi : a.xcd_start[8] + (wi - hcount) * 8 + xcd;
    if (seg >= a.nfirst) return;
    const int jstart = a.ptr[seg], jend = a.ptr[seg + 1];
    const int row = a.segrow[seg];
    float* outp = a.out + (size_t)seg * (size_t)a.k;

    int est[V], eld[V];
    bool ev[V];
    Vec<W> acc[V], rr[V];
    const float* rp = a.R + (size_t)row * (size_t)a.ldr;
#pragma unroll
    for (int i = 0; i < V; ++i) {
        est[i] = (i * LPN + l) * W;
        ev[i] = est[i] < a.k;
        eld[i] = ev[i] ? est[i] : 0;
        acc[i] = Vec<W>::zero();
        // lanes past k hold zeros: they contribute nothing to the dot products (masked here, once, not per nonzero)
        rr[i] = ev[i] ? Vec<W>::load(rp + eld[i]) : Vec<W>::zero();
    }
    const int q = l * (64 / LPN) + g;
    int rem = jend - jstart, j0 = jstart;
    int ccol;
    float cval;
    load_chunk<true, SV>(a, j0, 0, rem, q, ccol, cval);
    while (rem > 0) {
        int ncol;
        float nval;
        load_chunk<true, SV>(a, j0, 64, rem - 64, q, ncol, nval);
        float keep;
        if (rem >= 64) keep = fused_chunk<W, V, LPN, true, SV>(a, ccol, cval, 64, g, l, eld, ev, rr, acc);
        else keep = fused_chunk<W, V, LPN, false, SV>(a, ccol, cval, rem, g, l, eld, ev, rr, acc);
        if (a.qout != nullptr && q < rem) {
            const int p = j0 + q;
            a.qout[a.qperm != nullptr ? a.qperm[p] : p] = keep;
        }
        ccol = ncol;
        cval = nval;
        j0 += 64;
        rem -= 64;
    }
#pragma unroll
    for (int m = LPN; m < 64; m <<= 1) {
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] = vec_xor_add<W>(acc[i], m);
    }
    if (g == 0) {
#pragma unroll
        for (int i = 0; i < V; ++i)
            if (ev[i]) acc[i].store(outp + est[i]);
    }
}

template <int W, int V, int LPN>
__global__ __launch_bounds__(BM_BLOCK) void k_fused_rows(GatherArgs a) {
    fused_rows_body<W, V, LPN, false>(a);
}
// V in the caller's order and a row that takes the whole wave: each value by a scalar load (SV above)
template <int W, int V>
__global__ __launch_bounds__(BM_BLOCK) void k_fused_rows_sv(GatherArgs a) {
    fused_rows_body<W, V, 64, true>(a);
}

// The same chain by columns (an LDA E-step: Q = op(V, DDS(A, B, S)), C = beta*C + A * Q): the column of B
// stays in registers, every nonzero's column of A is gathered once for the dot product and the accumulation.
// Segments, overflow partials and the order of the additions are those of k_gather_axpy<..., false>; the dot
// products are those of the DDS kernels. a.R = B (column stride a.ldr), a.A = A.
template <int W, int V, int LPN>
__global__ __launch_bounds__(BM_BLOCK) void k_fused_cols(GatherArgs a) {
    const int lane = threadIdx.x & 63;
    const long long w = (long long)blockIdx.x * BM_WAVES_PER_BLOCK + wave_uniform(threadIdx.x >> 6);
    const int g = lane / LPN, l = lane % LPN;
    int jstart, jend, col;
    float* outp;
    bool accumulate;
    if (w < a.nfirst) {
        // (on a class-ordered pattern: the classes [poff, poff + pspan) of the column's 16 groups; plain CSC: 1, 0, 1)
        const long long pi = w * a.pstride + a.poff;
        const int s = a.ptr[pi], e = a.ptr[pi + a.pspan];
        col = (int)w;
        jstart = s;
        jend = (e - s > a.seglen) ? s + a.seglen : e;
        outp = a.out + (size_t)w * (size_t)a.ldo;
        accumulate = a.beta != 0;
    } else {
        if (a.ovf == nullptr) return;
        const long long x = w - a.nfirst;
        if (x >= a.ovf[a.nfirst]) return;
        int lo = 0, hi = a.nfirst;       // ovf[lo] <= x < ovf[hi]
        while (hi - lo > 1) {
            const int mid = (int)(((long long)lo + hi) >> 1);
            if (a.ovf[mid] <= x) lo = mid; else hi = mid;
        }
        const long long qseg = x - a.ovf[lo] + 1;
        const long long s = (long long)a.ptr[lo] + qseg * a.seglen;
        const long long e = a.ptr[lo + 1];
        col = lo;
        jstart = (int)s;
        jend = (int)((e - s > a.seglen) ? s + a.seglen : e);
        outp = a.partial + (size_t)x * (size_t)a.k;
        accumulate = false;
    }
    int est[V], eld[V];
    bool ev[V];
    Vec<W> acc[V], rr[V];
    const float* rp = a.R + (size_t)col * (size_t)a.ldr;
#pragma unroll
    for (int i = 0; i < V; ++i) {
        est[i] = (i * LPN + l) * W;
        ev[i] = est[i] < a.k;
        eld[i] = ev[i] ? est[i] : 0;
        acc[i] = Vec<W>::zero();
        // lanes past k hold zeros: they contribute nothing to the dot products (masked here, once, not per nonzero)
        rr[i] = ev[i] ? Vec<W>::load(rp + eld[i]) : Vec<W>::zero();
    }
    constexpr bool EARLY_ADDEND = V <= 2;            // as in k_gather_axpy
    Vec<W> addend[V];
    if constexpr (EARLY_ADDEND) {
#pragma unroll
        for (int i = 0; i < V; ++i)
            addend[i] = (accumulate && g == 0 && ev[i]) ? Vec<W>::load(outp + est[i]) : Vec<W>::zero();
    }
    const int q = l * (64 / LPN) + g;
    int rem = jend - jstart, j0 = jstart;
    int crow;
    float cval;
    load_chunk<false>(a, j0, 0, rem, q, crow, cval);
    while (rem > 0) {
        int nrow;
        float nval;
        load_chunk<false>(a, j0, 64, rem - 64, q, nrow, nval);
        float keep;
        if (rem >= 64) keep = fused_chunk<W, V, LPN, true>(a, crow, cval, 64, g, l, eld, ev, rr, acc);
        else keep = fused_chunk<W, V, LPN, false>(a, crow, cval, rem, g, l, eld, ev, rr, acc);
        if (a.qout != nullptr && q < rem) a.qout[a.perm != nullptr ? a.perm[j0 + q] : j0 + q] = keep;
        crow = nrow;
        cval = nval;
        j0 += 64;
        rem -= 64;
    }
#pragma unroll
    for (int m = LPN; m < 64; m <<= 1) {
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] = vec_xor_add<W>(acc[i], m);
    }
    if (g == 0) {
#pragma unroll
        for (int i = 0; i < V; ++i) {
            if (ev[i]) {
                float* o = outp + est[i];
                Vec<W> r = acc[i];
                if constexpr (EARLY_ADDEND) r.add(addend[i]);
                else if (accumulate) r.add(Vec<W>::load(o));
                r.store(o);
            }
        }
    }
}

// C[:,c] += sum of the overflow partials of column c, in segment order.
__global__ __launch_bounds__(BM_BLOCK) void k_overflow_reduce(int k, int ldc, int ncols, const int* __restrict__ ovf,
                                                              const float* __restrict__ partial,
                                                              float* __restrict__ C) {
    const int lane = threadIdx.x & 63;
    const long long w = (long long)blockIdx.x * BM_WAVES_PER_BLOCK + (threadIdx.x >> 6);
    if (w >= ncols) return;
    const int s = ovf[w], e = ovf[w + 1];
    if (s == e) return;
    for (int el = lane; el < k; el += 64) {
        float acc = C[(size_t)w * ldc + el];
        for (int q = s; q < e; ++q) acc += partial[(size_t)q * k + el];
        C[(size_t)w * ldc + el] = acc;
    }
}

// Overflow table of a small or medium matrix in two launches: out[c] = number of extra segments
// in the columns before c, out[ncols] = their total. Pass 1 scans each block of 256 columns and
// leaves block-local prefixes and block totals; in pass 2 every block sums the totals of the blocks
// before it (at most OVF2_MAX_BLOCKS of them) and shifts its prefixes.
constexpr int OVF2_MAX_BLOCKS = 1024;
__global__ __launch_bounds__(BM_BLOCK) void k_overflow_local(int ncols, const int* __restrict__ jc, int seglen,
                                                             int* __restrict__ out, int* __restrict__ bsum) {
    __shared__ int smem[8];
    const long long c = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    int extra = 0;
    if (c < ncols) {
        const int len = jc[c + 1] - jc[c];
        if (len > seglen) extra = (len - 1) / seglen;
    }
    int total;
    const int ex = block_exclusive_scan_256(extra, total, smem);
    if (c < ncols) out[c] = ex;
    if (threadIdx.x == 0) bsum[blockIdx.x] = total;
}

__global__ __launch_bounds__(BM_BLOCK) void k_overflow_shift(int ncols, int* __restrict__ out,
                                                             const int* __restrict__ bsum) {
    __shared__ int smem[8];
    int before = 0;
    for (int b = threadIdx.x; b < (int)blockIdx.x; b += BM_BLOCK) before += bsum[b];
    int total;
    (void)block_exclusive_scan_256(before, total, smem);      // total = sum over the whole block
    const long long c = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (c < ncols) out[c] += total;
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) out[ncols] = total + bsum[blockIdx.x];
}

__global__ __launch_bounds__(BM_BLOCK) void k_extra_segments(int ncols, const int* __restrict__ jc, int seglen,
                                                             int* __restrict__ extra) {
    const long long c = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (c >= ncols) return;
    const int len = jc[c + 1] - jc[c];
    extra[c] = len > seglen ? (len - 1) / seglen : 0;
}

// Plan stage 2: rows handled by groups of LPR lanes.
// Rows [row0, row0+nrows) of the plan; output column (row - row0) of C with stride ldc.
template <int W>
__global__ __launch_bounds__(BM_BLOCK) void k_reduce_segments(int k, int ldc, int row0, int nrows, int lpr,
                                                              const int* __restrict__ rowptr,
                                                              const int* __restrict__ rowseg,
                                                              const float* __restrict__ partial,
                                                              float* __restrict__ C, int beta,
                                                              const int* __restrict__ rowptr2,
                                                              const int* __restrict__ rowseg2,
                                                              const int* __restrict__ flag) {
    const long long t = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long row = t / lpr;
    const int l = (int)(t % lpr);
    if (row >= nrows) return;
    if (rowptr2 != nullptr && *flag == 0) { rowptr = rowptr2; rowseg = rowseg2; }
    const int s = rowptr[row0 + row], e = rowptr[row0 + row + 1];
    for (int el = l * W; el < k; el += lpr * W) {
        float* o = C + (size_t)row * ldc + el;
        Vec<W> acc = beta ? Vec<W>::load(o) : Vec<W>::zero();
        // eight partials in flight at a time; the additions keep their segment order
        int q = s;
        for (; q + 8 <= e; q += 8) {
            Vec<W> p[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) p[u] = Vec<W>::load(partial + (size_t)rowseg[q + u] * k + el);
#pragma unroll
            for (int u = 0; u < 8; ++u) acc.add(p[u]);
        }
        for (; q < e; ++q) acc.add(Vec<W>::load(partial + (size_t)rowseg[q] * k + el));
        acc.store(o);
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Scalar loads of the values where a nonzero's row takes the whole wave (k > 128; k > 32 with one float per lane).
// With two nonzeros per step (k = 128, rows of 512 bytes) the scalar cache does not keep up with the gathers: on a
// 400 M-nonzero pattern the walk over the rows cut by panels took 4.4 ms longer with scalar loads, the rest 0.4 ms.
constexpr int kScalarValuesMinLanes = 64;

template <bool PLAN>
hipError_t launch_gather(const Shape& sh, const GatherArgs& a, long long nwaves, hipStream_t s) {
    if (nwaves <= 0) return hipSuccess;
    long long nblk = (nwaves + BM_WAVES_PER_BLOCK - 1) / BM_WAVES_PER_BLOCK;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    dim3 grid((unsigned)nblk), block(BM_BLOCK);
#define BM_CASE(W_, V_, L_)                                                              \
    if (sh.W == W_ && sh.V == V_ && sh.LPN == L_) {                                      \
        if (PLAN && a.seglist != nullptr)                                                \
            hipLaunchKernelGGL((k_gather_listed<W_, V_, L_>), grid, block, 0, s, a);     \
        else if (L_ >= kScalarValuesMinLanes && a.perm != nullptr && !a.win_on && opt_scalar_values())    \
            hipLaunchKernelGGL((k_gather_axpy_sv<W_, V_, (L_ >= kScalarValuesMinLanes ? L_ : 64), PLAN>), grid, block, 0, s, a); \
        else                                                                             \
            hipLaunchKernelGGL((k_gather_axpy<W_, V_, L_, PLAN>), grid, block, 0, s, a); \
        return hipGetLastError();                                                        \
    }
#define BM_CASES(W_)                                                                     \
    BM_CASE(W_, 1, 1) BM_CASE(W_, 1, 2) BM_CASE(W_, 1, 4) BM_CASE(W_, 1, 8) BM_CASE(W_, 1, 16) \
    BM_CASE(W_, 1, 32) BM_CASE(W_, 1, 64) BM_CASE(W_, 2, 64) BM_CASE(W_, 4, 64)
    BM_CASES(1)
    BM_CASES(4)
#undef BM_CASES
#undef BM_CASE
    return hipErrorInvalidValue;
}

}  // namespace

// Columns wider than 4*64 vectors are processed in passes of V = 4 inside the kernel.
static Shape clamp_shape(Shape sh) {
    if (sh.V > 4) sh.V = 4;
    return sh;
}

size_t overflow_table_ints(int ncols) {
    // table area (2*ncols + 2 ints, rounded to 64) followed by the scan's block sums
    const size_t area = ((2 * (size_t)ncols + 2) + 63) & ~size_t(63);
    return area + scan_tmp_ints(ncols);
}

hipError_t build_overflow_table_in(int ncols, int nnz, const int* jc, int seglen, int* buf, int** d_ovf, hipStream_t s) {
    *d_ovf = nullptr;
    if (nnz <= seglen || ncols <= 0) return hipSuccess;
    unsigned nblk = (unsigned)(((long long)ncols + BM_BLOCK - 1) / BM_BLOCK);
    if (nblk <= (unsigned)OVF2_MAX_BLOCKS) {
        int* bsum = buf + ncols + 1;
        hipLaunchKernelGGL(k_overflow_local, dim3(nblk), dim3(BM_BLOCK), 0, s, ncols, jc, seglen, buf, bsum);
        hipLaunchKernelGGL(k_overflow_shift, dim3(nblk), dim3(BM_BLOCK), 0, s, ncols, buf, bsum);
        *d_ovf = buf;
        return hipGetLastError();
    }
    int* tmp = buf + (((2 * (size_t)ncols + 2) + 63) & ~size_t(63));
    int* extra = buf;
    int* ovf = buf + ncols + 1;
    hipLaunchKernelGGL(k_extra_segments, dim3(nblk), dim3(BM_BLOCK), 0, s, ncols, jc, seglen, extra);
    hipError_t err = scan_exclusive_i32(extra, ovf, ncols, tmp, s);
    if (err != hipSuccess) return err;
    *d_ovf = ovf;
    return hipGetLastError();
}

hipError_t build_overflow_table(int ncols, int nnz, const int* jc, int seglen, int** d_ovf, hipStream_t s) {
    *d_ovf = nullptr;
    if (nnz <= seglen || ncols <= 0) return hipSuccess;
    hipError_t err;
    int* buf = (int*)ws_get(WS_OVF, sizeof(int) * overflow_table_ints(ncols), &err, s);
    if (!buf) return err;
    return build_overflow_table_in(ncols, nnz, jc, seglen, buf, d_ovf, s);
}

namespace {
void init_args(GatherArgs& a) {
    a.win_on = 0; a.win_off = 0; a.win_len = 0;
    a.segrow = nullptr; a.row_off = 0; a.row_len = 0;
    for (int x = 0; x < 9; ++x) a.xcd_start[x] = 0;
    a.pstride = 1; a.poff = 0; a.pspan = 1;
    a.R = nullptr; a.ldr = 0; a.opn = 0; a.qout = nullptr; a.qperm = nullptr;
    a.skip = nullptr; a.flag = nullptr; a.seglist = nullptr;
}
}  // namespace

hipError_t dsmult_csc(int k, int ncols, int nnz, const float* A, const float* vals, const int* ir,
                      const int* jc, float* C, int beta, hipStream_t s, const ColTable* tab) {
    return dsmult_csc_ex(k, k, k, ncols, nnz, A, vals, ir, jc, C, beta, Window{0, 0, 0}, s, tab);
}

hipError_t dsmult_csc_ex(int k, int lda, int ldc, int ncols, int nnz, const float* A, const float* vals,
                         const int* ir, const int* jc, float* C, int beta, Window rows, hipStream_t s,
                         const ColTable* tab) {
    if (k <= 0 || ncols <= 0) return hipSuccess;
    int seglen = opt_seglen();
    int* ovf = nullptr;
    float* partial = nullptr;
    long long novf_max = 0;
    hipError_t err;
    if (tab) {
        // the caller knows the pattern's overflow segments: nothing to build, nothing to allocate
        seglen = tab->seglen;
        if (tab->novf > 0) {
            ovf = const_cast<int*>(tab->ovf);
            novf_max = tab->novf;
            partial = (float*)ws_get(WS_PARTIAL, sizeof(float) * (size_t)novf_max * (size_t)k, &err, s);
            if (!partial) return err;
        }
    } else {
        err = build_overflow_table(ncols, nnz, jc, seglen, &ovf, s);
        if (err != hipSuccess) return err;
        if (ovf) {
            novf_max = nnz / seglen;
            partial = (float*)ws_get(WS_PARTIAL, sizeof(float) * (size_t)novf_max * (size_t)k, &err, s);
            if (!partial) return err;
        }
    }
    const bool al = aligned16(A) && aligned16(C) && aligned16(partial) && lda % 4 == 0 && ldc % 4 == 0;
    Shape sh = clamp_shape(pick_shape(k, al));
    GatherArgs a;
    init_args(a);
    a.k = k; a.lda = lda; a.ldo = ldc; a.nfirst = ncols; a.seglen = seglen; a.beta = beta;
    a.A = A; a.vals = vals; a.idx = ir; a.perm = nullptr; a.ptr = jc; a.ovf = ovf;
    a.out = C; a.partial = partial;
    a.win_on = rows.on; a.win_off = rows.off; a.win_len = rows.len;
    err = launch_gather<false>(sh, a, (long long)ncols + novf_max, s);
    if (err != hipSuccess) return err;
    if (ovf) {
        unsigned nblk = (unsigned)(((long long)ncols + BM_WAVES_PER_BLOCK - 1) / BM_WAVES_PER_BLOCK);
        hipLaunchKernelGGL(k_overflow_reduce, dim3(nblk), dim3(BM_BLOCK), 0, s, k, ldc, ncols, ovf, partial, C);
        err = hipGetLastError();
    }
    return err;
}

// A*S over a class-ordered pattern in `nphase` passes, one launch each: pass p only gathers the rows
// of classes [8*p/nphase, 8*(p+1)/nphase), and the passes follow each other on the stream. While
// a pass runs, every L2 of the device only sees that pass's share of the rows, so it holds
// nphase times as many of the rows that matter as when all rows compete for it; the price is one
// read-modify-write of C per extra pass. The order of the additions (pass by pass, class by class,
// stored order inside a class) depends on the pattern alone.
hipError_t dsmult_phased(int k, int ncols, const float* A, const float* vals, const int* cir, const int* cperm,
                         const int* cptr, int nphase, float* C, int beta, hipStream_t s) {
    if (k <= 0 || ncols <= 0) return hipSuccess;
    if (nphase != 1 && nphase != 2 && nphase != 4 && nphase != 8) return hipErrorInvalidValue;
    const bool al = aligned16(A) && aligned16(C);
    Shape sh = clamp_shape(pick_shape(k, al));
    GatherArgs a;
    init_args(a);
    a.k = k; a.lda = k; a.ldo = k; a.nfirst = ncols; a.seglen = 0x7fffffff;
    a.A = A; a.vals = vals; a.idx = cir; a.perm = cperm; a.ptr = cptr; a.ovf = nullptr;
    a.out = C; a.partial = nullptr;
    a.pstride = 16; a.pspan = 16 / nphase;
    for (int p = 0; p < nphase; ++p) {
        a.poff = p * a.pspan;
        a.beta = p == 0 ? beta : 1;
        hipError_t err = launch_gather<false>(sh, a, (long long)ncols, s);
        if (err != hipSuccess) return err;
    }
    return hipSuccess;
}

namespace {
hipError_t gather_segments_impl(int k, int lda, int nseg, const int* xcd_start, const float* A,
                                const float* vals, const int* pc, const int* perm, const int* segstart,
                                float* partial, Window cols, const int* segrow, Window rowsel, hipStream_t s,
                                const unsigned char* skip, int* flag);
}

hipError_t gather_segments(int k, int nseg, const int* xcd_start, const float* A, const float* vals,
                           const int* pc, const int* perm, const int* segstart, float* partial,
                           hipStream_t s, const unsigned char* skip, int* flag) {
    return gather_segments_impl(k, k, nseg, xcd_start, A, vals, pc, perm, segstart, partial,
                                Window{0, 0, 0}, nullptr, Window{0, 0, 0}, s, skip, flag);
}

hipError_t gather_segments_listed(int k, int n, const int* list, const int* flag, const float* A, const float* vals,
                                  const int* pc, const int* perm, const int* segstart, float* partial, hipStream_t s) {
    if (k <= 0 || n <= 0) return hipSuccess;
    Shape sh = clamp_shape(pick_shape(k, aligned16(A) && aligned16(partial)));
    GatherArgs a;
    init_args(a);
    a.k = k; a.lda = k; a.ldo = k; a.nfirst = n; a.seglen = 0; a.beta = 0;
    a.A = A; a.vals = vals; a.idx = pc; a.perm = perm; a.ptr = segstart; a.ovf = nullptr;
    a.out = partial; a.partial = nullptr;
    a.seglist = list; a.flag = const_cast<int*>(flag);
    return launch_gather<true>(sh, a, n, s);
}

hipError_t gather_segments_ex(int k, int lda, int nseg, const int* xcd_start, const float* A,
                              const float* vals, const int* pc, const int* perm, const int* segstart,
                              float* partial, Window cols, const int* segrow, Window rowsel, hipStream_t s) {
    return gather_segments_impl(k, lda, nseg, xcd_start, A, vals, pc, perm, segstart, partial, cols, segrow, rowsel, s,
                                nullptr, nullptr);
}

namespace {
hipError_t gather_segments_impl(int k, int lda, int nseg, const int* xcd_start, const float* A,
                                const float* vals, const int* pc, const int* perm, const int* segstart,
                                float* partial, Window cols, const int* segrow, Window rowsel, hipStream_t s,
                                const unsigned char* skip, int* flag) {
    if (k <= 0 || nseg <= 0) return hipSuccess;
    Shape sh = clamp_shape(pick_shape(k, aligned16(A) && aligned16(partial) && lda % 4 == 0));
    GatherArgs a;
    init_args(a);
    a.k = k; a.lda = lda; a.ldo = k; a.nfirst = nseg; a.seglen = 0; a.beta = 0;
    a.A = A; a.vals = vals; a.idx = pc; a.perm = perm; a.ptr = segstart; a.ovf = nullptr;
    a.out = partial; a.partial = nullptr;
    a.win_on = cols.on; a.win_off = cols.off; a.win_len = cols.len;
    if (rowsel.on) { a.segrow = segrow; a.row_off = rowsel.off; a.row_len = rowsel.len; }
    a.skip = skip; a.flag = flag;
    int maxheavy = 0;
    for (int x = 0; x < 9; ++x) a.xcd_start[x] = xcd_start[x];
    for (int x = 0; x < 8; ++x) maxheavy = std::max(maxheavy, a.xcd_start[x + 1] - a.xcd_start[x]);
    const long long nlight = (long long)nseg - a.xcd_start[8];
    // waves per XCD, rounded up to whole workgroups, times 8 XCDs
    const long long per_xcd = (long long)maxheavy + (nlight + 7) / 8;
    const long long blocks_per_xcd = (per_xcd + BM_WAVES_PER_BLOCK - 1) / BM_WAVES_PER_BLOCK;
    return launch_gather<true>(sh, a, blocks_per_xcd * 8 * BM_WAVES_PER_BLOCK, s);
}
}  // namespace

hipError_t fused_segments(int k, int ldr, int lda, int nseg, const int* xcd_start, const int* segrow,
                          const float* R, const float* A, const float* vals, const int* pc, const int* perm,
                          const int* qperm, int opn, const int* segstart, float* partial, float* qout,
                          hipStream_t s) {
    if (k <= 0 || nseg <= 0) return hipSuccess;
    Shape sh = pick_shape(k, aligned16(A) && aligned16(R) && aligned16(partial) && lda % 4 == 0 && ldr % 4 == 0);
    if (sh.V > 4) return hipErrorInvalidValue;          // one pass must cover k
    GatherArgs a;
    init_args(a);
    a.k = k; a.lda = lda; a.ldo = k; a.nfirst = nseg; a.seglen = 0; a.beta = 0;
    a.A = A; a.vals = vals; a.idx = pc; a.perm = perm; a.ptr = segstart; a.ovf = nullptr;
    a.out = partial; a.partial = nullptr;
    a.segrow = segrow;
    a.R = R; a.ldr = ldr; a.opn = opn; a.qout = qout; a.qperm = qperm;
    int maxheavy = 0;
    for (int x = 0; x < 9; ++x) a.xcd_start[x] = xcd_start[x];
    for (int x = 0; x < 8; ++x) maxheavy = std::max(maxheavy, a.xcd_start[x + 1] - a.xcd_start[x]);
    const long long nlight = (long long)nseg - a.xcd_start[8];
    const long long per_xcd = (long long)maxheavy + (nlight + 7) / 8;
    const long long blocks_per_xcd = (per_xcd + BM_WAVES_PER_BLOCK - 1) / BM_WAVES_PER_BLOCK;
    const long long nblk = blocks_per_xcd * 8;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    dim3 grid((unsigned)nblk), block(BM_BLOCK);
#define BM_CASE(W_, V_, L_)                                                              \
    if (sh.W == W_ && sh.V == V_ && sh.LPN == L_) {                                      \
        if (L_ >= kScalarValuesMinLanes && a.perm != nullptr && opt_scalar_values())     \
            hipLaunchKernelGGL((k_fused_rows_sv<W_, V_>), grid, block, 0, s, a);         \
        else                                                                             \
            hipLaunchKernelGGL((k_fused_rows<W_, V_, L_>), grid, block, 0, s, a);        \
        return hipGetLastError();                                                        \
    }
#define BM_CASES(W_)                                                                     \
    BM_CASE(W_, 1, 1) BM_CASE(W_, 1, 2) BM_CASE(W_, 1, 4) BM_CASE(W_, 1, 8) BM_CASE(W_, 1, 16) \
    BM_CASE(W_, 1, 32) BM_CASE(W_, 1, 64) BM_CASE(W_, 2, 64) BM_CASE(W_, 4, 64)
    BM_CASES(1)
    BM_CASES(4)
#undef BM_CASES
#undef BM_CASE
    return hipErrorInvalidValue;
}

hipError_t fused_columns(int k, int ncols, int nnz, const float* A, const float* B, const float* vals, const int* ir,
                         const int* jc, int opn, float* Q, float* C, int beta, hipStream_t s, const ColTable* tab) {
    if (k <= 0 || ncols <= 0) return hipSuccess;
    int seglen = opt_seglen();
    int* ovf = nullptr;
    float* partial = nullptr;
    long long novf_max = 0;
    hipError_t err;
    if (tab) {
        seglen = tab->seglen;
        if (tab->novf > 0) {
            ovf = const_cast<int*>(tab->ovf);
            novf_max = tab->novf;
        }
    } else {
        err = build_overflow_table(ncols, nnz, jc, seglen, &ovf, s);
        if (err != hipSuccess) return err;
        if (ovf) novf_max = nnz / seglen;
    }
    if (ovf) {
        partial = (float*)ws_get(WS_PARTIAL, sizeof(float) * (size_t)novf_max * (size_t)k, &err, s);
        if (!partial) return err;
    }
    const bool al = aligned16(A) && aligned16(B) && aligned16(C) && aligned16(partial);
    Shape sh = pick_shape(k, al);
    if (sh.V > 4) return hipErrorInvalidValue;          // one pass must cover k
    GatherArgs a;
    init_args(a);
    a.k = k; a.lda = k; a.ldo = k; a.nfirst = ncols; a.seglen = seglen; a.beta = beta;
    a.A = A; a.vals = vals; a.idx = ir; a.perm = nullptr; a.ptr = jc; a.ovf = ovf;
    a.out = C; a.partial = partial;
    a.R = B; a.ldr = k; a.opn = opn; a.qout = Q;
    const long long nwaves = (long long)ncols + novf_max;
    const long long nblk = (nwaves + BM_WAVES_PER_BLOCK - 1) / BM_WAVES_PER_BLOCK;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    dim3 grid((unsigned)nblk), block(BM_BLOCK);
    bool launched = false;
#define BM_CASE(W_, V_, L_)                                                              \
    if (!launched && sh.W == W_ && sh.V == V_ && sh.LPN == L_) {                         \
        hipLaunchKernelGGL((k_fused_cols<W_, V_, L_>), grid, block, 0, s, a);            \
        launched = true;                                                                 \
    }
#define BM_CASES(W_)                                                                     \
    BM_CASE(W_, 1, 1) BM_CASE(W_, 1, 2) BM_CASE(W_, 1, 4) BM_CASE(W_, 1, 8) BM_CASE(W_, 1, 16) \
    BM_CASE(W_, 1, 32) BM_CASE(W_, 1, 64) BM_CASE(W_, 2, 64) BM_CASE(W_, 4, 64)
    BM_CASES(1)
    BM_CASES(4)
#undef BM_CASES
#undef BM_CASE
    if (!launched) return hipErrorInvalidValue;
    if ((err = hipGetLastError()) != hipSuccess) return err;
    if (ovf) {
        unsigned rblk = (unsigned)(((long long)ncols + BM_WAVES_PER_BLOCK - 1) / BM_WAVES_PER_BLOCK);
        hipLaunchKernelGGL(k_overflow_reduce, dim3(rblk), dim3(BM_BLOCK), 0, s, k, k, ncols, ovf, partial, C);
        err = hipGetLastError();
    }
    return err;
}

// The chain by columns over a class-ordered pattern in `nphase` passes (see dsmult_phased): pass p takes the row
// classes [8p/nphase, 8(p+1)/nphase) of every column, computes their products q (written through cperm) and adds their
// share to C, so that every L2 sees 1/nphase of the rows at a time; the first pass honours beta, the others accumulate.
hipError_t fused_columns_phased(int k, int ncols, const float* A, const float* B, const float* vals, const int* cir,
                                const int* cperm, const int* cptr, int nphase, int opn, float* Q, float* C, int beta,
                                hipStream_t s) {
    if (k <= 0 || ncols <= 0) return hipSuccess;
    if (nphase != 1 && nphase != 2 && nphase != 4 && nphase != 8) return hipErrorInvalidValue;
    Shape sh = pick_shape(k, aligned16(A) && aligned16(B) && aligned16(C));
    if (sh.V > 4) return hipErrorInvalidValue;          // one pass must cover k
    GatherArgs a;
    init_args(a);
    a.k = k; a.lda = k; a.ldo = k; a.nfirst = ncols; a.seglen = 0x7fffffff;
    a.A = A; a.vals = vals; a.idx = cir; a.perm = cperm; a.ptr = cptr; a.ovf = nullptr;
    a.out = C; a.partial = nullptr;
    a.R = B; a.ldr = k; a.opn = opn; a.qout = Q;
    a.pstride = 16; a.pspan = 16 / nphase;
    const long long nblk = ((long long)ncols + BM_WAVES_PER_BLOCK - 1) / BM_WAVES_PER_BLOCK;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    dim3 grid((unsigned)nblk), block(BM_BLOCK);
    for (int p = 0; p < nphase; ++p) {
        a.poff = p * a.pspan;
        a.beta = p == 0 ? beta : 1;
        bool launched = false;
#define BM_CASE(W_, V_, L_)                                                              \
        if (!launched && sh.W == W_ && sh.V == V_ && sh.LPN == L_) {                     \
            hipLaunchKernelGGL((k_fused_cols<W_, V_, L_>), grid, block, 0, s, a);        \
            launched = true;                                                             \
        }
#define BM_CASES(W_)                                                                     \
        BM_CASE(W_, 1, 1) BM_CASE(W_, 1, 2) BM_CASE(W_, 1, 4) BM_CASE(W_, 1, 8) BM_CASE(W_, 1, 16) \
        BM_CASE(W_, 1, 32) BM_CASE(W_, 1, 64) BM_CASE(W_, 2, 64) BM_CASE(W_, 4, 64)
        BM_CASES(1)
        BM_CASES(4)
#undef BM_CASES
#undef BM_CASE
        if (!launched) return hipErrorInvalidValue;
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    return hipSuccess;
}

hipError_t reduce_segments(int k, int nrows, const int* rowptr, const int* rowseg,
                           const float* partial, float* C, int beta, hipStream_t s, const int* rowptr2,
                           const int* rowseg2, const int* flag) {
    return reduce_segments_ex(k, k, 0, nrows, rowptr, rowseg, partial, C, beta, s, rowptr2, rowseg2, flag);
}

hipError_t reduce_segments_ex(int k, int ldc, int row0, int nrows, const int* rowptr, const int* rowseg,
                              const float* partial, float* C, int beta, hipStream_t s, const int* rowptr2,
                              const int* rowseg2, const int* flag) {
    if (rowptr2 == nullptr || rowseg2 == nullptr || flag == nullptr) { rowptr2 = nullptr; rowseg2 = nullptr; flag = nullptr; }
    if (k <= 0 || nrows <= 0) return hipSuccess;
    const bool al = aligned16(C) && aligned16(partial) && (k % 4 == 0) && (ldc % 4 == 0);
    const int W = al ? 4 : 1;
    int nv = (k + W - 1) / W;
    int lpr = pow2ceil(nv) < 64 ? pow2ceil(nv) : 64;
    long long threads = (long long)nrows * lpr;
    long long nblk = (threads + BM_BLOCK - 1) / BM_BLOCK;
    if (nblk > 0x7fffffffLL) return hipErrorInvalidValue;
    if (al) hipLaunchKernelGGL(k_reduce_segments<4>, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, k, ldc, row0, nrows, lpr, rowptr, rowseg, partial, C, beta, rowptr2, rowseg2, flag);
    else hipLaunchKernelGGL(k_reduce_segments<1>, dim3((unsigned)nblk), dim3(BM_BLOCK), 0, s, k, ldc, row0, nrows, lpr, rowptr, rowseg, partial, C, beta, rowptr2, rowseg2, flag);
    return hipGetLastError();
}

}  // namespace bm
