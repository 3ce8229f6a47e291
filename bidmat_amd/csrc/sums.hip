// Column / row reductions of sparse values and of dense matrices. All are streaming,
// bandwidth-bound kernels; every result is the same from run to run: float sums have a fixed order
// (two-stage, no atomics), and the one kernel that adds in arrival order adds exact integers.
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

// Row sums straight from the column-ordered arrays (row index and value per nonzero, any order),
// for values the caller has just produced. A float sum taken in arrival order would change from
// run to run, so the sums are taken exactly instead: with E the binary exponent of the largest
// finite magnitude and cb the bits of the nonzero count, every value is rounded once to a multiple
// of 2^(E + cb - 61) (values within 2^-(37 - cb) of the largest keep all 24 bits; the step is
// below 2^-34 of the largest for up to 2^27 nonzeros) and added as a 64-bit integer, which cannot
// overflow and does not depend on the order. One rounding to float at the end. A row holding NaN or
// infinities of both signs sums to NaN, one with infinities of one sign to that infinity.
//
// Pass 1 finds the largest finite magnitude (per-block maxima) and clears the flags; pass 3 converts.
// Pass 2 comes in two forms. Atomic adds to global memory leave the XCD (its L2 is not shared with
// the other seven) and run at a small fraction of the rate of loads, so the form for up to
// 16 * RS_RANGE_SLOTS rows uses none: the rows are dealt to R = 1..16 ranges by their low bits, a
// workgroup owns one range with all its accumulators in LDS, and the R workgroups of a group stream
// the same stretch of (row, value) pairs, each adding only the rows of its range. The R workgroups of
// a group sit on one XCD and start together, so the stretch comes from HBM once and R - 1 times from
// that XCD's L2. Every workgroup stores its table, and pass 3 adds the tables of all groups. For more
// rows than that, each workgroup keeps a direct-mapped table of row accumulators in LDS, claimed by
// the first row that hashes to a slot (the frequent rows claim theirs within the first few hundred
// nonzeros), sends the rest to accumulators in global memory, and flushes its table at the end.
constexpr int RS_SLOTS_LOG = 12, RS_SLOTS = 1 << RS_SLOTS_LOG, RS_BLOCK = 512, RS_MAXPART = 1024;
constexpr int RS_RANGE_SLOTS = 16384, RS_RANGE_BLOCK = 1024, RS_MAX_LOGR = 4;
constexpr size_t RS_RANGE_LDS = 8 * (size_t)RS_RANGE_SLOTS + 8 * 128 * (RS_RANGE_BLOCK / 64);   // tables + rings
constexpr int RS_MAXBLOCKS = 768;     // three tables fit the LDS of each of the 256 CUs
constexpr int RS_NAN = 1, RS_PINF = 2, RS_NINF = 4, RS_BADROW = 8;

__global__ __launch_bounds__(BM_BLOCK) void k_rowsum_prepare(long long nnz, const float* __restrict__ vals,
                                                            unsigned* __restrict__ part, int nrows,
                                                            unsigned long long* __restrict__ acc,
                                                            int* __restrict__ flags) {
    const long long gsz = (long long)gridDim.x * BM_BLOCK, t = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    for (long long r = t; r < nrows; r += gsz) { acc[r] = 0ull; flags[r] = 0; }
    if (t == 0) flags[nrows] = 0;
    unsigned m = 0;
    const long long n4 = nnz >> 2;
    const uint4* v4 = reinterpret_cast<const uint4*>(vals);
    const bool aligned = (reinterpret_cast<uintptr_t>(vals) & 15) == 0;
    auto take = [&](unsigned b) { b &= 0x7fffffffu; if (b < 0x7f800000u && b > m) m = b; };
    if (aligned) {
        for (long long i = t; i < n4; i += gsz) { const uint4 q = v4[i]; take(q.x); take(q.y); take(q.z); take(q.w); }
        for (long long i = (n4 << 2) + t; i < nnz; i += gsz) take(__float_as_uint(vals[i]));
    } else {
        for (long long i = t; i < nnz; i += gsz) take(__float_as_uint(vals[i]));
    }
    for (int o = 32; o > 0; o >>= 1) { const unsigned y = __shfl_xor(m, o, 64); m = y > m ? y : m; }
    __shared__ unsigned wm[BM_BLOCK / 64];
    if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < BM_BLOCK / 64; ++w) m = wm[w] > m ? wm[w] : m;
        part[blockIdx.x] = m;
    }
}

// The power of two every value is multiplied with, as two factors that each fit a float.
struct RsScale { float s1, s2; int sh; };
__device__ __forceinline__ RsScale rs_scale(unsigned maxbits, long long nnz) {
    int e = (int)(maxbits >> 23) - 127;                       // |v| < 2^(e+1) for every finite v
    if (e < -126) e = -126;
    const int cb = 64 - __clzll((unsigned long long)nnz);       // nnz < 2^cb
    RsScale r;
    r.sh = 61 - e - cb;                                       // |sum of q| < 2^(e+1+cb+sh) = 2^62
    const int a = r.sh / 2, b = r.sh - a;                     // |sh| <= 61 + 126 + 1: halves fit a float
    r.s1 = __uint_as_float((unsigned)(a + 127) << 23);
    r.s2 = __uint_as_float((unsigned)(b + 127) << 23);
    return r;
}

// q = round-to-nearest-even(v * 2^sh) as a 64-bit integer; |q| <= 2^61. v finite. The magnitude is split
// into its part above 2^32 and the rest; both are exact floats because the product has 24 significant bits.
__device__ __forceinline__ long long rs_quantise(float v, const RsScale& sc) {
    const float x = __builtin_rintf((__builtin_fabsf(v) * sc.s1) * sc.s2);
    const float hi = __builtin_floorf(x * 2.3283064365386963e-10f);
    const float lo = __builtin_fmaf(hi, -4294967296.f, x);
    const long long mag = (long long)(((unsigned long long)(unsigned)hi << 32) | (unsigned long long)(unsigned)lo);
    return (__float_as_uint(v) >> 31) ? -mag : mag;
}

__global__ __launch_bounds__(RS_BLOCK) void k_rowsum_exact(long long nnz, int nrows, const int* __restrict__ ir,
                                                          const float* __restrict__ vals,
                                                          const unsigned* __restrict__ part, int nparts,
                                                          unsigned long long* __restrict__ acc,
                                                          int* __restrict__ flags, long long per_block) {
    __shared__ unsigned long long lacc[RS_SLOTS];
    __shared__ int ltag[RS_SLOTS];
    __shared__ unsigned wm[RS_BLOCK / 64];
    for (int i = threadIdx.x; i < RS_SLOTS; i += RS_BLOCK) { lacc[i] = 0ull; ltag[i] = -1; }
    unsigned m = 0;
    for (int i = threadIdx.x; i < nparts; i += RS_BLOCK) { const unsigned y = part[i]; m = y > m ? y : m; }
    for (int o = 32; o > 0; o >>= 1) { const unsigned y = __shfl_xor(m, o, 64); m = y > m ? y : m; }
    if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = m;
    __syncthreads();
    m = wm[0];
    for (int w = 1; w < RS_BLOCK / 64; ++w) m = wm[w] > m ? wm[w] : m;
    const RsScale sc = rs_scale(m, nnz);

    auto add = [&](int row, float v) {
        const unsigned b = __float_as_uint(v);
        if ((unsigned)row >= (unsigned)nrows) { atomicOr(&flags[nrows], RS_BADROW); return; }
        if ((b & 0x7f800000u) == 0x7f800000u) {
            atomicOr(&flags[row], (b & 0x007fffffu) ? RS_NAN : (b >> 31) ? RS_NINF : RS_PINF);
            return;
        }
        const long long q = rs_quantise(v, sc);
        if (q == 0) return;
        const int slot = (int)(((unsigned)row * 0x9E3779B1u) >> (32 - RS_SLOTS_LOG));
        int tag = ltag[slot];
        if (tag == -1) { tag = atomicCAS(&ltag[slot], -1, row); if (tag == -1) tag = row; }
        if (tag == row) atomicAdd(&lacc[slot], (unsigned long long)q);
        else atomicAdd(&acc[row], (unsigned long long)q);
    };

    const long long lo = (long long)blockIdx.x * per_block, hi = lo + per_block < nnz ? lo + per_block : nnz;
    const bool aligned = ((reinterpret_cast<uintptr_t>(vals) | reinterpret_cast<uintptr_t>(ir)) & 15) == 0;
    if (aligned) {                                            // per_block is a multiple of 4
        const int4* r4 = reinterpret_cast<const int4*>(ir);
        const float4* v4 = reinterpret_cast<const float4*>(vals);
        const long long q0 = lo >> 2, q1 = hi >> 2;
        long long i = q0 + threadIdx.x;
        for (; i + RS_BLOCK < q1; i += 2 * RS_BLOCK) {
            const int4 ra = r4[i], rb = r4[i + RS_BLOCK];
            const float4 va = v4[i], vb = v4[i + RS_BLOCK];
            add(ra.x, va.x); add(ra.y, va.y); add(ra.z, va.z); add(ra.w, va.w);
            add(rb.x, vb.x); add(rb.y, vb.y); add(rb.z, vb.z); add(rb.w, vb.w);
        }
        for (; i < q1; i += RS_BLOCK) {
            const int4 ra = r4[i]; const float4 va = v4[i];
            add(ra.x, va.x); add(ra.y, va.y); add(ra.z, va.z); add(ra.w, va.w);
        }
        for (long long j = (q1 << 2) + threadIdx.x; j < hi; j += RS_BLOCK) add(ir[j], vals[j]);
    } else {
        for (long long j = lo + threadIdx.x; j < hi; j += RS_BLOCK) add(ir[j], vals[j]);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < RS_SLOTS; i += RS_BLOCK) {
        const int tag = ltag[i];
        const unsigned long long q = lacc[i];
        if (tag >= 0 && q != 0ull) atomicAdd(&acc[tag], q);
    }
}

// Of the (row, value) pairs a workgroup streams only one in R is its own, so a wave first packs its own pairs
// into a small ring in LDS (a compare, a ballot and one LDS store per pair met) and runs the arithmetic only on
// full sets of 64 taken from the ring: the conversion and the LDS atomic then cost a 1/R share per pair met.
constexpr int RS_RING = 128;                      // pairs per wave: at most 63 waiting + 64 new
template <int LOGR>
__global__ __launch_bounds__(RS_RANGE_BLOCK) void k_rowsum_ranged(long long nnz, int nrows, int nslots,
                                                                 const int* __restrict__ ir,
                                                                 const float* __restrict__ vals,
                                                                 const unsigned* __restrict__ part, int nparts,
                                                                 unsigned long long* __restrict__ tables,
                                                                 int* __restrict__ flags, long long per_group) {
    extern __shared__ unsigned long long racc[];  // nslots accumulators, then RS_RING entries per wave
    __shared__ unsigned wm[RS_RANGE_BLOCK / 64];
    constexpr int R = 1 << LOGR;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int range = idx & (R - 1);
    const int g = xcd * ((gridDim.x >> 3) >> LOGR) + (idx >> LOGR);   // groups of one XCD are consecutive
    int* ring = reinterpret_cast<int*>(racc + nslots) + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) * (2 * RS_RING);
    const int lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < nslots; i += RS_RANGE_BLOCK) racc[i] = 0ull;
    unsigned m = 0;
    for (int i = threadIdx.x; i < nparts; i += RS_RANGE_BLOCK) { const unsigned y = part[i]; m = y > m ? y : m; }
    for (int o = 32; o > 0; o >>= 1) { const unsigned y = __shfl_xor(m, o, 64); m = y > m ? y : m; }
    if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = m;
    __syncthreads();
    m = wm[0];
    for (int w = 1; w < RS_RANGE_BLOCK / 64; ++w) m = wm[w] > m ? wm[w] : m;
    const RsScale sc = rs_scale(m, nnz);

    int tail = 0;                                 // pairs waiting in the ring; the same in every lane
    // Many lanes adding to one LDS address are served one after the other, and with rows drawn from a power law
    // half the lanes of a set may hold the same row. The wave therefore keeps one row apart (`hot`, the same in
    // every lane) whose values each lane adds up in registers; when fewer than four lanes of a set hold it, the
    // row of the set's first other lane takes its place. Integer sums: any choice gives the same result.
    int hot = -1;
    unsigned long long hacc = 0ull;
    auto flush_hot = [&]() {
        if (hacc != 0ull) { atomicAdd(&racc[hot >> LOGR], hacc); hacc = 0ull; }
    };
    // Called by all 64 lanes together.
    auto consume = [&](int2 e, bool on) {
        const int row = e.x;
        const unsigned b = (unsigned)e.y;
        bool ok = on;
        if (ok && (unsigned)row >= (unsigned)nrows) { atomicOr(&flags[nrows], RS_BADROW); ok = false; }
        if (ok && (b & 0x7f800000u) == 0x7f800000u) {
            atomicOr(&flags[row], (b & 0x007fffffu) ? RS_NAN : (b >> 31) ? RS_NINF : RS_PINF);
            ok = false;
        }
        const unsigned long long q = ok ? (unsigned long long)rs_quantise(__uint_as_float(b), sc) : 0ull;
        const bool ishot = ok && row == hot;
        const int nhot = __builtin_popcountll(__ballot(ishot));
        if (ishot) hacc += q;
        else if (q != 0ull) atomicAdd(&racc[row >> LOGR], q);
        if (nhot < 4) {
            const unsigned long long others = __ballot(ok && !ishot);
            if (others != 0ull) {
                flush_hot();
                hot = __builtin_amdgcn_readlane(row, __builtin_ctzll(others));
            }
        }
    };
    // Called by all 64 lanes together, lanes without a pair with a row of another range (R > 1) or valid == false
    // (R == 1). Fewer than 64 pairs wait when it is entered, at [0, tail): rows at ring[i], values at
    // ring[RS_RING + i]; a full set is taken from the front and the rest moves down.
    auto push = [&](bool valid, int row, float v) {
        const bool mine = R == 1 ? valid : (row & (R - 1)) == range;
        const unsigned long long mask = __builtin_amdgcn_ballot_w64(mine);
        if (mine) {
            const int cnt = (int)__builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32),
                                                           __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
            int* at = ring + tail;
            at[cnt] = row;
            at[cnt + RS_RING] = (int)__float_as_uint(v);
        }
        tail += __builtin_popcountll(mask);
        if (tail >= 64) {
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            const int2 e = make_int2(ring[lane], ring[lane + RS_RING]);
            const int2 up = make_int2(ring[lane + 64], ring[lane + 64 + RS_RING]);
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            tail -= 64;
            if (lane < tail) { ring[lane] = up.x; ring[lane + RS_RING] = up.y; }
            consume(e, true);
        }
    };
    const int other = range ^ 1;                  // a row of another range when R > 1

    const long long lo = (long long)g * per_group, hi = lo + per_group < nnz ? lo + per_group : nnz;
    const bool aligned = ((reinterpret_cast<uintptr_t>(vals) | reinterpret_cast<uintptr_t>(ir)) & 15) == 0;
    long long done = lo;                          // pairs [lo, done) have been pushed
    if (aligned && hi > lo) {                     // lo is a multiple of 4
        const int4* r4 = reinterpret_cast<const int4*>(ir);
        const float4* v4 = reinterpret_cast<const float4*>(vals);
        const long long q0 = lo >> 2, q1 = hi >> 2;
        // the loads of the next step are on their way while this step's pairs are packed
        int4 ra, rb;
        float4 va, vb;
        bool oa, ob;
        auto fetch = [&](long long base) {
            const long long ia = base + threadIdx.x, ib = ia + RS_RANGE_BLOCK;
            oa = ia < q1; ob = ib < q1;
            ra = rb = make_int4(other, other, other, other);
            va = vb = make_float4(0.f, 0.f, 0.f, 0.f);
            if (oa) { ra = r4[ia]; va = v4[ia]; }
            if (ob) { rb = r4[ib]; vb = v4[ib]; }
        };
        fetch(q0);
        for (long long base = q0; base < q1; base += 2 * RS_RANGE_BLOCK) {
            const int4 ca = ra, cb = rb;
            const float4 wa = va, wb = vb;
            const bool pa = oa, pb = ob;
            fetch(base + 2 * RS_RANGE_BLOCK);
            push(pa, ca.x, wa.x); push(pa, ca.y, wa.y); push(pa, ca.z, wa.z); push(pa, ca.w, wa.w);
            push(pb, cb.x, wb.x); push(pb, cb.y, wb.y); push(pb, cb.z, wb.z); push(pb, cb.w, wb.w);
        }
        done = q1 << 2;
    }
    for (long long base = done; base < hi; base += RS_RANGE_BLOCK) {
        const long long j = base + threadIdx.x;
        const bool ok = j < hi;
        push(ok, ok ? ir[j] : other, ok ? vals[j] : 0.f);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    consume(make_int2(ring[lane], ring[lane + RS_RING]), lane < tail);
    flush_hot();
    __syncthreads();
    unsigned long long* mine = tables + ((size_t)g * R + range) * (size_t)nslots;
    for (int i = threadIdx.x; i < nslots; i += RS_RANGE_BLOCK) mine[i] = racc[i];
}

// out[slot * R + range] (+)= sum over groups of tables[group][range][slot], scaled back.
__global__ __launch_bounds__(BM_BLOCK) void k_rowsum_finish_ranged(long long nnz, int nrows, int nslots, int logr,
                                                                  int ngroups, const unsigned* __restrict__ part,
                                                                  int nparts,
                                                                  const unsigned long long* __restrict__ tables,
                                                                  const int* __restrict__ flags,
                                                                  float* __restrict__ out, int beta) {
    __shared__ unsigned wm[BM_BLOCK / 64];
    unsigned m = 0;
    for (int i = threadIdx.x; i < nparts; i += BM_BLOCK) { const unsigned y = part[i]; m = y > m ? y : m; }
    for (int o = 32; o > 0; o >>= 1) { const unsigned y = __shfl_xor(m, o, 64); m = y > m ? y : m; }
    if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = m;
    __syncthreads();
    m = wm[0];
    for (int w = 1; w < BM_BLOCK / 64; ++w) m = wm[w] > m ? wm[w] : m;
    const RsScale sc = rs_scale(m, nnz);
    const long long t = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const int R = 1 << logr;
    if (t >= (long long)nslots * R || (flags[nrows] & RS_BADROW)) return;
    const int range = (int)(t / nslots), slot = (int)(t - (long long)range * nslots);
    const long long r = ((long long)slot << logr) + range;
    if (r >= nrows) return;
    unsigned long long a = 0ull;
    for (int g = 0; g < ngroups; ++g) a += tables[((size_t)g * R + range) * (size_t)nslots + slot];
    const int f = flags[r];
    float v;
    if ((f & RS_NAN) || ((f & RS_PINF) && (f & RS_NINF))) v = __uint_as_float(0x7fc00000u);
    else if (f & RS_PINF) v = INFINITY;
    else if (f & RS_NINF) v = -INFINITY;
    else v = (float)ldexp((double)(long long)a, -sc.sh);
    out[r] = beta ? out[r] + v : v;
}

__global__ __launch_bounds__(BM_BLOCK) void k_rowsum_finish(long long nnz, int nrows, const unsigned* __restrict__ part,
                                                           int nparts, const unsigned long long* __restrict__ acc,
                                                           const int* __restrict__ flags, float* __restrict__ out,
                                                           int beta) {
    __shared__ unsigned wm[BM_BLOCK / 64];
    unsigned m = 0;
    for (int i = threadIdx.x; i < nparts; i += BM_BLOCK) { const unsigned y = part[i]; m = y > m ? y : m; }
    for (int o = 32; o > 0; o >>= 1) { const unsigned y = __shfl_xor(m, o, 64); m = y > m ? y : m; }
    if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = m;
    __syncthreads();
    m = wm[0];
    for (int w = 1; w < BM_BLOCK / 64; ++w) m = wm[w] > m ? wm[w] : m;
    const RsScale sc = rs_scale(m, nnz);
    const long long r = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (r >= nrows || (flags[nrows] & RS_BADROW)) return;       // a row index outside the output: write nothing
    const int f = flags[r];
    float v;
    if ((f & RS_NAN) || ((f & RS_PINF) && (f & RS_NINF))) v = __uint_as_float(0x7fc00000u);
    else if (f & RS_PINF) v = INFINITY;
    else if (f & RS_NINF) v = -INFINITY;
    else v = (float)ldexp((double)(long long)acc[r], -sc.sh);
    out[r] = beta ? out[r] + v : v;
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

// Whether a workgroup may take the LDS the ranged row sums ask for (144 KiB of the 160 KiB of a gfx950 CU).
bool rowsum_lds_fits() {
    static int fits[64];                      // 0 = not asked yet, 1 = yes, 2 = no
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
    if (!fits[dev]) {
        int v = 0;
        const bool ok = hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess &&
                        (size_t)v >= RS_RANGE_LDS + 256;
        fits[dev] = ok ? 1 : 2;
    }
    return fits[dev] == 1;
}

hipError_t spsum_rows_exact(int nrows, long long nnz, const int* ir, const float* vals, float* out, int beta,
                            int* bad_rows, hipStream_t s) {
    if (nrows <= 0) return hipSuccess;
    hipError_t err;
    // [ part: RS_MAXPART u32 | acc: nrows u64 | flags: nrows + 1 int ]
    const size_t bytes = sizeof(unsigned) * RS_MAXPART + sizeof(unsigned long long) * (size_t)nrows +
                         sizeof(int) * ((size_t)nrows + 1);
    char* base = (char*)ws_get(WS_ROWSUM, bytes, &err, s);
    if (!base) return err;
    unsigned* part = (unsigned*)base;
    unsigned long long* acc = (unsigned long long*)(base + sizeof(unsigned) * RS_MAXPART);
    int* flags = (int*)(acc + nrows);
    long long want = (nnz / 4 + BM_BLOCK - 1) / BM_BLOCK, rows_blk = ((long long)nrows + BM_BLOCK - 1) / BM_BLOCK;
    if (want < rows_blk) want = rows_blk;
    const int nparts = (int)(want < 1 ? 1 : want > RS_MAXPART ? RS_MAXPART : want);
    int logr = 0;
    while (logr <= RS_MAX_LOGR && ((long long)RS_RANGE_SLOTS << logr) < nrows) ++logr;
    const bool ranged = logr <= RS_MAX_LOGR && opt_rowsum_form() != 2 && rowsum_lds_fits();
    hipLaunchKernelGGL(k_rowsum_prepare, dim3(nparts), dim3(BM_BLOCK), 0, s, nnz, vals, part, nrows, acc, flags);
    if (ranged) {
        // 256 workgroups at most, one per CU: 8 XCDs x (groups per XCD) x R ranges.
        const int R = 1 << logr, nslots = (nrows + R - 1) >> logr;
        int gpx = (32 >> logr) < 1 ? 1 : (32 >> logr);                         // groups per XCD
        const long long want_groups = (nnz + 8 * RS_RANGE_BLOCK - 1) / (8 * RS_RANGE_BLOCK);
        while (gpx > 1 && 8LL * (gpx / 2) >= want_groups) gpx /= 2;
        const int ngroups = 8 * gpx;
        const long long per_group = (((nnz + ngroups - 1) / ngroups) + 3) & ~3LL;
        const size_t table_bytes = sizeof(unsigned long long) * (size_t)ngroups * R * nslots;
        unsigned long long* tables = (unsigned long long*)ws_get(WS_ROWSUM_TABLES, table_bytes, &err, s);
        if (!tables) return err;
        const size_t lds = sizeof(unsigned long long) * (size_t)nslots + sizeof(int2) * RS_RING * (RS_RANGE_BLOCK / 64);
        const unsigned nblk = (unsigned)(ngroups * R);
#define BM_RANGED(L)                                                                                              \
    case L: {                                                                                                     \
        static bool set[64] = {};                                                                                 \
        int dev = 0;                                                                                              \
        (void)hipGetDevice(&dev);                                                                                 \
        if (dev >= 0 && dev < 64 && !set[dev]) {                                                                  \
            err = hipFuncSetAttribute(reinterpret_cast<const void*>(k_rowsum_ranged<L>),                          \
                                      hipFuncAttributeMaxDynamicSharedMemorySize,                                 \
                                      (int)RS_RANGE_LDS);                                                         \
            if (err != hipSuccess) return err;                                                                    \
            set[dev] = true;                                                                                      \
        }                                                                                                         \
        hipLaunchKernelGGL(k_rowsum_ranged<L>, dim3(nblk), dim3(RS_RANGE_BLOCK), lds, s, nnz, nrows, nslots, ir,  \
                           vals, part, nparts, tables, flags, per_group);                                         \
    } break;
        switch (logr) {
            BM_RANGED(0) BM_RANGED(1) BM_RANGED(2) BM_RANGED(3) BM_RANGED(4)
        }
#undef BM_RANGED
        const long long fblk = ((long long)nslots * R + BM_BLOCK - 1) / BM_BLOCK;
        hipLaunchKernelGGL(k_rowsum_finish_ranged, dim3((unsigned)fblk), dim3(BM_BLOCK), 0, s, nnz, nrows, nslots, logr,
                           ngroups, part, nparts, tables, flags, out, beta);
    } else {
        if (nnz > 0) {
            long long nblk = (nnz + 8 * RS_BLOCK - 1) / (8 * RS_BLOCK);             // at least 8 nonzeros a lane
            if (nblk > RS_MAXBLOCKS) nblk = RS_MAXBLOCKS;
            long long per_block = ((nnz + nblk - 1) / nblk + 3) & ~3LL;
            nblk = (nnz + per_block - 1) / per_block;
            hipLaunchKernelGGL(k_rowsum_exact, dim3((unsigned)nblk), dim3(RS_BLOCK), 0, s, nnz, nrows, ir, vals, part,
                               nparts, acc, flags, per_block);
        }
        const long long fblk = ((long long)nrows + BM_BLOCK - 1) / BM_BLOCK;
        hipLaunchKernelGGL(k_rowsum_finish, dim3((unsigned)fblk), dim3(BM_BLOCK), 0, s, nnz, nrows, part, nparts, acc,
                           flags, out, beta);
    }
    if ((err = hipGetLastError()) != hipSuccess) return err;
    if (bad_rows) {                                                           // blocking callers only
        int f = 0;
        if ((err = hipMemcpyAsync(&f, flags + nrows, sizeof(int), hipMemcpyDeviceToHost, s)) != hipSuccess) return err;
        if ((err = hipStreamSynchronize(s)) != hipSuccess) return err;
        *bad_rows = (f & RS_BADROW) != 0;
    }
    return hipSuccess;
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
