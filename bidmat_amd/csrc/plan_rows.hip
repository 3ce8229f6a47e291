// Row side of a plan without a general sort. The plan order is "by key, then by position in the CSC
// arrays", with key = (panel slot, heavy rank) for nonzeros of heavy rows and key = row for the others.
// The columns of a panel are contiguous in CSC order, so the heavy nonzeros only need a stable counting
// sort PER PANEL over the heavy ranks (a few thousand bins, kept in LDS), and the light nonzeros one
// stable radix sort by row in passes of at most 8 bits. Ranks follow the position in the input (a wave
// ranks its 64 entries by ballots, the waves of a workgroup take turns on the tile's LDS counters), so
// the result is the unique stable order: the same arrays, bit for bit, as sorting (key, position) pairs.
//
// Data movement: a store of 4 bytes to a place of its own costs the memory system a whole request, and a
// CU holds only about a hundred of them in flight, so every scatter here goes through LDS first: the
// heavy nonzeros' places are a permutation that is applied in two steps (entries are grouped by blocks
// of 8192 destination positions, then every block is put in order inside LDS and written out whole), and
// the light passes sort a tile inside LDS and write runs. Integer work only.
#include "plan.hpp"
#include "common.hpp"
#include "kernels.hpp"
#include "scan.hpp"
#include "workspace.hpp"

namespace bm {
namespace {

constexpr int RB_CHUNK = BM_BLOCK;                 // entries a workgroup ranks per step
constexpr int RB_TILE_NNZ = 48 * 1024;             // aimed-at nonzeros per (panel, column range) tile
constexpr int RB_LIGHT_TILE = 16 * RB_CHUNK;       // entries per tile of the light-row passes (staged in LDS)
constexpr int RB_LIGHT_BITS = 8;                   // at most 256 bins per light pass: runs of 16 and more per tile
constexpr int RB_SUB = 8 * RB_CHUNK;               // entries a workgroup of the grouping step stages in LDS
constexpr int RB_SUBS_PER_TILE = 32;               // a tile holds at most 65535 nonzeros
constexpr int RB_DBLOCK = 8192;                    // destination positions per block of the placement step
constexpr int RB_MAX_DBINS = 512;                  // destination blocks one panel's heavy stretch may span

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

inline int bits_for(unsigned long long maxval) {
    int b = 1;
    while (b < 32 && (maxval >> b) != 0) ++b;
    return b;
}

// Rank of every lane among the lanes of its wave that hold the same key (in lane order), and the size
// of that group. nbits: bits of the key that can differ.
__device__ __forceinline__ void wave_match(unsigned key, bool valid, int nbits, int& rank, int& count) {
    unsigned long long peers = __ballot(valid);
    for (int b = 0; b < nbits; ++b) {
        const bool bit = (key >> b) & 1u;
        const unsigned long long m = __ballot(bit);
        peers &= bit ? m : ~m;
    }
    const unsigned long long below = (1ULL << (threadIdx.x & 63)) - 1ULL;
    rank = __popcll(peers & below);
    count = __popcll(peers);
}

// Workgroup barrier that orders LDS accesses only. __syncthreads() also waits for every global store the
// wave has in flight, and the ranking loops issue scattered stores between their LDS turns: four such
// waits per step made the stores' latency, not the ranking, the time of these kernels.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// The waves of the workgroup take their turn on the tile's running positions pos[] (LDS): a wave reads
// the position of each of its keys, then the first lane of every group of equal keys moves it on by the
// group's size. Returns where this lane's entry goes. All threads must call it.
__device__ __forceinline__ int take_positions(int* pos, unsigned key, bool valid, int nbits) {
    int rank, count;
    wave_match(key, valid, nbits, rank, count);
    const int wave = threadIdx.x >> 6;
    int mine = 0;
    for (int w = 0; w < BM_WAVES_PER_BLOCK; ++w) {
        if (wave == w && valid) {
            mine = pos[key];                       // every lane of a group reads before its leader writes:
            if (rank == 0) pos[key] = mine + count;    // LDS operations of one wave execute in order
        }
        lds_barrier();
    }
    return mine + rank;
}

// The same for N entries per lane: a wave owns N * 64 consecutive entries of the input (entry u of lane l is
// its (u * 64 + l)-th) and takes its turn once for all of them, so the workgroup meets at four barriers per
// N * 256 entries. at[u] receives the places.
template <int N, typename T>
__device__ __forceinline__ void take_positions_n(T* pos, const unsigned (&key)[N], const bool (&valid)[N], int nbits,
                                                 int (&at)[N]) {
    int rank[N], count[N];
#pragma unroll
    for (int u = 0; u < N; ++u) wave_match(key[u], valid[u], nbits, rank[u], count[u]);
    const int wave = threadIdx.x >> 6;
    for (int w = 0; w < BM_WAVES_PER_BLOCK; ++w) {
        if (wave == w) {
#pragma unroll
            for (int u = 0; u < N; ++u) {
                if (valid[u]) {
                    const int mine = (int)pos[key[u]];
                    if (rank[u] == 0) pos[key[u]] = (T)(mine + count[u]);
                    at[u] = mine + rank[u];
                }
            }
        }
        lds_barrier();
    }
}

// A panel's column range is cut into tiles; tile t of panel P covers columns [P*panel_cols + t*tcols, ...).
struct Tiling {
    int ncols, npanels, panel_cols, tpp, tcols, p8, nheavy;
    __host__ __device__ int tiles() const { return npanels * tpp; }
    __device__ void columns(int tile, int& c0, int& c1) const {
        const int P = tile / tpp, t = tile - P * tpp;
        const long long pend = (long long)(P + 1) * panel_cols < ncols ? (long long)(P + 1) * panel_cols : ncols;
        long long a = (long long)P * panel_cols + (long long)t * tcols, b = a + tcols;
        if (a > pend) a = pend;
        if (b > pend) b = pend;
        c0 = (int)a; c1 = (int)b;
    }
    // panels are ordered by the XCD that will own them: panel p -> slot (p % 8) * p8 + p / 8
    __host__ __device__ int slot(int P) const { return (P & 7) * p8 + (P >> 3); }
};

// Exclusive scan of v[0..n) in LDS by the whole workgroup (n <= 8 * BM_BLOCK), in place. Its barriers order
// LDS accesses only (global operations of the caller stay in flight across it).
__device__ __forceinline__ void lds_exclusive_scan(int* v, int n, int* smem8) {
    constexpr int PER = 8;
    int x[PER], sum = 0;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int idx = (int)threadIdx.x * PER + i;
        x[i] = idx < n ? v[idx] : 0;
        sum += x[i];
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int inc = sum;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int t = __shfl_up(inc, d, 64);
        if (lane >= d) inc += t;
    }
    if (lane == 63) smem8[wave] = inc;
    lds_barrier();
    int run = inc - sum;
#pragma unroll
    for (int w = 0; w < BM_WAVES_PER_BLOCK; ++w)
        if (w < wave) run += smem8[w];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int idx = (int)threadIdx.x * PER + i;
        if (idx < n) v[idx] = run;
        run += x[i];
    }
    lds_barrier();
}

// ---- pass 1 over the pattern, one workgroup per tile: the rank of every nonzero among the tile's nonzeros
// with the same key (heavy rank, or `nheavy` for all light rows), in CSC order, and the tile's count per key.
// what[j] = key << 16 | rank; hist[tile*(nheavy+1) + key]. Every row index is checked here. A tile with more
// than 65535 nonzeros sets *toolong (the caller then sorts instead).
__global__ __launch_bounds__(BM_BLOCK) void k_tile_rank(Tiling tg, int nrows, int nbits, const int* __restrict__ jc,
                                                        const int* __restrict__ ir, const int* __restrict__ hcode,
                                                        int* __restrict__ hist, unsigned* __restrict__ what,
                                                        int* __restrict__ bad, int* __restrict__ toolong) {
    // ranks and counts inside a tile stay below 65536: 16-bit counters halve the LDS a workgroup holds, and
    // eight workgroups instead of seven fit a CU
    extern __shared__ unsigned short pos[];
    const int nb = tg.nheavy + 1;
    for (int i = threadIdx.x; i < nb; i += BM_BLOCK) pos[i] = 0;
    __syncthreads();
    int c0, c1;
    tg.columns(blockIdx.x, c0, c1);
    const int js = jc[c0], je = jc[c1];
    if (je - js > 0xffff) {
        if (threadIdx.x == 0) *toolong = 1;
        return;
    }
    constexpr int UN = 4;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // Two steps ahead: while step s is ranked (a chain of LDS turns), the codes of step s+1 and the rows of
    // step s+2 are on their way.
    auto rows_of = [&](int jb, int (&r)[UN]) {
        const int j0 = jb + wave * (UN * 64) + lane;
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int j = j0 + u * 64;
            r[u] = j < je ? ir[j] : 0;
            if ((unsigned)r[u] >= (unsigned)nrows) { *bad = 1; r[u] = 0; }
        }
    };
    int r1[UN], r2[UN], h0[UN], h1[UN];
    rows_of(js, r1);
#pragma unroll
    for (int u = 0; u < UN; ++u) h0[u] = hcode[r1[u]];
    rows_of(js + UN * RB_CHUNK, r1);
    for (int jb = js; jb < je; jb += UN * RB_CHUNK) {
        // wave w owns the UN * 64 consecutive nonzeros from jb + w * UN * 64 on
        const int j0 = jb + wave * (UN * 64) + lane;
#pragma unroll
        for (int u = 0; u < UN; ++u) h1[u] = hcode[r1[u]];                  // step s+1
        rows_of(jb + 2 * UN * RB_CHUNK, r2);                               // step s+2
        int at[UN];
        unsigned key[UN];
        bool valid[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            valid[u] = j0 + u * 64 < je;
            key[u] = h0[u] >= 0 ? (unsigned)h0[u] : (unsigned)tg.nheavy;
            at[u] = 0;
        }
        take_positions_n<UN, unsigned short>(pos, key, valid, nbits, at);
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            if (valid[u]) what[j0 + u * 64] = (key[u] << 16) | (unsigned)at[u];
            h0[u] = h1[u];
            r1[u] = r2[u];
        }
    }
    __syncthreads();
    int* mine = hist + (size_t)blockIdx.x * nb;
    for (int i = threadIdx.x; i < nb; i += BM_BLOCK) mine[i] = (int)pos[i];
}

// ---- per (panel, bin): the tiles' counts become exclusive prefixes inside the panel; the panel's total
// goes to keytot[slot(panel)*nheavy + rank] (heavy bins) / ltot[panel] (light bin).
__global__ __launch_bounds__(BM_BLOCK) void k_panel_prefix(Tiling tg, int* __restrict__ hist, int* __restrict__ keytot,
                                                           int* __restrict__ ltot) {
    const int nb = tg.nheavy + 1;
    const long long idx = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (idx >= (long long)tg.npanels * nb) return;
    const int P = (int)(idx / nb), bin = (int)(idx - (long long)P * nb);
    int run = 0;
    for (int t = 0; t < tg.tpp; ++t) {
        int* p = hist + (size_t)(P * tg.tpp + t) * nb + bin;
        const int v = *p;
        *p = run;
        run += v;
    }
    if (bin < tg.nheavy) keytot[(size_t)tg.slot(P) * tg.nheavy + bin] = run;
    else ltot[P] = run;
}

// hist[tile][key] (count of the key in the panel's earlier tiles) += keybase[slot(panel)*nheavy + key] for the
// heavy keys, += lbase[panel] for the light bin: the first place of the tile's nonzeros of every key.
__global__ __launch_bounds__(BM_BLOCK) void k_add_base(Tiling tg, const int* __restrict__ keybase, const int* __restrict__ lbase,
                                                       int* __restrict__ hist) {
    const int nb = tg.nheavy + 1;
    const long long idx = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (idx >= (long long)tg.tiles() * nb) return;
    const int tile = (int)(idx / nb), key = (int)(idx - (long long)tile * nb);
    const int P = tile / tg.tpp;
    hist[idx] += key < tg.nheavy ? keybase[(size_t)tg.slot(P) * tg.nheavy + key] : lbase[P];
}

// First and last column of every (tile, sub) span of RB_SUB nonzeros: subcols[2*(tile*SUBS+sub) + {0,1}]
// (-1: the span is empty). One thread per span.
__global__ __launch_bounds__(BM_BLOCK) void k_sub_columns(Tiling tg, const int* __restrict__ jc, int* __restrict__ subcols) {
    const long long idx = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (idx >= (long long)tg.tiles() * RB_SUBS_PER_TILE) return;
    const int tile = (int)(idx / RB_SUBS_PER_TILE), sub = (int)(idx - (long long)tile * RB_SUBS_PER_TILE);
    int c0, c1;
    tg.columns(tile, c0, c1);
    const int tje = jc[c1];
    const long long js = (long long)jc[c0] + (long long)sub * RB_SUB;
    if (js >= tje) { subcols[2 * idx] = -1; subcols[2 * idx + 1] = -1; return; }
    const int je = (int)(js + RB_SUB < tje ? js + RB_SUB : tje);
    int lo = c0, hi = c1 - 1;
    while (lo < hi) { const int mid = (lo + hi + 1) >> 1; if (jc[mid] <= (int)js) lo = mid; else hi = mid - 1; }
    subcols[2 * idx] = lo;
    hi = c1 - 1;
    while (lo < hi) { const int mid = (lo + hi + 1) >> 1; if (jc[mid] <= je - 1) lo = mid; else hi = mid - 1; }
    subcols[2 * idx + 1] = lo;
}

// ---- pass 2 over the pattern, workgroup (tile, sub): RB_SUB consecutive nonzeros of a tile. A heavy
// nonzero's place is dest = keybase[its key] + (count of the key in the panel's earlier tiles) + its rank.
// The places of a panel's heavy nonzeros fill one stretch of the plan arrays; the stretch is cut into blocks
// of RB_DBLOCK positions, and this step only brings every entry (dest, column, position) into the scratch
// region of its block: the workgroup sorts its entries by block inside LDS, reserves room in each block's
// region with one atomic per block (the order inside a region does not matter: the next step places by
// dest) and writes runs. Light nonzeros go, in CSC order, to (lrow, lcol, lpos).
__global__ __launch_bounds__(BM_BLOCK) void k_group(Tiling tg, int heavy_total, const int* __restrict__ jc,
                                                    const int* __restrict__ ir, const unsigned* __restrict__ what,
                                                    const int* __restrict__ hist, const int* __restrict__ keybase,
                                                    const int* __restrict__ subcols, int* __restrict__ fill,
                                                    int* __restrict__ td, int* __restrict__ tc, int* __restrict__ tj,
                                                    int* __restrict__ lrow, int* __restrict__ lcol, int* __restrict__ lpos) {
    __shared__ int sd[RB_SUB], sc[RB_SUB], sj[RB_SUB + 1];
    __shared__ int cnt[RB_MAX_DBINS], lstart[RB_MAX_DBINS], gbase[RB_MAX_DBINS];
    __shared__ int smem8[8];
    int* const cols = sj;                 // the column pointers live where the staged positions go later
    const int tile = blockIdx.x, sub = blockIdx.y;
    const int cfirst = subcols[2 * ((size_t)tile * RB_SUBS_PER_TILE + sub)];
    if (cfirst < 0) return;                                        // no nonzeros in this span
    const int clast = subcols[2 * ((size_t)tile * RB_SUBS_PER_TILE + sub) + 1];
    int c0, c1;
    tg.columns(tile, c0, c1);
    const int tje = jc[c1];
    const int js = jc[c0] + sub * RB_SUB;
    const int je = js + RB_SUB < tje ? js + RB_SUB : tje;
    const int P = tile / tg.tpp;
    const int nb = tg.nheavy + 1;
    const int* kb = keybase + (size_t)tg.slot(P) * tg.nheavy;
    const int* hp = hist + (size_t)tile * nb;                    // first place of the tile's nonzeros of every key
    const int stretch0 = kb[0], stretch1 = kb[tg.nheavy];       // the panel's heavy nonzeros: plan positions [stretch0, stretch1)
    const int bfirst = stretch0 / RB_DBLOCK;
    const int nbins = stretch1 > stretch0 ? (stretch1 - 1) / RB_DBLOCK - bfirst + 1 : 0;
    const int lfirst = hp[tg.nheavy];                              // first light slot of this tile
    const int ncl = clast - cfirst + 1;
    const bool cols_in_lds = ncl <= RB_SUB;
    if (cols_in_lds)
        for (int i = threadIdx.x; i <= ncl; i += BM_BLOCK) cols[i] = jc[cfirst + i];
    for (int i = threadIdx.x; i < nbins; i += BM_BLOCK) cnt[i] = 0;
    __syncthreads();

    constexpr int PER = RB_SUB / BM_BLOCK;
    int d[PER], c[PER];
    unsigned w[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const int j = js + u * BM_BLOCK + (int)threadIdx.x;
        w[u] = j < je ? what[j] : 0xffffffffu;
    }
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const int j = js + u * BM_BLOCK + (int)threadIdx.x;
        d[u] = -1; c[u] = 0;
        if (j < je) {
            const int key = (int)(w[u] >> 16), rank = (int)(w[u] & 0xffffu);
            // column of j: the last one that starts at or before j
            int lo = 0, hi = ncl - 1;
            if (cols_in_lds) {
                while (lo < hi) { const int mid = (lo + hi + 1) >> 1; if (cols[mid] <= j) lo = mid; else hi = mid - 1; }
            } else {
                while (lo < hi) { const int mid = (lo + hi + 1) >> 1; if (jc[cfirst + mid] <= j) lo = mid; else hi = mid - 1; }
            }
            c[u] = cfirst + lo;
            if (key < tg.nheavy) {
                d[u] = hp[key] + rank;
                atomicAdd(&cnt[d[u] / RB_DBLOCK - bfirst], 1);
            } else {
                const int q = lfirst + rank;
                lrow[q] = ir[j]; lcol[q] = c[u]; lpos[q] = j;
            }
        }
    }
    __syncthreads();
    if (nbins == 0) return;
    // room in every destination block's region (the reply of the atomic is only needed for the write-out, so it
    // stays in a register across the staging), then the entries in block order inside LDS
    int room[(RB_MAX_DBINS + BM_BLOCK - 1) / BM_BLOCK];
#pragma unroll
    for (int t = 0; t < (RB_MAX_DBINS + BM_BLOCK - 1) / BM_BLOCK; ++t) {
        const int i = t * BM_BLOCK + (int)threadIdx.x;
        room[t] = 0;
        if (i < nbins) {
            const int k = cnt[i];
            if (k > 0) room[t] = atomicAdd(&fill[bfirst + i], k);
            lstart[i] = k;
        }
    }
    lds_barrier();
    lds_exclusive_scan(lstart, nbins, smem8);
    for (int i = threadIdx.x; i < nbins; i += BM_BLOCK) cnt[i] = lstart[i];      // running slots
    lds_barrier();
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        if (d[u] >= 0) {
            const int slot = atomicAdd(&cnt[d[u] / RB_DBLOCK - bfirst], 1);
            sd[slot] = d[u]; sc[slot] = c[u]; sj[slot] = js + u * BM_BLOCK + (int)threadIdx.x;
        }
    }
#pragma unroll
    for (int t = 0; t < (RB_MAX_DBINS + BM_BLOCK - 1) / BM_BLOCK; ++t) {
        const int i = t * BM_BLOCK + (int)threadIdx.x;
        if (i < nbins) gbase[i] = room[t];
    }
    __syncthreads();
    const int nheavy_here = cnt[nbins - 1];                       // the last bin's running slot: all staged entries
    for (int i = threadIdx.x; i < nheavy_here; i += BM_BLOCK) {
        const int dd = sd[i];
        const int b = dd / RB_DBLOCK - bfirst;
        const size_t o = (size_t)(bfirst + b) * RB_DBLOCK + (size_t)(gbase[b] + (i - lstart[b]));
        td[o] = dd; tc[o] = sc[i]; tj[o] = sj[i];
    }
}

// ---- the placement, one workgroup per block of RB_DBLOCK plan positions: its entries sit, in any order,
// in the block's scratch region; they are put in place inside LDS and the block is written out whole.
constexpr int RB_FILL_THREADS = 1024;
__global__ __launch_bounds__(RB_FILL_THREADS) void k_fill_block(int heavy_total, const int* __restrict__ td,
                                                                const int* __restrict__ tc, const int* __restrict__ tj,
                                                                int* __restrict__ pc, int* __restrict__ perm) {
    __shared__ int lc[RB_DBLOCK], lj[RB_DBLOCK];
    const long long base = (long long)blockIdx.x * RB_DBLOCK;
    const int n = (int)(heavy_total - base < RB_DBLOCK ? heavy_total - base : RB_DBLOCK);
    for (int i = threadIdx.x; i < n; i += RB_FILL_THREADS) {
        const int at = td[base + i] - (int)base;
        lc[at] = tc[base + i];
        lj[at] = tj[base + i];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += RB_FILL_THREADS) {
        pc[base + i] = lc[i];
        perm[base + i] = lj[i];
    }
}

// ---- light rows: one stable pass by bits [shift, shift+bits) of the row.
// counts go to table[bin*ntiles + tile], so that one flat exclusive scan of the table gives every
// (bin, tile) its first output position.
__global__ __launch_bounds__(BM_BLOCK) void k_light_count(int n, int shift, int nbins, int ntiles,
                                                          const int* __restrict__ lrow, int* __restrict__ table) {
    __shared__ int bins[1 << RB_LIGHT_BITS];
    for (int i = threadIdx.x; i < nbins; i += BM_BLOCK) bins[i] = 0;
    __syncthreads();
    const long long s = (long long)blockIdx.x * RB_LIGHT_TILE;
    const long long e = s + RB_LIGHT_TILE < n ? s + RB_LIGHT_TILE : n;
    for (long long i = s + threadIdx.x; i < e; i += BM_BLOCK) atomicAdd(&bins[(lrow[i] >> shift) & (nbins - 1)], 1);
    __syncthreads();
    for (int i = threadIdx.x; i < nbins; i += BM_BLOCK) table[(size_t)i * ntiles + blockIdx.x] = bins[i];
}

// The tile is put in order inside LDS (stable: ranks by take_positions), then written out bin by bin, so
// that neighbouring threads write neighbouring places. counts: the table k_light_count wrote, first: its
// exclusive scan. LAST: the pass by the top bits writes the plan arrays (from position `heavy_total` on)
// and the sorted rows.
template <bool LAST>
__global__ __launch_bounds__(BM_BLOCK) void k_light_scatter(int n, int shift, int nbins, int nbits, int ntiles,
                                                            const int* __restrict__ counts, const int* __restrict__ first,
                                                            const int* __restrict__ lrow, const int* __restrict__ lcol,
                                                            const int* __restrict__ lpos, int* __restrict__ orow,
                                                            int* __restrict__ ocol, int* __restrict__ opos,
                                                            int heavy_total) {
    __shared__ int sr[RB_LIGHT_TILE], sc[RB_LIGHT_TILE], sp[RB_LIGHT_TILE];
    __shared__ int lstart[1 << RB_LIGHT_BITS], run[1 << RB_LIGHT_BITS], gfirst[1 << RB_LIGHT_BITS];
    __shared__ int smem8[8];
    for (int i = threadIdx.x; i < nbins; i += BM_BLOCK) {
        lstart[i] = counts[(size_t)i * ntiles + blockIdx.x];
        gfirst[i] = first[(size_t)i * ntiles + blockIdx.x];
    }
    __syncthreads();
    lds_exclusive_scan(lstart, nbins, smem8);
    for (int i = threadIdx.x; i < nbins; i += BM_BLOCK) run[i] = lstart[i];
    __syncthreads();
    const long long s = (long long)blockIdx.x * RB_LIGHT_TILE;
    const long long e = s + RB_LIGHT_TILE < n ? s + RB_LIGHT_TILE : n;
    constexpr int UN = 4;
    for (long long ib = s; ib < e; ib += UN * RB_CHUNK) {
        int r[UN], c[UN], p[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const long long i = ib + u * RB_CHUNK + threadIdx.x;
            const bool valid = i < e;
            r[u] = valid ? lrow[i] : 0; c[u] = valid ? lcol[i] : 0; p[u] = valid ? lpos[i] : 0;
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            if (ib + u * RB_CHUNK >= e) break;                       // uniform over the workgroup
            const bool valid = ib + u * RB_CHUNK + threadIdx.x < e;
            const unsigned key = (unsigned)(r[u] >> shift) & (unsigned)(nbins - 1);
            const int at = take_positions(run, key, valid, nbits);
            if (valid) { sr[at] = r[u]; sc[at] = c[u]; sp[at] = p[u]; }
        }
    }
    __syncthreads();
    const int m = (int)(e - s);
    for (int i = threadIdx.x; i < m; i += BM_BLOCK) {
        const int r = sr[i];
        const int b = (r >> shift) & (nbins - 1);
        const int o = gfirst[b] + (i - lstart[b]);
        orow[o] = r;
        ocol[LAST ? heavy_total + o : o] = sc[i];
        opos[LAST ? heavy_total + o : o] = sp[i];
    }
}

// ---- segments. Keys in plan order: the heavy keys (slot, rank), then the rows (light ones non-empty).
// Key q occupies plan positions [a, b); a segment starts at a and at every multiple of seglen inside.
struct KeyRanges {
    int nkh;                 // heavy keys: 8 * p8 * nheavy
    int nrows;
    int heavy_total;
    int seglen;
    const int* keybase;      // [nkh + 1]
    const int* lrowptr;      // [nrows + 1]  light nonzeros before row r
    __device__ void range(int q, int& a, int& b) const {
        if (q < nkh) { a = keybase[q]; b = keybase[q + 1]; }
        else { a = heavy_total + lrowptr[q - nkh]; b = heavy_total + lrowptr[q - nkh + 1]; }
    }
    __device__ int segments(int a, int b) const { return b > a ? 1 + (b - 1) / seglen - a / seglen : 0; }
};

__global__ __launch_bounds__(BM_BLOCK) void k_seg_count(KeyRanges kr, int* __restrict__ segcnt) {
    const long long q = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (q >= (long long)kr.nkh + kr.nrows) return;
    int a, b;
    kr.range((int)q, a, b);
    segcnt[q] = kr.segments(a, b);
}

__global__ __launch_bounds__(BM_BLOCK) void k_seg_emit(KeyRanges kr, int nheavy, const int* __restrict__ segbase,
                                                       const int* __restrict__ hrow, int* __restrict__ segstart,
                                                       int* __restrict__ segrow) {
    const long long q = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (q >= (long long)kr.nkh + kr.nrows) return;
    int a, b;
    kr.range((int)q, a, b);
    const int n = kr.segments(a, b);
    if (n == 0) return;
    const int row = q < kr.nkh ? hrow[q % nheavy] : (int)(q - kr.nkh);
    const int base = segbase[q];
    segstart[base] = a;
    segrow[base] = row;
    const int first = a / kr.seglen;
    for (int s = 1; s < n; ++s) {
        segstart[base + s] = (first + s) * kr.seglen;
        segrow[base + s] = row;
    }
}

// segments per row: a heavy row's keys are (slot, its rank) for every slot; a light row has its own key
__global__ __launch_bounds__(BM_BLOCK) void k_row_segcount(int nkh, int nslots, int nheavy, int nrows,
                                                           const int* __restrict__ hcode, const int* __restrict__ hrow,
                                                           const int* __restrict__ segcnt, int* __restrict__ rowcnt) {
    const long long t = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    if (t < nheavy) {
        int n = 0;
        for (int s = 0; s < nslots; ++s) n += segcnt[(size_t)s * nheavy + t];
        rowcnt[hrow[t]] = n;
    }
    if (t < nrows && hcode[t] < 0) rowcnt[t] = segcnt[(size_t)nkh + t];
}

// rowseg: the ids of a row's segments in ascending order. A heavy row has one key per panel slot: a wave takes
// the row, its lanes the slots (64 at a time, a prefix sum over the lanes gives every slot its place); a light
// row is one thread's.
__global__ __launch_bounds__(BM_BLOCK) void k_rowseg_fill(int nkh, int nslots, int nheavy, int nrows,
                                                          const int* __restrict__ hcode, const int* __restrict__ hrow,
                                                          const int* __restrict__ segcnt, const int* __restrict__ segbase,
                                                          const int* __restrict__ rowptr, int* __restrict__ rowseg) {
    const long long t = (long long)blockIdx.x * BM_BLOCK + threadIdx.x;
    const long long w = t >> 6;
    const int lane = threadIdx.x & 63;
    if (w < nheavy) {
        int d = rowptr[hrow[w]];
        for (int s0 = 0; s0 < nslots; s0 += 64) {
            const int sl = s0 + lane;
            const size_t q = (size_t)(sl < nslots ? sl : 0) * nheavy + (size_t)w;
            const int n = sl < nslots ? segcnt[q] : 0;
            const int base = sl < nslots ? segbase[q] : 0;
            int inc = n;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int y = __shfl_up(inc, o, 64);
                if (lane >= o) inc += y;
            }
            const int at = d + inc - n;
            for (int i = 0; i < n; ++i) rowseg[at + i] = base + i;
            d += __shfl(inc, 63, 64);
        }
    }
    if (t < nrows && hcode[t] < 0) {
        const size_t q = (size_t)nkh + t;
        const int n = segcnt[q], base = segbase[q], d = rowptr[t];
        for (int i = 0; i < n; ++i) rowseg[d + i] = base + i;
    }
}

// out[x] = first segment of XCD group x (x < 8) / first light segment (x == 8); out[9] = number of segments
__global__ void k_group_starts(int nkh, int per_xcd, int nkeys, const int* __restrict__ segbase, int* __restrict__ out) {
    const int x = threadIdx.x;
    if (x < 8) out[x] = segbase[nkh > 0 ? x * per_xcd : 0];
    if (x == 8) out[8] = segbase[nkh];
    if (x == 9) out[9] = segbase[nkeys];
}

// out[0] = the largest number of heavy nonzeros of one panel slot (keybase has nslots*nheavy + 1 entries). One workgroup.
__global__ __launch_bounds__(BM_BLOCK) void k_max_stretch(int nslots, int nheavy, const int* __restrict__ keybase, int* __restrict__ out) {
    __shared__ int sm[BM_BLOCK];
    int m = 0;
    for (int sl = threadIdx.x; sl < nslots; sl += BM_BLOCK) {
        const int v = keybase[(size_t)(sl + 1) * nheavy] - keybase[(size_t)sl * nheavy];
        m = v > m ? v : m;
    }
    sm[threadIdx.x] = m;
    __syncthreads();
    for (int d = BM_BLOCK / 2; d > 0; d >>= 1) {
        if ((int)threadIdx.x < d) sm[threadIdx.x] = sm[threadIdx.x] > sm[threadIdx.x + d] ? sm[threadIdx.x] : sm[threadIdx.x + d];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = sm[0];
}

#define RB_CHECK(expr)                                          \
    do {                                                        \
        hipError_t _e = (expr);                                 \
        if (_e != hipSuccess) return _e;                        \
    } while (0)

template <typename K>
hipError_t allow_lds(K kernel, size_t bytes) {
    if (bytes <= (48u << 10)) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

}  // namespace

int rows_binned_max_heavy() { return 24 * 1024 - 1; }      // keys fit 15 bits beside a 16-bit rank; (nheavy + 1) 16-bit LDS counters per workgroup

// *unfit = 1 (and hipSuccess) when the pattern does not fit this builder (a tile of more than 65535 nonzeros, a
// panel whose heavy nonzeros span more than RB_MAX_DBINS destination blocks): the caller sorts instead.
hipError_t build_rows_binned(bidmat_plan* plan, const int* ir, const int* jc, const int* hcode, const int* hrow,
                             int nheavy, int p8, int* bad, int* unfit, hipStream_t s) {
    *unfit = 0;
    const int nrows = plan->nrows, ncols = plan->ncols, nnz = plan->nnz;
    if (nheavy > rows_binned_max_heavy()) { *unfit = 1; return hipSuccess; }
    Tiling tg;
    tg.ncols = ncols; tg.npanels = plan->npanels; tg.panel_cols = plan->panel_cols; tg.p8 = p8; tg.nheavy = nheavy;
    {
        const long long per_panel = ((long long)nnz + tg.npanels - 1) / tg.npanels;
        long long tpp = (per_panel + RB_TILE_NNZ - 1) / RB_TILE_NNZ;
        if (tpp < 1) tpp = 1;
        if (tpp > tg.panel_cols) tpp = tg.panel_cols;
        tg.tpp = (int)tpp;
        tg.tcols = (tg.panel_cols + tg.tpp - 1) / tg.tpp;
    }
    const int ntiles = tg.tiles();
    const int nb = nheavy + 1;
    const int nslots = nheavy > 0 ? 8 * p8 : 0;
    const long long nkh_ll = (long long)nslots * nheavy;
    if (nkh_ll + nrows + 1 > 0x7fffffffLL || (long long)ntiles * nb > 0x7fffffffLL || ntiles > 0x7fffffff / RB_SUBS_PER_TILE) {
        *unfit = 1;
        return hipSuccess;
    }
    const int nkh = (int)nkh_ll;
    const int nkeys = nkh + nrows;
    const size_t lds = sizeof(unsigned short) * (size_t)nb;

    // ---- temporaries, stage A (sizes known now)
    hipError_t werr;
    Arena ta;
    int *hist = nullptr, *keytot = nullptr, *keybase = nullptr, *ltot = nullptr, *lbase = nullptr, *scantmp = nullptr, *small = nullptr;
    unsigned* what = nullptr;
    int* subcols = nullptr;
    const size_t scan_n = (size_t)(nkeys > ntiles ? nkeys : ntiles) + 1;
    for (int pass = 0; pass < 2; ++pass) {
        ta.used = 0;
        hist = ta.take<int>((size_t)ntiles * nb);
        keytot = ta.take<int>((size_t)nkh + 1);
        keybase = ta.take<int>((size_t)nkh + 2);
        ltot = ta.take<int>((size_t)tg.npanels + 1);
        lbase = ta.take<int>((size_t)tg.npanels + 2);
        scantmp = ta.take<int>(scan_tmp_ints((long long)scan_n));
        small = ta.take<int>(16);
        what = ta.take<unsigned>((size_t)nnz);
        subcols = ta.take<int>(2 * (size_t)ntiles * RB_SUBS_PER_TILE);
        if (pass == 0) {
            ta.base = static_cast<char*>(ws_get(WS_PLAN_ROWS_A, ta.used, &werr, s));
            if (!ta.base) return werr;
        }
    }

    // ---- ranks inside the tiles and counts per (tile, key); prefixes inside panels; scan over keys
    RB_CHECK(allow_lds(k_tile_rank, lds));
    RB_CHECK(fill_i32(keytot, (long long)nkh + 1, 0, s));
    RB_CHECK(fill_i32(small, 16, 0, s));
    hipLaunchKernelGGL(k_tile_rank, dim3((unsigned)ntiles), dim3(BM_BLOCK), lds, s, tg, nrows, bits_for((unsigned long long)nheavy), jc, ir,
                       hcode, hist, what, bad, small + 10);
    hipLaunchKernelGGL(k_panel_prefix, dim3(blocks_for((long long)tg.npanels * nb)), dim3(BM_BLOCK), 0, s, tg, hist, keytot, ltot);
    RB_CHECK(scan_exclusive_i32(keytot, keybase, nkh, scantmp, s));              // keybase[nkh] = all heavy nonzeros
    RB_CHECK(scan_exclusive_i32(ltot, lbase, tg.npanels, scantmp, s));           // lbase[npanels] = all light nonzeros
    hipLaunchKernelGGL(k_max_stretch, dim3(1), dim3(BM_BLOCK), 0, s, nslots, nheavy, keybase, small + 11);
    RB_CHECK(hipGetLastError());
    int totals[2] = {0, 0}, badv = 0, flags[2] = {0, 0};
    RB_CHECK(hipMemcpyAsync(&totals[0], keybase + nkh, sizeof(int), hipMemcpyDeviceToHost, s));
    RB_CHECK(hipMemcpyAsync(&totals[1], lbase + tg.npanels, sizeof(int), hipMemcpyDeviceToHost, s));
    RB_CHECK(hipMemcpyAsync(&badv, bad, sizeof(int), hipMemcpyDeviceToHost, s));
    RB_CHECK(hipMemcpyAsync(flags, small + 10, sizeof(flags), hipMemcpyDeviceToHost, s));
    RB_CHECK(hipStreamSynchronize(s));
    if (badv) return hipErrorInvalidValue;                 // the ranking pass has seen every row index
    if (flags[0] || flags[1] > (RB_MAX_DBINS - 2) * RB_DBLOCK) { *unfit = 1; return hipSuccess; }
    const int heavy_total = totals[0], nlight = totals[1];
    if ((long long)heavy_total + nlight != nnz) return hipErrorInvalidValue;    // a column pointer that does not describe nnz entries

    // ---- temporaries, stage B (sized by the numbers of heavy and light nonzeros)
    int rb = bits_for((unsigned long long)(nrows > 1 ? nrows - 1 : 1));
    const int npass = (rb + RB_LIGHT_BITS - 1) / RB_LIGHT_BITS;
    const int pbits = (rb + npass - 1) / npass;
    const int lbins = 1 << pbits;
    const int ltiles = (int)(((long long)nlight + RB_LIGHT_TILE - 1) / RB_LIGHT_TILE);
    const int dblocks = (int)(((long long)heavy_total + RB_DBLOCK - 1) / RB_DBLOCK);
    Arena tb;
    int *lr[2] = {nullptr, nullptr}, *lc[2] = {nullptr, nullptr}, *lp[2] = {nullptr, nullptr};
    int *table = nullptr, *table2 = nullptr, *lrowptr = nullptr, *segcnt = nullptr, *segbase = nullptr, *rowcnt = nullptr, *scantmp2 = nullptr;
    int *td = nullptr, *tc = nullptr, *tj = nullptr, *fill = nullptr;
    const size_t tab_n = (size_t)lbins * (size_t)(ltiles > 0 ? ltiles : 1);
    const size_t hpad = (size_t)dblocks * RB_DBLOCK;
    for (int pass = 0; pass < 2; ++pass) {
        tb.used = 0;
        for (int x = 0; x < 2; ++x) {
            lr[x] = tb.take<int>((size_t)nlight);
            lc[x] = tb.take<int>((size_t)nlight);
            lp[x] = tb.take<int>((size_t)nlight);
        }
        td = tb.take<int>(hpad);
        tc = tb.take<int>(hpad);
        tj = tb.take<int>(hpad);
        fill = tb.take<int>((size_t)dblocks + 1);
        table = tb.take<int>(tab_n + 1);
        table2 = tb.take<int>(tab_n + 2);
        lrowptr = tb.take<int>((size_t)nrows + 2);
        segcnt = tb.take<int>((size_t)nkeys + 1);
        segbase = tb.take<int>((size_t)nkeys + 2);
        rowcnt = tb.take<int>((size_t)nrows + 1);
        scantmp2 = tb.take<int>(scan_tmp_ints((long long)(tab_n > (size_t)nkeys ? tab_n : (size_t)nkeys) + 1));
        if (pass == 0) {
            tb.base = static_cast<char*>(ws_get(WS_PLAN_ROWS_B, tb.used, &werr, s));
            if (!tb.base) return werr;
        }
    }

    // ---- heavy nonzeros to their places (grouped by destination block, then placed block by block), light ones
    // packed in CSC order
    RB_CHECK(fill_i32(fill, (long long)dblocks + 1, 0, s));
    hipLaunchKernelGGL(k_sub_columns, dim3(blocks_for((long long)ntiles * RB_SUBS_PER_TILE)), dim3(BM_BLOCK), 0, s, tg, jc, subcols);
    hipLaunchKernelGGL(k_add_base, dim3(blocks_for((long long)ntiles * nb)), dim3(BM_BLOCK), 0, s, tg, keybase, lbase, hist);
    hipLaunchKernelGGL(k_group, dim3((unsigned)ntiles, RB_SUBS_PER_TILE), dim3(BM_BLOCK), 0, s, tg, heavy_total, jc, ir, what, hist,
                       keybase, subcols, fill, td, tc, tj, lr[0], lc[0], lp[0]);
    if (dblocks > 0)
        hipLaunchKernelGGL(k_fill_block, dim3((unsigned)dblocks), dim3(RB_FILL_THREADS), 0, s, heavy_total, td, tc, tj, plan->pc, plan->perm);
    RB_CHECK(hipGetLastError());

    // ---- light nonzeros: stable passes by row, low bits first
    if (nlight > 0) {
        int cur = 0;
        for (int p = 0; p < npass; ++p) {
            const int shift = p * pbits;
            const bool last = p == npass - 1;
            hipLaunchKernelGGL(k_light_count, dim3((unsigned)ltiles), dim3(BM_BLOCK), 0, s, nlight, shift, lbins, ltiles, lr[cur], table);
            RB_CHECK(scan_exclusive_i32(table, table2, (long long)tab_n, scantmp2, s));
            if (last)
                hipLaunchKernelGGL(k_light_scatter<true>, dim3((unsigned)ltiles), dim3(BM_BLOCK), 0, s, nlight, shift, lbins, pbits, ltiles,
                                   table, table2, lr[cur], lc[cur], lp[cur], lr[cur ^ 1], plan->pc, plan->perm, heavy_total);
            else
                hipLaunchKernelGGL(k_light_scatter<false>, dim3((unsigned)ltiles), dim3(BM_BLOCK), 0, s, nlight, shift, lbins, pbits, ltiles,
                                   table, table2, lr[cur], lc[cur], lp[cur], lr[cur ^ 1], lc[cur ^ 1], lp[cur ^ 1], 0);
            RB_CHECK(hipGetLastError());
            cur ^= 1;
        }
        // lr[cur]: the rows of the light nonzeros in plan order
        RB_CHECK(sorted_lower_bounds(nrows, nlight, lr[cur], lrowptr, s));
    } else {
        RB_CHECK(fill_i32(lrowptr, (long long)nrows + 1, 0, s));
    }

    // ---- segments
    KeyRanges kr;
    kr.nkh = nkh; kr.nrows = nrows; kr.heavy_total = heavy_total; kr.seglen = plan->seglen;
    kr.keybase = keybase; kr.lrowptr = lrowptr;
    hipLaunchKernelGGL(k_seg_count, dim3(blocks_for(nkeys)), dim3(BM_BLOCK), 0, s, kr, segcnt);
    RB_CHECK(scan_exclusive_i32(segcnt, segbase, nkeys, scantmp2, s));
    hipLaunchKernelGGL(k_group_starts, dim3(1), dim3(64), 0, s, nkh, p8 * nheavy, nkeys, segbase, small);
    RB_CHECK(hipGetLastError());
    int starts[10];
    RB_CHECK(hipMemcpyAsync(starts, small, sizeof(starts), hipMemcpyDeviceToHost, s));
    RB_CHECK(hipStreamSynchronize(s));
    const int nseg = starts[9];
    plan->nseg = nseg;
    for (int x = 0; x < 9; ++x) plan->xcd_start[x] = starts[x];
    {
        Arena own;
        for (int pass = 0; pass < 2; ++pass) {
            own.used = 0;
            plan->segstart = own.take<int>((size_t)nseg + 1);
            plan->segrow = own.take<int>((size_t)nseg);
            plan->rowseg = own.take<int>((size_t)nseg);
            if (pass == 0) {
                hipError_t perr;
                plan->block_seg = pool_alloc(own.used, &perr);
                RB_CHECK(perr);
                own.base = static_cast<char*>(plan->block_seg);
                plan->row_bytes += own.used;
            }
        }
    }
    hipLaunchKernelGGL(k_seg_emit, dim3(blocks_for(nkeys)), dim3(BM_BLOCK), 0, s, kr, nheavy > 0 ? nheavy : 1, segbase, hrow,
                       plan->segstart, plan->segrow);
    RB_CHECK(fill_i32(plan->segstart + nseg, 1, nnz, s));
    // ---- a row's segments, in ascending order
    hipLaunchKernelGGL(k_row_segcount, dim3(blocks_for(nrows > nheavy ? nrows : nheavy)), dim3(BM_BLOCK), 0, s, nkh, nslots, nheavy,
                       nrows, hcode, hrow, segcnt, rowcnt);
    RB_CHECK(scan_exclusive_i32(rowcnt, plan->rowptr, nrows, scantmp2, s));
    hipLaunchKernelGGL(k_rowseg_fill, dim3(blocks_for((long long)nrows > 64LL * nheavy ? (long long)nrows : 64LL * nheavy)), dim3(BM_BLOCK), 0, s, nkh, nslots, nheavy,
                       nrows, hcode, hrow, segcnt, segbase, plan->rowptr, plan->rowseg);
    RB_CHECK(hipGetLastError());
    RB_CHECK(hipStreamSynchronize(s));
    const size_t keep = (size_t)opt_plan_keep_mb() << 20;
    if (ta.used > keep) RB_CHECK(ws_drop(WS_PLAN_ROWS_A, s));
    if (tb.used > keep) RB_CHECK(ws_drop(WS_PLAN_ROWS_B, s));
    return hipSuccess;
}

}  // namespace bm
