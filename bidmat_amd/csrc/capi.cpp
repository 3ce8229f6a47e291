// C ABI of libbidmathip.so: argument validation, the reference-shaped blocking launchers, the
// native stream-taking entry points, plan handles + the fingerprint-keyed plan cache used by the
// reference-shaped entries, and the device-memory helpers.
#include "../../include/bidmat_hip.h"
#include "common.hpp"
#include "kernels.hpp"
#include "plan.hpp"
#include "workspace.hpp"
#include <algorithm>
#include <atomic>
#include <cstring>
#include <cstdio>
#include <cstdlib>
#include <list>
#include <memory>
#include <mutex>

#define API extern "C" __attribute__((visibility("default")))

namespace bm {
namespace {
std::atomic<int> g_seglen{1024};
std::atomic<int> g_panel_kb{4096};
std::atomic<int> g_heavy_min{8};
std::atomic<int> g_col_classes{-1};
std::atomic<int> g_class_strip{16};
std::atomic<int> g_class_hot{-1};
std::atomic<int> g_class_threads{1024};
std::atomic<int> g_class_phases{2};
std::atomic<int> g_plan_keep_mb{4096};
std::atomic<int> g_cache_cols_after{2};
std::atomic<int> g_cache_plans{4};
std::atomic<int> g_check_plan{0};
std::atomic<int> g_plan_builder{0};
std::atomic<int> g_rowsum_form{0};
std::atomic<int> g_class_shift{-1};
std::atomic<int> g_plan_pool_mb{4096};
std::atomic<int> g_dense_rows{128};
std::atomic<int> g_dense_min_pct{15};
std::atomic<int> g_dense_min_nnz{1 << 22};
std::atomic<int> g_dense_cb{0};
std::atomic<int> g_scalar_values{1};
}  // namespace
int opt_plan_pool_mb() { return g_plan_pool_mb.load(std::memory_order_relaxed); }
int opt_dense_rows() { return g_dense_rows.load(std::memory_order_relaxed); }
int opt_dense_min_pct() { return g_dense_min_pct.load(std::memory_order_relaxed); }
int opt_dense_min_nnz() { return g_dense_min_nnz.load(std::memory_order_relaxed); }
int opt_dense_cb() { return g_dense_cb.load(std::memory_order_relaxed); }
int opt_scalar_values() { return g_scalar_values.load(std::memory_order_relaxed); }
int opt_plan_builder() { return g_plan_builder.load(std::memory_order_relaxed); }
int opt_class_shift() { return g_class_shift.load(std::memory_order_relaxed); }
int opt_rowsum_form() { return g_rowsum_form.load(std::memory_order_relaxed); }
int opt_check_plan() { return g_check_plan.load(std::memory_order_relaxed); }
int opt_class_threads() { return g_class_threads.load(std::memory_order_relaxed); }
int opt_plan_keep_mb() { return g_plan_keep_mb.load(std::memory_order_relaxed); }
int opt_class_phases() { return g_class_phases.load(std::memory_order_relaxed); }
int opt_class_hot() { return g_class_hot.load(std::memory_order_relaxed); }
int opt_class_strip() { return g_class_strip.load(std::memory_order_relaxed); }
int opt_col_classes() { return g_col_classes.load(std::memory_order_relaxed); }
int opt_heavy_min() { return g_heavy_min.load(std::memory_order_relaxed); }
int opt_seglen() { return g_seglen.load(std::memory_order_relaxed); }
int opt_panel_kb() { return g_panel_kb.load(std::memory_order_relaxed); }
}  // namespace bm

namespace {

constexpr int kInvalid = (int)hipErrorInvalidValue;

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// Blocking epilogue of the reference-shaped launchers (Arith.cu:57-59).
inline int finish_blocking(hipError_t launch_err) {
    hipError_t sync_err = hipStreamSynchronize(nullptr);
    if (launch_err != hipSuccess) return (int)launch_err;
    if (sync_err != hipSuccess) return (int)sync_err;
    return (int)hipGetLastError();
}

// ---- plan cache for entries that only receive (ir, ic): keyed by a fingerprint of both index
// arrays, so a caller that refills the same device buffers with another pattern never meets a
// stale plan. An entry starts without a plan; A*^S / row sums build the row side at once (they cannot
// run without it), A*S / DDS build the column side from their "cache_cols_after"-th call on the
// pattern (default: the second), so a pattern that is used once costs no build.
struct CacheEntry {
    int device;
    int ncols, nnz, nrows, k_hint;
    unsigned long long fa, fb;
    int col_uses;                           // A*S / DDS calls that met this pattern
    std::shared_ptr<bidmat_plan> plan;      // callers hold a reference while they use the plan (may be empty)
};
using PlanRef = std::shared_ptr<bidmat_plan>;
PlanRef own(bidmat_plan* p) { return PlanRef(p, [](bidmat_plan* q) { (void)bm::plan_free(q); }); }
std::mutex g_cache_mu;
std::list<CacheEntry> g_cache;          // most recently used first
// the class-ordered DDS kernel walks a column's class in one wave: very long columns stay with the
// segment-splitting kernel
constexpr int kMaxClassedColumn = 1 << 16;
// A*S in passes over the classes adds a column's share of a pass in one running sum: kept to columns short enough
// for that to cost no accuracy (a 60 000-nonzero column came out at 1.3e-5 relative, against 1.9e-6 from the
// kernel that cuts columns into segments); longer ones stay with the segment-splitting kernel
constexpr int kMaxPhasedColumn = 1 << 13;

enum Need { NEED_ROWS, NEED_COLS };

// Finds (or makes) the cache entry of the pattern (ir, ic) and returns its plan with the side `need`
// built when that side is due; *out stays empty when A*S / DDS should run without a plan. *jc_out
// (nullable) receives the pattern's column pointer, built in the same pass over ic into the default
// stream's scratch: valid until the caller's next scratch request for WS_JC.
// zcheck != nullptr: *all_zero tells whether the nz floats there are all +0.0f (checked in the same pass).
hipError_t cached_plan(int ncols, int nnz, const int* ir, const int* ic, int k_hint, Need need, PlanRef* out,
                       int** jc_out = nullptr, const float* zcheck = nullptr, long long nz = 0, bool* all_zero = nullptr) {
    out->reset();
    hipError_t err;
    int dev = 0;
    if ((err = hipGetDevice(&dev)) != hipSuccess) return err;
    hipStream_t s = nullptr;
    unsigned long long* d_misc = (unsigned long long*)bm::ws_get(bm::WS_MISC, sizeof(unsigned long long) * bm::pattern_digest_words(), &err);
    if (!d_misc) return err;
    int* jc = (int*)bm::ws_get(bm::WS_JC, sizeof(int) * ((size_t)ncols + 1), &err);
    if (!jc) return err;
    if (jc_out) *jc_out = jc;
    // misc layout: [0..1] two digests of the (ic, ir) pair sequence, [2] (as int) max row
    if ((err = bm::pattern_digest(ir, ic, nnz, d_misc, s, ncols, jc, zcheck, nz)) != hipSuccess) return err;
    unsigned long long h[4];
    if ((err = hipMemcpy(h, d_misc, sizeof(h), hipMemcpyDeviceToHost)) != hipSuccess) return err;
    if (all_zero) *all_zero = zcheck != nullptr && h[3] == 0;
    int maxrow;
    memcpy(&maxrow, &h[2], sizeof(int));
    const int nrows = maxrow + 1;

    std::lock_guard<std::mutex> lock(g_cache_mu);
    auto hit = g_cache.end();
    for (auto it = g_cache.begin(); it != g_cache.end(); ++it) {
        // panels are sized for k_hint: a request that names k only takes a plan built for that k
        const bool k_ok = k_hint <= 0 || (it->k_hint > 0 ? it->k_hint : 256) == k_hint;
        // (no addresses in the key: the same pattern uploaded into other buffers is the same pattern)
        if (k_ok && it->device == dev && it->ncols == ncols && it->nnz == nnz && it->nrows == nrows &&
            it->fa == h[0] && it->fb == h[1]) {
            hit = it;
            break;
        }
    }
    if (hit == g_cache.end()) {
        const size_t cap = (size_t)std::max(1, bm::g_cache_plans.load());
        while (g_cache.size() >= cap) g_cache.pop_back();           // its plan is freed when its last user lets go
        g_cache.push_front(CacheEntry{dev, ncols, nnz, nrows, k_hint, h[0], h[1], 0, PlanRef()});
    } else {
        g_cache.splice(g_cache.begin(), g_cache, hit);
    }
    CacheEntry& e = g_cache.front();
    int side = bm::PLAN_ROWS;
    if (need == NEED_COLS) {
        side = bm::PLAN_COLS;
        const int after = bm::g_cache_cols_after.load();
        if (e.col_uses < 0x7fffffff) ++e.col_uses;
        if (after <= 0 || e.col_uses < after) {
            // not due yet: use the column side only if an earlier call has built it
            if (e.plan && (e.plan->sides & bm::PLAN_COLS)) *out = e.plan;
            return hipSuccess;
        }
    }
    if (!e.plan) {
        bidmat_plan* p = nullptr;
        if ((err = bm::plan_build(nrows, ncols, nnz, ir, jc, k_hint, &p, side)) != hipSuccess) return err;
        e.plan = own(p);
    } else if (!(e.plan->sides & side)) {
        if ((err = bm::plan_extend(e.plan.get(), ir, jc, side)) != hipSuccess) return err;
    }
    *out = e.plan;
    return hipSuccess;
}

// The nseg*k partial sums of one call through a plan: scratch of the stream the call runs on, so a plan holds
// pattern data only and calls on different streams do not meet.
float* row_partial(const bidmat_plan* plan, int k, hipStream_t s, hipError_t* err, size_t extra_floats = 0) {
    return (float*)bm::ws_get(bm::WS_ROWPARTIAL, sizeof(float) * ((size_t)plan->nseg * (size_t)k + extra_floats), err, s);
}

// vals == nullptr: the values stored in the plan by bidmat_plan_set_values (already in plan order)
// between != nullptr: an event recorded after stage 1 (the gathers), before stage 2 (the row reduction)
hipError_t run_dsmultT(bidmat_plan* plan, int k, const float* A, const float* vals, float* C, int beta,
                       hipStream_t s, hipEvent_t between = nullptr) {
    hipError_t err;
    if (!vals && !plan->pvals && plan->nnz > 0) return hipErrorInvalidValue;
    // With values of the caller's (stored order) and a k the dense product is written for, the plan's dense rows go
    // through the matrix cores: their partial sums follow the segments' in the scratch, then the flag that tells
    // whether A held a value that is not finite (the dense rows' segments are then gathered after all).
    const bool dense = (vals != nullptr || plan->dvals != nullptr) && plan->ndense > 0 && bm::dense_rows_fit(k) && bm::opt_dense_rows() > 0;
    const size_t dfloats = dense ? (size_t)(plan->ndblocks + bm::dense_rows_fold(plan->ndblocks)) * (size_t)plan->ndense * (size_t)k : 0;
    float* partial = row_partial(plan, k, s, &err, dense ? dfloats + 64 : 0);
    if (!partial) return err;
    float* dpart = partial + (size_t)plan->nseg * (size_t)k;
    int* flag = dense ? reinterpret_cast<int*>(dpart + dfloats) : nullptr;
    if ((err = bm::gather_segments(k, plan->nseg, plan->xcd_start, A, vals ? vals : plan->pvals, plan->pc,
                                   vals ? plan->perm : nullptr, plan->segstart, partial, s,
                                   dense ? plan->dskip : nullptr, flag)) != hipSuccess) return err;
    if (dense) {
        if ((err = bm::dense_rows_stage(k, plan->ncols, plan->ndense, plan->dcb, plan->ndblocks, A, vals, plan->dpos, plan->dvals,
                                        dpart, flag, s)) != hipSuccess) return err;
        if ((err = bm::gather_segments_listed(k, plan->ndseg, plan->dseglist, flag, A, vals ? vals : plan->pvals, plan->pc,
                                              vals ? plan->perm : nullptr, plan->segstart, partial, s)) != hipSuccess) return err;
    }
    if (between && (err = hipEventRecord(between, s)) != hipSuccess) return err;
    return bm::reduce_segments(k, plan->nrows, plan->rowptr, plan->rowseg, partial, C, beta, s,
                               dense ? plan->rowptr2 : nullptr, dense ? plan->rowseg2 : nullptr, flag);
}

hipError_t run_spsum_rows(bidmat_plan* plan, const float* vals, float* out, int beta, hipStream_t s) {
    hipError_t err;
    if (!vals && !plan->pvals && plan->nnz > 0) return hipErrorInvalidValue;
    float* partial = row_partial(plan, 1, s, &err);
    if (!partial) return err;
    if ((err = bm::spsum_segments(plan->nseg, plan->xcd_start, vals ? vals : plan->pvals, vals ? plan->perm : nullptr,
                                  plan->segstart, partial, s)) != hipSuccess)
        return err;
    return bm::reduce_segments(1, plan->nrows, plan->rowptr, plan->rowseg, partial, out, beta, s);
}

bool plan_on_current_device(const bidmat_plan* p) {
    int dev = -1;
    return p && hipGetDevice(&dev) == hipSuccess && dev == p->device;
}

// the plan's column table as the kernels take it
bm::ColTable col_table(const bidmat_plan* plan) {
    return bm::ColTable{plan->col_seglen, plan->ovf, (long long)plan->novf};
}

inline bool ranges_overlap(const float* a, const float* b, long long n) {
    const uintptr_t x = reinterpret_cast<uintptr_t>(a), y = reinterpret_cast<uintptr_t>(b);
    const uintptr_t len = (uintptr_t)n * sizeof(float);
    return x < y + len && y < x + len;
}

// The fused step reads V[j] and writes P[j] from the same lane, so P == V (the in-place update) is sound
// as long as k is covered in one pass; wider k keeps running sums in P between passes, and a V that
// overlaps P at another offset is read by other lanes than the ones that write it.
bool fused_operand_ok(int k, long long nnz, const float* A, const float* B, const float* V, const float* P) {
    if (!V || !ranges_overlap(V, P, nnz)) return true;
    if (V != P) return false;
    const bool al = ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0;
    const bm::Shape sh = bm::pick_shape(k, al);
    return k <= sh.W * (sh.V > 4 ? 4 : sh.V) * sh.LPN;
}

// Checked mode (option "check_plan"): the pattern handed to a plan-taking call must be the one the plan
// was built from. Compares a digest of (Sir, Sjc) with the one taken at build time; plans built while
// the option was off carry no digest and pass.
int plan_pattern_ok(const bidmat_plan* plan, const int* Sir, const int* Sjc) {
    if (!bm::opt_check_plan() || !plan->has_digest) return 0;
    unsigned long long d[2];
    hipError_t e = bm::plan_digest(plan->nnz, plan->ncols, Sir, Sjc, d);
    if (e != hipSuccess) return (int)e;
    return (d[0] == plan->digest[0] && d[1] == plan->digest[1]) ? 0 : kInvalid;
}

// C = beta*C + A*S through the column side of a plan.
int dsmult_through_plan(bidmat_plan* plan, int k, const float* A, const float* Sdata, const int* Sir, const int* Sjc,
                        float* C, int beta, hipStream_t s) {
    if (!(plan->sides & bm::PLAN_COLS)) return kInvalid;
    const int nphase = bm::opt_class_phases();
    const bool phased = plan->ncls == 8 && plan->hcap == 0 && nphase > 0 && plan->maxlen <= kMaxPhasedColumn && plan->nnz > 0;
    if (!Sdata && !phased) return kInvalid;
    // Sdata == NULL: the values stored by bidmat_plan_set_values, which exist in class order only
    if (!Sjc || !C || (plan->nnz > 0 && (!A || !Sir || (!Sdata && !(phased && plan->cvals))))) return kInvalid;
    if (int bad = plan_pattern_ok(plan, Sir, Sjc)) return bad;
    if (phased)
        return (int)bm::dsmult_phased(k, plan->ncols, A, Sdata ? Sdata : plan->cvals, plan->cir, Sdata ? plan->cperm : nullptr,
                                      plan->cptr, nphase, C, beta, s);
    const bm::ColTable tab = col_table(plan);
    return (int)bm::dsmult_csc(k, plan->ncols, plan->nnz, A, Sdata, Sir, Sjc, C, beta, s, &tab);
}

// DDS through the column side of a plan. stored: the epilogue operand is the plan's stored values (V ignored).
int dds_through_plan(bidmat_plan* plan, int k, const float* A, const float* B, const int* Sir, const int* Sjc, const float* V,
                     bool stored, int opn, float* P, int beta, hipStream_t s) {
    if (!(plan->sides & bm::PLAN_COLS)) return kInvalid;
    if ((V || stored) && (beta != 0 || opn < 0 || opn > 14)) return kInvalid;
    if (plan->ncols == 0 || plan->nnz == 0) return 0;
    if (!Sjc || !Sir || !P || (k > 0 && (!A || !B))) return kInvalid;
    if (!stored && !fused_operand_ok(k, plan->nnz, A, B, V, P)) return kInvalid;
    if (int bad = plan_pattern_ok(plan, Sir, Sjc)) return bad;
    const bool classed = plan->ncls == 8 && k > 0 && plan->maxlen <= kMaxClassedColumn &&
                         (size_t)plan->hcap * (size_t)k * sizeof(float) <= bm::dds_classed_lds_budget();
    if (stored) {
        V = plan->ncls == 8 ? (classed ? plan->cvals : nullptr) : plan->svals;
        if (!V) return kInvalid;              // bidmat_plan_set_values has not been called (or k does not fit the ordering)
    }
    if (classed) {
        const hipError_t e = bm::dds_classed(k, plan->ncols, A, B, plan->cir, plan->cperm, plan->cptr, plan->hcap, plan->hotrows,
                                             P, beta, s, V, opn, stored);
        // A launch that the device refuses (e.g. less LDS per workgroup than the ordering was built for)
        // leaves nothing enqueued: the plain kernel gives the same bits. Stored values exist in class
        // order only, so that form reports the error.
        if (e == hipSuccess || stored) return (int)e;
        (void)hipGetLastError();
    }
    const bm::ColTable tab = col_table(plan);
    return (int)bm::dds_csc(k, plan->ncols, plan->nnz, A, B, Sir, Sjc, P, beta, s, V, opn, &tab);
}

}  // namespace

// ======================================================================== reference-shaped

API int bidmat_dsmult(int nrows, int ncols, int nnz, const float* A, const float* Bdata,
                      const int* Bir, const int* Bic, float* C) {
    auto lock = bm::device_lock();
    if (nrows < 0 || ncols < 0 || nnz < 0) return kInvalid;
    if (nrows == 0 || ncols == 0 || nnz == 0) return 0;           // C += 0
    if (!A || !Bdata || !Bir || !Bic || !C) return kInvalid;
    hipError_t err;
    if (bm::g_cache_cols_after.load() > 0) {
        // a pattern met before runs through the column side of its cached plan
        // (callers clear C before they call, GMat.scala:1047: a C found all zero is overwritten, not read)
        PlanRef plan;
        int* jc = nullptr;
        bool zero = false;
        err = cached_plan(ncols, nnz, Bir, Bic, nrows, NEED_COLS, &plan, &jc, C, (long long)nrows * ncols, &zero);
        if (err != hipSuccess) return finish_blocking(err);
        const int beta = zero ? 0 : 1;
        if (plan) return finish_blocking((hipError_t)dsmult_through_plan(plan.get(), nrows, A, Bdata, Bir, jc, C, beta, nullptr));
        return finish_blocking(bm::dsmult_csc(nrows, ncols, nnz, A, Bdata, Bir, jc, C, beta, nullptr));
    }
    int* jc = (int*)bm::ws_get(bm::WS_JC, sizeof(int) * ((size_t)ncols + 1), &err);
    if (!jc) return (int)err;
    err = bm::coo_compress_cols(ncols, nnz, Bic, jc, nullptr);
    if (err == hipSuccess) err = bm::dsmult_csc(nrows, ncols, nnz, A, Bdata, Bir, jc, C, 1, nullptr);
    return finish_blocking(err);
}

API int bidmat_dsmultT(int nrows, int ncols, int nnz, const float* A, const float* Bdata,
                       const int* Bir, const int* Bic, float* C) {
    auto lock = bm::device_lock();
    if (nrows < 0 || ncols < 0 || nnz < 0) return kInvalid;
    if (nrows == 0 || ncols == 0 || nnz == 0) return 0;
    if (!A || !Bdata || !Bir || !Bic || !C) return kInvalid;
    PlanRef plan;
    hipError_t err = cached_plan(ncols, nnz, Bir, Bic, nrows, NEED_ROWS, &plan);
    if (err == hipSuccess) err = run_dsmultT(plan.get(), nrows, A, Bdata, C, 1, nullptr);
    return finish_blocking(err);
}

API int bidmat_dsmultTile(int nr, int nc, int kk, int nnz, const float* A, int lda, const float* Bdata,
                          const int* Bir, const int* Bic, int broff, int bcoff, float* C, int ldc) {
    auto lock = bm::device_lock();
    if (nr < 0 || nc < 0 || kk < 0 || nnz < 0 || broff < 0 || bcoff < 0 || lda < nr || ldc < nr) return kInvalid;
    if (nr == 0 || nc == 0 || kk == 0 || nnz == 0) return 0;
    if (!A || !Bdata || !Bir || !Bic || !C) return kInvalid;
    // the launcher does not receive S's column count: it is max(Bic)+1, and Bic is non-decreasing
    int last = 0;
    hipError_t err = hipMemcpy(&last, Bic + (nnz - 1), sizeof(int), hipMemcpyDeviceToHost);
    if (err != hipSuccess) return (int)err;
    if (last < 0 || last == 0x7fffffff) return kInvalid;
    const int ncolsS = last + 1;
    if (bcoff >= ncolsS) return 0;                       // the tile holds no stored column
    const int nc_eff = nc < ncolsS - bcoff ? nc : ncolsS - bcoff;
    int* jc = (int*)bm::ws_get(bm::WS_JC, sizeof(int) * ((size_t)ncolsS + 1), &err);
    if (!jc) return (int)err;
    err = bm::coo_compress_cols(ncolsS, nnz, Bic, jc, nullptr);
    if (err == hipSuccess)
        err = bm::dsmult_csc_ex(nr, lda, ldc, nc_eff, nnz, A, Bdata, Bir, jc + bcoff, C, 1, bm::Window{1, broff, kk}, nullptr);
    return finish_blocking(err);
}

API int bidmat_dsmultTileT(int nr, int nc, int kk, int nnz, const float* A, int lda, const float* Bdata,
                           const int* Bir, const int* Bic, int broff, int bcoff, float* C, int ldc) {
    auto lock = bm::device_lock();
    if (nr < 0 || nc < 0 || kk < 0 || nnz < 0 || broff < 0 || bcoff < 0 || lda < nr || ldc < nr) return kInvalid;
    if (nr == 0 || nc == 0 || kk == 0 || nnz == 0) return 0;
    if (!A || !Bdata || !Bir || !Bic || !C) return kInvalid;
    int last = 0;
    hipError_t err = hipMemcpy(&last, Bic + (nnz - 1), sizeof(int), hipMemcpyDeviceToHost);
    if (err != hipSuccess) return (int)err;
    if (last < 0 || last == 0x7fffffff) return kInvalid;
    PlanRef plan;
    err = cached_plan(last + 1, nnz, Bir, Bic, nr, NEED_ROWS, &plan);
    if (err != hipSuccess) return finish_blocking(err);
    if (broff >= plan->nrows) return 0;                  // the tile holds no stored row
    const int nrows_eff = nc < plan->nrows - broff ? nc : plan->nrows - broff;
    float* partial = row_partial(plan.get(), nr, nullptr, &err);
    if (partial)
        err = bm::gather_segments_ex(nr, lda, plan->nseg, plan->xcd_start, A, Bdata, plan->pc, plan->perm,
                                     plan->segstart, partial, bm::Window{1, bcoff, kk}, plan->segrow,
                                     bm::Window{1, broff, nrows_eff}, nullptr);
    if (partial && err == hipSuccess)
        err = bm::reduce_segments_ex(nr, ldc, broff, nrows_eff, plan->rowptr, plan->rowseg, partial, C, 1, nullptr);
    return finish_blocking(err);
}

API int bidmat_sdoprow(int nrows, int ncols, int nnz, float* A, const int* Aic, const float* B, int len, int opn) {
    if (nrows < 0 || ncols < 0 || nnz < 0 || opn < 0 || opn > 14) return kInvalid;
    if (nnz == 0) return 0;
    if (!A || !B || (len > 1 && !Aic)) return kInvalid;
    if (len > 1 && len < ncols) return kInvalid;         // a row vector has one entry per column
    return finish_blocking(bm::sdop(nnz, A, Aic, B, len, opn, nullptr));
}

API int bidmat_sdopcol(int nrows, int ncols, int nnz, float* A, const int* Air, const float* B, int len, int opn) {
    if (nrows < 0 || ncols < 0 || nnz < 0 || opn < 0 || opn > 14) return kInvalid;
    if (nnz == 0) return 0;
    if (!A || !B || (len > 1 && !Air)) return kInvalid;
    if (len > 1 && len < nrows) return kInvalid;         // a column vector has one entry per row
    return finish_blocking(bm::sdop(nnz, A, Air, B, len, opn, nullptr));
}

API int bidmat_dds(int nrows, int nnz, const float* A, const float* B, const int* Cir,
                   const int* Cic, float* P) {
    auto lock = bm::device_lock();
    if (nrows < 0 || nnz < 0) return kInvalid;
    if (nnz == 0) return 0;
    if (!Cir || !Cic || !P || (nrows > 0 && (!A || !B))) return kInvalid;
    // the launcher has no column count: it is max(Cic)+1, and Cic is non-decreasing
    int last = 0;
    hipError_t err = hipMemcpy(&last, Cic + (nnz - 1), sizeof(int), hipMemcpyDeviceToHost);
    if (err != hipSuccess) return (int)err;
    if (last < 0 || last == 0x7fffffff) return kInvalid;
    const int ncols = last + 1;
    if (bm::g_cache_cols_after.load() > 0 && nrows > 0) {
        // a pattern met before runs through the column side of its cached plan
        // (callers clear P before they call, GSMat.scala:662: a P found all zero is overwritten, not read)
        PlanRef plan;
        int* jc = nullptr;
        bool zero = false;
        err = cached_plan(ncols, nnz, Cir, Cic, nrows, NEED_COLS, &plan, &jc, P, nnz, &zero);
        if (err != hipSuccess) return finish_blocking(err);
        const int beta = zero ? 0 : 1;
        if (plan) return finish_blocking((hipError_t)dds_through_plan(plan.get(), nrows, A, B, Cir, jc, nullptr, false, 0, P, beta, nullptr));
        return finish_blocking(bm::dds_csc(nrows, ncols, nnz, A, B, Cir, jc, P, beta, nullptr));
    }
    int* jc = (int*)bm::ws_get(bm::WS_JC, sizeof(int) * ((size_t)ncols + 1), &err);
    if (!jc) return (int)err;
    err = bm::coo_compress_cols(ncols, nnz, Cic, jc, nullptr);
    if (err == hipSuccess) err = bm::dds_csc(nrows, ncols, nnz, A, B, Cir, jc, P, 1, nullptr);
    return finish_blocking(err);
}

API int bidmat_spsum(int nrows, int ncols, int nnz, const int* Air, const int* Aic, const float* P,
                     float* B, int n) {
    auto lock = bm::device_lock();
    if (nrows < 0 || ncols < 0 || nnz < 0) return kInvalid;
    if (nnz == 0) return 0;
    if (!Air || !Aic || !P || !B) return kInvalid;
    hipError_t err;
    if (n == 1) {
        int* jc = (int*)bm::ws_get(bm::WS_JC, sizeof(int) * ((size_t)ncols + 1), &err);
        if (!jc) return (int)err;
        err = bm::coo_compress_cols(ncols, nnz, Aic, jc, nullptr);
        if (err == hipSuccess) err = bm::spsum_cols(ncols, nnz, P, jc, B, 1, nullptr);
    } else {
        int bad = 0;
        err = bm::spsum_rows_exact(nrows, nnz, Air, P, B, 1, &bad, nullptr);
        if (err == hipSuccess && bad) err = hipErrorInvalidValue;                   // row index outside B
    }
    return finish_blocking(err);
}

API int bidmat_reduce1op(int nrows, int ncols, const float* A, float* B, float initv, int opn) {
    auto lock = bm::device_lock();
    if (nrows < 0 || ncols < 0) return kInvalid;
    if (ncols == 0) return 0;
    if (!B || (nrows > 0 && !A)) return kInvalid;
    return finish_blocking(bm::reduce1op(nrows, ncols, A, B, initv, opn, nullptr));
}

API int bidmat_reduce2op(int nrows, int ncols, const float* A, float* B, float initv, int opn) {
    auto lock = bm::device_lock();
    if (nrows < 0 || ncols < 0) return kInvalid;
    if (nrows == 0) return 0;
    if (!B || (ncols > 0 && !A)) return kInvalid;
    return finish_blocking(bm::reduce2op(nrows, ncols, A, B, initv, opn, nullptr));
}

API int bidmat_applyop(const float* A, int Anrows, int Ancols, const float* B, int Bnrows, int Bncols,
                       float* C, int opn) {
    if (Anrows < 0 || Ancols < 0 || Bnrows < 0 || Bncols < 0) return kInvalid;
    if (opn < 0 || opn > 14) return kInvalid;
    if ((long long)(Anrows > Bnrows ? Anrows : Bnrows) * (Ancols > Bncols ? Ancols : Bncols) == 0) return 0;
    if (!A || !B || !C) return kInvalid;
    return finish_blocking(bm::applyop(A, Anrows, Ancols, B, Bnrows, Bncols, C, opn, nullptr));
}

// ======================================================================== native entries

API int bidmat_dsmult_csc(int k, int ncols, int nnz, const float* A, const float* Sdata,
                          const int* Sir, const int* Sjc, float* C, int beta, void* stream) {
    auto lock = bm::device_lock();
    if (k < 0 || ncols < 0 || nnz < 0 || (beta != 0 && beta != 1)) return kInvalid;
    if (k == 0 || ncols == 0) return 0;
    if (!Sjc || !C || (nnz > 0 && (!A || !Sdata || !Sir))) return kInvalid;
    return (int)bm::dsmult_csc(k, ncols, nnz, A, Sdata, Sir, Sjc, C, beta, as_stream(stream));
}

API int bidmat_dds_csc(int k, int ncols, int nnz, const float* A, const float* B, const int* Sir,
                       const int* Sjc, float* P, int beta, void* stream) {
    auto lock = bm::device_lock();
    if (k < 0 || ncols < 0 || nnz < 0 || (beta != 0 && beta != 1)) return kInvalid;
    if (ncols == 0 || nnz == 0) return 0;
    if (!Sjc || !Sir || !P || (k > 0 && (!A || !B))) return kInvalid;
    return (int)bm::dds_csc(k, ncols, nnz, A, B, Sir, Sjc, P, beta, as_stream(stream));
}

API int bidmat_dds_csc_static(int k, int ncols, int nnz, const float* A, const float* B, const int* Sir,
                              const int* Sjc, float* P, int beta, void* stream) {
    // a mutex allocates nothing: host threads that share a stream cannot interleave "table built" and
    // "kernel enqueued" on the one scratch array (calls on different streams of a device still race on it)
    auto lock = bm::device_lock();
    if (k < 0 || ncols < 0 || nnz < 0 || (beta != 0 && beta != 1)) return kInvalid;
    if (ncols > bm::dds_static_max_cols()) return kInvalid;      // beyond the fixed scratch array
    if (ncols == 0 || nnz == 0) return 0;
    if (!Sjc || !Sir || !P || (k > 0 && (!A || !B))) return kInvalid;
    return (int)bm::dds_csc_static(k, ncols, nnz, A, B, Sir, Sjc, P, beta, as_stream(stream));
}

API int bidmat_dds_static_max_cols(void) { return bm::dds_static_max_cols(); }

API int bidmat_dds_csc_op(int k, int ncols, int nnz, const float* A, const float* B, const int* Sir,
                          const int* Sjc, const float* V, int opn, float* P, void* stream) {
    auto lock = bm::device_lock();
    if (k < 0 || ncols < 0 || nnz < 0 || opn < 0 || opn > 14) return kInvalid;
    if (ncols == 0 || nnz == 0) return 0;
    if (!Sjc || !Sir || !P || !V || (k > 0 && (!A || !B))) return kInvalid;
    if (!fused_operand_ok(k, nnz, A, B, V, P)) return kInvalid;
    return (int)bm::dds_csc(k, ncols, nnz, A, B, Sir, Sjc, P, 0, as_stream(stream), V, opn);
}

API int bidmat_dds_dsmult_csc(int k, int ncols, int nnz, const float* A, const float* B, const int* Sir, const int* Sjc,
                              const float* V, int opn, float* Q, float* C, int beta, void* stream) {
    auto lock = bm::device_lock();
    if (k < 0 || ncols < 0 || nnz < 0 || opn < 0 || opn > 14 || (beta != 0 && beta != 1)) return kInvalid;
    if (k == 0 || ncols == 0) return 0;
    if (!Sjc || !C || !A || !B || (nnz > 0 && (!Sir || !V))) return kInvalid;
    if (Q && V != Q && ranges_overlap(V, Q, nnz)) return kInvalid;      // in place (Q == V) or apart
    return (int)bm::fused_columns(k, ncols, nnz, A, B, V, Sir, Sjc, opn, Q, C, beta, as_stream(stream));
}

API int bidmat_dds_dsmult_plan(bidmat_plan* plan, int k, const float* A, const float* B, const int* Sir, const int* Sjc,
                               const float* V, int opn, float* Q, float* C, int beta, void* stream) {
    auto lock = bm::device_lock();
    if (!plan || k < 0 || opn < 0 || opn > 14 || (beta != 0 && beta != 1)) return kInvalid;
    if (!plan_on_current_device(plan)) return (int)hipErrorInvalidDevice;
    if (!(plan->sides & bm::PLAN_COLS)) return kInvalid;
    if (k == 0 || plan->ncols == 0) return 0;
    if (!Sjc || !C || !A || !B || (plan->nnz > 0 && (!Sir || !V))) return kInvalid;
    if (Q && V != Q && ranges_overlap(V, Q, plan->nnz)) return kInvalid;      // in place (Q == V) or apart
    const int bad = plan_pattern_ok(plan, Sir, Sjc);
    if (bad) return bad;
    hipStream_t s = as_stream(stream);
    // with a class order (and no hot-row ranks in it, no column too long for one running sum per pass): in passes
    const int nphase = bm::opt_class_phases();
    const bool phased = plan->ncls == 8 && plan->hcap == 0 && nphase > 0 && plan->maxlen <= kMaxPhasedColumn && plan->nnz > 0;
    if (phased) {
        const hipError_t e = bm::fused_columns_phased(k, plan->ncols, A, B, V, plan->cir, plan->cperm, plan->cptr, nphase, opn,
                                                      Q, C, beta, s);
        return (int)e;
    }
    const bm::ColTable tab = col_table(plan);
    return (int)bm::fused_columns(k, plan->ncols, plan->nnz, A, B, V, Sir, Sjc, opn, Q, C, beta, s, &tab);
}

API int bidmat_dds0(int nrows, int ncols, const float* A, const float* B, const int* Cir, const int* Cjc,
                    float* P) {
    auto lock = bm::device_lock();
    if (nrows < 0 || ncols < 0) return kInvalid;
    if (ncols == 0) return 0;
    if (!Cjc) return kInvalid;
    // the launcher has no nonzero count: it is the last column pointer
    int nnz = 0;
    hipError_t err = hipMemcpy(&nnz, Cjc + ncols, sizeof(int), hipMemcpyDeviceToHost);
    if (err != hipSuccess) return (int)err;
    if (nnz < 0) return kInvalid;
    if (nnz == 0) return 0;
    if (!Cir || !P || (nrows > 0 && (!A || !B))) return kInvalid;
    return finish_blocking(bm::dds_csc(nrows, ncols, nnz, A, B, Cir, Cjc, P, 0, nullptr));
}

API int bidmat_plan_create(int nrows, int ncols, int nnz, const int* Sir, const int* Sjc, int k_hint,
                           bidmat_plan** plan) {
    auto lock = bm::device_lock();
    if (!plan) return kInvalid;
    *plan = nullptr;
    if (nrows < 0 || ncols < 0 || nnz < 0 || k_hint < 0) return kInvalid;
    if (nnz > 0 && (!Sir || !Sjc)) return kInvalid;
    return (int)bm::plan_build(nrows, ncols, nnz, Sir, Sjc, k_hint, plan);
}

API int bidmat_plan_destroy(bidmat_plan* plan) {
    if (!plan) return 0;
    auto lock = bm::device_lock();          // no call of another thread is between its scratch lookup and its launch
    return (int)bm::plan_free(plan);
}

API long long bidmat_plan_bytes(const bidmat_plan* plan) {
    if (!plan) return 0;
    return (long long)(plan->row_bytes + plan->col_bytes +
                       ((plan->pvals ? 1 : 0) + (plan->cvals ? 1 : 0) + (plan->svals ? 1 : 0)) * (size_t)plan->nnz * sizeof(float));
}

API int bidmat_plan_segments(const bidmat_plan* plan) { return plan ? plan->nseg : 0; }

API long long bidmat_plan_info(const bidmat_plan* plan, const char* name) {
    if (!plan || !name) return -1;
    if (!strcmp(name, "nrows")) return plan->nrows;
    if (!strcmp(name, "ncols")) return plan->ncols;
    if (!strcmp(name, "nnz")) return plan->nnz;
    if (!strcmp(name, "sides")) return plan->sides;
    if (!strcmp(name, "nseg")) return plan->nseg;
    if (!strcmp(name, "nheavy")) return plan->nheavy;
    if (!strcmp(name, "npanels")) return plan->npanels;
    if (!strcmp(name, "panel_cols")) return plan->panel_cols;
    if (!strcmp(name, "seglen")) return plan->seglen;
    if (!strcmp(name, "col_classes")) return plan->ncls;
    if (!strcmp(name, "class_hot")) return plan->hcap;
    if (!strcmp(name, "longest_column")) return plan->maxlen;
    if (!strcmp(name, "dense_rows")) return plan->ndense;
    if (!strcmp(name, "dense_blocks")) return plan->ndblocks;
    if (!strcmp(name, "dense_block_cols")) return plan->dcb;
    if (!strcmp(name, "dense_segments")) return plan->ndseg;
    if (!strncmp(name, "xcd_start", 9) && name[9] >= '0' && name[9] <= '8' && !name[10]) return plan->xcd_start[name[9] - '0'];
    return -1;
}

API int bidmat_plan_array(const bidmat_plan* plan, const char* name, const void** dptr, long long* count) {
    if (!plan || !name || !dptr || !count) return kInvalid;
    *dptr = nullptr;
    *count = 0;
    const bool rows = (plan->sides & bm::PLAN_ROWS) != 0;
    const bool cls = (plan->sides & bm::PLAN_COLS) != 0 && plan->ncls == 8;
    struct { const char* n; const void* p; long long c; } tab[] = {
        {"pc", plan->pc, rows ? plan->nnz : 0}, {"perm", plan->perm, rows ? plan->nnz : 0},
        {"segstart", plan->segstart, rows && plan->segstart ? (long long)plan->nseg + 1 : 0},
        {"segrow", plan->segrow, rows ? plan->nseg : 0}, {"rowseg", plan->rowseg, rows ? plan->nseg : 0},
        {"rowptr", plan->rowptr, rows ? (long long)plan->nrows + 1 : 0},
        {"cir", plan->cir, cls ? plan->nnz : 0}, {"cperm", plan->cperm, cls ? plan->nnz : 0},
        {"cptr", plan->cptr, cls ? 16LL * plan->ncols + 1 : 0},
        {"ovf", plan->ovf, plan->ovf ? (long long)plan->ncols + 1 : 0},
        {"drow", plan->drow, plan->ndense}, {"drank", plan->drank, plan->ndense > 0 ? plan->nrows : 0},
        {"dpos", plan->dpos, (long long)plan->ndense * plan->ncols},
    };
    for (auto& t : tab)
        if (!strcmp(name, t.n)) { *dptr = t.c > 0 ? t.p : nullptr; *count = t.p ? t.c : 0; return 0; }
    return kInvalid;
}

API int bidmat_dsmultT_plan(bidmat_plan* plan, int k, const float* A, const float* Sdata, float* C,
                            int beta, void* stream) {
    auto lock = bm::device_lock();
    if (!plan || k < 0 || (beta != 0 && beta != 1)) return kInvalid;
    if (!plan_on_current_device(plan)) return (int)hipErrorInvalidDevice;
    if (!(plan->sides & bm::PLAN_ROWS)) return kInvalid;
    if (k == 0 || plan->nrows == 0) return 0;
    if (!C || (plan->nnz > 0 && (!A || (!Sdata && !plan->pvals)))) return kInvalid;
    return (int)run_dsmultT(plan, k, A, Sdata, C, beta, as_stream(stream));
}

API int bidmat_dsmultT_plan_staged(bidmat_plan* plan, int k, const float* A, const float* Sdata, float* C,
                                   int beta, void* stream, void* event_between) {
    auto lock = bm::device_lock();
    if (!plan || k < 0 || (beta != 0 && beta != 1)) return kInvalid;
    if (!plan_on_current_device(plan)) return (int)hipErrorInvalidDevice;
    if (!(plan->sides & bm::PLAN_ROWS)) return kInvalid;
    if (k == 0 || plan->nrows == 0) return 0;
    if (!C || (plan->nnz > 0 && (!A || (!Sdata && !plan->pvals)))) return kInvalid;
    return (int)run_dsmultT(plan, k, A, Sdata, C, beta, as_stream(stream), (hipEvent_t)event_between);
}

API long long bidmat_plan_heavy_nnz(const bidmat_plan* plan) {
    if (!plan || !(plan->sides & bm::PLAN_ROWS) || plan->nseg == 0 || !plan_on_current_device(plan)) return 0;
    // heavy segments come first in plan order: the light ones start at segment xcd_start[8]
    if (plan->xcd_start[8] >= plan->nseg) return plan->nnz;
    int first_light = 0;
    if (hipMemcpy(&first_light, plan->segstart + plan->xcd_start[8], sizeof(int), hipMemcpyDeviceToHost) != hipSuccess) return -1;
    return first_light;
}

API int bidmat_dsmult_plan(bidmat_plan* plan, int k, const float* A, const float* Sdata, const int* Sir,
                           const int* Sjc, float* C, int beta, void* stream) {
    auto lock = bm::device_lock();
    if (!plan || k < 0 || (beta != 0 && beta != 1)) return kInvalid;
    if (!plan_on_current_device(plan)) return (int)hipErrorInvalidDevice;
    if (k == 0 || plan->ncols == 0) return 0;
    return dsmult_through_plan(plan, k, A, Sdata, Sir, Sjc, C, beta, as_stream(stream));
}

namespace {
int dds_plan_entry(bidmat_plan* plan, int k, const float* A, const float* B, const int* Sir, const int* Sjc, const float* V,
                   bool stored, int opn, float* P, int beta, void* stream) {
    auto lock = bm::device_lock();
    if (!plan || k < 0 || (beta != 0 && beta != 1)) return kInvalid;
    if (!plan_on_current_device(plan)) return (int)hipErrorInvalidDevice;
    return dds_through_plan(plan, k, A, B, Sir, Sjc, V, stored, opn, P, beta, as_stream(stream));
}
}  // namespace

API int bidmat_dds_plan(bidmat_plan* plan, int k, const float* A, const float* B, const int* Sir, const int* Sjc,
                        const float* V, int opn, float* P, int beta, void* stream) {
    return dds_plan_entry(plan, k, A, B, Sir, Sjc, V, false, opn, P, beta, stream);
}

API int bidmat_dds_plan_stored(bidmat_plan* plan, int k, const float* A, const float* B, const int* Sir, const int* Sjc,
                               int opn, float* P, void* stream) {
    return dds_plan_entry(plan, k, A, B, Sir, Sjc, nullptr, true, opn, P, 0, stream);
}

API int bidmat_dds_dsmultT_plan(bidmat_plan* plan, int k, const float* A, const float* B, const float* V, int opn,
                                float* Q, float* G, int beta, void* stream) {
    auto lock = bm::device_lock();
    if (!plan || k < 0 || (beta != 0 && beta != 1) || opn < 0 || opn > 14) return kInvalid;
    if (!plan_on_current_device(plan)) return (int)hipErrorInvalidDevice;
    if (!(plan->sides & bm::PLAN_ROWS)) return kInvalid;
    if (k == 0 || plan->nrows == 0) return 0;
    if (!G || (plan->nnz > 0 && (!A || !B || (!V && !plan->pvals)))) return kInvalid;
    hipStream_t s = as_stream(stream);
    hipError_t err;
    float* partial = row_partial(plan, k, s, &err);
    if (!partial) return (int)err;
    if ((err = bm::fused_segments(k, k, k, plan->nseg, plan->xcd_start, plan->segrow, A, B, V ? V : plan->pvals, plan->pc,
                                  V ? plan->perm : nullptr, plan->perm, opn, plan->segstart, partial, Q, s)) != hipSuccess)
        return (int)err;
    return (int)bm::reduce_segments(k, plan->nrows, plan->rowptr, plan->rowseg, partial, G, beta, s);
}

API int bidmat_plan_set_values(bidmat_plan* plan, const float* Sdata, void* stream) {
    if (!plan) return kInvalid;
    auto lock = bm::device_lock();
    if (!plan_on_current_device(plan)) return (int)hipErrorInvalidDevice;
    if (plan->nnz == 0) return 0;
    if (!Sdata) return kInvalid;
    return (int)bm::plan_set_values(plan, Sdata, as_stream(stream));
}

API int bidmat_plan_overflow_segments(const bidmat_plan* plan) { return plan ? plan->novf : 0; }

API int bidmat_spsum_cols(int ncols, int nnz, const float* Sdata, const int* Sjc, float* out, int beta,
                          void* stream) {
    if (ncols < 0 || nnz < 0 || (beta != 0 && beta != 1)) return kInvalid;
    if (ncols == 0) return 0;
    if (!Sjc || !out || (nnz > 0 && !Sdata)) return kInvalid;
    return (int)bm::spsum_cols(ncols, nnz, Sdata, Sjc, out, beta, as_stream(stream));
}

API int bidmat_spsum_rows_plan(bidmat_plan* plan, const float* Sdata, float* out, int beta, void* stream) {
    auto lock = bm::device_lock();
    if (!plan || (beta != 0 && beta != 1)) return kInvalid;
    if (!plan_on_current_device(plan)) return (int)hipErrorInvalidDevice;
    if (!(plan->sides & bm::PLAN_ROWS)) return kInvalid;
    if (plan->nrows == 0) return 0;
    if (!out || (plan->nnz > 0 && !Sdata && !plan->pvals)) return kInvalid;
    return (int)run_spsum_rows(plan, Sdata, out, beta, as_stream(stream));
}

API int bidmat_spsum_rows_csc(int nrows, int nnz, const int* Sir, const float* Sdata, float* out, int beta,
                              void* stream) {
    auto lock = bm::device_lock();
    if (nrows < 0 || nnz < 0 || (beta != 0 && beta != 1)) return kInvalid;
    if (nrows == 0) return 0;
    if (!out || (nnz > 0 && (!Sir || !Sdata))) return kInvalid;
    return (int)bm::spsum_rows_exact(nrows, nnz, Sir, Sdata, out, beta, nullptr, as_stream(stream));
}

API int bidmat_transpose(int nrows, int ncols, const float* in, int ldi, float* out, int ldo, void* stream) {
    if (nrows < 0 || ncols < 0 || ldi < nrows || ldo < ncols) return kInvalid;
    if (nrows == 0 || ncols == 0) return 0;
    if (!in || !out) return kInvalid;
    return (int)bm::transpose(nrows, ncols, in, ldi, out, ldo, as_stream(stream));
}

API int bidmat_sdtmult_csc(int nrows, int ncols, int nnz, int p, const float* Sdata, const int* Sir,
                           const int* Sjc, const float* A, int lda, float* C, int ldc, void* stream) {
    auto lock = bm::device_lock();
    if (nrows < 0 || ncols < 0 || nnz < 0 || p < 0 || lda < nrows || ldc < ncols) return kInvalid;
    if (ncols == 0 || p == 0) return 0;
    if (!Sjc || !C || (nnz > 0 && (!Sdata || !Sir || !A))) return kInvalid;
    hipStream_t s = as_stream(stream);
    hipError_t err;
    // At = A^T (p x nrows), Ct = At * S (p x ncols), C = Ct^T
    float* At = (float*)bm::ws_get(bm::WS_TRANS_IN, sizeof(float) * (size_t)p * (size_t)(nrows > 0 ? nrows : 1), &err, s);
    if (!At) return (int)err;
    float* Ct = (float*)bm::ws_get(bm::WS_TRANS_OUT, sizeof(float) * (size_t)p * (size_t)ncols, &err, s);
    if (!Ct) return (int)err;
    if ((err = bm::transpose(nrows, p, A, lda, At, p, s)) != hipSuccess) return (int)err;
    if ((err = bm::dsmult_csc(p, ncols, nnz, At, Sdata, Sir, Sjc, Ct, 0, s)) != hipSuccess) return (int)err;
    return (int)bm::transpose(p, ncols, Ct, p, C, ldc, s);
}

API int bidmat_sdmult_plan(bidmat_plan* plan, int p, const float* Sdata, const float* A, int lda, float* C,
                           int ldc, void* stream) {
    auto lock = bm::device_lock();
    if (!plan || p < 0) return kInvalid;
    if (!plan_on_current_device(plan)) return (int)hipErrorInvalidDevice;
    if (lda < plan->ncols || ldc < plan->nrows || !(plan->sides & bm::PLAN_ROWS)) return kInvalid;
    if (plan->nrows == 0 || p == 0) return 0;
    if (!C || (plan->nnz > 0 && (!Sdata || !A))) return kInvalid;
    hipStream_t s = as_stream(stream);
    hipError_t err;
    // At = A^T (p x ncols), Ct = At *^ S (p x nrows), C = Ct^T
    float* At = (float*)bm::ws_get(bm::WS_TRANS_IN, sizeof(float) * (size_t)p * (size_t)(plan->ncols > 0 ? plan->ncols : 1), &err, s);
    if (!At) return (int)err;
    float* Ct = (float*)bm::ws_get(bm::WS_TRANS_OUT, sizeof(float) * (size_t)p * (size_t)plan->nrows, &err, s);
    if (!Ct) return (int)err;
    if ((err = bm::transpose(plan->ncols, p, A, lda, At, p, s)) != hipSuccess) return (int)err;
    if ((err = run_dsmultT(plan, p, At, Sdata, Ct, 0, s)) != hipSuccess) return (int)err;
    return (int)bm::transpose(p, plan->nrows, Ct, p, C, ldc, s);
}

API int bidmat_csc_expand_cols(int ncols, int nnz, const int* Sjc, int* Sic, void* stream) {
    if (ncols < 0 || nnz < 0) return kInvalid;
    if (nnz == 0) return 0;
    if (!Sjc || !Sic) return kInvalid;
    return (int)bm::csc_expand_cols(ncols, nnz, Sjc, Sic, as_stream(stream));
}

API int bidmat_csc_implicit_rows(int ncols, int nnz, const int* Sjc, int* Sir, void* stream) {
    if (ncols < 0 || nnz < 0) return kInvalid;
    if (nnz == 0) return 0;
    if (!Sjc || !Sir) return kInvalid;
    return (int)bm::csc_implicit_rows(ncols, nnz, Sjc, Sir, as_stream(stream));
}

API int bidmat_csc_validate(int nrows, int ncols, int nnz, const int* Sir, const int* Sjc, int* rule) {
    auto lock = bm::device_lock();
    if (!rule) return kInvalid;
    *rule = 0;
    if (nrows < 0 || ncols < 0 || nnz < 0 || !Sjc) return kInvalid;
    hipError_t err;
    int* d_flags = (int*)bm::ws_get(bm::WS_MISC, 64, &err);
    if (!d_flags) return (int)err;
    err = bm::csc_validate(nrows, ncols, nnz, Sir, Sjc, d_flags, nullptr);
    int flags = 0;
    if (err == hipSuccess) err = hipMemcpy(&flags, d_flags, sizeof(int), hipMemcpyDeviceToHost);
    if (err != hipSuccess) return (int)err;
    for (int r = 1; r <= 6; ++r)
        if (flags & (1 << r)) { *rule = r; break; }
    return 0;
}

API int bidmat_csc_colslice_range(int ncols, int col1, int col2, const int* Sjc, int* start, int* nnz) {
    if (ncols < 0 || col1 < 0 || col2 < col1 || col2 > ncols || !Sjc || !start || !nnz) return kInvalid;
    int lo = 0, hi = 0;
    hipError_t e = hipMemcpy(&lo, Sjc + col1, sizeof(int), hipMemcpyDeviceToHost);
    if (e == hipSuccess) e = hipMemcpy(&hi, Sjc + col2, sizeof(int), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return (int)e;
    if (lo < 0 || hi < lo) return kInvalid;
    *start = lo;
    *nnz = hi - lo;
    return 0;
}

API int bidmat_csc_colslice(int col1, int col2, int start, int nnz, const int* Sjc, const int* Sir, const float* Sdata,
                            int* out_jc, int* out_ir, int* out_ic, float* out_data, void* stream) {
    if (col1 < 0 || col2 < col1 || start < 0 || nnz < 0) return kInvalid;
    if (!Sjc || !out_jc || (nnz > 0 && (!Sir || !Sdata || !out_ir || !out_data))) return kInvalid;
    return (int)bm::csc_colslice(col2 - col1, start, nnz, Sjc + col1, Sir, Sdata, out_jc, out_ir, out_ic, out_data,
                                 as_stream(stream));
}

API int bidmat_csc_transpose(int nrows, int ncols, int nnz, const float* Sdata, const int* Sir, const int* Sjc,
                             float* out_data, int* out_ir, int* out_jc) {
    auto lock = bm::device_lock();
    if (nrows < 0 || ncols < 0 || nnz < 0 || !out_jc) return kInvalid;
    if (nnz > 0 && (!Sdata || !Sir || !Sjc || !out_data || !out_ir)) return kInvalid;
    return finish_blocking(bm::csc_transpose(nrows, ncols, nnz, Sdata, Sir, Sjc, out_data, out_ir, out_jc, nullptr));
}

API int bidmat_full(const int* ir, const int* ic, const float* data, float* od, int nrows, int ncols, int nnz) {
    if (nrows < 0 || ncols < 0 || nnz < 0) return kInvalid;
    if (nnz == 0) return 0;
    if (!ir || !ic || !data || !od) return kInvalid;
    return finish_blocking(bm::full_from_coo(nrows, ncols, nnz, ir, ic, data, od, nrows, nullptr));
}

API int bidmat_nhot(int n, int ncols, const int* cats, int* out_ir, int* out_ic, int* out_jc, float* out_data,
                    int* maxcat) {
    auto lock = bm::device_lock();
    if (n < 0 || ncols < 0 || (long long)n * ncols > 0x7fffffffLL || !out_jc) return kInvalid;
    if ((long long)n * ncols > 0 && (!cats || !out_ir || !out_ic || !out_data)) return kInvalid;
    hipError_t err;
    int* d_max = (int*)bm::ws_get(bm::WS_MISC, 64, &err);
    if (!d_max) return (int)err;
    err = bm::nhot(n, ncols, cats, out_ir, out_ic, out_jc, out_data, d_max, nullptr);
    int m = -1;
    if (err == hipSuccess) err = hipMemcpy(&m, d_max, sizeof(int), hipMemcpyDeviceToHost);
    if (maxcat) *maxcat = m;
    return finish_blocking(err);
}

API int bidmat_index_shift(int* p, long long n, int delta, void* stream) {
    if (n < 0 || (n > 0 && !p)) return kInvalid;
    return (int)bm::index_shift(p, n, delta, as_stream(stream));
}

API int bidmat_coo_compress_cols(int ncols, int nnz, const int* Sic, int* Sjc, void* stream) {
    if (ncols < 0 || nnz < 0) return kInvalid;
    if (!Sjc || (nnz > 0 && !Sic)) return kInvalid;
    return (int)bm::coo_compress_cols(ncols, nnz, Sic, Sjc, as_stream(stream));
}

API int bidmat_applyop_flat(const float* A, const float* B, float* C, long long n, int opn, void* stream) {
    if (n < 0 || opn < 0 || opn > 14) return kInvalid;
    if (n == 0) return 0;
    if (!A || !B || !C) return kInvalid;
    // a flat array is a column vector longer than an int allows: walk it in int-sized pieces
    const long long piece = 1LL << 30;
    for (long long off = 0; off < n; off += piece) {
        const int len = (int)((n - off) < piece ? (n - off) : piece);
        hipError_t e = bm::applyop(A + off, len, 1, B + off, len, 1, C + off, opn, as_stream(stream));
        if (e != hipSuccess) return (int)e;
    }
    return 0;
}

// ======================================================================== memory / runtime

API int bidmat_device_count(int* count) { return count ? (int)hipGetDeviceCount(count) : kInvalid; }
API int bidmat_set_device(int dev) { return (int)hipSetDevice(dev); }
API int bidmat_get_device(int* dev) { return dev ? (int)hipGetDevice(dev) : kInvalid; }

API int bidmat_malloc(void** dptr, long long bytes) {
    if (!dptr || bytes < 0) return kInvalid;
    *dptr = nullptr;
    hipError_t e = hipMalloc(dptr, bytes > 0 ? (size_t)bytes : 256);
    if (e == hipSuccess && getenv("BIDMAT_DEBUG_MEM")) {
        size_t f = 0, t = 0;
        (void)hipMemGetInfo(&f, &t);
        fprintf(stderr, "[bidmathip] malloc %lld bytes, free fraction %.3f\n", bytes, t ? (double)f / t : 0.0);
    }
    return (int)e;
}
API int bidmat_free(void* dptr) { return dptr ? (int)hipFree(dptr) : 0; }
API int bidmat_memcpy_h2d(void* dst, const void* src, long long bytes) {
    if (bytes < 0 || (bytes > 0 && (!dst || !src))) return kInvalid;
    return bytes ? (int)hipMemcpy(dst, src, (size_t)bytes, hipMemcpyHostToDevice) : 0;
}
API int bidmat_memcpy_d2h(void* dst, const void* src, long long bytes) {
    if (bytes < 0 || (bytes > 0 && (!dst || !src))) return kInvalid;
    return bytes ? (int)hipMemcpy(dst, src, (size_t)bytes, hipMemcpyDeviceToHost) : 0;
}
API int bidmat_memcpy_d2d(void* dst, const void* src, long long bytes) {
    if (bytes < 0 || (bytes > 0 && (!dst || !src))) return kInvalid;
    return bytes ? (int)hipMemcpy(dst, src, (size_t)bytes, hipMemcpyDeviceToDevice) : 0;
}
API int bidmat_memcpy_h2d_async(void* dst, const void* src, long long bytes, void* stream) {
    if (bytes < 0 || (bytes > 0 && (!dst || !src))) return kInvalid;
    return bytes ? (int)hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyHostToDevice, as_stream(stream)) : 0;
}
API int bidmat_memcpy_d2h_async(void* dst, const void* src, long long bytes, void* stream) {
    if (bytes < 0 || (bytes > 0 && (!dst || !src))) return kInvalid;
    return bytes ? (int)hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToHost, as_stream(stream)) : 0;
}
API int bidmat_memset(void* dptr, int value, long long bytes) {
    if (bytes < 0 || (bytes > 0 && !dptr)) return kInvalid;
    if (!bytes) return 0;
    hipError_t e = hipMemset(dptr, value, (size_t)bytes);
    if (e != hipSuccess) return (int)e;
    return (int)hipStreamSynchronize(nullptr);
}
API int bidmat_mem_info(long long* free_bytes, long long* total_bytes) {
    size_t f = 0, t = 0;
    hipError_t e = hipMemGetInfo(&f, &t);
    if (free_bytes) *free_bytes = (long long)f;
    if (total_bytes) *total_bytes = (long long)t;
    return (int)e;
}
API int bidmat_synchronize(void) { return (int)hipDeviceSynchronize(); }
API int bidmat_host_alloc(void** hptr, long long bytes) {
    if (!hptr || bytes < 0) return kInvalid;
    return (int)hipHostMalloc(hptr, bytes > 0 ? (size_t)bytes : 256, hipHostMallocDefault);
}
API int bidmat_host_free(void* hptr) { return hptr ? (int)hipHostFree(hptr) : 0; }

API int bidmat_stream_create(void** stream) {
    if (!stream) return kInvalid;
    hipStream_t s;
    hipError_t e = hipStreamCreate(&s);      // default priority
    *stream = (e == hipSuccess) ? (void*)s : nullptr;
    return (int)e;
}
API int bidmat_stream_destroy(void* stream) {
    auto lock = bm::device_lock();
    if (!stream) return 0;
    hipError_t e = hipStreamSynchronize(as_stream(stream));
    hipError_t f = bm::ws_drop_stream(as_stream(stream));      // the stream's scratch goes with it
    hipError_t g = hipStreamDestroy(as_stream(stream));
    return (int)(e != hipSuccess ? e : (f != hipSuccess ? f : g));
}
API int bidmat_stream_synchronize(void* stream) { return (int)hipStreamSynchronize(as_stream(stream)); }
// ---- HIP graphs: record a sequence of stream-taking calls once, replay it with one launch
API int bidmat_graph_begin_capture(void* stream) {
    if (!stream) return kInvalid;                  // the default stream cannot be captured
    return (int)hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal);
}
API int bidmat_graph_end_capture(void* stream, void** graph_exec) {
    if (!stream || !graph_exec) return kInvalid;
    *graph_exec = nullptr;
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(as_stream(stream), &g);
    if (e != hipSuccess) return (int)e;
    hipGraphExec_t x = nullptr;
    e = hipGraphInstantiate(&x, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) return (int)e;
    *graph_exec = (void*)x;
    return 0;
}
API int bidmat_graph_launch(void* graph_exec, void* stream) {
    if (!graph_exec) return kInvalid;
    return (int)hipGraphLaunch((hipGraphExec_t)graph_exec, as_stream(stream));
}
API int bidmat_graph_destroy(void* graph_exec) {
    return graph_exec ? (int)hipGraphExecDestroy((hipGraphExec_t)graph_exec) : 0;
}

API int bidmat_event_create(void** event) {
    if (!event) return kInvalid;
    hipEvent_t ev;
    hipError_t e = hipEventCreate(&ev);
    *event = (e == hipSuccess) ? (void*)ev : nullptr;
    return (int)e;
}
API int bidmat_event_destroy(void* event) { return event ? (int)hipEventDestroy((hipEvent_t)event) : 0; }
API int bidmat_event_record(void* event, void* stream) {
    return event ? (int)hipEventRecord((hipEvent_t)event, as_stream(stream)) : kInvalid;
}
API int bidmat_event_synchronize(void* event) { return event ? (int)hipEventSynchronize((hipEvent_t)event) : kInvalid; }
API int bidmat_event_elapsed_ms(void* start, void* stop, float* ms) {
    if (!start || !stop || !ms) return kInvalid;
    return (int)hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop);
}

API const char* bidmat_error_string(int err) { return hipGetErrorString((hipError_t)err); }

API const char* bidmat_version(void) { return "bidmathip 0.1 (gfx950, wave64, HIP)"; }

API int bidmat_device_info(char* arch, int arch_len, int* compute_units, long long* total_mem) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return (int)e;
    if (arch && arch_len > 0) {
        strncpy(arch, prop.gcnArchName, (size_t)arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (total_mem) *total_mem = (long long)prop.totalGlobalMem;
    return 0;
}

API int bidmat_set_option(const char* name, long long value) {
    if (!name) return kInvalid;
    if (!strcmp(name, "seglen")) {
        if (value < 64 || value > (1 << 24)) return kInvalid;
        bm::g_seglen.store((int)value);
        return 0;
    }
    if (!strcmp(name, "panel_kb")) {
        if (value < 16 || value > (1 << 22)) return kInvalid;
        bm::g_panel_kb.store((int)value);
        return 0;
    }
    if (!strcmp(name, "heavy_min")) {
        if (value < 1 || value > (1 << 20)) return kInvalid;
        bm::g_heavy_min.store((int)value);
        return 0;
    }
    if (!strcmp(name, "class_phases")) {
        if (value != 0 && value != 1 && value != 2 && value != 4 && value != 8) return kInvalid;
        bm::g_class_phases.store((int)value);
        return 0;
    }
    if (!strcmp(name, "plan_keep_mb")) {
        if (value < 0 || value > (1 << 20)) return kInvalid;
        bm::g_plan_keep_mb.store((int)value);
        return 0;
    }
    if (!strcmp(name, "cache_cols_after")) {
        if (value < 0 || value > (1 << 20)) return kInvalid;
        bm::g_cache_cols_after.store((int)value);
        return 0;
    }
    if (!strcmp(name, "cache_plans")) {
        if (value < 1 || value > 1024) return kInvalid;
        bm::g_cache_plans.store((int)value);
        return 0;
    }
    if (!strcmp(name, "check_plan")) {
        if (value != 0 && value != 1) return kInvalid;
        bm::g_check_plan.store((int)value);
        return 0;
    }
    if (!strcmp(name, "plan_builder")) {
        if (value != 0 && value != 1) return kInvalid;
        bm::g_plan_builder.store((int)value);
        return 0;
    }
    if (!strcmp(name, "class_shift")) {
        if (value < -1 || value > 16) return kInvalid;
        bm::g_class_shift.store((int)value);
        return 0;
    }
    if (!strcmp(name, "rowsum_form")) {
        if (value != 0 && value != 2) return kInvalid;
        bm::g_rowsum_form.store((int)value);
        return 0;
    }
    if (!strcmp(name, "plan_pool_mb")) {
        if (value < 0 || value > (1 << 20)) return kInvalid;
        bm::g_plan_pool_mb.store((int)value);
        return 0;
    }
    if (!strcmp(name, "class_threads")) {
        if (value != 256 && value != 512 && value != 1024) return kInvalid;
        bm::g_class_threads.store((int)value);
        return 0;
    }
    if (!strcmp(name, "class_hot")) {
        if (value < -1 || value > 1024) return kInvalid;
        bm::g_class_hot.store((int)value);
        return 0;
    }
    if (!strcmp(name, "class_strip")) {
        if (value < 1 || value > 64) return kInvalid;
        bm::g_class_strip.store((int)value);
        return 0;
    }
    if (!strcmp(name, "col_classes")) {
        if (value < -1 || value > 1) return kInvalid;
        bm::g_col_classes.store((int)value);
        return 0;
    }
    if (!strcmp(name, "dense_rows")) {
        if (value < 0 || value > bm::dense_rows_max() || value % 32 != 0) return kInvalid;
        bm::g_dense_rows.store((int)value);
        return 0;
    }
    if (!strcmp(name, "dense_min_pct")) {
        if (value < 1 || value > 100) return kInvalid;
        bm::g_dense_min_pct.store((int)value);
        return 0;
    }
    if (!strcmp(name, "dense_min_nnz")) {
        if (value < 0 || value > 0x7fffffffLL) return kInvalid;
        bm::g_dense_min_nnz.store((int)value);
        return 0;
    }
    if (!strcmp(name, "dense_cb")) {
        if (value < 0 || value > (1 << 24)) return kInvalid;
        bm::g_dense_cb.store((int)value);
        return 0;
    }
    if (!strcmp(name, "scalar_values")) {
        if (value != 0 && value != 1) return kInvalid;
        bm::g_scalar_values.store((int)value);
        return 0;
    }
    return kInvalid;
}

API long long bidmat_get_option(const char* name) {
    if (!name) return -1;
    if (!strcmp(name, "seglen")) return bm::opt_seglen();
    if (!strcmp(name, "panel_kb")) return bm::opt_panel_kb();
    if (!strcmp(name, "heavy_min")) return bm::opt_heavy_min();
    if (!strcmp(name, "col_classes")) return bm::opt_col_classes();
    if (!strcmp(name, "class_strip")) return bm::opt_class_strip();
    if (!strcmp(name, "class_hot")) return bm::opt_class_hot();
    if (!strcmp(name, "class_threads")) return bm::opt_class_threads();
    if (!strcmp(name, "class_phases")) return bm::opt_class_phases();
    if (!strcmp(name, "plan_keep_mb")) return bm::opt_plan_keep_mb();
    if (!strcmp(name, "cache_cols_after")) return bm::g_cache_cols_after.load();
    if (!strcmp(name, "cache_plans")) return bm::g_cache_plans.load();
    if (!strcmp(name, "check_plan")) return bm::opt_check_plan();
    if (!strcmp(name, "plan_builder")) return bm::opt_plan_builder();
    if (!strcmp(name, "rowsum_form")) return bm::opt_rowsum_form();
    if (!strcmp(name, "class_shift")) return bm::opt_class_shift();
    if (!strcmp(name, "plan_pool_mb")) return bm::opt_plan_pool_mb();
    if (!strcmp(name, "dense_rows")) return bm::opt_dense_rows();
    if (!strcmp(name, "dense_min_pct")) return bm::opt_dense_min_pct();
    if (!strcmp(name, "dense_min_nnz")) return bm::opt_dense_min_nnz();
    if (!strcmp(name, "dense_cb")) return bm::opt_dense_cb();
    if (!strcmp(name, "scalar_values")) return bm::opt_scalar_values();
    return -2;
}

API int bidmat_release_caches(void) {
    auto lock = bm::device_lock();
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    (void)hipDeviceSynchronize();
    {
        std::lock_guard<std::mutex> lock(g_cache_mu);
        for (auto it = g_cache.begin(); it != g_cache.end();) {
            if (it->device == dev) it = g_cache.erase(it);
            else ++it;
        }
    }
    hipError_t p = bm::pool_release();
    hipError_t w = bm::ws_release();
    return (int)(p != hipSuccess ? p : w);
}
