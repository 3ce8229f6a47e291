// Handle-based C exports of the host-side mirror, so that scripts (the parity tests) can drive
// GMat / GSMat operators without a C++ toolchain. A handle owns one shared_ptr; release it with
// bmh_release. Functions that can throw return NULL / -1 and leave the text in bmh_last_error().
#include "bidmat.hpp"
#include "../../include/bidmat_hip.h"
#include <cstring>

using namespace BIDMat;

#define API extern "C" __attribute__((visibility("default")))

namespace {
struct Handle {
    GMatP g;
    GSMatP s;
};
thread_local std::string g_err;

template <typename F>
void* guard_ptr(F f) {
    try { return f(); } catch (const std::exception& e) { g_err = e.what(); return nullptr; }
}
template <typename F>
int guard_int(F f) {
    try { f(); return 0; } catch (const std::exception& e) { g_err = e.what(); return -1; }
}
Handle* H(void* h) { return static_cast<Handle*>(h); }
GMatP G(void* h) { return h ? H(h)->g : nullptr; }
GSMatP S(void* h) { return h ? H(h)->s : nullptr; }
void* wrap(GMatP g) { auto* h = new Handle(); h->g = std::move(g); return h; }
void* wrap(GSMatP s) { auto* h = new Handle(); h->s = std::move(s); return h; }
}  // namespace

API const char* bmh_last_error() { return g_err.c_str(); }
API void bmh_release(void* h) { delete H(h); }
API const char* bmh_type(void* h) { return H(h)->g ? "GMat" : "GSMat"; }
API long long bmh_guid(void* h) { return H(h)->g ? H(h)->g->GUID : H(h)->s->GUID; }
API int bmh_same_object(void* a, void* b) {
    return (H(a)->g && H(a)->g == H(b)->g) || (H(a)->s && H(a)->s == H(b)->s);
}

// 1 when two sparse matrices point at the same device index arrays
API int bmh_same_pattern(void* a, void* b) { return S(a)->pir == S(b)->pir && S(a)->pjc == S(b)->pjc && S(a)->pic == S(b)->pic; }
// 1 when the matrix's pattern has a plan by now
API int bmh_has_plan(void* s) { return S(s)->planHolder && S(s)->planHolder->plan != nullptr; }

API void* bmh_gmat_from_host(int nr, int nc, const float* data) {
    return guard_ptr([&] { return wrap(GMat::fromFMat(FMat(nr, nc, data))); });
}
API void* bmh_gmat_zeros(int nr, int nc) { return guard_ptr([&] { return wrap(GMat::zeros(nr, nc)); }); }
API int bmh_gmat_dims(void* h, int* nr, int* nc) { *nr = G(h)->nrows; *nc = G(h)->ncols; return 0; }
API int bmh_gmat_to_host(void* h, float* out) {
    return guard_int([&] { FMat f = G(h)->toFMat(); memcpy(out, f.data.data(), sizeof(float) * f.data.size()); });
}

// host arrays carry the index base Mat::ioneBased, exactly like a host SMat
API void* bmh_gsmat_from_host(int nr, int nc, int nnz, const float* data, const int* ir, const int* jc) {
    return guard_ptr([&] { return wrap(GSMat::fromHost(nr, nc, nnz, data, ir, jc, Mat::ioneBased)); });
}
API int bmh_gsmat_dims(void* h, int* nr, int* nc, int* nnz) {
    *nr = S(h)->nrows; *nc = S(h)->ncols; *nnz = S(h)->nnz();
    return 0;
}
// copies the matrix back as a host SMat and runs SparseMat.check on it
API int bmh_gsmat_to_host(void* h, float* data, int* ir, int* jc) {
    return guard_int([&] {
        S(h)->toHost(data, ir, jc);
        SMat::checkArrays(S(h)->nrows, S(h)->ncols, S(h)->nnz(), ir, jc);
    });
}
// the device column pointer, 0-based (to check that DDS results carry it)
API int bmh_gsmat_device_jc(void* h, int* jc) {
    return bidmat_memcpy_d2h(jc, S(h)->pjc, (long long)sizeof(int) * ((long long)S(h)->ncols + 1));
}

API void* bmh_mult(void* a, void* s, void* out) { return guard_ptr([&] { return wrap(G(a)->GSMult(S(s), G(out))); }); }
API void* bmh_madd(void* a, void* s, void* out) { return guard_ptr([&] { return wrap(G(a)->madd(S(s), G(out))); }); }
API void* bmh_multT(void* a, void* s, void* out) { return guard_ptr([&] { return wrap(G(a)->GSMultT(S(s), G(out))); }); }
API void* bmh_maddT(void* a, void* s, void* out) { return guard_ptr([&] { return wrap(G(a)->maddT(S(s), G(out))); }); }
API void* bmh_tile_mult(void* a, int nr, int nc, int kk, int aroff, int acoff, void* b, int broff, int bcoff,
                        void* c, int croff, int ccoff, int transposed) {
    return guard_ptr([&] {
        return wrap(transposed ? G(a)->tileMultNT(nr, nc, kk, aroff, acoff, S(b), broff, bcoff, G(c), croff, ccoff)
                               : G(a)->tileMult(nr, nc, kk, aroff, acoff, S(b), broff, bcoff, G(c), croff, ccoff));
    });
}
API void* bmh_sdmult(void* s, void* a, void* out, int transposed) {
    return guard_ptr([&] { return wrap(transposed ? S(s)->SDTMult(G(a), G(out)) : S(s)->SDMult(G(a), G(out))); });
}
API void* bmh_gsdop(void* s, void* b, void* out, int op) {
    return guard_ptr([&] { return wrap(S(s)->GSDop(G(b), S(out), op)); });
}
API void* bmh_nhot(const int* cats, int n, int ncols, int ncats) {
    return guard_ptr([&] {
        std::vector<int> c(cats, cats + (size_t)n * (size_t)ncols);
        return wrap(GSMat::nHot(c, n, ncols, ncats));
    });
}
API void* bmh_t(void* s, void* out) { return guard_ptr([&] { return wrap(S(s)->t(S(out))); }); }
API void* bmh_full(void* s, void* out) { return guard_ptr([&] { return wrap(S(s)->full(G(out))); }); }
API void* bmh_colslice(void* s, int col1, int col2, void* out) {
    return guard_ptr([&] { return wrap(S(s)->colslice(col1, col2, S(out))); });
}
API void* bmh_dds(void* a, void* b, void* c, void* out) {
    return guard_ptr([&] { return wrap(GSMat::DDS(G(a), G(b), S(c), S(out))); });
}
API void* bmh_sum_sparse(void* s, int n, void* out) { return guard_ptr([&] { return wrap(S(s)->sum(n, G(out))); }); }
API void* bmh_sum_dense(void* a, int n, void* out) { return guard_ptr([&] { return wrap(sum(G(a), n, G(out))); }); }
API void* bmh_reduce(void* a, void* out, int dir, float initv, int op) {
    return guard_ptr([&] { return wrap(G(a)->reduceOp(G(out), dir, initv, op)); });
}
API void* bmh_gop(void* a, void* b, void* out, int op) { return guard_ptr([&] { return wrap(G(a)->gOp(G(b), G(out), op)); }); }
API void* bmh_contents(void* s) { return guard_ptr([&] { return wrap(S(s)->contents()); }); }
API void* bmh_with_values(void* s, void* vals) { return guard_ptr([&] { return wrap(S(s)->withValues(G(vals))); }); }

// ---- matrix files (host arrays carry Mat::ioneBased)
API int bmh_save_smat(const char* fname, int nr, int nc, int nnz, const float* data, const int* ir, const int* jc) {
    return guard_int([&] {
        SMat a(nr, nc, nnz);
        memcpy(a.data.data(), data, sizeof(float) * (size_t)nnz);
        memcpy(a.ir.data(), ir, sizeof(int) * (size_t)nnz);
        memcpy(a.jc.data(), jc, sizeof(int) * ((size_t)nc + 1));
        HMat::saveSMat(fname, a);
    });
}
// two calls: first with null arrays to learn the sizes, then with arrays to fill
API int bmh_load_smat(const char* fname, int* nr, int* nc, int* nnz, float* data, int* ir, int* jc) {
    return guard_int([&] {
        SMat a = HMat::loadSMat(fname);
        *nr = a.nrows; *nc = a.ncols; *nnz = a.nnz();
        if (data) {
            memcpy(data, a.data.data(), sizeof(float) * a.data.size());
            memcpy(ir, a.ir.data(), sizeof(int) * a.ir.size());
            memcpy(jc, a.jc.data(), sizeof(int) * a.jc.size());
        }
    });
}
API int bmh_save_fmat(const char* fname, int nr, int nc, const float* data) {
    return guard_int([&] { HMat::saveFMat(fname, FMat(nr, nc, data)); });
}
API int bmh_load_fmat(const char* fname, int* nr, int* nc, float* data) {
    return guard_int([&] {
        FMat a = HMat::loadFMat(fname);
        *nr = a.nrows; *nc = a.ncols;
        if (data) memcpy(data, a.data.data(), sizeof(float) * a.data.size());
    });
}
API void* bmh_load_gsmat(const char* fname) { return guard_ptr([&] { return wrap(HMat::loadGSMat(fname)); }); }

API long long bmh_nflops() { return Mat::nflops.load(); }
API void bmh_flip() { flip(); }
API double bmh_gflop(float* secs) { auto r = gflop(); if (secs) *secs = r.second; return r.first; }

API int bmh_set_flag(const char* name, double v) {
    if (!strcmp(name, "ioneBased")) Mat::ioneBased = (int)v;
    else if (!strcmp(name, "useGPUcache")) Mat::useGPUcache = v != 0;
    else if (!strcmp(name, "recycleGrow")) Mat::recycleGrow = v;
    else if (!strcmp(name, "debugMem")) Mat::debugMem = v != 0;
    else if (!strcmp(name, "numThreads")) Mat::numThreads = (int)v;
    else return -1;
    return 0;
}
API double bmh_get_flag(const char* name) {
    if (!strcmp(name, "ioneBased")) return Mat::ioneBased;
    if (!strcmp(name, "useGPUcache")) return Mat::useGPUcache;
    if (!strcmp(name, "recycleGrow")) return Mat::recycleGrow;
    if (!strcmp(name, "debugMem")) return Mat::debugMem;
    if (!strcmp(name, "numThreads")) return Mat::numThreads;
    return -1;
}
API void bmh_clear_caches() { Mat::clearCaches(); }

// SparseMat.check on host arrays (no device needed): 0 = valid, else -1 with the reference's message
API int bmh_smat_check(int nr, int nc, int nnz, const int* ir, const int* jc) {
    return guard_int([&] {
        SMat a(nr, nc, nnz);
        memcpy(a.ir.data(), ir, sizeof(int) * (size_t)nnz);
        memcpy(a.jc.data(), jc, sizeof(int) * ((size_t)nc + 1));
        a.check();
    });
}
