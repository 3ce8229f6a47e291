#include "bidmat.hpp"
#include "../../include/bidmat_hip.h"
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <functional>
#include <mutex>

namespace BIDMat {

// ------------------------------------------------------------------ globals
int Mat::ioneBased = 1;
bool Mat::useGPUcache = false;
double Mat::recycleGrow = 1.2;
bool Mat::debugMem = false;
int Mat::numThreads = 8;
std::atomic<long long> Mat::nflops{0};

namespace {
std::atomic<long long> g_guid{1000};
std::mutex g_cache_mu;
using Key = std::tuple<long long, long long, long long, long long, int>;
std::map<Key, GMatP> g_gcache;
std::map<Key, GSMatP> g_scache;

std::string fmt(const char* f, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, f);
    vsnprintf(buf, sizeof buf, f, ap);
    va_end(ap);
    return buf;
}

[[noreturn]] void fail(const std::string& msg) { throw std::runtime_error(msg); }

void hipcheck(int err, const char* what) {
    if (err != 0) fail(std::string(what) + " " + bidmat_error_string(err));
}

long long opHash(const char* name) { return (long long)std::hash<std::string>()(name); }

void checkThread(int myGPU, const char* where, long long guid) {
    int cur = getGPU();
    if (myGPU != cur) fail(fmt("%s wrong thread %d %d for mat %lld", where, myGPU, cur, guid));
}
}  // namespace

long long Mat::newGUID() { return g_guid.fetch_add(1); }

void Mat::clearCaches() {
    std::lock_guard<std::mutex> lock(g_cache_mu);
    g_gcache.clear();
    g_scache.clear();
}

int getGPU() {
    int d = 0;
    hipcheck(bidmat_get_device(&d), "getGPU");
    return d;
}
void setGPU(int dev) { hipcheck(bidmat_set_device(dev), "setGPU"); }
std::pair<float, long long> GPUmem() {
    long long f = 0, t = 0;
    hipcheck(bidmat_mem_info(&f, &t), "GPUmem");
    return {t ? (float)((double)f / (double)t) : 0.f, f};
}

// ------------------------------------------------------------------ timers
namespace {
std::chrono::steady_clock::time_point g_tic = std::chrono::steady_clock::now();
long long g_lastFlops = 0;
float toc() { return std::chrono::duration<float>(std::chrono::steady_clock::now() - g_tic).count(); }
}  // namespace
void flip() { g_lastFlops = Mat::nflops.load(); g_tic = std::chrono::steady_clock::now(); }
std::pair<float, float> flop() { float t = toc(); return {(float)(Mat::nflops.load() - g_lastFlops) / t, t}; }
std::pair<float, float> gflop() { float t = toc(); return {(float)(Mat::nflops.load() - g_lastFlops) / t / 1e9f, t}; }

// ------------------------------------------------------------------ FMat / SMat
FMat::FMat(int nr, int nc) : nrows(nr), ncols(nc), data((size_t)nr * nc, 0.f), GUID(Mat::newGUID()) {}
FMat::FMat(int nr, int nc, const float* src) : nrows(nr), ncols(nc), data(src, src + (size_t)nr * nc), GUID(Mat::newGUID()) {}

SMat::SMat(int nr, int nc, int nnz) : nrows(nr), ncols(nc), ir((size_t)nnz), jc((size_t)nc + 1, Mat::ioneBased),
                                      data((size_t)nnz), GUID(Mat::newGUID()) {}

void SMat::check() const { checkArrays(nrows, ncols, nnz(), ir.data(), jc.data()); }

void SMat::checkArrays(int nrows, int ncols, int nnz, const int* ir, const int* jc) {
    const int ioff = Mat::ioneBased;
    if (jc[0] != ioff) fail(fmt("jc(0) should be %d", ioff));
    for (int i = 0; i < ncols; ++i) {
        int j = jc[i] - ioff;
        if (jc[i] > jc[i + 1]) fail(fmt("jc(i) out of order %d %d %d", i, jc[i], jc[i + 1]));
        while (j < jc[i + 1] - ioff - 1 && j + 1 < nnz) {      // never read past the arrays
            if (ir[j + 1] <= ir[j]) fail(fmt("ir(j) out of order %d %d %d", j, ir[j], ir[j + 1]));
            if (ir[j] < ioff) fail(fmt("ir(%d)=%d too small", j, ir[j]));
            if (ir[j + 1] >= nrows + ioff) fail(fmt("ir(%d)=%d out of range %d", j + 1, ir[j + 1], nrows + ioff));
            ++j;
        }
    }
    if (jc[ncols] != nnz + ioff) fail(fmt("jc(ncols) should be %d", nnz));
}

FMat SMat::full() const {
    FMat out(nrows, ncols);
    const int ioff = Mat::ioneBased;
    for (int i = 0; i < ncols; ++i)
        for (int j = jc[i] - ioff; j < jc[i + 1] - ioff; ++j)
            out.data[(size_t)(ir[j] - ioff) + (size_t)i * nrows] += data[j];
    return out;
}

// ------------------------------------------------------------------ GMat
GMat::GMat(int nr, int nc, float* p, long long rs, bool o)
    : nrows(nr), ncols(nc), pdata(p), realsize(rs), GUID(Mat::newGUID()), myGPU(getGPU()), owns(o) {}

GMat::~GMat() { free(); }

void GMat::free() {
    if (owns && pdata) bidmat_free(pdata);
    pdata = nullptr;
}

GMatP GMat::make(int nr, int nc) {
    long long n = (long long)nr * nc;
    if (Mat::debugMem) fprintf(stderr, "GMat %d %d, %d %f\n", nr, nc, getGPU(), GPUmem().first);
    void* p = nullptr;
    hipcheck(bidmat_malloc(&p, n * (long long)sizeof(float)), "GPU alloc failed");
    return std::make_shared<GMat>(nr, nc, (float*)p, n, true);
}

GMatP GMat::zeros(int nr, int nc) {
    GMatP m = make(nr, nc);
    m->clear();
    return m;
}

GMat& GMat::clear() {
    hipcheck(bidmat_memset(pdata, 0, (long long)sizeof(float) * length()), "GMat.clear");
    return *this;
}

GMatP GMat::fromFMat(const FMat& a, GMatP out) {
    GMatP m = newOrCheckGMat(a.nrows, a.ncols, out);
    hipcheck(bidmat_memcpy_h2d(m->pdata, a.data.data(), (long long)sizeof(float) * a.length()), "GMat() copy");
    return m;
}

FMat GMat::toFMat() const {
    FMat out(nrows, ncols);
    hipcheck(bidmat_memcpy_d2h(out.data.data(), pdata, (long long)sizeof(float) * length()), "toFMat copy");
    return out;
}

GMatP GMat::newOrCheckGMat(int nr, int nc, GMatP outmat) {
    if (!outmat || (outmat->nrows == 0 && outmat->ncols == 0)) return make(nr, nc);
    if (outmat->nrows != nr || outmat->ncols != nc) {
        // recycle: reuse the buffer when it is large enough (GMat.scala:1315-1331)
        if (outmat->realsize >= (long long)nr * nc) {
            auto m = std::make_shared<GMat>(nr, nc, outmat->pdata, outmat->realsize, false);
            m->keepalive = outmat;
            return m;
        }
        return make(nr, nc);
    }
    return outmat;
}

GMatP GMat::newOrCheckGMat(int nr, int nc, GMatP outmat, long long g1, long long g2, long long oph) {
    GMatP m;
    if (outmat || !Mat::useGPUcache) {
        m = newOrCheckGMat(nr, nc, outmat);
    } else {
        Key key(g1, g2, 0, oph, getGPU());
        std::lock_guard<std::mutex> lock(g_cache_mu);
        auto it = g_gcache.find(key);
        GMatP res = it == g_gcache.end() ? nullptr : it->second;
        m = newOrCheckGMat(nr, nc, res);
        if (m != res) g_gcache[key] = m;
    }
    checkThread(m->myGPU, "newOrCheckGMat", m->GUID);
    return m;
}

namespace {
// C = beta*C + A*S: through the plan of S's pattern when it has one (or is due one), else the plain kernel
int dsmultDispatch(const GMat& A, GSMat& S, float* C, int beta) {
    if (bidmat_plan* p = S.planIfDue(A.nrows))
        return bidmat_dsmult_plan(p, A.nrows, A.pdata, S.pdata, S.pir, S.pjc, C, beta, nullptr);
    return bidmat_dsmult_csc(A.nrows, S.ncols, S.nnz(), A.pdata, S.pdata, S.pir, S.pjc, C, beta, nullptr);
}
}  // namespace

GMatP GMat::GSMult(const GSMatP& a, GMatP oldmat) {
    if (ncols != a->nrows) fail(fmt("GSMult dimensions mismatch (%d %d) (%d %d)", nrows, ncols, a->nrows, a->ncols));
    GMatP out = newOrCheckGMat(nrows, a->ncols, oldmat, GUID, a->GUID, opHash("GSMult"));
    // the reference clears `out` and accumulates (GMat.scala:1047-1048); beta = 0 overwrites instead
    Mat::nflops += 2LL * nrows * a->nnz();
    int err = dsmultDispatch(*this, *a, out->pdata, 0);
    if (err == 0) err = bidmat_stream_synchronize(nullptr);
    if (err != 0) fail(std::string("GMult: HIP kernel error in dsmult ") + bidmat_error_string(err));
    return out;
}

GMatP GMat::madd(const GSMatP& a, GMatP out) {
    if (ncols != a->nrows || nrows != out->nrows || a->ncols != out->ncols)
        fail(fmt("GSMadd dimensions mismatch (%d %d) (%d %d) (%d %d)", nrows, ncols, a->nrows, a->ncols, out->nrows, out->ncols));
    Mat::nflops += 2LL * nrows * a->nnz();
    int err = dsmultDispatch(*this, *a, out->pdata, 1);
    if (err == 0) err = bidmat_stream_synchronize(nullptr);
    if (err != 0) fail(std::string("GMult: HIP kernel error in dsmult ") + bidmat_error_string(err));
    return out;
}

GMatP GMat::GSMultT(const GSMatP& a, GMatP oldmat) {
    if (ncols != a->ncols) fail(fmt("GSMult dimensions mismatch (%d %d) (%d %d)", nrows, ncols, a->ncols, a->nrows));
    GMatP out = newOrCheckGMat(nrows, a->nrows, oldmat, GUID, a->GUID, opHash("GSMultT"));
    Mat::nflops += 2LL * nrows * a->nnz();
    int err = bidmat_dsmultT_plan(a->plan(nrows), nrows, pdata, a->pdata, out->pdata, 0, nullptr);
    if (err == 0) err = bidmat_stream_synchronize(nullptr);
    if (err != 0) fail(std::string("GMult: HIP kernel error in dsmultT ") + bidmat_error_string(err));
    return out;
}

GMatP GMat::maddT(const GSMatP& a, GMatP out) {
    if (ncols != a->ncols || nrows != out->nrows || a->nrows != out->ncols)
        fail(fmt("GSMadd dimensions mismatch (%d %d) (%d %d) (%d %d)", nrows, ncols, a->ncols, a->nrows, out->nrows, out->ncols));
    Mat::nflops += 2LL * nrows * a->nnz();
    int err = bidmat_dsmultT_plan(a->plan(nrows), nrows, pdata, a->pdata, out->pdata, 1, nullptr);
    if (err == 0) err = bidmat_stream_synchronize(nullptr);
    if (err != 0) fail(std::string("GMult: HIP kernel error in dsmultT ") + bidmat_error_string(err));
    return out;
}

GMatP GMat::tileMult(int nr, int nc, int kk, int aroff, int acoff, const GSMatP& b, int broff, int bcoff,
                     GMatP c, int croff, int ccoff) {
    if (aroff < 0 || acoff < 0 || broff < 0 || bcoff < 0 || croff < 0 || ccoff < 0 || nr < 0 || nc < 0 || kk < 0)
        fail("tileMult: cant have negative offsets or dimensions");
    if (aroff + nr > nrows || acoff + kk > ncols || broff + kk > b->nrows || bcoff + nc > b->ncols ||
        croff + nr > c->nrows || ccoff + nc > c->ncols)
        fail("tileMult: tile strays outside matrix dimensions");
    Mat::nflops += 2LL * nr * b->nnz();
    int err = bidmat_dsmultTile(nr, nc, kk, b->nnz(), pdata + (aroff + (long long)acoff * nrows), nrows, b->pdata,
                                b->pir, b->pic, broff, bcoff, c->pdata + (croff + (long long)ccoff * c->nrows), c->nrows);
    if (err != 0) fail(std::string("tileMult error ") + bidmat_error_string(err));
    return c;
}

GMatP GMat::tileMultNT(int nr, int nc, int kk, int aroff, int acoff, const GSMatP& b, int broff, int bcoff,
                       GMatP c, int croff, int ccoff) {
    if (aroff < 0 || acoff < 0 || broff < 0 || bcoff < 0 || croff < 0 || ccoff < 0 || nr < 0 || nc < 0 || kk < 0)
        fail("tileMultNT: cant have negative offsets or dimensions");
    if (aroff + nr > nrows || acoff + kk > ncols || broff + nc > b->nrows || bcoff + kk > b->ncols ||
        croff + nr > c->nrows || ccoff + nc > c->ncols)
        fail("tileMultNT: tile strays outside matrix dimensions");
    Mat::nflops += 2LL * nr * b->nnz() * kk / std::max(1, b->ncols);
    int err = bidmat_dsmultTileT(nr, nc, kk, b->nnz(), pdata + (aroff + (long long)acoff * nrows), nrows, b->pdata,
                                 b->pir, b->pic, broff, bcoff, c->pdata + (croff + (long long)ccoff * c->nrows), c->nrows);
    if (err != 0) fail(std::string("tileMultT error ") + bidmat_error_string(err));
    return c;
}

GMatP GMat::gOp(const GMatP& a, GMatP oldmat, int op) {
    // compatible shapes (ND.compatibleGDims for the 2-D case): equal, or a row/column/scalar on either side
    const int nr = std::max(nrows, a->nrows), nc = std::max(ncols, a->ncols);
    const bool ok = (nrows == a->nrows || nrows == 1 || a->nrows == 1) && (ncols == a->ncols || ncols == 1 || a->ncols == 1) &&
                    ((nrows == a->nrows && ncols == a->ncols) || (a->nrows == 1 && a->ncols == 1) || (nrows == 1 && ncols == 1) ||
                     (nrows == a->nrows && (a->ncols == 1 || ncols == 1)) || (ncols == a->ncols && (a->nrows == 1 || nrows == 1)));
    if (!ok) fail(fmt("DenseMat Op: dimensions mismatch (%d %d) (%d %d)", nrows, ncols, a->nrows, a->ncols));
    GMatP out = newOrCheckGMat(nr, nc, oldmat, GUID, a->GUID, op);
    Mat::nflops += std::max(length(), a->length());
    int err = bidmat_applyop(pdata, nrows, ncols, a->pdata, a->nrows, a->ncols, out->pdata, op);
    if (err != 0) fail(fmt("HIP kernel error %d in applyop", err));
    return out;
}

GMatP GMat::reduceOp(GMatP oldmat, int dir, float initval, int op) {
    if (dir == 1 || (dir == 0 && nrows > 1)) {
        GMatP out = newOrCheckGMat(1, ncols, oldmat, GUID, 1, op);
        int err = bidmat_reduce1op(nrows, ncols, pdata, out->pdata, initval, op);
        if (err != 0) fail(std::string("HIP kernel error in reduce1op ") + bidmat_error_string(err));
        Mat::nflops += length();
        return out;
    } else if (dir == 2 || dir == 0) {
        GMatP out = newOrCheckGMat(nrows, 1, oldmat, GUID, 2, op);
        int err = bidmat_reduce2op(nrows, ncols, pdata, out->pdata, initval, op);
        if (err != 0) fail(std::string("HIP kernel error in reduce2op ") + bidmat_error_string(err));
        Mat::nflops += length();
        return out;
    }
    fail("dimension must be 1 or 2");
}

// ------------------------------------------------------------------ pinned staging
Staging::Staging(size_t chunk_bytes) : chunk_(chunk_bytes) {
    int err = bidmat_stream_create(&stream_);
    for (int i = 0; i < 2 && err == 0; ++i) {
        err = bidmat_host_alloc(&stage_[i], (long long)chunk_);
        if (err == 0) err = bidmat_event_create(&ev_[i]);
    }
    if (err != 0) {
        const std::string msg = std::string("HIP error creating staging buffers ") + bidmat_error_string(err);
        this->~Staging();
        fail(msg);
    }
}

Staging::~Staging() {
    if (stream_) bidmat_stream_synchronize(stream_);
    for (int i = 0; i < 2; ++i) {
        if (stage_[i]) bidmat_host_free(stage_[i]);
        if (ev_[i]) bidmat_event_destroy(ev_[i]);
        stage_[i] = ev_[i] = nullptr;
    }
    if (stream_) bidmat_stream_destroy(stream_);
    stream_ = nullptr;
}

void Staging::upload(void* dst, size_t bytes, const std::function<void(void*, size_t)>& fill) {
    char* d = static_cast<char*>(dst);
    while (bytes > 0) {
        const size_t n = bytes < chunk_ ? bytes : chunk_;
        if (busy_[which_]) hipcheck(bidmat_event_synchronize(ev_[which_]), "staging wait");
        fill(stage_[which_], n);
        hipcheck(bidmat_memcpy_h2d_async(d, stage_[which_], (long long)n, stream_), "staged upload");
        hipcheck(bidmat_event_record(ev_[which_], stream_), "staging event");
        busy_[which_] = true;
        which_ ^= 1;
        d += n;
        bytes -= n;
    }
}

void Staging::upload(void* dst, const void* src, size_t bytes) {
    const char* p = static_cast<const char*>(src);
    upload(dst, bytes, [&p](void* buf, size_t n) { memcpy(buf, p, n); p += n; });
}

void Staging::download(void* dst, const void* src, size_t bytes, int add) {
    // the copy into buffer b is enqueued one step ahead of the host draining buffer b^1
    char* out = static_cast<char*>(dst);
    const char* s = static_cast<const char*>(src);
    wait();
    size_t pending[2] = {0, 0};
    char* where[2] = {nullptr, nullptr};
    auto drain = [&](int b) {
        if (!pending[b]) return;
        hipcheck(bidmat_event_synchronize(ev_[b]), "staging wait");
        if (add == 0) {
            memcpy(where[b], stage_[b], pending[b]);
        } else {
            const int* in = static_cast<const int*>(stage_[b]);
            int* o = reinterpret_cast<int*>(where[b]);
            for (size_t i = 0; i < pending[b] / sizeof(int); ++i) o[i] = in[i] + add;
        }
        pending[b] = 0;
    };
    int b = 0;
    while (bytes > 0) {
        const size_t n = bytes < chunk_ ? bytes : chunk_;
        drain(b);
        hipcheck(bidmat_memcpy_d2h_async(stage_[b], s, (long long)n, stream_), "staged download");
        hipcheck(bidmat_event_record(ev_[b], stream_), "staging event");
        pending[b] = n;
        where[b] = out;
        out += n; s += n; bytes -= n;
        b ^= 1;
    }
    drain(b);
    drain(b ^ 1);
    busy_[0] = busy_[1] = false;
}

void Staging::wait() {
    hipcheck(bidmat_stream_synchronize(stream_), "staging sync");
    busy_[0] = busy_[1] = false;
}

// ------------------------------------------------------------------ GSMat
PlanHolder::~PlanHolder() {
    if (plan) bidmat_plan_destroy(plan);
}

Pattern::Pattern(int ncols, int realnnz) {
    void* p = nullptr;
    int err = bidmat_malloc(&p, (long long)sizeof(int) * realnnz); pir = (int*)p;
    if (err == 0) { err = bidmat_malloc(&p, (long long)sizeof(int) * realnnz); pic = (int*)p; }
    if (err == 0) { err = bidmat_malloc(&p, (long long)sizeof(int) * ((long long)ncols + 1)); pjc = (int*)p; }
    if (err != 0) {
        this->~Pattern();
        fail(std::string("HIP error in GSMat() ") + bidmat_error_string(err));
    }
}

Pattern::~Pattern() {
    if (pic) bidmat_free(pic);
    if (pir) bidmat_free(pir);
    if (pjc) bidmat_free(pjc);
    pic = pir = pjc = nullptr;
}

GSMat::GSMat(int nr, int nc, int nnz, int rn)
    : nrows(nr), ncols(nc), nnz0(nnz), pir(nullptr), pic(nullptr), pjc(nullptr), pdata(nullptr),
      realnnz(std::max(1, rn)), GUID(Mat::newGUID()), myGPU(getGPU()), planHolder(std::make_shared<PlanHolder>()) {
    if (Mat::debugMem) fprintf(stderr, "GSMat %d %d %d, %d %f\n", nr, nc, nnz, getGPU(), GPUmem().first);
    pattern = std::make_shared<Pattern>(ncols, realnnz);
    pir = pattern->pir; pic = pattern->pic; pjc = pattern->pjc;
    void* p = nullptr;
    int err = bidmat_malloc(&p, (long long)sizeof(float) * realnnz); pdata = (float*)p;
    if (err != 0) { free(); fail(std::string("HIP error in GSMat() ") + bidmat_error_string(err)); }
}

GSMat::GSMat(int nr, int nc, int nnz, int rn, const GSMat& like)
    : nrows(nr), ncols(nc), nnz0(nnz), pir(like.pir), pic(like.pic), pjc(like.pjc), pdata(nullptr),
      realnnz(std::max(1, rn)), GUID(Mat::newGUID()), myGPU(getGPU()), pattern(like.pattern), planHolder(like.planHolder) {
    if (Mat::debugMem) fprintf(stderr, "GSMat %d %d %d (shared pattern), %d %f\n", nr, nc, nnz, getGPU(), GPUmem().first);
    void* p = nullptr;
    int err = bidmat_malloc(&p, (long long)sizeof(float) * realnnz); pdata = (float*)p;
    if (err != 0) { free(); fail(std::string("HIP error in GSMat() ") + bidmat_error_string(err)); }
}

GSMat::~GSMat() { free(); }

void GSMat::free() {
    if (pdata) bidmat_free(pdata);
    pdata = nullptr;
    pattern.reset();                       // the arrays go with their last user
    pic = pir = pjc = nullptr;
}

void GSMat::ownPattern() {
    if (pattern.use_count() > 1) {
        pattern = std::make_shared<Pattern>(ncols, realnnz);
        pir = pattern->pir; pic = pattern->pic; pjc = pattern->pjc;
    }
    planHolder = std::make_shared<PlanHolder>();      // new indices: any older plan is stale
}

void GSMat::sharePattern(const GSMat& like) {
    pattern = like.pattern;
    pir = like.pir; pic = like.pic; pjc = like.pjc;
    planHolder = like.planHolder;
}

GSMatP GSMat::make(int nr, int nc, int nnz, int realnnz) { return std::make_shared<GSMat>(nr, nc, nnz, realnnz); }

GSMat& GSMat::clear() {
    hipcheck(bidmat_memset(pdata, 0, (long long)sizeof(float) * nnz0), "GSMat.clear");
    return *this;
}

// like != nullptr: a matrix that has to be made new takes `like`'s pattern instead of index arrays of its own
GSMatP GSMat::newOrCheckGSMat(int nr, int nc, int nnz, int realnnz, GSMatP oldmat, const GSMat* like) {
    auto fresh = [&](int rn) { return like ? std::make_shared<GSMat>(nr, nc, nnz, rn, *like) : make(nr, nc, nnz, rn); };
    if (!oldmat || (oldmat->nrows == 0 && oldmat->ncols == 0)) {
        if (Mat::useGPUcache) return fresh(std::max((int)(Mat::recycleGrow * nnz), realnnz));
        return fresh(realnnz);
    }
    if (oldmat->nrows == nr && oldmat->ncols == nc && nnz <= oldmat->realnnz) {
        oldmat->nnz0 = nnz;
        return oldmat;
    }
    // recycle (GSMat.scala:234-248): the column pointer depends on ncols, so a new shape gets new buffers
    GSMatP m = Mat::useGPUcache ? fresh((int)(Mat::recycleGrow * nnz)) : fresh(nnz);
    if (oldmat->nrows == nr && oldmat->ncols == nc) m->GUID = oldmat->GUID;
    return m;
}

GSMatP GSMat::newOrCheckGSMat(int nr, int nc, int nnz, int realnnz, GSMatP outmat, long long g1, long long g2,
                              long long g3, long long oph, const GSMat* like) {
    GSMatP m;
    if (outmat || !Mat::useGPUcache) {
        m = newOrCheckGSMat(nr, nc, nnz, realnnz, outmat, like);
    } else {
        Key key(g1, g2, g3, oph, getGPU());
        std::lock_guard<std::mutex> lock(g_cache_mu);
        auto it = g_scache.find(key);
        GSMatP res = it == g_scache.end() ? nullptr : it->second;
        m = newOrCheckGSMat(nr, nc, nnz, realnnz, res, like);
        if (m != res) g_scache[key] = m;
    }
    checkThread(m->myGPU, "newOrCheckGSMat3", m->GUID);
    return m;
}

GSMatP GSMat::fromSMat(const SMat& a, GSMatP b) {
    return fromHost(a.nrows, a.ncols, a.nnz(), a.data.data(), a.ir.data(), a.jc.data(), Mat::ioneBased, b, a.GUID);
}

// Upload of a host CSC matrix (GSMat.scala:620-647). The three arrays cross PCIe through pinned
// staging buffers with asynchronous copies; the index base is converted and the per-nonzero column
// indices are made on the device (the reference shifts in host loops and calls cusparseXcsr2coo,
// GSMat.scala:626-639); the pattern is checked on the device before any kernel trusts it.
GSMatP GSMat::fromHost(int nr, int nc, int n, const float* data, const int* ir, const int* jc, int ioff, GSMatP b,
                       long long guid) {
    if (guid == 0) guid = Mat::newGUID();                  // bare arrays: never share a cached output
    GSMatP out = newOrCheckGSMat(nr, nc, n, n, b, guid, 0, 0, opHash("fromSMat"));
    out->nnz0 = n;
    out->ownPattern();                                     // new indices: nothing shared, any older plan is stale
    Staging st;
    st.upload(out->pjc, jc, sizeof(int) * ((size_t)nc + 1));
    st.upload(out->pir, ir, sizeof(int) * (size_t)n);
    st.upload(out->pdata, data, sizeof(float) * (size_t)n);
    if (ioff != 0) {             // device indices are always 0-based (GSMat.scala:626-632)
        hipcheck(bidmat_index_shift(out->pir, n, -ioff, st.stream()), "GSMat.fromSMat");
        hipcheck(bidmat_index_shift(out->pjc, (long long)nc + 1, -ioff, st.stream()), "GSMat.fromSMat");
    }
    st.wait();
    int rule = 0;
    hipcheck(bidmat_csc_validate(nr, nc, n, out->pir, out->pjc, &rule), "GSMat.fromSMat");
    if (rule != 0) fail(fmt("GSMat.fromSMat: malformed sparse matrix (SparseMat.check rule %d)", rule));
    int err = bidmat_csc_expand_cols(nc, n, out->pjc, out->pic, nullptr);
    if (err == 0) err = bidmat_stream_synchronize(nullptr);
    if (err != 0) fail(std::string("HIP error in GSMat.fromSMat ") + bidmat_error_string(err));
    return out;
}

// Download (GSMat.scala:108-127). The reference downloads the per-nonzero column indices and
// compresses them on the host; the device already holds the column pointer, which is 200 times
// smaller, so that is what crosses PCIe. The index base is added while the staging buffers are drained.
SMat GSMat::toSMat() const {
    SMat out(nrows, ncols, nnz0);
    toHost(out.data.data(), out.ir.data(), out.jc.data());
    return out;
}

void GSMat::toHost(float* data, int* ir, int* jc) const {
    const int ioff = Mat::ioneBased;
    Staging st;
    st.download(jc, pjc, sizeof(int) * ((size_t)ncols + 1), ioff);
    st.download(ir, pir, sizeof(int) * (size_t)nnz0, ioff);
    st.download(data, pdata, sizeof(float) * (size_t)nnz0);
}

GMatP GSMat::contents() {
    auto out = std::make_shared<GMat>(nnz0, 1, pdata, realnnz, false);
    // the view does not own pdata: it keeps this matrix alive for as long as it exists
    // (matrices made with GSMat::make are always held by a shared_ptr)
    out->keepalive = weak_from_this().lock();
    return out;
}

bidmat_plan* GSMat::plan(int k_hint) {
    if (!planHolder->plan) {
        int err = bidmat_plan_create(nrows, ncols, nnz0, pir, pjc, k_hint, &planHolder->plan);
        if (err != 0) fail(std::string("HIP error building the row plan ") + bidmat_error_string(err));
        planHolder->k_hint = k_hint;
    }
    return planHolder->plan;
}

bidmat_plan* GSMat::planIfDue(int k_hint) {
    if (planHolder->plan) return planHolder->plan;
    if (++planHolder->uses < 2) return nullptr;
    return plan(k_hint);
}

GMatP GSMat::sum(int n, GMatP oldmat) {
    const int nn = n > 0 ? n : (nrows == 1 ? 2 : 1);
    GMatP out = GMat::newOrCheckGMat(nn == 1 ? 1 : nrows, nn == 1 ? ncols : 1, oldmat, GUID, n, opHash("sum"));
    Mat::nflops += nnz0;
    int err;
    if (nn == 1) err = bidmat_spsum_cols(ncols, nnz0, pdata, pjc, out->pdata, 0, nullptr);
    else if (nn == 2) err = bidmat_spsum_rows_csc(nrows, nnz0, pir, pdata, out->pdata, 0, nullptr);
    else fail("index must 1 or 2");
    if (err == 0) err = bidmat_stream_synchronize(nullptr);
    if (err != 0) fail(std::string("HIP error in GSMat.sum ") + bidmat_error_string(err));
    return out;
}

GSMatP GSMat::copy(GSMatP omat, long long key1, long long key2) {
    GSMatP out = newOrCheckGSMat(nrows, ncols, nnz0, realnnz, omat, GUID, key1, key2, opHash("copy"), this);
    if (out.get() != this) {
        // the copy has values of its own and points at the same index arrays (and plan): the indices of
        // a GSMat only ever change through calls that take private arrays first
        if (out->pattern != pattern) out->sharePattern(*this);
        hipcheck(bidmat_memcpy_d2d(out->pdata, pdata, (long long)sizeof(float) * nnz0), "GSMat.copy");
    }
    return out;
}

GSMatP GSMat::nHot(const std::vector<int>& cats, int n, int ncols, int ncats0) {
    if (n < 0 || ncols < 0 || (long long)cats.size() != (long long)n * ncols) fail("GSMat.nHot: category matrix has the wrong size");
    const int len = n * ncols;
    void* dcats = nullptr;
    hipcheck(bidmat_malloc(&dcats, (long long)sizeof(int) * len), "GSMat.nHot");
    GSMatP out;
    try {
        hipcheck(bidmat_memcpy_h2d(dcats, cats.data(), (long long)sizeof(int) * len), "GSMat.nHot category copy error");
        out = make(ncats0, ncols, len, len);
        int maxcat = -1;
        int err = bidmat_nhot(n, ncols, static_cast<const int*>(dcats), out->pir, out->pic, out->pjc, out->pdata, &maxcat);
        if (err != 0) fail(std::string("HIP error in GSMat.nHot ") + bidmat_error_string(err));
        if (ncats0 == 0) out->nrows = maxcat + 1;
        else if (maxcat >= ncats0) fail("GSMat.nHot: category outside the matrix");
    } catch (...) {
        (void)bidmat_free(dcats);
        throw;
    }
    hipcheck(bidmat_free(dcats), "GSMat.nHot");
    return out;
}

GSMatP GSMat::t(GSMatP omat) {
    GSMatP out = newOrCheckGSMat(ncols, nrows, nnz0, realnnz, omat, GUID, 0, 0, opHash("t"));
    out->nnz0 = nnz0;
    out->ownPattern();
    int err = bidmat_csc_transpose(nrows, ncols, nnz0, pdata, pir, pjc, out->pdata, out->pir, out->pjc);
    if (err == 0) err = bidmat_csc_expand_cols(out->ncols, nnz0, out->pjc, out->pic, nullptr);
    if (err == 0) err = bidmat_stream_synchronize(nullptr);
    if (err != 0) fail(std::string("HIP error in GSMat.t ") + bidmat_error_string(err));
    return out;
}

GMatP GSMat::full(GMatP omat) {
    GMatP out = GMat::newOrCheckGMat(nrows, ncols, omat, GUID, 0, opHash("full"));
    out->clear();
    int err = bidmat_full(pir, pic, pdata, out->pdata, nrows, ncols, nnz0);
    if (err != 0) fail(std::string("HIP full kernel error ") + bidmat_error_string(err));
    return out;
}

GSMatP GSMat::colslice(int col1, int col2, GSMatP omat) {
    if (col1 < 0 || col2 < col1 || col2 > ncols) fail("GSMat.colslice: column range outside the matrix");
    int starti = 0, newnnz = 0;
    hipcheck(bidmat_csc_colslice_range(ncols, col1, col2, pjc, &starti, &newnnz), "GSMAT.colslice");
    const int newncols = col2 - col1;
    GSMatP out = newOrCheckGSMat(nrows, newncols, newnnz, newnnz, omat, GUID, col1, col2, opHash("colslice"));
    out->ownPattern();                                      // another pattern: any plan is rebuilt on demand
    int err = bidmat_csc_colslice(col1, col2, starti, newnnz, pjc, pir, pdata, out->pjc, out->pir, out->pic, out->pdata, nullptr);
    if (err == 0) err = bidmat_stream_synchronize(nullptr);
    if (err != 0) fail(std::string("HIP error in GSMAT.colslice ") + bidmat_error_string(err));
    return out;
}

GSMatP GSMat::GSDop(const GMatP& b, GSMatP omat, int op) {
    if (b->nrows > 1 && b->ncols > 1) fail("Sorry only edge operators supported for GSMat op GMat");
    if (b->nrows != nrows && b->ncols != ncols && b->length() > 1) fail("GSMat op GMat: dimensions mismatch");
    Mat::nflops += nnz0;
    GSMatP out = copy(omat, b->GUID, op);
    int err;
    if (b->ncols > 1) err = bidmat_sdoprow(nrows, ncols, nnz0, out->pdata, out->pic, b->pdata, (int)b->length(), op);
    else err = bidmat_sdopcol(nrows, ncols, nnz0, out->pdata, out->pir, b->pdata, (int)b->length(), op);
    if (err != 0) fail(std::string("HIP error in GSMat.GSDop ") + bidmat_error_string(err));
    return out;
}

GMatP GSMat::SDMult(const GMatP& a, GMatP omat) {
    if (ncols != a->nrows) fail("SDMult dimensions mismatch");
    GMatP out = GMat::newOrCheckGMat(nrows, a->ncols, omat, GUID, a->GUID, opHash("SDMult"));
    int err = bidmat_sdmult_plan(plan(a->ncols), a->ncols, pdata, a->pdata, a->nrows, out->pdata, out->nrows, nullptr);
    if (err == 0) err = bidmat_stream_synchronize(nullptr);
    if (err != 0) fail(std::string("HIP error in GSMAT.SDMult ") + bidmat_error_string(err));
    Mat::nflops += 2LL * nnz0 * a->ncols;
    return out;
}

GMatP GSMat::SDTMult(const GMatP& a, GMatP omat) {
    if (nrows != a->nrows) fail("SDTMult dimensions mismatch");
    GMatP out = GMat::newOrCheckGMat(ncols, a->ncols, omat, GUID, a->GUID, opHash("SDTMult"));
    int err = bidmat_sdtmult_csc(nrows, ncols, nnz0, a->ncols, pdata, pir, pjc, a->pdata, a->nrows, out->pdata, out->nrows, nullptr);
    if (err == 0) err = bidmat_stream_synchronize(nullptr);
    if (err != 0) fail(std::string("HIP error in GSMAT.SDTMult ") + bidmat_error_string(err));
    Mat::nflops += 2LL * nnz0 * a->ncols;
    return out;
}

GSMatP GSMat::DDS(const GMatP& A, const GMatP& B, const GSMatP& C, GSMatP oldmat) {
    if (A->nrows != B->nrows || C->nrows != A->ncols || C->ncols != B->ncols)
        fail(fmt("dimensions mismatch %d,%d  %d,%d  %d,%d", A->nrows, A->ncols, B->nrows, B->ncols, C->nrows, C->ncols));
    GSMatP out = newOrCheckGSMat(C->nrows, C->ncols, C->nnz(), C->realnnz, oldmat, A->GUID, B->GUID, C->GUID, opHash("DDS"), C.get());
    // The result carries C's pattern: row indices, column indices AND the column pointer (the reference
    // copies pir and pic, 8 bytes per nonzero, and leaves out.pjc stale, GSMat.scala:656-661). Here the
    // result points at C's index arrays; whoever rewrites the indices of either matrix later takes
    // private arrays first (ownPattern).
    if (out != C && out->pattern != C->pattern) out->sharePattern(*C);
    int err;
    if (bidmat_plan* p = C->planIfDue(A->nrows))
        err = bidmat_dds_plan(p, A->nrows, A->pdata, B->pdata, C->pir, C->pjc, nullptr, 0, out->pdata, 0, nullptr);
    else
        err = bidmat_dds_csc(A->nrows, C->ncols, C->nnz(), A->pdata, B->pdata, C->pir, C->pjc, out->pdata, 0, nullptr);
    if (err == 0) err = bidmat_stream_synchronize(nullptr);
    if (err != 0) fail(fmt("GPU %d DDS kernel error %s", getGPU(), bidmat_error_string(err)));
    Mat::nflops += 2LL * C->nnz() * A->nrows;
    return out;
}

GSMatP GSMat::withValues(const GMatP& vals) const {
    if (vals->length() != nnz0) fail(fmt("withValues: %lld values for %d nonzeros", vals->length(), nnz0));
    GSMatP out = std::make_shared<GSMat>(nrows, ncols, nnz0, realnnz, *this);      // same index arrays, same plan
    hipcheck(bidmat_memcpy_d2d(out->pdata, vals->pdata, (long long)sizeof(float) * nnz0), "value copy error");
    return out;
}

// ------------------------------------------------------------------ operators / free functions
GMatP operator*(const GMatP& a, const GSMatP& s) { return a->GSMult(s, nullptr); }
GMatP xT(const GMatP& a, const GSMatP& s) { return a->GSMultT(s, nullptr); }
GMatP operator/(const GMatP& a, const GMatP& b) { return a->gOp(b, nullptr, op_div); }
GMatP operator*(const GSMatP& s, const GMatP& a) { return s->SDMult(a, nullptr); }
GMatP Tx(const GSMatP& s, const GMatP& a) { return s->SDTMult(a, nullptr); }
GSMatP DDS(const GMatP& a, const GMatP& b, const GSMatP& c, GSMatP omat) { return GSMat::DDS(a, b, c, omat); }
GMatP sum(const GSMatP& s, int n, GMatP omat) { return s->sum(n, omat); }
GMatP sum(const GMatP& a, int n, GMatP omat) { return a->reduceOp(omat, n, 0.f, op_add); }

}  // namespace BIDMat
