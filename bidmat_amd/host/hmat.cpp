// BIDMat matrix files for the sparse-dense path: SMat (type 231) and FMat (type 130), plus a
// streaming loader that fills a GSMat through pinned staging buffers.
#include "bidmat.hpp"
#include "../../include/bidmat_hip.h"
#include <zlib.h>
#include <cstdio>
#include <cstring>

namespace BIDMat {
namespace HMat {
namespace {

[[noreturn]] void fail(const std::string& m) { throw std::runtime_error(m); }

bool ends_with(const std::string& s, const char* suf) {
    const size_t n = strlen(suf);
    return s.size() >= n && s.compare(s.size() - n, n, suf) == 0;
}

// gzread also passes uncompressed files through unchanged, like the reference's plain stream.
struct Reader {
    gzFile f = nullptr;
    explicit Reader(const std::string& fname) {
        if (ends_with(fname, ".lz4")) fail("lz4-compressed matrix files are not supported: " + fname);
        f = gzopen(fname.c_str(), "rb");
        if (!f) fail("cannot open " + fname);
        gzbuffer(f, 1 << 20);
    }
    ~Reader() { if (f) gzclose(f); }
    void read(void* dst, size_t bytes, const char* what) {
        char* p = static_cast<char*>(dst);
        while (bytes > 0) {
            const unsigned chunk = bytes > (1u << 30) ? (1u << 30) : (unsigned)bytes;
            const int got = gzread(f, p, chunk);
            if (got <= 0) fail(std::string("unexpected end of file while reading ") + what);
            p += got;
            bytes -= (size_t)got;
        }
    }
};

struct Writer {
    gzFile gz = nullptr;
    FILE* fp = nullptr;
    explicit Writer(const std::string& fname) {
        if (ends_with(fname, ".lz4")) fail("lz4-compressed matrix files are not supported: " + fname);
        if (ends_with(fname, ".gz")) gz = gzopen(fname.c_str(), "wb");
        else fp = fopen(fname.c_str(), "wb");
        if (!gz && !fp) fail("cannot create " + fname);
    }
    ~Writer() {
        if (gz) gzclose(gz);
        if (fp) fclose(fp);
    }
    void write(const void* src, size_t bytes) {
        const char* p = static_cast<const char*>(src);
        while (bytes > 0) {
            const unsigned chunk = bytes > (1u << 30) ? (1u << 30) : (unsigned)bytes;
            const size_t put = gz ? (size_t)gzwrite(gz, p, chunk) : fwrite(p, 1, chunk, fp);
            if (put == 0) fail("write error");
            p += put;
            bytes -= put;
        }
    }
};

void read_sparse_header(Reader& r, int& nrows, int& ncols, int& nnz) {
    int h[4];
    r.read(h, sizeof h, "header");
    if (h[0] == 331) fail("loadSMat: type 331 (sparse without row indices) is not supported on this path");
    if (h[0] != 231) fail("loadSMat expected type field 231 or 331 but was " + std::to_string(h[0]));
    nrows = h[1]; ncols = h[2]; nnz = h[3];
    if (nrows < 0 || ncols < 0 || nnz < 0) fail("loadSMat: negative dimensions in header");
}

}  // namespace

SMat loadSMat(const std::string& fname) {
    Reader r(fname);
    int nrows, ncols, nnz;
    read_sparse_header(r, nrows, ncols, nnz);
    SMat out(nrows, ncols, nnz);
    r.read(out.jc.data(), sizeof(int) * ((size_t)ncols + 1), "jc");
    r.read(out.ir.data(), sizeof(int) * (size_t)nnz, "ir");
    r.read(out.data.data(), sizeof(float) * (size_t)nnz, "data");
    if (Mat::ioneBased == 1) {          // files are 0-based, host matrices carry Mat.ioneBased
        for (auto& v : out.jc) v += 1;
        for (auto& v : out.ir) v += 1;
    }
    return out;
}

void saveSMat(const std::string& fname, const SMat& m) {
    Writer w(fname);
    const int h[4] = {231, m.nrows, m.ncols, m.nnz()};      // 2 = sparse, 3 = float, 1 = int
    w.write(h, sizeof h);
    const int ioff = Mat::ioneBased;
    if (ioff == 0) {
        w.write(m.jc.data(), sizeof(int) * m.jc.size());
        w.write(m.ir.data(), sizeof(int) * m.ir.size());
    } else {
        std::vector<int> t(m.jc);
        for (auto& v : t) v -= ioff;
        w.write(t.data(), sizeof(int) * t.size());
        t = m.ir;
        for (auto& v : t) v -= ioff;
        w.write(t.data(), sizeof(int) * t.size());
    }
    w.write(m.data.data(), sizeof(float) * m.data.size());
}

FMat loadFMat(const std::string& fname) {
    Reader r(fname);
    int h[4];
    r.read(h, sizeof h, "header");
    if (h[0] != 130) fail("loadFMat expected type field 130 but was " + std::to_string(h[0]));
    if (h[1] < 0 || h[2] < 0) fail("loadFMat: negative dimensions in header");
    FMat out(h[1], h[2]);
    r.read(out.data.data(), sizeof(float) * out.data.size(), "data");
    return out;
}

void saveFMat(const std::string& fname, const FMat& m) {
    Writer w(fname);
    const int h[4] = {130, m.nrows, m.ncols, 0};             // 1 = dense, 3 = float
    w.write(h, sizeof h);
    w.write(m.data.data(), sizeof(float) * m.data.size());
}

GSMatP loadGSMat(const std::string& fname) {
    Reader r(fname);
    int nrows, ncols, nnz;
    read_sparse_header(r, nrows, ncols, nnz);
    GSMatP out = GSMat::make(nrows, ncols, nnz, nnz);
    // two pinned staging buffers: while one is on its way to the device the other is being read
    const size_t chunk = 8u << 20;
    void* stage[2] = {nullptr, nullptr};
    void* ev[2] = {nullptr, nullptr};
    void* stream = nullptr;
    auto cleanup = [&] {
        for (int i = 0; i < 2; ++i) {
            if (stage[i]) bidmat_host_free(stage[i]);
            if (ev[i]) bidmat_event_destroy(ev[i]);
        }
        if (stream) bidmat_stream_destroy(stream);
    };
    try {
        auto ok = [](int e, const char* what) { if (e != 0) fail(std::string(what) + " " + bidmat_error_string(e)); };
        ok(bidmat_stream_create(&stream), "stream");
        for (int i = 0; i < 2; ++i) {
            ok(bidmat_host_alloc(&stage[i], (long long)chunk), "pinned alloc");
            ok(bidmat_event_create(&ev[i]), "event");
        }
        bool busy[2] = {false, false};
        int which = 0;
        auto upload = [&](void* dst, size_t bytes, const char* what) {
            char* d = static_cast<char*>(dst);
            while (bytes > 0) {
                const size_t n = bytes < chunk ? bytes : chunk;
                if (busy[which]) ok(bidmat_event_synchronize(ev[which]), "event wait");
                r.read(stage[which], n, what);
                ok(bidmat_memcpy_h2d_async(d, stage[which], (long long)n, stream), "async copy");
                ok(bidmat_event_record(ev[which], stream), "event record");
                busy[which] = true;
                which ^= 1;
                d += n;
                bytes -= n;
            }
        };
        upload(out->pjc, sizeof(int) * ((size_t)ncols + 1), "jc");      // files are 0-based, like the device
        upload(out->pir, sizeof(int) * (size_t)nnz, "ir");
        upload(out->pdata, sizeof(float) * (size_t)nnz, "data");
        ok(bidmat_csc_expand_cols(ncols, nnz, out->pjc, out->pic, stream), "expand cols");
        ok(bidmat_stream_synchronize(stream), "sync");
    } catch (...) {
        cleanup();
        throw;
    }
    cleanup();
    return out;
}

}  // namespace HMat
}  // namespace BIDMat
