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

// norows: type 331, the file holds no row indices (HMat.scala:1246-1258)
void read_sparse_header(Reader& r, int& nrows, int& ncols, int& nnz, bool& norows) {
    int h[4];
    r.read(h, sizeof h, "header");
    if (h[0] != 231 && h[0] != 331) fail("loadSMat expected type field 231 or 331 but was " + std::to_string(h[0]));
    norows = h[0] == 331;
    nrows = h[1]; ncols = h[2]; nnz = h[3];
    if (nrows < 0 || ncols < 0 || nnz < 0) fail("loadSMat: negative dimensions in header");
}

// jc as read from a file (0-based): first pointer 0, non-decreasing, last pointer nnz
void check_file_jc(const int* jc, int ncols, int nnz) {
    if (jc[0] != 0) fail("loadSMat: malformed file, jc(0) should be 0");
    for (int i = 0; i < ncols; ++i)
        if (jc[i] > jc[i + 1]) fail("loadSMat: malformed file, jc(i) out of order " + std::to_string(i));
    if (jc[ncols] != nnz) fail("loadSMat: malformed file, jc(ncols) should be " + std::to_string(nnz));
}

}  // namespace

SMat loadSMat(const std::string& fname) {
    Reader r(fname);
    int nrows, ncols, nnz;
    bool norows;
    read_sparse_header(r, nrows, ncols, nnz, norows);
    SMat out(nrows, ncols, nnz);
    r.read(out.jc.data(), sizeof(int) * ((size_t)ncols + 1), "jc");
    check_file_jc(out.jc.data(), ncols, nnz);
    if (!norows) {
        r.read(out.ir.data(), sizeof(int) * (size_t)nnz, "ir");
        for (int j = 0; j < nnz; ++j)
            if ((unsigned)out.ir[j] >= (unsigned)nrows) fail("loadSMat: malformed file, ir(" + std::to_string(j) + ") out of range");
    } else {
        // the rows such a matrix implies: element j of a column sits in row j. (The reference's
        // SparseMat.explicitInds means this too; its inner loop bound, SparseMat.scala:86, stops after
        // one element per column.)
        for (int c = 0; c < ncols; ++c) {
            if (out.jc[c + 1] - out.jc[c] > nrows) fail("loadSMat: malformed file, column longer than the matrix is tall");
            for (int j = out.jc[c]; j < out.jc[c + 1]; ++j) out.ir[j] = j - out.jc[c];
        }
    }
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
    bool norows;
    read_sparse_header(r, nrows, ncols, nnz, norows);
    GSMatP out = GSMat::make(nrows, ncols, nnz, nnz);
    auto ok = [](int e, const char* what) { if (e != 0) fail(std::string(what) + " " + bidmat_error_string(e)); };
    Staging st;
    const char* what = "jc";
    auto from_file = [&](void* buf, size_t n) { r.read(buf, n, what); };
    st.upload(out->pjc, sizeof(int) * ((size_t)ncols + 1), from_file);      // files are 0-based, like the device
    if (!norows) {
        what = "ir";
        st.upload(out->pir, sizeof(int) * (size_t)nnz, from_file);
    }
    what = "data";
    st.upload(out->pdata, sizeof(float) * (size_t)nnz, from_file);
    st.wait();
    // nothing on the device has used the arrays yet: check them before the first kernel does
    int rule = 0;
    ok(bidmat_csc_validate(nrows, ncols, nnz, norows ? nullptr : out->pir, out->pjc, &rule), "validate");
    if (rule != 0) fail("loadGSMat: malformed file (SparseMat.check rule " + std::to_string(rule) + "): " + fname);
    if (norows) ok(bidmat_csc_implicit_rows(ncols, nnz, out->pjc, out->pir, nullptr), "implicit rows");
    ok(bidmat_csc_expand_cols(ncols, nnz, out->pjc, out->pic, nullptr), "expand cols");
    ok(bidmat_stream_synchronize(nullptr), "sync");
    if (norows) {
        // a column of such a file may not be longer than the matrix is tall
        ok(bidmat_csc_validate(nrows, ncols, nnz, out->pir, out->pjc, &rule), "validate");
        if (rule != 0) fail("loadGSMat: malformed file, column longer than the matrix is tall: " + fname);
    }
    return out;
}

}  // namespace HMat
}  // namespace BIDMat
