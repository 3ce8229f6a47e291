// Host-side mirror of BIDMat's operator interface for the sparse-dense product path
// (C++ stand-in for the Scala layer: no JVM/Scala toolchain exists on the build or GPU boxes).
// Same class and method names, argument meaning, flop accounting and exception texts as
//   GMat   src/main/scala/BIDMat/GMat.scala   (GSMult :1041, madd :1051, GSMultT :1076, maddT :1086,
//                                              gOp :1119, reduceOp :1182, clear :562, operators :1684-1688)
//   GSMat  src/main/scala/BIDMat/GSMat.scala  (fromSMat :620, toSMat :108, DDS :649, sum :250,
//                                              contents :21, free :225, newOrCheckGSMat :722-806)
//   SMat / FMat host containers, Mat globals (Mat.scala:646-724), flip/flop/gflop
//   (MatFunctions.scala:19-51), sum dispatch (SFunctions.scala:10-15, GFunctions.scala:227).
// Everything device-side goes through the C ABI of libbidmathip.so (include/bidmat_hip.h);
// this layer never touches HIP directly.
#pragma once
#include <atomic>
#include <map>
#include <functional>
#include <memory>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

struct bidmat_plan;

namespace BIDMat {

// ---- global flags and counters (object Mat, Mat.scala:670-724)
struct Mat {
    static int ioneBased;          // index base of host sparse matrices (1 like the reference)
    static bool useGPUcache;       // cache operator outputs under (operand GUIDs, op, GPU)
    static double recycleGrow;     // growth factor for recycled buffers
    static bool debugMem;          // print every device allocation
    static int numThreads;
    static std::atomic<long long> nflops;
    static long long newGUID();
    static void clearCaches();
};

enum BinOp { op_add = 0, op_sub, op_mul, op_div, op_gt, op_lt, op_eq, op_ge, op_le, op_ne,
             op_max, op_min, op_atan2, op_pow, op_ifpos };

// ---- host dense, column-major (FMat)
class FMat {
public:
    int nrows = 0, ncols = 0;
    std::vector<float> data;
    long long GUID;
    FMat(int nr, int nc);
    FMat(int nr, int nc, const float* src);
    long long length() const { return (long long)nrows * ncols; }
    std::string mytype() const { return "FMat"; }
};

// ---- host sparse CSC (SMat); ir / jc carry Mat::ioneBased
class SMat {
public:
    int nrows = 0, ncols = 0;
    std::vector<int> ir, jc;
    std::vector<float> data;
    long long GUID;
    SMat(int nr, int nc, int nnz);
    int nnz() const { return (int)data.size(); }
    // SparseMat.check (SparseMat.scala:710-740): throws with the reference's messages
    void check() const;
    // the same on caller-owned arrays (index base Mat::ioneBased)
    static void checkArrays(int nrows, int ncols, int nnz, const int* ir, const int* jc);
    FMat full() const;
    std::string mytype() const { return "SMat"; }
};

// Transfers between pageable host memory and the device through two pinned staging buffers and
// asynchronous copies on a stream of their own: while one buffer crosses PCIe the other is being
// filled (upload) or emptied (download). Used by GSMat.fromSMat / toSMat and HMat.loadGSMat.
class Staging {
public:
    explicit Staging(size_t chunk_bytes = size_t(8) << 20);
    ~Staging();
    Staging(const Staging&) = delete;
    Staging& operator=(const Staging&) = delete;
    // dst (device) <- bytes produced by fill(staging_buffer, n) in chunks
    void upload(void* dst, size_t bytes, const std::function<void(void*, size_t)>& fill);
    // dst (device) <- src (host)
    void upload(void* dst, const void* src, size_t bytes);
    // dst (host) <- src (device); add != 0: the data are int32 and `add` is added on the way
    void download(void* dst, const void* src, size_t bytes, int add = 0);
    void* stream() const { return stream_; }
    void wait();                      // until everything enqueued so far is complete
private:
    size_t chunk_;
    void* stage_[2] = {nullptr, nullptr};
    void* ev_[2] = {nullptr, nullptr};
    bool busy_[2] = {false, false};
    int which_ = 0;
    void* stream_ = nullptr;
};

class GSMat;
class GMat;
using GMatP = std::shared_ptr<GMat>;
using GSMatP = std::shared_ptr<GSMat>;

// ---- device dense (GMat)
class GMat {
public:
    int nrows, ncols;
    float* pdata;              // device, column-major, leading dimension nrows
    long long realsize;        // capacity in floats
    long long GUID;
    int myGPU;
    bool owns;
    std::shared_ptr<void> keepalive;   // a view (GSMat.contents) keeps its parent's buffer alive

    GMat(int nr, int nc, float* p, long long realsize, bool owns);
    ~GMat();
    static GMatP make(int nr, int nc);                       // GMat(nr, nc)  (GMat.scala:2338-2353)
    static GMatP zeros(int nr, int nc);
    static GMatP fromFMat(const FMat& a, GMatP out = nullptr);
    FMat toFMat() const;
    long long length() const { return (long long)nrows * ncols; }
    std::string mytype() const { return "GMat"; }
    GMat& clear();                                           // GMat.scala:562-566
    void free();

    // C = this * S and C += this * S
    GMatP GSMult(const GSMatP& a, GMatP oldmat);
    GMatP madd(const GSMatP& a, GMatP out);
    // C = this *^ S and C += this *^ S
    GMatP GSMultT(const GSMatP& a, GMatP oldmat);
    GMatP maddT(const GSMatP& a, GMatP out);
    // windowed products for tiled matrices (GMat.scala:961-997): c[croff.., ccoff..] += this[aroff.., acoff..] * b[broff.., bcoff..]
    GMatP tileMult(int nr, int nc, int kk, int aroff, int acoff, const GSMatP& b, int broff, int bcoff,
                   GMatP c, int croff, int ccoff);
    GMatP tileMultNT(int nr, int nc, int kk, int aroff, int acoff, const GSMatP& b, int broff, int bcoff,
                     GMatP c, int croff, int ccoff);
    // elementwise binary op with broadcasting, reductions
    GMatP gOp(const GMatP& a, GMatP oldmat, int op);
    GMatP reduceOp(GMatP oldmat, int dir, float initval, int op);

    static GMatP newOrCheckGMat(int nr, int nc, GMatP outmat);
    static GMatP newOrCheckGMat(int nr, int nc, GMatP outmat, long long g1, long long g2, long long opHash);
};

// The plan of a pattern, shared by all GSMats that carry the same pattern (a DDS result, V./R ...).
// A*^S and sparse row sums cannot run without a plan and build it at once; A*S and DDS run through it
// when it exists and build it on their second call on the pattern (`uses` counts them), so a pattern
// that is multiplied once never pays for a plan.
struct PlanHolder {
    bidmat_plan* plan = nullptr;
    int k_hint = 0;
    int uses = 0;
    ~PlanHolder();
};

// The index arrays of a device sparse matrix. Several GSMats may share one Pattern (the result of DDS
// has the pattern of its third operand: the reference copies 8 bytes per nonzero for it,
// GSMat.scala:656-661; here the result points at the same arrays). A GSMat that is about to have its
// indices rewritten takes a private Pattern first (GSMat::ownPattern).
struct Pattern {
    int* pir = nullptr;
    int* pic = nullptr;
    int* pjc = nullptr;
    Pattern(int ncols, int realnnz);       // allocates; throws on failure
    ~Pattern();
    Pattern(const Pattern&) = delete;
    Pattern& operator=(const Pattern&) = delete;
};

// ---- device sparse (GSMat): pir/pic/pjc/pdata, all 0-based on the device
class GSMat : public std::enable_shared_from_this<GSMat> {
public:
    int nrows, ncols;
    int nnz0;
    int* pir;                  // = pattern->pir etc.: the names the reference uses
    int* pic;
    int* pjc;
    float* pdata;
    int realnnz;
    long long GUID;
    int myGPU;
    std::shared_ptr<Pattern> pattern;
    std::shared_ptr<PlanHolder> planHolder;

    GSMat(int nr, int nc, int nnz, int realnnz);
    // a matrix with its own values and the pattern (and plan) of `like`
    GSMat(int nr, int nc, int nnz, int realnnz, const GSMat& like);
    ~GSMat();
    int nnz() const { return nnz0; }
    std::string mytype() const { return "GSMat"; }
    static GSMatP make(int nr, int nc, int nnz, int realnnz);
    static GSMatP fromSMat(const SMat& a, GSMatP b = nullptr);   // GSMat.scala:620-647
    // the same from bare host arrays in index base ioff (what fromSMat does with a.data / a.ir / a.jc)
    static GSMatP fromHost(int nr, int nc, int nnz, const float* data, const int* ir, const int* jc, int ioff,
                           GSMatP b = nullptr, long long guid = 0);
    // oneHot (n = 1) / nHot: cats is an n x ncols category matrix (column-major, 0-based);
    // ncats0 == 0: rows = largest category + 1  (GSMat.scala:686-720)
    static GSMatP nHot(const std::vector<int>& cats, int n, int ncols, int ncats0);
    SMat toSMat() const;                                         // GSMat.scala:108-127
    // the same into caller-owned arrays (nnz values, nnz rows, ncols+1 column pointers, base Mat::ioneBased)
    void toHost(float* data, int* ir, int* jc) const;
    GMatP contents();                                            // GSMat.scala:21-25
    GSMat& clear();
    void free();
    GMatP sum(int n, GMatP oldmat);                              // GSMat.scala:250-261
    GSMatP GSDop(const GMatP& b, GSMatP omat, int op);           // this op edge vector (GSMat.scala:315-330)
    GSMatP copy(GSMatP omat, long long key1, long long key2);    // GSMat.copy / copyTo
    GSMatP t(GSMatP omat = nullptr);                             // transpose, on the device (GSMat.scala:218-223)
    GMatP full(GMatP omat = nullptr);                            // dense image (GSMat.scala:206-216)
    GSMatP colslice(int col1, int col2, GSMatP omat = nullptr);  // columns [col1, col2)  (GSMat.scala:77-104)
    GMatP SDMult(const GMatP& a, GMatP omat);                    // this * a    (GSMat.scala:265-289)
    GMatP SDTMult(const GMatP& a, GMatP omat);                   // this ^* a   (GSMat.scala:291-313)
    static GSMatP DDS(const GMatP& A, const GMatP& B, const GSMatP& C, GSMatP oldmat);   // GSMat.scala:649-667
    // a sparse matrix with this pattern and other values (the V./R step keeps V's pattern)
    GSMatP withValues(const GMatP& vals) const;
    // the plan of this pattern, built now if there is none
    bidmat_plan* plan(int k_hint);
    // for A*S / DDS: the plan if there is one or if this is at least the second such call on the
    // pattern (then it is built), otherwise nullptr (the caller runs without a plan)
    bidmat_plan* planIfDue(int k_hint);
    // private index arrays, about to be rewritten: nothing another matrix shares, no plan
    void ownPattern();
    // point at the pattern (and plan) of `like`
    void sharePattern(const GSMat& like);

    static GSMatP newOrCheckGSMat(int nr, int nc, int nnz, int realnnz, GSMatP oldmat, const GSMat* like = nullptr);
    static GSMatP newOrCheckGSMat(int nr, int nc, int nnz, int realnnz, GSMatP outmat, long long g1,
                                  long long g2, long long g3, long long opHash, const GSMat* like = nullptr);
};

// ---- operators (GMat.scala:1684-1688, 1972-1976) and free functions
GMatP operator*(const GMatP& a, const GSMatP& s);                 // a * s
GMatP xT(const GMatP& a, const GSMatP& s);                        // a *^ s  (alias xT in the reference)
GMatP operator*(const GSMatP& s, const GMatP& a);                 // s * a   (GSMat.scala:334)
GMatP Tx(const GSMatP& s, const GMatP& a);                        // s ^* a  (GSMat.scala:335-336)
GMatP operator/(const GMatP& a, const GMatP& b);                  // elementwise
GSMatP DDS(const GMatP& a, const GMatP& b, const GSMatP& c, GSMatP omat = nullptr);
GMatP sum(const GSMatP& s, int n = 0, GMatP omat = nullptr);      // SFunctions.scala:10-15
GMatP sum(const GMatP& a, int n = 0, GMatP omat = nullptr);       // GFunctions.scala:227
// host reference path: FMat * SMat, FMat *^ SMat, DDS on host are NOT provided here (the CPU
// restatement of those loops lives with the tests); these mirror only the GPU dispatch.

// ---- matrix files (HMat.scala): little-endian int32 header [type, nrows, ncols, nnz], then
// for a sparse float matrix (type 231) jc[ncols+1], ir[nnz], data[nnz] with 0-based indices on
// disk (HMat.scala:1232-1266, 1444-1480); type 331 is the same without ir (HMat.scala:1246-1258):
// the j-th stored element of a column sits in row j (SparseMat.explicitInds, SparseMat.scala:79-93),
// and the loaders make those rows explicit; for a dense float matrix (type 130) the column-major
// floats (HMat.scala:337-399, 876-891). Names ending in .gz are gzip streams; .lz4 is refused.
namespace HMat {
SMat loadSMat(const std::string& fname);
void saveSMat(const std::string& fname, const SMat& m);
FMat loadFMat(const std::string& fname);
void saveFMat(const std::string& fname, const FMat& m);
// Reads a type-231 / 331 file straight into a GSMat: chunks go through two pinned staging buffers
// and asynchronous copies, so reading the file and crossing PCIe overlap. The pattern is checked on
// the device (column pointers in order and inside the file's nnz, rows inside the matrix) before
// any kernel trusts it; a malformed file throws.
GSMatP loadGSMat(const std::string& fname);
}  // namespace HMat

// timers (MatFunctions.scala:19-51)
void flip();
std::pair<float, float> flop();
std::pair<float, float> gflop();

int getGPU();
void setGPU(int dev);
std::pair<float, long long> GPUmem();     // (free fraction, free bytes)  GFunctions.scala:208-213

}  // namespace BIDMat
