// Seeded synthetic inputs for the benchmark configurations and the tests (host code, OpenMP).
// Every number is a pure function of (seed, stream, counter) through a counter-based hash, so
// results do not depend on the thread count.
//
// Shapes follow the reference's own generators in spirit (Random.scala:58-170: sprand with
// row/column distributions, simplePowerLaw, paretoGen) but nothing here is taken from them.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

#define EXPORT extern "C" __attribute__((visibility("default")))

namespace {

inline uint64_t mix64(uint64_t x) {
    x += 0x9e3779b97f4a7c15ULL;
    x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ULL;
    x = (x ^ (x >> 27)) * 0x94d049bb133111ebULL;
    return x ^ (x >> 31);
}
inline uint64_t rnd(uint64_t seed, uint64_t stream, uint64_t ctr) {
    return mix64(mix64(seed ^ (stream * 0xd1342543de82ef95ULL)) + ctr * 0x2545f4914f6cdd1dULL);
}
// U[0,1) with 53 bits
inline double u01(uint64_t r) { return (double)(r >> 11) * (1.0 / 9007199254740992.0); }

}  // namespace

// out[i] ~ U[lo,hi)
EXPORT void gen_uniform(float* out, long long n, uint64_t seed, float lo, float hi) {
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < n; ++i) {
        float u = (float)(rnd(seed, 1, (uint64_t)i) >> 40) * (1.0f / 16777216.0f);   // 24 bits, < 1
        out[i] = lo + (hi - lo) * u;
    }
}

// out[i] ~ U(0,1]  (1 - U[0,1), never zero)
EXPORT void gen_uniform_open0(float* out, long long n, uint64_t seed) {
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < n; ++i) {
        float u = (float)(rnd(seed, 2, (uint64_t)i) >> 40) * (1.0f / 16777216.0f);
        out[i] = 1.0f - u;
    }
}

// out[i] ~ N(mean, sigma^2), Box-Muller on two counter draws
EXPORT void gen_normal(float* out, long long n, uint64_t seed, float mean, float sigma) {
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < n; ++i) {
        double u1 = 1.0 - u01(rnd(seed, 3, (uint64_t)i));     // (0,1]
        double u2 = u01(rnd(seed, 4, (uint64_t)i));
        double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2);
        out[i] = (float)(mean + sigma * z);
    }
}

// out[i] ~ Exp(1) == Gamma(1,1)
EXPORT void gen_exponential(float* out, long long n, uint64_t seed) {
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < n; ++i) {
        double u = 1.0 - u01(rnd(seed, 5, (uint64_t)i));
        float v = (float)(-std::log(u));
        out[i] = v > 0.f ? v : 1e-30f;
    }
}

EXPORT void gen_lengths_const(int* len, int ncols, int L) {
    for (int c = 0; c < ncols; ++c) len[c] = L;
}

// Poisson(lambda) per column (Knuth's product method in double; lambda <= ~600), clipped to maxlen.
EXPORT void gen_lengths_poisson(int* len, int ncols, double lambda, uint64_t seed, int maxlen) {
    const double limit = std::exp(-lambda);
#pragma omp parallel for schedule(static)
    for (int c = 0; c < ncols; ++c) {
        double p = 1.0;
        int k = 0;
        uint64_t ctr = 0;
        for (;;) {
            p *= u01(rnd(seed, 6 + ((uint64_t)c << 8), ctr++));
            if (p <= limit) break;
            ++k;
        }
        len[c] = k > maxlen ? maxlen : k;
    }
}

// floor(xm * Pareto(alpha)) clipped to [lo, hi]
EXPORT void gen_lengths_pareto(int* len, int ncols, double xm, double alpha, int lo, int hi, uint64_t seed) {
#pragma omp parallel for schedule(static)
    for (int c = 0; c < ncols; ++c) {
        double u = 1.0 - u01(rnd(seed, 7, (uint64_t)c));       // (0,1]
        double x = xm * std::pow(u, -1.0 / alpha);
        double f = std::floor(x);
        int L = f > (double)hi ? hi : (int)f;
        if (L < lo) L = lo;
        len[c] = L;
    }
}

// jc[0]=0, jc[c+1]=jc[c]+len[c]; returns nnz or -1 if it does not fit in int32.
EXPORT long long gen_jc_from_lengths(const int* len, int ncols, int* jc) {
    long long acc = 0;
    jc[0] = 0;
    for (int c = 0; c < ncols; ++c) {
        acc += len[c];
        if (acc > 0x7fffffffLL) return -1;
        jc[c + 1] = (int)acc;
    }
    return acc;
}

// Row indices of every column: draws from the row distribution until the column holds
// jc[c+1]-jc[c] DISTINCT rows, then sorts them ascending.
//   dist 0: uniform over [0,nrows);  dist 1: Zipf, P(row r) ~ (r+1)^-s.
// Returns 0, or -1 if a column asks for more distinct rows than exist.
EXPORT int gen_rows(int nrows, int ncols, const int* jc, int* ir, int dist, double s, uint64_t seed) {
    std::vector<double> cdf;
    if (dist == 1) {
        cdf.resize((size_t)nrows);
        double acc = 0.0;
        for (int r = 0; r < nrows; ++r) { acc += std::pow((double)(r + 1), -s); cdf[(size_t)r] = acc; }
        for (int r = 0; r < nrows; ++r) cdf[(size_t)r] /= acc;
        cdf[(size_t)nrows - 1] = 1.0;
    }
    int bad = 0;
#pragma omp parallel
    {
        std::vector<uint64_t> seen(((size_t)nrows + 63) / 64, 0);
#pragma omp for schedule(dynamic, 256)
        for (int c = 0; c < ncols; ++c) {
            const int L = jc[c + 1] - jc[c];
            if (L > nrows) { bad = 1; continue; }
            int* out = ir + jc[c];
            int got = 0;
            uint64_t ctr = 0;
            while (got < L) {
                const double u = u01(rnd(seed, 8 + ((uint64_t)c << 8), ctr++));
                int r;
                if (dist == 1) {
                    r = (int)(std::upper_bound(cdf.begin(), cdf.end(), u) - cdf.begin());
                    if (r >= nrows) r = nrows - 1;
                } else {
                    r = (int)(u * nrows);
                    if (r >= nrows) r = nrows - 1;
                }
                uint64_t& word = seen[(size_t)r >> 6];
                const uint64_t bit = 1ULL << (r & 63);
                if (!(word & bit)) { word |= bit; out[got++] = r; }
            }
            for (int i = 0; i < L; ++i) seen[(size_t)out[i] >> 6] = 0;
            std::sort(out, out + L);
        }
    }
    return bad ? -1 : 0;
}

EXPORT int gen_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
