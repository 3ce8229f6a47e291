// JNI entry points for a Scala/Java host (class edu.berkeley.bid.HIPMAT). They forward to the
// C ABI one to one; device addresses travel as jlong, so no JCuda Pointer objects and no cached
// field ids are needed (the reference unwraps jcuda.Pointer in PointerUtils.cpp:353-363 and
// caches field ids in JNI_OnLoad, BIDMat_CUMAT.cpp:11-29).
// Compiled only where a JDK's <jni.h> is on the include path; elsewhere this file is empty.
#if defined(__has_include)
#if __has_include(<jni.h>)
#define BIDMAT_HAVE_JNI 1
#endif
#endif

#ifdef BIDMAT_HAVE_JNI
#include <jni.h>
#include "../../include/bidmat_hip.h"

#define P(T, x) reinterpret_cast<T*>(static_cast<intptr_t>(x))
#define JFN(ret, name) extern "C" JNIEXPORT ret JNICALL Java_edu_berkeley_bid_HIPMAT_##name

// replaces Java_edu_berkeley_bid_CUMAT_dsmult (BIDMat_CUMAT.cpp:722-733)
JFN(jint, dsmult)(JNIEnv*, jclass, jint nr, jint nc, jint nnz, jlong A, jlong Bdata, jlong Bir, jlong Bic, jlong C) {
    return bidmat_dsmult(nr, nc, nnz, P(const float, A), P(const float, Bdata), P(const int, Bir), P(const int, Bic), P(float, C));
}
// replaces Java_edu_berkeley_bid_CUMAT_dsmultT (BIDMat_CUMAT.cpp:761-772)
JFN(jint, dsmultT)(JNIEnv*, jclass, jint nr, jint nc, jint nnz, jlong A, jlong Bdata, jlong Bir, jlong Bic, jlong C) {
    return bidmat_dsmultT(nr, nc, nnz, P(const float, A), P(const float, Bdata), P(const int, Bir), P(const int, Bic), P(float, C));
}
// replaces Java_edu_berkeley_bid_CUMAT_dsmultTile (BIDMat_CUMAT.cpp:1456-1471), transpose flag included
JFN(jint, dsmultTile)(JNIEnv*, jclass, jint nr, jint nc, jint kk, jint nnz, jlong A, jint lda, jlong Bdata, jlong Bir, jlong Bic,
                      jint broff, jint bcoff, jlong C, jint ldc, jint transpose) {
    if (transpose)
        return bidmat_dsmultTileT(nr, nc, kk, nnz, P(const float, A), lda, P(const float, Bdata), P(const int, Bir), P(const int, Bic), broff, bcoff, P(float, C), ldc);
    return bidmat_dsmultTile(nr, nc, kk, nnz, P(const float, A), lda, P(const float, Bdata), P(const int, Bir), P(const int, Bic), broff, bcoff, P(float, C), ldc);
}
// replace Java_edu_berkeley_bid_CUMAT_sdoprow / sdopcol
JFN(jint, sdoprow)(JNIEnv*, jclass, jint nr, jint nc, jint nnz, jlong A, jlong Aic, jlong B, jint len, jint op) {
    return bidmat_sdoprow(nr, nc, nnz, P(float, A), P(const int, Aic), P(const float, B), len, op);
}
JFN(jint, sdopcol)(JNIEnv*, jclass, jint nr, jint nc, jint nnz, jlong A, jlong Air, jlong B, jint len, jint op) {
    return bidmat_sdopcol(nr, nc, nnz, P(float, A), P(const int, Air), P(const float, B), len, op);
}
// replaces Java_edu_berkeley_bid_CUMAT_dds (BIDMat_CUMAT.cpp:774-785)
JFN(jint, dds)(JNIEnv*, jclass, jint nr, jint nnz, jlong A, jlong B, jlong Cir, jlong Cic, jlong Pv) {
    return bidmat_dds(nr, nnz, P(const float, A), P(const float, B), P(const int, Cir), P(const int, Cic), P(float, Pv));
}
// replaces Java_edu_berkeley_bid_CUMAT_dds0 (BIDMat_CUMAT.cpp:787-798): column pointer instead of column indices
JFN(jint, dds0)(JNIEnv*, jclass, jint nr, jint nc, jlong A, jlong B, jlong Cir, jlong Cjc, jlong Pv) {
    return bidmat_dds0(nr, nc, P(const float, A), P(const float, B), P(const int, Cir), P(const int, Cjc), P(float, Pv));
}
// replaces Java_edu_berkeley_bid_CUMAT_spsum (BIDMat_CUMAT.cpp:873-882)
JFN(jint, spsum)(JNIEnv*, jclass, jint nr, jint nc, jint nnz, jlong Air, jlong Aic, jlong Pv, jlong B, jint n) {
    return bidmat_spsum(nr, nc, nnz, P(const int, Air), P(const int, Aic), P(const float, Pv), P(float, B), n);
}
// replaces Java_edu_berkeley_bid_CUMAT_reduce1op / reduce2op (BIDMat_CUMAT.cpp:800-808, 838-846)
JFN(jint, reduce1op)(JNIEnv*, jclass, jint nr, jint nc, jlong A, jlong B, jfloat initv, jint opn) {
    return bidmat_reduce1op(nr, nc, P(const float, A), P(float, B), initv, opn);
}
JFN(jint, reduce2op)(JNIEnv*, jclass, jint nr, jint nc, jlong A, jlong B, jfloat initv, jint opn) {
    return bidmat_reduce2op(nr, nc, P(const float, A), P(float, B), initv, opn);
}
// replaces Java_edu_berkeley_bid_CUMAT_applyop
JFN(jint, applyop)(JNIEnv*, jclass, jlong A, jint Anr, jint Anc, jlong B, jint Bnr, jint Bnc, jlong C, jint opn) {
    return bidmat_applyop(P(const float, A), Anr, Anc, P(const float, B), Bnr, Bnc, P(float, C), opn);
}
// native entries (column pointer + beta), used by the patched GMat.madd / GSMat.DDS
JFN(jint, dsmultCsc)(JNIEnv*, jclass, jint k, jint nc, jint nnz, jlong A, jlong Sdata, jlong Sir, jlong Sjc, jlong C, jint beta) {
    int e = bidmat_dsmult_csc(k, nc, nnz, P(const float, A), P(const float, Sdata), P(const int, Sir), P(const int, Sjc), P(float, C), beta, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
JFN(jint, ddsCsc)(JNIEnv*, jclass, jint k, jint nc, jint nnz, jlong A, jlong B, jlong Sir, jlong Sjc, jlong Pv, jint beta) {
    int e = bidmat_dds_csc(k, nc, nnz, P(const float, A), P(const float, B), P(const int, Sir), P(const int, Sjc), P(float, Pv), beta, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
// DDS with the elementwise step fused in: Pv[j] = op(V[j], dot_j) (GSMat.DDS + GMat.gOp in one launch)
JFN(jint, ddsCscOp)(JNIEnv*, jclass, jint k, jint nc, jint nnz, jlong A, jlong B, jlong Sir, jlong Sjc, jlong V, jint opn, jlong Pv) {
    int e = bidmat_dds_csc_op(k, nc, nnz, P(const float, A), P(const float, B), P(const int, Sir), P(const int, Sjc),
                              P(const float, V), opn, P(float, Pv), nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
JFN(jlong, planCreate)(JNIEnv*, jclass, jint nr, jint nc, jint nnz, jlong Sir, jlong Sjc, jint khint) {
    bidmat_plan* p = nullptr;
    int e = bidmat_plan_create(nr, nc, nnz, P(const int, Sir), P(const int, Sjc), khint, &p);
    return e ? -(jlong)e : (jlong)reinterpret_cast<intptr_t>(p);
}
JFN(jint, planDestroy)(JNIEnv*, jclass, jlong plan) { return bidmat_plan_destroy(P(bidmat_plan, plan)); }
JFN(jint, dsmultTPlan)(JNIEnv*, jclass, jlong plan, jint k, jlong A, jlong Sdata, jlong C, jint beta) {
    int e = bidmat_dsmultT_plan(P(bidmat_plan, plan), k, P(const float, A), P(const float, Sdata), P(float, C), beta, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
// A*S and DDS through a plan (one launch when no column is long), values kept in plan order
JFN(jint, dsmultPlan)(JNIEnv*, jclass, jlong plan, jint k, jlong A, jlong Sdata, jlong Sir, jlong Sjc, jlong C, jint beta) {
    int e = bidmat_dsmult_plan(P(bidmat_plan, plan), k, P(const float, A), P(const float, Sdata), P(const int, Sir),
                               P(const int, Sjc), P(float, C), beta, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
JFN(jint, ddsPlan)(JNIEnv*, jclass, jlong plan, jint k, jlong A, jlong B, jlong Sir, jlong Sjc, jlong V, jint opn, jlong Pv, jint beta) {
    int e = bidmat_dds_plan(P(bidmat_plan, plan), k, P(const float, A), P(const float, B), P(const int, Sir), P(const int, Sjc),
                            P(const float, V), opn, P(float, Pv), beta, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
JFN(jint, ddsPlanStored)(JNIEnv*, jclass, jlong plan, jint k, jlong A, jlong B, jlong Sir, jlong Sjc, jint opn, jlong Pv) {
    int e = bidmat_dds_plan_stored(P(bidmat_plan, plan), k, P(const float, A), P(const float, B), P(const int, Sir), P(const int, Sjc),
                                   opn, P(float, Pv), nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
JFN(jint, planSetValues)(JNIEnv*, jclass, jlong plan, jlong Sdata) {
    int e = bidmat_plan_set_values(P(bidmat_plan, plan), P(const float, Sdata), nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
// sparse sums without the per-nonzero column array (GSMat.sum, GSMat.scala:250-261)
JFN(jint, spsumCols)(JNIEnv*, jclass, jint nc, jint nnz, jlong Sdata, jlong Sjc, jlong out, jint beta) {
    int e = bidmat_spsum_cols(nc, nnz, P(const float, Sdata), P(const int, Sjc), P(float, out), beta, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
JFN(jint, spsumRowsPlan)(JNIEnv*, jclass, jlong plan, jlong Sdata, jlong out, jint beta) {
    int e = bidmat_spsum_rows_plan(P(bidmat_plan, plan), P(const float, Sdata), P(float, out), beta, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
JFN(jint, spsumRowsCsc)(JNIEnv*, jclass, jint nr, jint nnz, jlong Sir, jlong Sdata, jlong out, jint beta) {
    int e = bidmat_spsum_rows_csc(nr, nnz, P(const int, Sir), P(const float, Sdata), P(float, out), beta, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
// Q = op(V, DDS(A, B, S)), G = beta*G + B *^ Q in one launch (V == 0: the values stored in the plan; Q == 0: not written)
JFN(jint, ddsDsmultTPlan)(JNIEnv*, jclass, jlong plan, jint k, jlong A, jlong B, jlong V, jint opn, jlong Q, jlong G, jint beta) {
    int e = bidmat_dds_dsmultT_plan(P(bidmat_plan, plan), k, P(const float, A), P(const float, B), P(const float, V), opn,
                                    P(float, Q), P(float, G), beta, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
// Q = op(V, DDS(A, B, S)), C = beta*C + A * Q in one launch (Q == 0: not written; Q == V: in place)
JFN(jint, ddsDsmultCsc)(JNIEnv*, jclass, jint k, jint nc, jint nnz, jlong A, jlong B, jlong Sir, jlong Sjc, jlong V, jint opn,
                        jlong Q, jlong C, jint beta) {
    int e = bidmat_dds_dsmult_csc(k, nc, nnz, P(const float, A), P(const float, B), P(const int, Sir), P(const int, Sjc),
                                  P(const float, V), opn, P(float, Q), P(float, C), beta, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
// the same through a plan's column side (in passes over the row classes when the plan has a class order)
JFN(jint, ddsDsmultPlan)(JNIEnv*, jclass, jlong plan, jint k, jlong A, jlong B, jlong Sir, jlong Sjc, jlong V, jint opn, jlong Q,
                         jlong C, jint beta) {
    int e = bidmat_dds_dsmult_plan(P(bidmat_plan, plan), k, P(const float, A), P(const float, B), P(const int, Sir),
                                   P(const int, Sjc), P(const float, V), opn, P(float, Q), P(float, C), beta, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
// S^T * A and S * A (replace the cusparseScsrmm calls of GSMat.SDTMult / SDMult, GSMat.scala:265-313)
JFN(jint, sdtmultCsc)(JNIEnv*, jclass, jint nr, jint nc, jint nnz, jint p, jlong Sdata, jlong Sir, jlong Sjc, jlong A,
                      jint lda, jlong C, jint ldc) {
    int e = bidmat_sdtmult_csc(nr, nc, nnz, p, P(const float, Sdata), P(const int, Sir), P(const int, Sjc),
                               P(const float, A), lda, P(float, C), ldc, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
JFN(jint, sdmultPlan)(JNIEnv*, jclass, jlong plan, jint p, jlong Sdata, jlong A, jint lda, jlong C, jint ldc) {
    int e = bidmat_sdmult_plan(P(bidmat_plan, plan), p, P(const float, Sdata), P(const float, A), lda, P(float, C), ldc, nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
JFN(jint, setOption)(JNIEnv* env, jclass, jstring name, jlong value) {
    const char* n = env->GetStringUTFChars(name, nullptr);
    if (!n) return 1;
    int e = bidmat_set_option(n, value);
    env->ReleaseStringUTFChars(name, n);
    return e;
}
JFN(jint, releaseCaches)(JNIEnv*, jclass) { return bidmat_release_caches(); }
// GSMat.oneHot / nHot (GSMat.scala:686-720); returns -(error) or the largest category + 1
JFN(jint, nhot)(JNIEnv*, jclass, jint n, jint nc, jlong cats, jlong oir, jlong oic, jlong ojc, jlong odata) {
    int maxcat = -1;
    int e = bidmat_nhot(n, nc, P(const int, cats), P(int, oir), P(int, oic), P(int, ojc), P(float, odata), &maxcat);
    return e ? -e : maxcat + 1;
}
// GSMat.colslice (GSMat.scala:77-104): range[0] = first nonzero, range[1] = number of nonzeros
JFN(jint, cscColsliceRange)(JNIEnv* env, jclass, jint nc, jint col1, jint col2, jlong Sjc, jintArray range) {
    int start = 0, nnz = 0;
    int e = bidmat_csc_colslice_range(nc, col1, col2, P(const int, Sjc), &start, &nnz);
    if (e) return e;
    jint* r = static_cast<jint*>(env->GetPrimitiveArrayCritical(range, nullptr));
    r[0] = start; r[1] = nnz;
    env->ReleasePrimitiveArrayCritical(range, r, 0);
    return 0;
}
JFN(jint, cscColslice)(JNIEnv*, jclass, jint col1, jint col2, jint start, jint nnz, jlong Sjc, jlong Sir, jlong Sdata,
                       jlong ojc, jlong oir, jlong oic, jlong odata) {
    int e = bidmat_csc_colslice(col1, col2, start, nnz, P(const int, Sjc), P(const int, Sir), P(const float, Sdata),
                                P(int, ojc), P(int, oir), P(int, oic), P(float, odata), nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
// GSMat.t without the host round trip, and the launcher behind GSMat.full (CUMAT.full)
JFN(jint, cscTranspose)(JNIEnv*, jclass, jint nr, jint nc, jint nnz, jlong Sdata, jlong Sir, jlong Sjc, jlong odata, jlong oir, jlong ojc) {
    return bidmat_csc_transpose(nr, nc, nnz, P(const float, Sdata), P(const int, Sir), P(const int, Sjc), P(float, odata), P(int, oir), P(int, ojc));
}
JFN(jint, full)(JNIEnv*, jclass, jlong ir, jlong ic, jlong data, jlong od, jint nr, jint nc, jint nnz) {
    return bidmat_full(P(const int, ir), P(const int, ic), P(const float, data), P(float, od), nr, nc, nnz);
}
JFN(jint, cscExpandCols)(JNIEnv*, jclass, jint nc, jint nnz, jlong Sjc, jlong Sic) {
    int e = bidmat_csc_expand_cols(nc, nnz, P(const int, Sjc), P(int, Sic), nullptr);
    return e ? e : bidmat_stream_synchronize(nullptr);
}
JFN(jlong, malloc)(JNIEnv*, jclass, jlong bytes) {
    void* p = nullptr;
    return bidmat_malloc(&p, bytes) ? 0 : (jlong)reinterpret_cast<intptr_t>(p);
}
JFN(jint, free)(JNIEnv*, jclass, jlong p) { return bidmat_free(P(void, p)); }
JFN(jint, memset)(JNIEnv*, jclass, jlong p, jint v, jlong bytes) { return bidmat_memset(P(void, p), v, bytes); }
JFN(jint, copyFloatsToDevice)(JNIEnv* env, jclass, jlong dst, jfloatArray src, jlong n) {
    void* h = env->GetPrimitiveArrayCritical(src, nullptr);
    int e = bidmat_memcpy_h2d(P(void, dst), h, n * 4);
    env->ReleasePrimitiveArrayCritical(src, h, JNI_ABORT);
    return e;
}
JFN(jint, copyIntsToDevice)(JNIEnv* env, jclass, jlong dst, jintArray src, jlong n) {
    void* h = env->GetPrimitiveArrayCritical(src, nullptr);
    int e = bidmat_memcpy_h2d(P(void, dst), h, n * 4);
    env->ReleasePrimitiveArrayCritical(src, h, JNI_ABORT);
    return e;
}
JFN(jint, copyFloatsFromDevice)(JNIEnv* env, jclass, jfloatArray dst, jlong src, jlong n) {
    void* h = env->GetPrimitiveArrayCritical(dst, nullptr);
    int e = bidmat_memcpy_d2h(h, P(const void, src), n * 4);
    env->ReleasePrimitiveArrayCritical(dst, h, 0);
    return e;
}
JFN(jint, copyIntsFromDevice)(JNIEnv* env, jclass, jintArray dst, jlong src, jlong n) {
    void* h = env->GetPrimitiveArrayCritical(dst, nullptr);
    int e = bidmat_memcpy_d2h(h, P(const void, src), n * 4);
    env->ReleasePrimitiveArrayCritical(dst, h, 0);
    return e;
}
JFN(jstring, errorString)(JNIEnv* env, jclass, jint err) { return env->NewStringUTF(bidmat_error_string(err)); }
#endif  // BIDMAT_HAVE_JNI
