/* STAND-IN, test use only: the few JNI type names and JNIEnv members that
 * bidmat_amd/csrc/jni_shim.cpp mentions, so that a machine without a JDK can at least parse the
 * shim (g++ -fsyntax-only) and list the functions it defines. It is not a JNI implementation,
 * is never on the include path of the product build and is never shipped. */
#pragma once
#include <stdint.h>
#define JNIEXPORT
#define JNICALL
#define JNI_ABORT 2
typedef int jint;
typedef long long jlong;
typedef float jfloat;
typedef void* jclass;
typedef void* jobject;
typedef void* jstring;
typedef void* jarray;
typedef void* jfloatArray;
typedef void* jintArray;
struct JNIEnv {
    void* GetPrimitiveArrayCritical(jarray, void*);
    void ReleasePrimitiveArrayCritical(jarray, void*, int);
    jstring NewStringUTF(const char*);
    const char* GetStringUTFChars(jstring, void*);
    void ReleaseStringUTFChars(jstring, const char*);
};
