/*
 * Test-only stand-in for <jni.h>: just enough of the Java Native Interface (types, constants and the
 * JNIEnv members the shim calls, spelled as the JNI specification spells them) for
 * dragon-alpha-v1.2_amd/csrc/jni/dragon_jni.cpp to be compiled and its exports listed on a machine without
 * a JDK.  Every JNIEnv member is a do-nothing inline, so the resulting library can be loaded but not
 * driven; a real build uses the JDK's header (csrc/jni/build_jni.sh).
 */
#ifndef DRAGON_TEST_JNI_H
#define DRAGON_TEST_JNI_H

#include <stdint.h>
#include <stddef.h>

#define JNIEXPORT __attribute__((visibility("default")))
#define JNIIMPORT
#define JNICALL

typedef int32_t jint;
typedef int64_t jlong;
typedef int8_t jbyte;
typedef uint8_t jboolean;
typedef uint16_t jchar;
typedef int16_t jshort;
typedef float jfloat;
typedef double jdouble;
typedef jint jsize;

class _jobject {};
class _jclass : public _jobject {};
class _jthrowable : public _jobject {};
class _jstring : public _jobject {};
class _jarray : public _jobject {};
class _jlongArray : public _jarray {};
class _jfloatArray : public _jarray {};
typedef _jobject* jobject;
typedef _jclass* jclass;
typedef _jthrowable* jthrowable;
typedef _jstring* jstring;
typedef _jarray* jarray;
typedef _jlongArray* jlongArray;
typedef _jfloatArray* jfloatArray;
struct _jmethodID;
typedef _jmethodID* jmethodID;

#define JNI_FALSE 0
#define JNI_TRUE 1
#define JNI_OK 0
#define JNI_ERR (-1)
#define JNI_COMMIT 1
#define JNI_ABORT 2
#define JNI_VERSION_1_8 0x00010008

struct JNIEnv {
    jclass FindClass(const char*) { return nullptr; }
    jmethodID GetMethodID(jclass, const char*, const char*) { return nullptr; }
    jobject NewObject(jclass, jmethodID, ...) { return nullptr; }
    jint Throw(jthrowable) { return 0; }
    jstring NewStringUTF(const char*) { return nullptr; }
    jsize GetArrayLength(jarray) { return 0; }
    void GetLongArrayRegion(jlongArray, jsize, jsize, jlong*) {}
    jfloat* GetFloatArrayElements(jfloatArray, jboolean*) { return nullptr; }
    void ReleaseFloatArrayElements(jfloatArray, jfloat*, jint) {}
    void SetFloatArrayRegion(jfloatArray, jsize, jsize, const jfloat*) {}
};
struct JavaVM {
    jint GetEnv(void**, jint) { return JNI_ERR; }
};

#endif /* DRAGON_TEST_JNI_H */
