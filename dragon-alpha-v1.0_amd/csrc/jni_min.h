// Minimal JNI declarations for building the shim where no JDK is installed. Written from the public
// JNI specification ("Interface Function Table"): JNIEnv is a pointer to a pointer to a table of
// function pointers; only the slots this shim calls are typed, by their specified index:
//     6 FindClass, 14 ThrowNew, 17 ExceptionClear, 204 GetLongArrayRegion.
// jlong = int64, jint = int32, jboolean = uint8. When a real <jni.h> is on the include path it is
// used instead (see jni_shim.cpp).
#pragma once
#include <stdint.h>

typedef int32_t jint;
typedef int64_t jlong;
typedef uint8_t jboolean;
typedef int32_t jsize;
struct _jobject;
typedef _jobject *jobject;
typedef jobject jclass;
typedef jobject jthrowable;
typedef jobject jarray;
typedef jarray jlongArray;

struct JNIEnv_;
typedef JNIEnv_ JNIEnv;

enum { JNI_SLOT_FindClass = 6, JNI_SLOT_ThrowNew = 14, JNI_SLOT_ExceptionClear = 17, JNI_SLOT_GetLongArrayRegion = 204,
       JNI_SLOT_COUNT = 235 };

struct JNINativeInterface_ {
    void *slot[JNI_SLOT_COUNT];
};

struct JNIEnv_ {
    const JNINativeInterface_ *functions;

    jclass FindClass(const char *name)
    {
        typedef jclass (*fn_t)(JNIEnv *, const char *);
        return reinterpret_cast<fn_t>(functions->slot[JNI_SLOT_FindClass])(this, name);
    }
    jint ThrowNew(jclass cls, const char *msg)
    {
        typedef jint (*fn_t)(JNIEnv *, jclass, const char *);
        return reinterpret_cast<fn_t>(functions->slot[JNI_SLOT_ThrowNew])(this, cls, msg);
    }
    void ExceptionClear()
    {
        typedef void (*fn_t)(JNIEnv *);
        reinterpret_cast<fn_t>(functions->slot[JNI_SLOT_ExceptionClear])(this);
    }
    void GetLongArrayRegion(jlongArray array, jsize start, jsize len, jlong *buf)
    {
        typedef void (*fn_t)(JNIEnv *, jlongArray, jsize, jsize, jlong *);
        reinterpret_cast<fn_t>(functions->slot[JNI_SLOT_GetLongArrayRegion])(this, array, start, len, buf);
    }
};

#define JNIEXPORT __attribute__((visibility("default")))
#define JNICALL
