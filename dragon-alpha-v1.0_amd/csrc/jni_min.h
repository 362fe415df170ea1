// Minimal JNI declarations for building the shim where no JDK is installed. Written from the public
// JNI specification ("Interface Function Table"): JNIEnv is a pointer to a pointer to a table of
// function pointers; only the slots this shim calls are typed, by their specified index:
//     6 FindClass, 14 ThrowNew, 17 ExceptionClear, 31 GetObjectClass, 94 GetFieldID, 104 / 105 / 109 / 110
//     Set{Object,Boolean,Int,Long}Field, 167 NewStringUTF, 176 NewByteArray, 179 NewIntArray,
//     200 / 203 / 204 / 205 Get{Byte,Int,Long,Float}ArrayRegion, 208 / 211 / 213 Set{Byte,Int,Float}ArrayRegion.
// jlong = int64, jint = int32, jboolean = uint8, jbyte = int8, jfloat = float. When a real <jni.h> is on the include path it is
// used instead (see jni_shim.cpp).
#pragma once
#include <stdint.h>

typedef int32_t jint;
typedef int64_t jlong;
typedef uint8_t jboolean;
typedef int8_t jbyte;
typedef float jfloat;
typedef int32_t jsize;
struct _jobject;
typedef _jobject *jobject;
typedef jobject jclass;
typedef jobject jthrowable;
typedef jobject jarray;
typedef jarray jlongArray;
typedef jarray jintArray;
typedef jarray jfloatArray;
typedef jarray jbyteArray;
typedef jobject jstring;
struct _jfieldID;
typedef _jfieldID *jfieldID;

struct JNIEnv_;
typedef JNIEnv_ JNIEnv;

enum { JNI_SLOT_FindClass = 6, JNI_SLOT_ThrowNew = 14, JNI_SLOT_ExceptionClear = 17, JNI_SLOT_GetObjectClass = 31,
       JNI_SLOT_GetFieldID = 94, JNI_SLOT_SetObjectField = 104, JNI_SLOT_SetBooleanField = 105, JNI_SLOT_SetIntField = 109,
       JNI_SLOT_SetLongField = 110, JNI_SLOT_NewStringUTF = 167, JNI_SLOT_NewByteArray = 176,
       JNI_SLOT_NewIntArray = 179, JNI_SLOT_GetByteArrayRegion = 200, JNI_SLOT_GetIntArrayRegion = 203,
       JNI_SLOT_GetLongArrayRegion = 204, JNI_SLOT_GetFloatArrayRegion = 205, JNI_SLOT_SetByteArrayRegion = 208,
       JNI_SLOT_SetIntArrayRegion = 211, JNI_SLOT_SetFloatArrayRegion = 213, JNI_SLOT_COUNT = 235 };

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
    jstring NewStringUTF(const char *utf)
    {
        typedef jstring (*fn_t)(JNIEnv *, const char *);
        return reinterpret_cast<fn_t>(functions->slot[JNI_SLOT_NewStringUTF])(this, utf);
    }
    jclass GetObjectClass(jobject obj)
    {
        typedef jclass (*fn_t)(JNIEnv *, jobject);
        return reinterpret_cast<fn_t>(functions->slot[JNI_SLOT_GetObjectClass])(this, obj);
    }
    jfieldID GetFieldID(jclass cls, const char *name, const char *sig)
    {
        typedef jfieldID (*fn_t)(JNIEnv *, jclass, const char *, const char *);
        return reinterpret_cast<fn_t>(functions->slot[JNI_SLOT_GetFieldID])(this, cls, name, sig);
    }
    // Set<Type>Field all have the shape (env, object, field, value)
    template <typename T>
    void set_field(int slot, jobject obj, jfieldID id, T value)
    {
        typedef void (*fn_t)(JNIEnv *, jobject, jfieldID, T);
        reinterpret_cast<fn_t>(functions->slot[slot])(this, obj, id, value);
    }
    void SetObjectField(jobject obj, jfieldID id, jobject v) { set_field(JNI_SLOT_SetObjectField, obj, id, v); }
    void SetBooleanField(jobject obj, jfieldID id, jboolean v) { set_field(JNI_SLOT_SetBooleanField, obj, id, v); }
    void SetIntField(jobject obj, jfieldID id, jint v) { set_field(JNI_SLOT_SetIntField, obj, id, v); }
    void SetLongField(jobject obj, jfieldID id, jlong v) { set_field(JNI_SLOT_SetLongField, obj, id, v); }
    jbyteArray NewByteArray(jsize len)
    {
        typedef jbyteArray (*fn_t)(JNIEnv *, jsize);
        return reinterpret_cast<fn_t>(functions->slot[JNI_SLOT_NewByteArray])(this, len);
    }
    jintArray NewIntArray(jsize len)
    {
        typedef jintArray (*fn_t)(JNIEnv *, jsize);
        return reinterpret_cast<fn_t>(functions->slot[JNI_SLOT_NewIntArray])(this, len);
    }
    // Get/Set<Type>ArrayRegion all have the shape (env, array, start, len, buf)
    template <typename T>
    void region(int slot, jarray array, jsize start, jsize len, T *buf)
    {
        typedef void (*fn_t)(JNIEnv *, jarray, jsize, jsize, T *);
        reinterpret_cast<fn_t>(functions->slot[slot])(this, array, start, len, buf);
    }
    void GetByteArrayRegion(jbyteArray a, jsize s, jsize n, jbyte *b) { region(JNI_SLOT_GetByteArrayRegion, a, s, n, b); }
    void GetIntArrayRegion(jintArray a, jsize s, jsize n, jint *b) { region(JNI_SLOT_GetIntArrayRegion, a, s, n, b); }
    void GetFloatArrayRegion(jfloatArray a, jsize s, jsize n, jfloat *b) { region(JNI_SLOT_GetFloatArrayRegion, a, s, n, b); }
    void SetByteArrayRegion(jbyteArray a, jsize s, jsize n, const jbyte *b) { region(JNI_SLOT_SetByteArrayRegion, a, s, n, b); }
    void SetIntArrayRegion(jintArray a, jsize s, jsize n, const jint *b) { region(JNI_SLOT_SetIntArrayRegion, a, s, n, b); }
    void SetFloatArrayRegion(jfloatArray a, jsize s, jsize n, const jfloat *b) { region(JNI_SLOT_SetFloatArrayRegion, a, s, n, b); }
};

#define JNIEXPORT __attribute__((visibility("default")))
#define JNICALL
