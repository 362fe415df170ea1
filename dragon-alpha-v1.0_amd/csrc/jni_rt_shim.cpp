// JNI entry points of the reference's runtime class z.dragon.engine.cuda.impl.Cuda (Cuda.java:19-182), forwarding to
// the C ABI of include/alpha_rt.h. Symbol names are the JNI long names the reference's sources use (overloaded natives
// carry their argument signature: Cuda_Stream.cuh:15-61, Cuda_Event.cuh:43-62, Cuda_float.cuh:141-400). Java arrays are
// moved with Get/Set<Type>ArrayRegion into a host temporary, or into the caller's pinned buffer for the *_v2 natives.
// A non-zero status raises a Java exception (same class search as the conv shim); value-returning natives return 0.
#if __has_include(<jni.h>)
#include <jni.h>
#else
#include "jni_min.h"
#endif
#include <stdint.h>
#include <stdio.h>

#include <vector>

#include "../../include/alpha_rt.h"

namespace {

void raise(JNIEnv *env, int status)
{
    if (status == 0) return;
    char msg[320];
    snprintf(msg, sizeof(msg), "alpha-rt-hip error %d: %s", status, alpha_rt_last_error());
    static const char *const classes[] = {"z/dragon/engine/cuda/impl/CudaException", "z/jcuda/exception/CudaException",
                                          "java/lang/RuntimeException"};
    for (const char *name : classes) {
        jclass cls = env->FindClass(name);
        if (cls != nullptr) {
            env->ThrowNew(cls, msg);
            return;
        }
        env->ExceptionClear();
    }
    fprintf(stderr, "%s\n", msg);
}

// the handles of a Java long[] (stream arrays)
struct Streams {
    std::vector<int64_t> v;
    Streams(JNIEnv *env, jlongArray arr, jint length)
    {
        if (length > 0 && arr != nullptr) {
            v.resize((size_t)length);
            env->GetLongArrayRegion(arr, 0, length, reinterpret_cast<jlong *>(v.data()));
        }
    }
    const int64_t *data() const { return v.data(); }
    int size() const { return (int)v.size(); }
};

template <typename T> T *host(jlong a) { return reinterpret_cast<T *>(static_cast<intptr_t>(a)); }

// device -> Java array. `buf` = pinned staging buffer of the _v2 natives, or 0.
template <typename T, typename Setter>
void get_nd(JNIEnv *env, jlong stream, jlong address, jlong buf, jint height, jint width, jint stride, bool two_d, Setter set)
{
    const long n_out = two_d ? (long)height * width : (long)width;
    const long n_dev = two_d ? (long)height * stride : (long)width;
    if (n_out <= 0) return;
    std::vector<T> tmp;
    T *h = host<T>(buf);
    if (!h) {
        tmp.resize((size_t)n_dev);
        h = tmp.data();
    }
    const int rc = two_d ? alpha_rt_get2D(stream, address, h, height, width, stride, (int)sizeof(T), h)
                         : alpha_rt_get1D(stream, address, h, width, (int)sizeof(T), nullptr);
    if (rc) return raise(env, rc);
    set(h, (jint)n_out);
}
// Java array -> device
template <typename T, typename Getter>
void set_nd(JNIEnv *env, jlong stream, jlong address, jlong buf, jint height, jint width, jint stride, bool two_d, Getter get)
{
    const long n_in = two_d ? (long)height * width : (long)width;
    const long n_dev = two_d ? (long)height * stride : (long)width;
    if (n_in <= 0) return;
    std::vector<T> tmp;
    T *h = host<T>(buf);
    if (!h) {
        tmp.resize((size_t)n_dev);
        h = tmp.data();
    }
    get(h, (jint)n_in);   // dense rows at the start of the buffer; set2D expands them in place
    raise(env, two_d ? alpha_rt_set2D(stream, address, h, height, width, stride, (int)sizeof(T), h)
                     : alpha_rt_set1D(stream, address, h, width, (int)sizeof(T), nullptr));
}
// byte[] -> float tensor
void set_bytes_nd(JNIEnv *env, jlong stream, jlong address, jbyteArray value, jlong buf, jint height, jint width, jint stride, bool two_d)
{
    const long n_in = two_d ? (long)height * width : (long)width;
    if (n_in <= 0) return;
    std::vector<jbyte> bytes((size_t)n_in);
    env->GetByteArrayRegion(value, 0, (jint)n_in, bytes.data());
    raise(env, two_d ? alpha_rt_set2D_bytes(stream, address, bytes.data(), height, width, stride, host<float>(buf))
                     : alpha_rt_set1D_bytes(stream, address, bytes.data(), width, host<float>(buf)));
}

}  // namespace

#define CUDA_NATIVE(ret, name) extern "C" JNIEXPORT ret JNICALL Java_z_dragon_engine_cuda_impl_Cuda_##name

// ---- memory (Cuda_memory.cuh) ---------------------------------------------------------------------------------------------
CUDA_NATIVE(jlong, malloc)(JNIEnv *env, jclass, jlong size)
{
    int64_t a = 0;
    raise(env, alpha_rt_malloc(size, &a));
    return a;
}
CUDA_NATIVE(void, free)(JNIEnv *env, jclass, jlong address) { raise(env, alpha_rt_free(address)); }
CUDA_NATIVE(jlong, mallocHost)(JNIEnv *env, jclass, jlong size)
{
    int64_t a = 0;
    raise(env, alpha_rt_mallocHost(size, &a));
    return a;
}
CUDA_NATIVE(void, freeHost)(JNIEnv *env, jclass, jlong address) { raise(env, alpha_rt_freeHost(address)); }
CUDA_NATIVE(void, memsetAsync)(JNIEnv *env, jclass, jlong stream, jlong address, jint value, jlong size)
{
    raise(env, alpha_rt_memsetAsync(stream, address, value, size));
}
CUDA_NATIVE(void, memcpyAsyncHostToDevice)(JNIEnv *env, jclass, jlong s, jlong dst, jlong src, jlong size)
{
    raise(env, alpha_rt_memcpyAsyncHostToDevice(s, dst, src, size));
}
CUDA_NATIVE(void, memcpyAsyncHostToHost)(JNIEnv *env, jclass, jlong s, jlong dst, jlong src, jlong size)
{
    raise(env, alpha_rt_memcpyAsyncHostToHost(s, dst, src, size));
}
CUDA_NATIVE(void, memcpyAsyncDeviceToHost)(JNIEnv *env, jclass, jlong s, jlong dst, jlong src, jlong size)
{
    raise(env, alpha_rt_memcpyAsyncDeviceToHost(s, dst, src, size));
}
CUDA_NATIVE(void, memcpyAsyncDeviceToDevice)(JNIEnv *env, jclass, jlong s, jlong dst, jlong src, jlong size)
{
    raise(env, alpha_rt_memcpyAsyncDeviceToDevice(s, dst, src, size));
}
CUDA_NATIVE(void, memcpyAsyncDefault)(JNIEnv *env, jclass, jlong s, jlong dst, jlong src, jlong size)
{
    raise(env, alpha_rt_memcpyAsyncDefault(s, dst, src, size));
}

// ---- device (Cuda_Device.cuh) -----------------------------------------------------------------------------------------------
CUDA_NATIVE(jint, getDeviceId)(JNIEnv *env, jclass)
{
    int v = 0;
    raise(env, alpha_rt_getDeviceId(&v));
    return v;
}
CUDA_NATIVE(jint, getDeviceCount)(JNIEnv *env, jclass)
{
    int v = 0;
    raise(env, alpha_rt_getDeviceCount(&v));
    return v;
}
CUDA_NATIVE(void, setDevice)(JNIEnv *env, jclass, jint dev) { raise(env, alpha_rt_setDevice(dev)); }
CUDA_NATIVE(void, resetDevice)(JNIEnv *env, jclass) { raise(env, alpha_rt_resetDevice()); }
CUDA_NATIVE(void, deviceSynchronize)(JNIEnv *env, jclass) { raise(env, alpha_rt_deviceSynchronize()); }
CUDA_NATIVE(jboolean, isDeviceP2PAccessEnabled)(JNIEnv *env, jclass, jint d1, jint d2)
{
    int v = 0;
    raise(env, alpha_rt_isDeviceP2PAccessEnabled(d1, d2, &v));
    return v ? 1 : 0;
}
CUDA_NATIVE(void, enableDeviceP2PAccess)(JNIEnv *env, jclass, jint d2) { raise(env, alpha_rt_enableDeviceP2PAccess(d2)); }
CUDA_NATIVE(void, disableDeviceP2PAccess)(JNIEnv *env, jclass, jint d2) { raise(env, alpha_rt_disableDeviceP2PAccess(d2)); }

// ---- streams (Cuda_Stream.cuh) ------------------------------------------------------------------------------------------------
CUDA_NATIVE(jintArray, getStreamPriorityRange)(JNIEnv *env, jclass)
{
    int r[2] = {0, 0};
    raise(env, alpha_rt_getStreamPriorityRange(&r[0], &r[1]));
    jintArray arr = env->NewIntArray(2);
    if (arr != nullptr) {
        const jint v[2] = {r[0], r[1]};
        env->SetIntArrayRegion(arr, 0, 2, v);
    }
    return arr;
}
CUDA_NATIVE(jlong, newStream_1Blocking__)(JNIEnv *env, jclass)
{
    int64_t s = 0;
    raise(env, alpha_rt_newStream_Blocking(&s));
    return s;
}
CUDA_NATIVE(jlong, newStream_1Blocking__I)(JNIEnv *env, jclass, jint priority)
{
    int64_t s = 0;
    raise(env, alpha_rt_newStream_Blocking_priority(priority, &s));
    return s;
}
CUDA_NATIVE(jlong, newStream_1NonBlocking__)(JNIEnv *env, jclass)
{
    int64_t s = 0;
    raise(env, alpha_rt_newStream_NonBlocking(&s));
    return s;
}
CUDA_NATIVE(jlong, newStream_1NonBlocking__I)(JNIEnv *env, jclass, jint priority)
{
    int64_t s = 0;
    raise(env, alpha_rt_newStream_NonBlocking_priority(priority, &s));
    return s;
}
CUDA_NATIVE(void, deleteStream__J)(JNIEnv *env, jclass, jlong stream) { raise(env, alpha_rt_deleteStream(stream)); }
CUDA_NATIVE(void, deleteStream___3JI)(JNIEnv *env, jclass, jlongArray arr, jint length)
{
    Streams s(env, arr, length);
    raise(env, alpha_rt_deleteStreams(s.data(), s.size()));
}
CUDA_NATIVE(jboolean, streamQuery)(JNIEnv *env, jclass, jlong stream)
{
    int done = 0;
    raise(env, alpha_rt_streamQuery(stream, &done));
    return done ? 1 : 0;
}
CUDA_NATIVE(void, streamSynchronize__J)(JNIEnv *env, jclass, jlong stream) { raise(env, alpha_rt_streamSynchronize(stream)); }
CUDA_NATIVE(void, streamSynchronize___3JI)(JNIEnv *env, jclass, jlongArray arr, jint length)
{
    Streams s(env, arr, length);
    raise(env, alpha_rt_streamsSynchronize(s.data(), s.size()));
}

// ---- events (Cuda_Event.cuh) --------------------------------------------------------------------------------------------------
CUDA_NATIVE(jlong, newEvent_1Default)(JNIEnv *env, jclass)
{
    int64_t e = 0;
    raise(env, alpha_rt_newEvent_Default(&e));
    return e;
}
CUDA_NATIVE(jlong, newEvent_1BlockingSync)(JNIEnv *env, jclass)
{
    int64_t e = 0;
    raise(env, alpha_rt_newEvent_BlockingSync(&e));
    return e;
}
CUDA_NATIVE(jlong, newEvent_1DisableTiming)(JNIEnv *env, jclass)
{
    int64_t e = 0;
    raise(env, alpha_rt_newEvent_DisableTiming(&e));
    return e;
}
CUDA_NATIVE(jlong, newEvent_1Interprocess)(JNIEnv *env, jclass)
{
    int64_t e = 0;
    raise(env, alpha_rt_newEvent_Interprocess(&e));
    return e;
}
CUDA_NATIVE(void, deleteEvent)(JNIEnv *env, jclass, jlong event) { raise(env, alpha_rt_deleteEvent(event)); }
CUDA_NATIVE(void, eventRecord__JJ)(JNIEnv *env, jclass, jlong event, jlong stream) { raise(env, alpha_rt_eventRecord(event, stream)); }
CUDA_NATIVE(void, eventRecord__J_3JI)(JNIEnv *env, jclass, jlong event, jlongArray arr, jint length)
{
    Streams s(env, arr, length);
    raise(env, alpha_rt_eventRecord_streams(event, s.data(), s.size()));
}
CUDA_NATIVE(void, eventSynchronize)(JNIEnv *env, jclass, jlong event) { raise(env, alpha_rt_eventSynchronize(event)); }
CUDA_NATIVE(void, eventSynchronize_1delete)(JNIEnv *env, jclass, jlong event)   // Cuda_Event.cuh:73-80 (no Java declaration)
{
    const int rc = alpha_rt_eventSynchronize(event);
    raise(env, rc ? rc : alpha_rt_deleteEvent(event));
}
CUDA_NATIVE(jfloat, eventElapsedTime)(JNIEnv *env, jclass, jlong start, jlong stop)
{
    float ms = 0.f;
    raise(env, alpha_rt_eventElapsedTime(start, stop, &ms));
    return ms;
}
CUDA_NATIVE(void, streamWaitEvent_1default)(JNIEnv *env, jclass, jlong stream, jlong event)
{
    raise(env, alpha_rt_streamWaitEvent_default(stream, event));
}
CUDA_NATIVE(void, streamWaitEvent_1external)(JNIEnv *env, jclass, jlong stream, jlong event)
{
    raise(env, alpha_rt_streamWaitEvent_external(stream, event));
}
CUDA_NATIVE(void, streamsWaitEvent_1default)(JNIEnv *env, jclass, jlongArray arr, jint length, jlong event)
{
    Streams s(env, arr, length);
    raise(env, alpha_rt_streamsWaitEvent_default(s.data(), s.size(), event));
}
CUDA_NATIVE(void, streamsWaitEvent_1external)(JNIEnv *env, jclass, jlongArray arr, jint length, jlong event)
{
    Streams s(env, arr, length);
    raise(env, alpha_rt_streamsWaitEvent_external(s.data(), s.size(), event));
}

// ---- error text (Cuda_Exception.cuh) ------------------------------------------------------------------------------------------
CUDA_NATIVE(jstring, getExceptionName)(JNIEnv *env, jclass, jint type) { return env->NewStringUTF(alpha_rt_getExceptionName(type)); }
CUDA_NATIVE(jstring, getExceptionInfo)(JNIEnv *env, jclass, jint type) { return env->NewStringUTF(alpha_rt_getExceptionInfo(type)); }
CUDA_NATIVE(jint, getLastExceptionType)(JNIEnv *, jclass) { return alpha_rt_getLastExceptionType(); }

// ---- float tensors (Cuda_float.cuh) ----------------------------------------------------------------------------------------------
#define FSET(arr) [&](jfloat *h, jint n) { env->SetFloatArrayRegion(arr, 0, n, h); }
#define FGET(arr) [&](jfloat *h, jint n) { env->GetFloatArrayRegion(arr, 0, n, h); }
#define ISET(arr) [&](jint *h, jint n) { env->SetIntArrayRegion(arr, 0, n, h); }
#define IGET(arr) [&](jint *h, jint n) { env->GetIntArrayRegion(arr, 0, n, h); }
#define BSET(arr) [&](jbyte *h, jint n) { env->SetByteArrayRegion(arr, 0, n, h); }
#define BGET(arr) [&](jbyte *h, jint n) { env->GetByteArrayRegion(arr, 0, n, h); }

CUDA_NATIVE(void, get1D)(JNIEnv *env, jclass, jlong s, jlong a, jfloatArray v, jint length)
{
    get_nd<jfloat>(env, s, a, 0, 1, length, length, false, FSET(v));
}
CUDA_NATIVE(void, get1D_1v2)(JNIEnv *env, jclass, jlong s, jlong a, jfloatArray v, jlong buf, jint length)
{
    get_nd<jfloat>(env, s, a, buf, 1, length, length, false, FSET(v));
}
CUDA_NATIVE(void, get2D)(JNIEnv *env, jclass, jlong s, jlong a, jfloatArray v, jint h, jint w, jint st)
{
    get_nd<jfloat>(env, s, a, 0, h, w, st, true, FSET(v));
}
CUDA_NATIVE(void, get2D_1v2)(JNIEnv *env, jclass, jlong s, jlong a, jfloatArray v, jlong buf, jint h, jint w, jint st)
{
    get_nd<jfloat>(env, s, a, buf, h, w, st, true, FSET(v));
}
CUDA_NATIVE(void, set1D__JJFI)(JNIEnv *env, jclass, jlong s, jlong a, jfloat value, jint length)
{
    raise(env, alpha_rt_set1D_value(s, a, value, length));
}
CUDA_NATIVE(void, set2D__JJFIII)(JNIEnv *env, jclass, jlong s, jlong a, jfloat value, jint h, jint w, jint st)
{
    raise(env, alpha_rt_set2D_value(s, a, value, h, w, st));
}
CUDA_NATIVE(void, set1D__JJ_3BI)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jint length)
{
    set_bytes_nd(env, s, a, v, 0, 1, length, length, false);
}
CUDA_NATIVE(void, set1D_1v2__JJ_3BJI)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jlong buf, jint length)
{
    set_bytes_nd(env, s, a, v, buf, 1, length, length, false);
}
CUDA_NATIVE(void, set1D__JJ_3FI)(JNIEnv *env, jclass, jlong s, jlong a, jfloatArray v, jint length)
{
    set_nd<jfloat>(env, s, a, 0, 1, length, length, false, FGET(v));
}
CUDA_NATIVE(void, set1D_1v2__JJ_3FJI)(JNIEnv *env, jclass, jlong s, jlong a, jfloatArray v, jlong buf, jint length)
{
    set_nd<jfloat>(env, s, a, buf, 1, length, length, false, FGET(v));
}
CUDA_NATIVE(void, set2D__JJ_3BIII)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jint h, jint w, jint st)
{
    set_bytes_nd(env, s, a, v, 0, h, w, st, true);
}
CUDA_NATIVE(void, set2D_1v2__JJ_3BJIII)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jlong buf, jint h, jint w, jint st)
{
    set_bytes_nd(env, s, a, v, buf, h, w, st, true);
}
CUDA_NATIVE(void, set2D__JJ_3FIII)(JNIEnv *env, jclass, jlong s, jlong a, jfloatArray v, jint h, jint w, jint st)
{
    set_nd<jfloat>(env, s, a, 0, h, w, st, true, FGET(v));
}
CUDA_NATIVE(void, set2D_1v2__JJ_3FJIII)(JNIEnv *env, jclass, jlong s, jlong a, jfloatArray v, jlong buf, jint h, jint w, jint st)
{
    set_nd<jfloat>(env, s, a, buf, h, w, st, true, FGET(v));
}
CUDA_NATIVE(void, setFrom1Dto2D)(JNIEnv *env, jclass, jlong s, jlong src, jint len, jlong dst, jint h, jint w, jint st)
{
    raise(env, alpha_rt_setFrom1Dto2D(s, src, len, dst, h, w, st));
}
CUDA_NATIVE(void, setFrom2Dto1D)(JNIEnv *env, jclass, jlong s, jlong src, jint h, jint w, jint st, jlong dst, jint len)
{
    raise(env, alpha_rt_setFrom2Dto1D(s, src, h, w, st, dst, len));
}
CUDA_NATIVE(void, setFrom2Dto2D)(JNIEnv *env, jclass, jlong s, jlong src, jint h, jint w, jint st, jlong dst, jint dh, jint dw, jint dst_stride)
{
    raise(env, alpha_rt_setFrom2Dto2D(s, src, h, w, st, dst, dh, dw, dst_stride));
}

// ---- int32 tensors (Cuda_int.cuh) ---------------------------------------------------------------------------------------------------
CUDA_NATIVE(void, get1D_1int)(JNIEnv *env, jclass, jlong s, jlong a, jintArray v, jint length)
{
    get_nd<jint>(env, s, a, 0, 1, length, length, false, ISET(v));
}
CUDA_NATIVE(void, get2D_1int)(JNIEnv *env, jclass, jlong s, jlong a, jintArray v, jint h, jint w, jint st)
{
    get_nd<jint>(env, s, a, 0, h, w, st, true, ISET(v));
}
CUDA_NATIVE(void, get1D_1v2_1int)(JNIEnv *env, jclass, jlong s, jlong a, jintArray v, jlong buf, jint length)
{
    get_nd<jint>(env, s, a, buf, 1, length, length, false, ISET(v));
}
CUDA_NATIVE(void, get2D_1v2_1int)(JNIEnv *env, jclass, jlong s, jlong a, jintArray v, jlong buf, jint h, jint w, jint st)
{
    get_nd<jint>(env, s, a, buf, h, w, st, true, ISET(v));
}
CUDA_NATIVE(void, set1D_1int)(JNIEnv *env, jclass, jlong s, jlong a, jintArray v, jint length)
{
    set_nd<jint>(env, s, a, 0, 1, length, length, false, IGET(v));
}
CUDA_NATIVE(void, set2D_1int)(JNIEnv *env, jclass, jlong s, jlong a, jintArray v, jint h, jint w, jint st)
{
    set_nd<jint>(env, s, a, 0, h, w, st, true, IGET(v));
}
CUDA_NATIVE(void, set1D_1v2_1int)(JNIEnv *env, jclass, jlong s, jlong a, jintArray v, jlong buf, jint length)
{
    set_nd<jint>(env, s, a, buf, 1, length, length, false, IGET(v));
}
CUDA_NATIVE(void, set2D_1v2_1int)(JNIEnv *env, jclass, jlong s, jlong a, jintArray v, jlong buf, jint h, jint w, jint st)
{
    set_nd<jint>(env, s, a, buf, h, w, st, true, IGET(v));
}

// ---- int8 tensors (Cuda_char.cuh) ---------------------------------------------------------------------------------------------------
CUDA_NATIVE(void, get1D_1char)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jint length)
{
    get_nd<jbyte>(env, s, a, 0, 1, length, length, false, BSET(v));
}
CUDA_NATIVE(void, get2D_1char)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jint h, jint w, jint st)
{
    get_nd<jbyte>(env, s, a, 0, h, w, st, true, BSET(v));
}
CUDA_NATIVE(void, get1D_1v2_1char)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jlong buf, jint length)
{
    get_nd<jbyte>(env, s, a, buf, 1, length, length, false, BSET(v));
}
CUDA_NATIVE(void, get2D_1v2_1char)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jlong buf, jint h, jint w, jint st)
{
    get_nd<jbyte>(env, s, a, buf, h, w, st, true, BSET(v));
}
CUDA_NATIVE(void, set1D_1char)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jint length)
{
    set_nd<jbyte>(env, s, a, 0, 1, length, length, false, BGET(v));
}
CUDA_NATIVE(void, set2D_1char)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jint h, jint w, jint st)
{
    set_nd<jbyte>(env, s, a, 0, h, w, st, true, BGET(v));
}
CUDA_NATIVE(void, set1D_1v2_1char)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jlong buf, jint length)
{
    set_nd<jbyte>(env, s, a, buf, 1, length, length, false, BGET(v));
}
CUDA_NATIVE(void, set2D_1v2_1char)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jlong buf, jint h, jint w, jint st)
{
    set_nd<jbyte>(env, s, a, buf, h, w, st, true, BGET(v));
}
CUDA_NATIVE(void, set2D_1v2_1char_1W3S4)(JNIEnv *env, jclass, jlong s, jlong a, jbyteArray v, jlong buf1, jlong buf2, jint height)
{
    if (height <= 0) return;
    std::vector<jbyte> bytes((size_t)height * 3);
    env->GetByteArrayRegion(v, 0, height * 3, bytes.data());
    raise(env, alpha_rt_set2D_char_W3S4(s, a, bytes.data(), host<int8_t>(buf1), host<int8_t>(buf2), height));
}
