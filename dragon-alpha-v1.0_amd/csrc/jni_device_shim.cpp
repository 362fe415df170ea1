// The reference's class z.dragon.engine.cuda.impl.CudaDevice on HIP: alpha_rt_getDeviceProperties fills the C struct of
// include/alpha_rt.h from hipGetDeviceProperties, and the one JNI native of that class, setProperty(int device_id)
// (CudaDevice.java:29; src/cu32_src/CudaDevice/CudaDevice/A.cu:7-330), copies every member into the Java field of the
// same name - table-driven: (field name, JNI signature, kind, offset in the struct, element count).
// One deliberate difference: the reference writes maxTexture1DLinear into the field "maxTexture1DMipmap" a second time
// (A.cu:204-205); here each of the two values goes to its own field.
#if __has_include(<jni.h>)
#include <jni.h>
#else
#include "jni_min.h"
#endif
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdio.h>
#include <string.h>

#include "../../include/alpha_rt.h"

namespace {

thread_local char g_err[256] = "";

template <typename T, int N>
void copy_ints(int (&dst)[N], const T (&src)[N])
{
    for (int i = 0; i < N; i++) dst[i] = (int)src[i];
}

enum Kind { K_STRING, K_BYTES, K_INT, K_BOOL, K_LONG, K_INTS };
struct Field {
    const char *name, *sig;
    Kind kind;
    size_t offset;
    int count;
};
#define F_(member, sig, kind, count) {#member, sig, kind, offsetof(alpha_device_properties, member), count}
const Field FIELDS[] = {
    F_(name, "Ljava/lang/String;", K_STRING, 0),
    F_(uuid, "[B", K_BYTES, 16),
    F_(luid, "[B", K_BYTES, 8),
    F_(luidDeviceNodeMask, "I", K_INT, 1),
    F_(major, "I", K_INT, 1), F_(minor, "I", K_INT, 1),
    F_(pciBusID, "I", K_INT, 1), F_(pciDeviceID, "I", K_INT, 1), F_(pciDomainID, "I", K_INT, 1),
    F_(multiGpuBoardGroupID, "I", K_INT, 1),
    F_(computeMode, "I", K_INT, 1),
    F_(deviceOverlap, "Z", K_BOOL, 1), F_(integrated, "Z", K_BOOL, 1), F_(kernelExecTimeoutEnabled, "Z", K_BOOL, 1),
    F_(unifiedAddressing, "Z", K_BOOL, 1), F_(canMapHostMemory, "Z", K_BOOL, 1),
    F_(canUseHostPointerForRegisteredMem, "Z", K_BOOL, 1), F_(directManagedMemAccessFromHost, "Z", K_BOOL, 1),
    F_(concurrentKernels, "Z", K_BOOL, 1), F_(ECCEnabled, "Z", K_BOOL, 1), F_(tccDriver, "Z", K_BOOL, 1),
    F_(streamPrioritiesSupported, "Z", K_BOOL, 1), F_(globalL1CacheSupported, "Z", K_BOOL, 1),
    F_(localL1CacheSupported, "Z", K_BOOL, 1), F_(managedMemory, "Z", K_BOOL, 1), F_(multiGpuBoard, "Z", K_BOOL, 1),
    F_(hostNativeAtomicSupported, "Z", K_BOOL, 1), F_(pageableMemoryAccess, "Z", K_BOOL, 1),
    F_(cooperativeLaunch, "Z", K_BOOL, 1), F_(concurrentManagedAccess, "Z", K_BOOL, 1),
    F_(computePreemptionSupported, "Z", K_BOOL, 1),
    F_(clockRate, "I", K_INT, 1), F_(memoryClockRate, "I", K_INT, 1), F_(memoryBusWidth, "I", K_INT, 1),
    F_(totalGlobalMemory, "J", K_LONG, 1), F_(totalConstMemory, "J", K_LONG, 1),
    F_(l2CacheSize, "I", K_INT, 1), F_(persistingL2CacheMaxSize, "I", K_INT, 1), F_(multiProcessorCount, "I", K_INT, 1),
    F_(asyncEngineCount, "I", K_INT, 1),
    F_(maxGridSize, "[I", K_INTS, 3),
    F_(singleToDoublePrecisionPerfRatio, "I", K_INT, 1), F_(accessPolicyMaxWindowSize, "I", K_INT, 1),
    F_(memoryPitch, "J", K_LONG, 1),
    F_(maxThreadsPerMultiProcessor, "I", K_INT, 1),
    F_(sharedMemPerMultiprocessor, "J", K_LONG, 1),
    F_(regsPerMultiprocessor, "I", K_INT, 1), F_(maxBlocksPerMultiProcessor, "I", K_INT, 1),
    F_(sharedMemPerBlock, "J", K_LONG, 1), F_(reservedSharedMemPerBlock, "J", K_LONG, 1), F_(sharedMemPerBlockOptin, "J", K_LONG, 1),
    F_(regsPerBlock, "I", K_INT, 1), F_(maxThreadsPerBlock, "I", K_INT, 1),
    F_(maxThreadsDim, "[I", K_INTS, 3),
    F_(warpSize, "I", K_INT, 1),
    F_(textureAlignment, "J", K_LONG, 1), F_(texturePitchAlignment, "J", K_LONG, 1),
    F_(maxTexture1D, "I", K_INT, 1), F_(maxTexture1DMipmap, "I", K_INT, 1), F_(maxTexture1DLinear, "I", K_INT, 1),
    F_(maxTexture2D, "[I", K_INTS, 2), F_(maxTexture2DMipmap, "[I", K_INTS, 2), F_(maxTexture2DLinear, "[I", K_INTS, 3),
    F_(maxTexture2DGather, "[I", K_INTS, 2), F_(maxTexture3D, "[I", K_INTS, 3), F_(maxTexture3DAlt, "[I", K_INTS, 3),
    F_(maxTexture1DLayered, "[I", K_INTS, 2), F_(maxTexture2DLayered, "[I", K_INTS, 3), F_(maxTextureCubemapLayered, "[I", K_INTS, 2),
    F_(surfaceAlignment, "J", K_LONG, 1),
    F_(maxSurface1D, "I", K_INT, 1),
    F_(maxSurface2D, "[I", K_INTS, 2), F_(maxSurface3D, "[I", K_INTS, 3), F_(maxSurface1DLayered, "[I", K_INTS, 2),
    F_(maxSurface2DLayered, "[I", K_INTS, 3),
    F_(maxSurfaceCubemap, "I", K_INT, 1),
    F_(maxSurfaceCubemapLayered, "[I", K_INTS, 2),
};
#undef F_

void raise(JNIEnv *env, int status)
{
    char msg[320];
    snprintf(msg, sizeof(msg), "alpha-rt-hip error %d: %s", status, g_err);
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

}  // namespace

extern "C" __attribute__((visibility("default"))) int alpha_rt_getDeviceProperties(int device_id, alpha_device_properties *out)
{
    if (out == nullptr) {
        snprintf(g_err, sizeof(g_err), "alpha_rt_getDeviceProperties: null result pointer");
        return (int)hipErrorInvalidValue;
    }
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess) count = 0;
    if (device_id < 0 || device_id >= count) {   // refused here: a failed runtime call would leave its error for the next caller to find
        (void)hipGetLastError();
        snprintf(g_err, sizeof(g_err), "alpha_rt_getDeviceProperties: device %d of %d", device_id, count);
        return (int)hipErrorInvalidDevice;
    }
    hipDeviceProp_t p;
    const hipError_t e = hipGetDeviceProperties(&p, device_id);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        snprintf(g_err, sizeof(g_err), "alpha_rt_getDeviceProperties: %s", hipGetErrorString(e));
        return (int)e;
    }
    alpha_device_properties &o = *out;
    memset(&o, 0, sizeof(o));
    strncpy(o.name, p.name, sizeof(o.name) - 1);
    memcpy(o.uuid, p.uuid.bytes, 16);
    memcpy(o.luid, p.luid, 8);
    o.luidDeviceNodeMask = (int)p.luidDeviceNodeMask;
    o.major = p.major; o.minor = p.minor;
    o.pciBusID = p.pciBusID; o.pciDeviceID = p.pciDeviceID; o.pciDomainID = p.pciDomainID;
    o.multiGpuBoardGroupID = p.multiGpuBoardGroupID;
    o.computeMode = p.computeMode;
    o.deviceOverlap = p.deviceOverlap; o.integrated = p.integrated; o.kernelExecTimeoutEnabled = p.kernelExecTimeoutEnabled;
    o.unifiedAddressing = p.unifiedAddressing; o.canMapHostMemory = p.canMapHostMemory;
    o.canUseHostPointerForRegisteredMem = p.canUseHostPointerForRegisteredMem;
    o.directManagedMemAccessFromHost = p.directManagedMemAccessFromHost;
    o.concurrentKernels = p.concurrentKernels; o.ECCEnabled = p.ECCEnabled; o.tccDriver = p.tccDriver;
    o.streamPrioritiesSupported = p.streamPrioritiesSupported;
    o.globalL1CacheSupported = p.globalL1CacheSupported; o.localL1CacheSupported = p.localL1CacheSupported;
    o.managedMemory = p.managedMemory; o.multiGpuBoard = p.isMultiGpuBoard;
    o.hostNativeAtomicSupported = p.hostNativeAtomicSupported; o.pageableMemoryAccess = p.pageableMemoryAccess;
    o.cooperativeLaunch = p.cooperativeLaunch; o.concurrentManagedAccess = p.concurrentManagedAccess;
    o.computePreemptionSupported = p.computePreemptionSupported;
    o.clockRate = p.clockRate; o.memoryClockRate = p.memoryClockRate; o.memoryBusWidth = p.memoryBusWidth;
    o.totalGlobalMemory = (int64_t)p.totalGlobalMem; o.totalConstMemory = (int64_t)p.totalConstMem;
    o.l2CacheSize = p.l2CacheSize; o.persistingL2CacheMaxSize = p.persistingL2CacheMaxSize;
    o.multiProcessorCount = p.multiProcessorCount; o.asyncEngineCount = p.asyncEngineCount;
    copy_ints(o.maxGridSize, p.maxGridSize);
    o.singleToDoublePrecisionPerfRatio = p.singleToDoublePrecisionPerfRatio;
    o.accessPolicyMaxWindowSize = p.accessPolicyMaxWindowSize;
    o.memoryPitch = (int64_t)p.memPitch;
    o.maxThreadsPerMultiProcessor = p.maxThreadsPerMultiProcessor;
    o.sharedMemPerMultiprocessor = (int64_t)p.sharedMemPerMultiprocessor;
    o.regsPerMultiprocessor = p.regsPerMultiprocessor; o.maxBlocksPerMultiProcessor = p.maxBlocksPerMultiProcessor;
    o.sharedMemPerBlock = (int64_t)p.sharedMemPerBlock; o.reservedSharedMemPerBlock = (int64_t)p.reservedSharedMemPerBlock;
    o.sharedMemPerBlockOptin = (int64_t)p.sharedMemPerBlockOptin;
    o.regsPerBlock = p.regsPerBlock; o.maxThreadsPerBlock = p.maxThreadsPerBlock;
    copy_ints(o.maxThreadsDim, p.maxThreadsDim);
    o.warpSize = p.warpSize;
    o.textureAlignment = (int64_t)p.textureAlignment; o.texturePitchAlignment = (int64_t)p.texturePitchAlignment;
    o.maxTexture1D = p.maxTexture1D; o.maxTexture1DMipmap = p.maxTexture1DMipmap; o.maxTexture1DLinear = p.maxTexture1DLinear;
    copy_ints(o.maxTexture2D, p.maxTexture2D); copy_ints(o.maxTexture2DMipmap, p.maxTexture2DMipmap);
    copy_ints(o.maxTexture2DLinear, p.maxTexture2DLinear); copy_ints(o.maxTexture2DGather, p.maxTexture2DGather);
    copy_ints(o.maxTexture3D, p.maxTexture3D); copy_ints(o.maxTexture3DAlt, p.maxTexture3DAlt);
    copy_ints(o.maxTexture1DLayered, p.maxTexture1DLayered); copy_ints(o.maxTexture2DLayered, p.maxTexture2DLayered);
    copy_ints(o.maxTextureCubemapLayered, p.maxTextureCubemapLayered);
    o.surfaceAlignment = (int64_t)p.surfaceAlignment;
    o.maxSurface1D = p.maxSurface1D;
    copy_ints(o.maxSurface2D, p.maxSurface2D); copy_ints(o.maxSurface3D, p.maxSurface3D);
    copy_ints(o.maxSurface1DLayered, p.maxSurface1DLayered); copy_ints(o.maxSurface2DLayered, p.maxSurface2DLayered);
    o.maxSurfaceCubemap = p.maxSurfaceCubemap;
    copy_ints(o.maxSurfaceCubemapLayered, p.maxSurfaceCubemapLayered);
    return 0;
}

// Fills the Java object from a struct: the part of setProperty that needs no device (the tests drive it with a struct
// of known values through the exported helper below).
static void fill_java_object(JNIEnv *env, jobject device, const alpha_device_properties &props)
{
    jclass cls = env->GetObjectClass(device);
    const char *base = reinterpret_cast<const char *>(&props);
    for (const Field &f : FIELDS) {
        jfieldID id = env->GetFieldID(cls, f.name, f.sig);
        if (id == nullptr) {   // a Java class without this field (an older CudaDevice): the other fields are still filled
            env->ExceptionClear();   // no JNI call may follow while the NoSuchFieldError is pending
            continue;
        }
        const char *src = base + f.offset;
        switch (f.kind) {
        case K_STRING: env->SetObjectField(device, id, env->NewStringUTF(src)); break;
        case K_BYTES: {
            jbyteArray arr = env->NewByteArray(f.count);
            env->SetByteArrayRegion(arr, 0, f.count, reinterpret_cast<const jbyte *>(src));
            env->SetObjectField(device, id, arr);
            break;
        }
        case K_INT: env->SetIntField(device, id, *reinterpret_cast<const int *>(src)); break;
        case K_BOOL: env->SetBooleanField(device, id, (jboolean)(*reinterpret_cast<const int *>(src) != 0)); break;
        case K_LONG: env->SetLongField(device, id, (jlong) * reinterpret_cast<const int64_t *>(src)); break;
        case K_INTS: {
            jintArray arr = env->NewIntArray(f.count);
            env->SetIntArrayRegion(arr, 0, f.count, reinterpret_cast<const jint *>(src));
            env->SetObjectField(device, id, arr);
            break;
        }
        }
    }
}

// CudaDevice/A.cu:7  Java: CudaDevice.setProperty (instance method: the second argument is the CudaDevice object)
extern "C" JNIEXPORT void JNICALL Java_z_dragon_engine_cuda_impl_CudaDevice_setProperty(JNIEnv *env, jobject device, jint device_id)
{
    alpha_device_properties props;
    const int rc = alpha_rt_getDeviceProperties((int)device_id, &props);
    if (rc != 0) {
        raise(env, rc);
        return;
    }
    fill_java_object(env, device, props);
}

// Test hook: the field-by-field copy into a Java object from a caller-supplied struct (no device involved).
extern "C" __attribute__((visibility("default"))) void alpha_rt_selfcheck_fillDeviceObject(JNIEnv *env, jobject device,
                                                                                           const alpha_device_properties *props)
{
    if (props) fill_java_object(env, device, *props);
}
