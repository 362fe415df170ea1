/*
 * alpha_rt.h — C ABI of the runtime natives of Dragon-Alpha's class z.dragon.engine.cuda.impl.Cuda
 * (src/alpha_src/z/dragon/engine/cuda/impl/Cuda.java:19-182; implemented in the reference by
 * src/cu32_src/Cuda/Cuda/Cuda_memory.cuh, Cuda_Device.cuh, Cuda_Stream.cuh, Cuda_Event.cuh, Cuda_Exception.cuh,
 * Cuda_float.cuh, Cuda_int.cuh, Cuda_char.cuh), on HIP. The conv natives of alpha_conv.h take device addresses and
 * stream handles as 64-bit integers; these are the functions that produce them, so that a process can run the conv path
 * end to end through this library alone. One C function per Java native (overloads get a suffix), same argument order;
 * Java arrays become host pointers, return values become out-parameters, the status is returned:
 * 0 or a hipError_t value (text from alpha_rt_last_error(), thread-local).
 *
 * Handles are the HIP objects cast to int64 (hipStream_t, hipEvent_t, device and pinned-host pointers), as the
 * reference casts the CUDA ones (Cuda_memory.cuh:8-9, Cuda_Stream.cuh:19).
 */
#ifndef ALPHA_RT_H
#define ALPHA_RT_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char *alpha_rt_last_error(void);

/* ---- memory: Cuda.java:19-38, Cuda_memory.cuh:4-106 -------------------------------------------------------------- */
int alpha_rt_malloc(int64_t size, int64_t *address);
int alpha_rt_free(int64_t address);
int alpha_rt_mallocHost(int64_t size, int64_t *address);        /* pinned host memory */
int alpha_rt_freeHost(int64_t address);
int alpha_rt_memsetAsync(int64_t stream, int64_t address, int value, int64_t size);
int alpha_rt_memcpyAsyncHostToDevice(int64_t stream, int64_t dst, int64_t src, int64_t size);
int alpha_rt_memcpyAsyncHostToHost(int64_t stream, int64_t dst, int64_t src, int64_t size);
int alpha_rt_memcpyAsyncDeviceToHost(int64_t stream, int64_t dst, int64_t src, int64_t size);
int alpha_rt_memcpyAsyncDeviceToDevice(int64_t stream, int64_t dst, int64_t src, int64_t size);
int alpha_rt_memcpyAsyncDefault(int64_t stream, int64_t dst, int64_t src, int64_t size);

/* ---- device: Cuda.java:52-63, Cuda_Device.cuh:4-66 ----------------------------------------------------------------- */
int alpha_rt_getDeviceId(int *id);
int alpha_rt_getDeviceCount(int *count);
int alpha_rt_setDevice(int dev_id);
int alpha_rt_resetDevice(void);

/* The device description the reference's class CudaDevice holds (CudaDevice.java:31-215), filled by its one native
 * `setProperty(int device_id)` (src/cu32_src/CudaDevice/CudaDevice/A.cu:7-330) from cudaGetDeviceProperties. Here it is
 * filled from hipGetDeviceProperties: same field names and meanings; `major.minor` is the gfx target version (9.5 for
 * gfx950), warpSize is 64, multiProcessorCount is the number of compute units. The JNI symbol
 * Java_z_dragon_engine_cuda_impl_CudaDevice_setProperty copies every member into the Java field of the same name. */
typedef struct alpha_device_properties {
    char name[256];
    unsigned char uuid[16];
    unsigned char luid[8];
    int luidDeviceNodeMask;
    int major, minor;
    int pciBusID, pciDeviceID, pciDomainID;
    int multiGpuBoardGroupID;
    int computeMode;
    int deviceOverlap, integrated, kernelExecTimeoutEnabled, unifiedAddressing, canMapHostMemory;
    int canUseHostPointerForRegisteredMem, directManagedMemAccessFromHost, concurrentKernels, ECCEnabled, tccDriver;
    int streamPrioritiesSupported, globalL1CacheSupported, localL1CacheSupported, managedMemory, multiGpuBoard;
    int hostNativeAtomicSupported, pageableMemoryAccess, cooperativeLaunch, concurrentManagedAccess, computePreemptionSupported;
    int clockRate, memoryClockRate, memoryBusWidth;
    int64_t totalGlobalMemory, totalConstMemory;
    int l2CacheSize, persistingL2CacheMaxSize, multiProcessorCount, asyncEngineCount;
    int maxGridSize[3];
    int singleToDoublePrecisionPerfRatio, accessPolicyMaxWindowSize;
    int64_t memoryPitch;
    int maxThreadsPerMultiProcessor;
    int64_t sharedMemPerMultiprocessor;
    int regsPerMultiprocessor, maxBlocksPerMultiProcessor;
    int64_t sharedMemPerBlock, reservedSharedMemPerBlock, sharedMemPerBlockOptin;
    int regsPerBlock, maxThreadsPerBlock;
    int maxThreadsDim[3];
    int warpSize;
    int64_t textureAlignment, texturePitchAlignment;
    int maxTexture1D, maxTexture1DMipmap, maxTexture1DLinear;
    int maxTexture2D[2], maxTexture2DMipmap[2], maxTexture2DLinear[3], maxTexture2DGather[2];
    int maxTexture3D[3], maxTexture3DAlt[3], maxTexture1DLayered[2], maxTexture2DLayered[3], maxTextureCubemapLayered[2];
    int64_t surfaceAlignment;
    int maxSurface1D;
    int maxSurface2D[2], maxSurface3D[3], maxSurface1DLayered[2], maxSurface2DLayered[3];
    int maxSurfaceCubemap;
    int maxSurfaceCubemapLayered[2];
} alpha_device_properties;

/* CudaDevice/A.cu:7-12 (cudaGetDeviceProperties) */
int alpha_rt_getDeviceProperties(int device_id, alpha_device_properties *out);
int alpha_rt_deviceSynchronize(void);
int alpha_rt_isDeviceP2PAccessEnabled(int dev1_id, int dev2_id, int *enabled);
int alpha_rt_enableDeviceP2PAccess(int dev2_id);
int alpha_rt_disableDeviceP2PAccess(int dev2_id);

/* ---- streams: Cuda.java:72-98, Cuda_Stream.cuh:4-103. The priority arguments are accepted and ignored: every stream is
 * created at the default priority (range reported as [0, 0]). ------------------------------------------------------- */
int alpha_rt_getStreamPriorityRange(int *low, int *high);
int alpha_rt_newStream_Blocking(int64_t *stream);
int alpha_rt_newStream_Blocking_priority(int priority, int64_t *stream);
int alpha_rt_newStream_NonBlocking(int64_t *stream);
int alpha_rt_newStream_NonBlocking_priority(int priority, int64_t *stream);
int alpha_rt_deleteStream(int64_t stream);                                   /* 0 is skipped, as in the reference */
int alpha_rt_deleteStreams(const int64_t *streams, int length);
int alpha_rt_streamQuery(int64_t stream, int *completed);
int alpha_rt_streamSynchronize(int64_t stream);
int alpha_rt_streamsSynchronize(const int64_t *streams, int length);

/* ---- events: Cuda.java:102-119, Cuda_Event.cuh:4-135 ----------------------------------------------------------------- */
int alpha_rt_newEvent_Default(int64_t *event);
int alpha_rt_newEvent_BlockingSync(int64_t *event);
int alpha_rt_newEvent_DisableTiming(int64_t *event);
int alpha_rt_newEvent_Interprocess(int64_t *event);
int alpha_rt_deleteEvent(int64_t event);
int alpha_rt_eventRecord(int64_t event, int64_t stream);
/* The reference's array form does not record anything: it synchronises every stream of the array on the host
 * (Cuda_Event.cuh:53-62). Kept: callers rely on the work being complete when it returns. */
int alpha_rt_eventRecord_streams(int64_t event, const int64_t *streams, int length);
int alpha_rt_eventSynchronize(int64_t event);
int alpha_rt_eventElapsedTime(int64_t start_event, int64_t stop_event, float *ms);
int alpha_rt_streamWaitEvent_default(int64_t stream, int64_t event);
int alpha_rt_streamWaitEvent_external(int64_t stream, int64_t event);
int alpha_rt_streamsWaitEvent_default(const int64_t *streams, int length, int64_t event);
int alpha_rt_streamsWaitEvent_external(const int64_t *streams, int length, int64_t event);

/* ---- error text: Cuda.java:123-125, Cuda_Exception.cuh:4-22 ------------------------------------------------------------ */
const char *alpha_rt_getExceptionName(int type);
const char *alpha_rt_getExceptionInfo(int type);
int alpha_rt_getLastExceptionType(void);

/* ---- host <-> device arrays: Cuda.java:129-182; Cuda_float.cuh, Cuda_int.cuh, Cuda_char.cuh -----------------------------
 * elem = bytes per element (4: float and int natives, 1: char natives). A 2-D tensor has `height` rows of `stride`
 * elements of which the first `width` are data and the rest padding: get2D compacts rows to `width`, set2D expands them
 * and writes zeros into the padding. `staging` is the pinned host buffer of the *_v2 natives (at least height*stride
 * elements) or NULL (a temporary is allocated, as the plain natives do); `value` may be the staging buffer itself
 * (compaction and expansion then happen in place, as in the reference). All of them synchronise the stream before
 * returning, as the reference does. */
int alpha_rt_get1D(int64_t stream, int64_t address, void *value, int length, int elem, void *staging);
int alpha_rt_get2D(int64_t stream, int64_t address, void *value, int height, int width, int stride, int elem, void *staging);
int alpha_rt_set1D(int64_t stream, int64_t address, const void *value, int length, int elem, void *staging);
int alpha_rt_set2D(int64_t stream, int64_t address, const void *value, int height, int width, int stride, int elem, void *staging);
/* set1D(byte[]) / set2D(byte[]) of the float natives: each signed byte becomes a float (Cuda_float.cuh:172-214, 258-310) */
int alpha_rt_set1D_bytes(int64_t stream, int64_t address, const int8_t *value, int length, float *staging);
int alpha_rt_set2D_bytes(int64_t stream, int64_t address, const int8_t *value, int height, int width, int stride, float *staging);
/* set2D_v2_char_W3S4: rows of 3 bytes expanded to 4 (pictures with 3 channels), two pinned buffers (Cuda_char.cuh:241-265) */
int alpha_rt_set2D_char_W3S4(int64_t stream, int64_t address, const int8_t *value, int8_t *buf1, int8_t *buf2, int height);
/* fills on the device, enqueued only (Cuda_float.cuh:141-166, Cuda_float_set1D.cuh, Cuda_float_set2D.cuh) */
int alpha_rt_set1D_value(int64_t stream, int64_t address, float value, int length);
int alpha_rt_set2D_value(int64_t stream, int64_t address, float value, int height, int width, int stride);
/* device-side re-strides of float tensors, enqueued only (Cuda_float_set1to2.cuh, _set2to1.cuh, _set2to2.cuh):
 * element k of the dense side <-> row k / width, column k % width of the strided side; padding is left untouched */
int alpha_rt_setFrom1Dto2D(int64_t stream, int64_t src, int src_length, int64_t dst, int dst_height, int dst_width, int dst_stride);
int alpha_rt_setFrom2Dto1D(int64_t stream, int64_t src, int src_height, int src_width, int src_stride, int64_t dst, int dst_length);
int alpha_rt_setFrom2Dto2D(int64_t stream, int64_t src, int src_height, int src_width, int src_stride,
                           int64_t dst, int dst_height, int dst_width, int dst_stride);

#ifdef __cplusplus
}
#endif
#endif /* ALPHA_RT_H */
