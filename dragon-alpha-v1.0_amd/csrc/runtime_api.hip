// HIP implementation of the runtime natives declared in include/alpha_rt.h: thin wrappers around the HIP runtime for
// memory, devices, streams and events, the host<->device array transfers with their 2-D compaction/expansion, and three
// small device kernels (fills and re-strides). Nothing here is on the convolution path; it exists so that a process can
// obtain the device addresses and stream handles that path consumes from the same library.
#include "../../include/alpha_rt.h"
#include "common.hpp"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace {

thread_local char g_err[256] = "";

int status(hipError_t e, const char *fn)
{
    if (e == hipSuccess) return 0;
    snprintf(g_err, sizeof(g_err), "%s: %s (%s)", fn, hipGetErrorString(e), hipGetErrorName(e));
    return (int)e;
}
int invalid(const char *fn, const char *what)
{
    snprintf(g_err, sizeof(g_err), "%s: %s", fn, what);
    return (int)hipErrorInvalidValue;
}

inline hipStream_t S(int64_t s) { return reinterpret_cast<hipStream_t>(static_cast<intptr_t>(s)); }
inline hipEvent_t E(int64_t e) { return reinterpret_cast<hipEvent_t>(static_cast<intptr_t>(e)); }
inline void *P(int64_t a) { return reinterpret_cast<void *>(static_cast<intptr_t>(a)); }

int copy(const char *fn, int64_t stream, int64_t dst, int64_t src, int64_t size, hipMemcpyKind kind)
{
    if (size < 0) return invalid(fn, "negative size");
    if (size == 0) return 0;
    return status(hipMemcpyAsync(P(dst), P(src), (size_t)size, kind, S(stream)), fn);
}

// ---- device kernels: grid-stride, 128-bit where the layout allows ------------------------------------------------------
__global__ __launch_bounds__(256) void fill_kernel(float *__restrict__ X, float value, int lengthv, int width, int stride)
{
    // element k is data when k % stride < width, padding (zero) otherwise; width == stride for the 1-D fill
    // 64-bit loop index: k + gridDim.x*256 must not wrap for lengths close to 2^31
    for (long k = (long)blockIdx.x * 256 + threadIdx.x; k < lengthv; k += (long)gridDim.x * 256) X[k] = ((int)k % stride) < width ? value : 0.f;
}
__global__ __launch_bounds__(256) void restride_kernel(const float *__restrict__ X, int XW, int XS, float *__restrict__ Y,
                                                       int YW, int YS, int length)
{
    for (long kk = (long)blockIdx.x * 256 + threadIdx.x; kk < length; kk += (long)gridDim.x * 256) {
        const int k = (int)kk;
        Y[(size_t)(k / YW) * YS + (k % YW)] = X[(size_t)(k / XW) * XS + (k % XW)];
    }
}

// memset by kernel rather than hipMemsetAsync, so that the call behaves the same when the caller's stream is being
// captured into a graph: words where address and size allow, bytes otherwise
__global__ __launch_bounds__(256) void memset_words_kernel(uint32_t *__restrict__ p, uint32_t word, size_t n)
{
    for (size_t k = (size_t)blockIdx.x * 256 + threadIdx.x; k < n; k += (size_t)gridDim.x * 256) p[k] = word;
}
__global__ __launch_bounds__(256) void memset_bytes_kernel(uint8_t *__restrict__ p, uint8_t byte, size_t n)
{
    for (size_t k = (size_t)blockIdx.x * 256 + threadIdx.x; k < n; k += (size_t)gridDim.x * 256) p[k] = byte;
}

int grid_for(int n)
{
    int g = (n + 255) / 256;
    return g < 1 ? 1 : (g > 4096 ? 4096 : g);
}

struct Temp {   // host temporary of the plain (non-v2) natives
    void *p = nullptr;
    bool owned = false;
    Temp(void *staging, size_t bytes)
    {
        if (staging) p = staging;
        else { p = malloc(bytes ? bytes : 1); owned = true; }
    }
    ~Temp() { if (owned) free(p); }
};

}  // namespace

#pragma GCC visibility push(default)
extern "C" {

const char *alpha_rt_last_error(void) { return g_err; }

// ---- memory ---------------------------------------------------------------------------------------------------------------
int alpha_rt_malloc(int64_t size, int64_t *address)
{
    if (!address || size < 0) return invalid(__func__, "null result pointer or negative size");
    void *p = nullptr;
    const int rc = status(hipMalloc(&p, (size_t)size), __func__);
    *address = (int64_t)(intptr_t)p;
    return rc;
}
int alpha_rt_free(int64_t address) { return status(hipFree(P(address)), __func__); }
int alpha_rt_mallocHost(int64_t size, int64_t *address)
{
    if (!address || size < 0) return invalid(__func__, "null result pointer or negative size");
    void *p = nullptr;
    const int rc = status(hipHostMalloc(&p, (size_t)size, hipHostMallocDefault), __func__);
    *address = (int64_t)(intptr_t)p;
    return rc;
}
int alpha_rt_freeHost(int64_t address) { return status(hipHostFree(P(address)), __func__); }
int alpha_rt_memsetAsync(int64_t stream, int64_t address, int value, int64_t size)
{
    if (size < 0) return invalid(__func__, "negative size");
    if (size == 0) return 0;
    const uint32_t b = (uint32_t)value & 0xffu;
    if (((uintptr_t)address & 3u) == 0 && (size & 3) == 0) {
        const size_t n = (size_t)size >> 2;
        const size_t g = (n + 255) / 256;
        hipLaunchKernelGGL(memset_words_kernel, dim3((unsigned)(g > 8192 ? 8192 : g)), dim3(256), 0, S(stream),
                           static_cast<uint32_t *>(P(address)), b * 0x01010101u, n);
    } else {
        const size_t g = ((size_t)size + 255) / 256;
        hipLaunchKernelGGL(memset_bytes_kernel, dim3((unsigned)(g > 8192 ? 8192 : g)), dim3(256), 0, S(stream),
                           static_cast<uint8_t *>(P(address)), (uint8_t)b, (size_t)size);
    }
    return status(hipGetLastError(), __func__);
}
int alpha_rt_memcpyAsyncHostToDevice(int64_t stream, int64_t dst, int64_t src, int64_t size)
{
    return copy(__func__, stream, dst, src, size, hipMemcpyHostToDevice);
}
int alpha_rt_memcpyAsyncHostToHost(int64_t stream, int64_t dst, int64_t src, int64_t size)
{
    return copy(__func__, stream, dst, src, size, hipMemcpyHostToHost);
}
int alpha_rt_memcpyAsyncDeviceToHost(int64_t stream, int64_t dst, int64_t src, int64_t size)
{
    return copy(__func__, stream, dst, src, size, hipMemcpyDeviceToHost);
}
int alpha_rt_memcpyAsyncDeviceToDevice(int64_t stream, int64_t dst, int64_t src, int64_t size)
{
    return copy(__func__, stream, dst, src, size, hipMemcpyDeviceToDevice);
}
int alpha_rt_memcpyAsyncDefault(int64_t stream, int64_t dst, int64_t src, int64_t size)
{
    return copy(__func__, stream, dst, src, size, hipMemcpyDefault);
}

// ---- device ---------------------------------------------------------------------------------------------------------------
int alpha_rt_getDeviceId(int *id) { return id ? status(hipGetDevice(id), __func__) : invalid(__func__, "null"); }
int alpha_rt_getDeviceCount(int *count) { return count ? status(hipGetDeviceCount(count), __func__) : invalid(__func__, "null"); }
int alpha_rt_setDevice(int dev_id) { return status(hipSetDevice(dev_id), __func__); }
// hipDeviceReset drops what the library configured on the device (function attributes, the address of the static
// scratch array) and frees every allocation, including the scratch pools of engines: destroy engines before a reset.
// The generation counter makes the conv launchers configure their kernels again afterwards.
int alpha_rt_resetDevice(void)
{
    const int rc = status(hipDeviceReset(), __func__);
    alpha::device_generation().fetch_add(1, std::memory_order_acq_rel);
    return rc;
}
int alpha_rt_deviceSynchronize(void) { return status(hipDeviceSynchronize(), __func__); }
int alpha_rt_isDeviceP2PAccessEnabled(int dev1_id, int dev2_id, int *enabled)
{
    if (!enabled) return invalid(__func__, "null");
    return status(hipDeviceCanAccessPeer(enabled, dev1_id, dev2_id), __func__);
}
int alpha_rt_enableDeviceP2PAccess(int dev2_id) { return status(hipDeviceEnablePeerAccess(dev2_id, 0), __func__); }
int alpha_rt_disableDeviceP2PAccess(int dev2_id) { return status(hipDeviceDisablePeerAccess(dev2_id), __func__); }

// ---- streams (always the default priority) ----------------------------------------------------------------------------------
int alpha_rt_getStreamPriorityRange(int *low, int *high)
{
    if (!low || !high) return invalid(__func__, "null");
    *low = 0;
    *high = 0;
    return 0;
}
static int new_stream(const char *fn, unsigned flags, int64_t *stream)
{
    if (!stream) return invalid(fn, "null");
    hipStream_t s = nullptr;
    const int rc = status(hipStreamCreateWithFlags(&s, flags), fn);
    *stream = (int64_t)(intptr_t)s;
    return rc;
}
int alpha_rt_newStream_Blocking(int64_t *stream) { return new_stream(__func__, hipStreamDefault, stream); }
int alpha_rt_newStream_Blocking_priority(int, int64_t *stream) { return new_stream(__func__, hipStreamDefault, stream); }
int alpha_rt_newStream_NonBlocking(int64_t *stream) { return new_stream(__func__, hipStreamNonBlocking, stream); }
int alpha_rt_newStream_NonBlocking_priority(int, int64_t *stream) { return new_stream(__func__, hipStreamNonBlocking, stream); }
int alpha_rt_deleteStream(int64_t stream)
{
    if (!stream) return 0;
    return status(hipStreamDestroy(S(stream)), __func__);
}
int alpha_rt_deleteStreams(const int64_t *streams, int length)
{
    if (length > 0 && !streams) return invalid(__func__, "null");
    for (int i = 0; i < length; i++)
        if (int rc = alpha_rt_deleteStream(streams[i])) return rc;
    return 0;
}
int alpha_rt_streamQuery(int64_t stream, int *completed)
{
    if (!completed) return invalid(__func__, "null");
    const hipError_t e = hipStreamQuery(S(stream));
    *completed = e == hipSuccess;
    if (e == hipSuccess || e == hipErrorNotReady) return 0;
    return status(e, __func__);
}
int alpha_rt_streamSynchronize(int64_t stream) { return status(hipStreamSynchronize(S(stream)), __func__); }
int alpha_rt_streamsSynchronize(const int64_t *streams, int length)
{
    if (length > 0 && !streams) return invalid(__func__, "null");
    for (int i = 0; i < length; i++)
        if (int rc = status(hipStreamSynchronize(S(streams[i])), __func__)) return rc;
    return 0;
}

// ---- events ---------------------------------------------------------------------------------------------------------------
static int new_event(const char *fn, unsigned flags, int64_t *event)
{
    if (!event) return invalid(fn, "null");
    hipEvent_t e = nullptr;
    const int rc = status(hipEventCreateWithFlags(&e, flags), fn);
    *event = (int64_t)(intptr_t)e;
    return rc;
}
int alpha_rt_newEvent_Default(int64_t *event) { return new_event(__func__, hipEventDefault, event); }
int alpha_rt_newEvent_BlockingSync(int64_t *event) { return new_event(__func__, hipEventBlockingSync, event); }
int alpha_rt_newEvent_DisableTiming(int64_t *event) { return new_event(__func__, hipEventDisableTiming, event); }
int alpha_rt_newEvent_Interprocess(int64_t *event)
{
    return new_event(__func__, hipEventInterprocess | hipEventDisableTiming, event);   // HIP requires both flags together
}
int alpha_rt_deleteEvent(int64_t event) { return status(hipEventDestroy(E(event)), __func__); }
int alpha_rt_eventRecord(int64_t event, int64_t stream) { return status(hipEventRecord(E(event), S(stream)), __func__); }
int alpha_rt_eventRecord_streams(int64_t, const int64_t *streams, int length) { return alpha_rt_streamsSynchronize(streams, length); }
int alpha_rt_eventSynchronize(int64_t event) { return status(hipEventSynchronize(E(event)), __func__); }
int alpha_rt_eventElapsedTime(int64_t start_event, int64_t stop_event, float *ms)
{
    if (!ms) return invalid(__func__, "null");
    return status(hipEventElapsedTime(ms, E(start_event), E(stop_event)), __func__);
}
int alpha_rt_streamWaitEvent_default(int64_t stream, int64_t event) { return status(hipStreamWaitEvent(S(stream), E(event), 0), __func__); }
int alpha_rt_streamWaitEvent_external(int64_t stream, int64_t event) { return status(hipStreamWaitEvent(S(stream), E(event), 0), __func__); }
int alpha_rt_streamsWaitEvent_default(const int64_t *streams, int length, int64_t event)
{
    if (length > 0 && !streams) return invalid(__func__, "null");
    for (int i = 0; i < length; i++)
        if (int rc = status(hipStreamWaitEvent(S(streams[i]), E(event), 0), __func__)) return rc;
    return 0;
}
int alpha_rt_streamsWaitEvent_external(const int64_t *streams, int length, int64_t event)
{
    return alpha_rt_streamsWaitEvent_default(streams, length, event);
}

// ---- error text -------------------------------------------------------------------------------------------------------------
const char *alpha_rt_getExceptionName(int type) { return hipGetErrorName((hipError_t)type); }
const char *alpha_rt_getExceptionInfo(int type) { return hipGetErrorString((hipError_t)type); }
int alpha_rt_getLastExceptionType(void) { return (int)hipGetLastError(); }

// ---- host <-> device arrays ---------------------------------------------------------------------------------------------------
int alpha_rt_get1D(int64_t stream, int64_t address, void *value, int length, int elem, void *staging)
{
    if (length < 0 || (elem != 1 && elem != 4) || (length > 0 && !value)) return invalid(__func__, "bad length, element size or pointer");
    if (length == 0) return 0;
    const size_t bytes = (size_t)length * elem;
    void *host = staging ? staging : value;   // without a staging buffer the copy lands in the caller's array directly
    if (int rc = status(hipMemcpyAsync(host, P(address), bytes, hipMemcpyDeviceToHost, S(stream)), __func__)) return rc;
    if (int rc = status(hipStreamSynchronize(S(stream)), __func__)) return rc;
    if (staging) memcpy(value, staging, bytes);
    return 0;
}
int alpha_rt_get2D(int64_t stream, int64_t address, void *value, int height, int width, int stride, int elem, void *staging)
{
    if (height < 0 || width < 1 || stride < width || (elem != 1 && elem != 4) || (height > 0 && !value))
        return invalid(__func__, "needs height >= 0, 1 <= width <= stride, element size 1 or 4");
    if (height == 0) return 0;
    const size_t bytes = (size_t)height * stride * elem;
    Temp tmp(staging, bytes);
    if (!tmp.p) return invalid(__func__, "out of host memory");
    if (int rc = status(hipMemcpyAsync(tmp.p, P(address), bytes, hipMemcpyDeviceToHost, S(stream)), __func__)) return rc;
    if (int rc = status(hipStreamSynchronize(S(stream)), __func__)) return rc;
    const char *src = static_cast<const char *>(tmp.p);
    char *dst = static_cast<char *>(value);
    // ascending rows with memmove: compacting in place (value == staging) never overwrites a row not yet moved
    for (int i = 0; i < height; i++) memmove(dst + (size_t)i * width * elem, src + (size_t)i * stride * elem, (size_t)width * elem);
    return 0;
}
int alpha_rt_set1D(int64_t stream, int64_t address, const void *value, int length, int elem, void *staging)
{
    if (length < 0 || (elem != 1 && elem != 4) || (length > 0 && !value)) return invalid(__func__, "bad length, element size or pointer");
    if (length == 0) return 0;
    const size_t bytes = (size_t)length * elem;
    const void *host = value;
    if (staging) { memcpy(staging, value, bytes); host = staging; }
    if (int rc = status(hipMemcpyAsync(P(address), host, bytes, hipMemcpyHostToDevice, S(stream)), __func__)) return rc;
    return status(hipStreamSynchronize(S(stream)), __func__);
}
int alpha_rt_set2D(int64_t stream, int64_t address, const void *value, int height, int width, int stride, int elem, void *staging)
{
    if (height < 0 || width < 1 || stride < width || (elem != 1 && elem != 4) || (height > 0 && !value))
        return invalid(__func__, "needs height >= 0, 1 <= width <= stride, element size 1 or 4");
    if (height == 0) return 0;
    const size_t bytes = (size_t)height * stride * elem;
    Temp tmp(staging, bytes);
    if (!tmp.p) return invalid(__func__, "out of host memory");
    const char *src = static_cast<const char *>(value);
    char *dst = static_cast<char *>(tmp.p);
    // descending rows with memmove: expanding in place (value == staging) never overwrites a row not yet moved
    for (int i = height - 1; i >= 0; i--) {
        memmove(dst + (size_t)i * stride * elem, src + (size_t)i * width * elem, (size_t)width * elem);
        memset(dst + ((size_t)i * stride + width) * elem, 0, (size_t)(stride - width) * elem);
    }
    if (int rc = status(hipMemcpyAsync(P(address), tmp.p, bytes, hipMemcpyHostToDevice, S(stream)), __func__)) return rc;
    return status(hipStreamSynchronize(S(stream)), __func__);
}
int alpha_rt_set1D_bytes(int64_t stream, int64_t address, const int8_t *value, int length, float *staging)
{
    if (length < 0 || (length > 0 && !value)) return invalid(__func__, "bad length or pointer");
    if (length == 0) return 0;
    Temp tmp(staging, (size_t)length * 4);
    if (!tmp.p) return invalid(__func__, "out of host memory");
    float *f = static_cast<float *>(tmp.p);
    for (int i = 0; i < length; i++) f[i] = (float)value[i];
    if (int rc = status(hipMemcpyAsync(P(address), f, (size_t)length * 4, hipMemcpyHostToDevice, S(stream)), __func__)) return rc;
    return status(hipStreamSynchronize(S(stream)), __func__);
}
int alpha_rt_set2D_bytes(int64_t stream, int64_t address, const int8_t *value, int height, int width, int stride, float *staging)
{
    if (height < 0 || width < 1 || stride < width || (height > 0 && !value)) return invalid(__func__, "needs height >= 0, 1 <= width <= stride");
    if (height == 0) return 0;
    const size_t n = (size_t)height * stride;
    Temp tmp(staging, n * 4);
    if (!tmp.p) return invalid(__func__, "out of host memory");
    float *f = static_cast<float *>(tmp.p);
    for (int i = 0; i < height; i++) {
        for (int j = 0; j < width; j++) f[(size_t)i * stride + j] = (float)value[(size_t)i * width + j];
        for (int j = width; j < stride; j++) f[(size_t)i * stride + j] = 0.f;
    }
    if (int rc = status(hipMemcpyAsync(P(address), f, n * 4, hipMemcpyHostToDevice, S(stream)), __func__)) return rc;
    return status(hipStreamSynchronize(S(stream)), __func__);
}
int alpha_rt_set2D_char_W3S4(int64_t stream, int64_t address, const int8_t *value, int8_t *buf1, int8_t *buf2, int height)
{
    if (height < 0 || (height > 0 && (!value || !buf1 || !buf2))) return invalid(__func__, "bad height or pointer");
    if (height == 0) return 0;
    memcpy(buf1, value, (size_t)height * 3);   // the reference stages the Java array in buf1 first
    for (int i = 0; i < height; i++) {
        buf2[4 * (size_t)i + 0] = buf1[3 * (size_t)i + 0];
        buf2[4 * (size_t)i + 1] = buf1[3 * (size_t)i + 1];
        buf2[4 * (size_t)i + 2] = buf1[3 * (size_t)i + 2];
        buf2[4 * (size_t)i + 3] = 0;
    }
    if (int rc = status(hipMemcpyAsync(P(address), buf2, (size_t)height * 4, hipMemcpyHostToDevice, S(stream)), __func__)) return rc;
    return status(hipStreamSynchronize(S(stream)), __func__);
}

int alpha_rt_set1D_value(int64_t stream, int64_t address, float value, int length)
{
    if (length < 0) return invalid(__func__, "negative length");
    if (length == 0) return 0;
    hipLaunchKernelGGL(fill_kernel, dim3(grid_for(length)), dim3(256), 0, S(stream), static_cast<float *>(P(address)), value, length, 1, 1);
    return status(hipGetLastError(), __func__);
}
int alpha_rt_set2D_value(int64_t stream, int64_t address, float value, int height, int width, int stride)
{
    if (height < 0 || width < 1 || stride < width) return invalid(__func__, "needs height >= 0, 1 <= width <= stride");
    if ((long)height * stride >= (1L << 31)) return invalid(__func__, "tensor too large");
    if (height == 0) return 0;
    const int n = height * stride;
    hipLaunchKernelGGL(fill_kernel, dim3(grid_for(n)), dim3(256), 0, S(stream), static_cast<float *>(P(address)), value, n, width, stride);
    return status(hipGetLastError(), __func__);
}
static int restride(const char *fn, int64_t stream, int64_t src, int XW, int XS, int64_t dst, int YW, int YS, long length)
{
    if (length < 0 || XW < 1 || YW < 1 || XS < XW || YS < YW || length >= (1L << 31)) return invalid(fn, "bad geometry");
    if (length == 0) return 0;
    hipLaunchKernelGGL(restride_kernel, dim3(grid_for((int)length)), dim3(256), 0, S(stream), static_cast<const float *>(P(src)), XW, XS,
                       static_cast<float *>(P(dst)), YW, YS, (int)length);
    return status(hipGetLastError(), fn);
}
int alpha_rt_setFrom1Dto2D(int64_t stream, int64_t src, int src_length, int64_t dst, int dst_height, int dst_width, int dst_stride)
{
    (void)dst_height;
    return restride(__func__, stream, src, src_length > 0 ? src_length : 1, src_length > 0 ? src_length : 1, dst, dst_width, dst_stride, src_length);
}
int alpha_rt_setFrom2Dto1D(int64_t stream, int64_t src, int src_height, int src_width, int src_stride, int64_t dst, int dst_length)
{
    (void)src_height;
    return restride(__func__, stream, src, src_width, src_stride, dst, dst_length > 0 ? dst_length : 1, dst_length > 0 ? dst_length : 1, dst_length);
}
int alpha_rt_setFrom2Dto2D(int64_t stream, int64_t src, int src_height, int src_width, int src_stride,
                           int64_t dst, int dst_height, int dst_width, int dst_stride)
{
    (void)src_height;
    return restride(__func__, stream, src, src_width, src_stride, dst, dst_width, dst_stride, (long)dst_height * dst_width);
}

}  // extern "C"
#pragma GCC visibility pop
