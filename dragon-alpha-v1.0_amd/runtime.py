"""ctypes mirror of the reference's runtime class z.dragon.engine.cuda.impl.Cuda (Cuda.java:19-182) over the C ABI of
include/alpha_rt.h. Method names and argument order are the Java ones; Java arrays are numpy arrays (float32, int32 or
int8, C-contiguous), natives that return a value return it, and a non-zero status raises AlphaConvError where the Java
side would see a CudaException. Test and tooling plumbing, like native.py."""
import ctypes

import numpy as np

from . import native

_I, _L, _P, _F = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_float
_bound = False


def _lib():
    global _bound
    L = native.lib()
    if not _bound:
        L.alpha_rt_last_error.restype = ctypes.c_char_p
        for name in ("alpha_rt_getExceptionName", "alpha_rt_getExceptionInfo"):
            getattr(L, name).restype = ctypes.c_char_p
            getattr(L, name).argtypes = [_I]
        sig = {
            "malloc": [_L, ctypes.POINTER(_L)], "free": [_L], "mallocHost": [_L, ctypes.POINTER(_L)], "freeHost": [_L],
            "memsetAsync": [_L, _L, _I, _L],
            "memcpyAsyncHostToDevice": [_L] * 4, "memcpyAsyncHostToHost": [_L] * 4, "memcpyAsyncDeviceToHost": [_L] * 4,
            "memcpyAsyncDeviceToDevice": [_L] * 4, "memcpyAsyncDefault": [_L] * 4,
            "getDeviceId": [ctypes.POINTER(_I)], "getDeviceCount": [ctypes.POINTER(_I)], "setDevice": [_I],
            "resetDevice": [], "deviceSynchronize": [], "isDeviceP2PAccessEnabled": [_I, _I, ctypes.POINTER(_I)],
            "enableDeviceP2PAccess": [_I], "disableDeviceP2PAccess": [_I],
            "getStreamPriorityRange": [ctypes.POINTER(_I), ctypes.POINTER(_I)],
            "newStream_Blocking": [ctypes.POINTER(_L)], "newStream_Blocking_priority": [_I, ctypes.POINTER(_L)],
            "newStream_NonBlocking": [ctypes.POINTER(_L)], "newStream_NonBlocking_priority": [_I, ctypes.POINTER(_L)],
            "deleteStream": [_L], "deleteStreams": [ctypes.POINTER(_L), _I], "streamQuery": [_L, ctypes.POINTER(_I)],
            "streamSynchronize": [_L], "streamsSynchronize": [ctypes.POINTER(_L), _I],
            "newEvent_Default": [ctypes.POINTER(_L)], "newEvent_BlockingSync": [ctypes.POINTER(_L)],
            "newEvent_DisableTiming": [ctypes.POINTER(_L)], "newEvent_Interprocess": [ctypes.POINTER(_L)],
            "deleteEvent": [_L], "eventRecord": [_L, _L], "eventRecord_streams": [_L, ctypes.POINTER(_L), _I],
            "eventSynchronize": [_L], "eventElapsedTime": [_L, _L, ctypes.POINTER(_F)],
            "streamWaitEvent_default": [_L, _L], "streamWaitEvent_external": [_L, _L],
            "streamsWaitEvent_default": [ctypes.POINTER(_L), _I, _L], "streamsWaitEvent_external": [ctypes.POINTER(_L), _I, _L],
            "getLastExceptionType": [],
            "get1D": [_L, _L, _P, _I, _I, _P], "get2D": [_L, _L, _P, _I, _I, _I, _I, _P],
            "set1D": [_L, _L, _P, _I, _I, _P], "set2D": [_L, _L, _P, _I, _I, _I, _I, _P],
            "set1D_bytes": [_L, _L, _P, _I, _P], "set2D_bytes": [_L, _L, _P, _I, _I, _I, _P],
            "set2D_char_W3S4": [_L, _L, _P, _P, _P, _I],
            "set1D_value": [_L, _L, _F, _I], "set2D_value": [_L, _L, _F, _I, _I, _I],
            "setFrom1Dto2D": [_L, _L, _I, _L, _I, _I, _I], "setFrom2Dto1D": [_L, _L, _I, _I, _I, _L, _I],
            "setFrom2Dto2D": [_L, _L, _I, _I, _I, _L, _I, _I, _I],
        }
        for name, args in sig.items():
            getattr(L, "alpha_rt_" + name).argtypes = args
        _bound = True
    return L


def _ck(rc):
    if rc != 0:
        raise native.AlphaConvError("runtime call failed (%d): %s" % (rc, _lib().alpha_rt_last_error().decode()))


def _out_long(fn, *args):
    v = _L(0)
    _ck(getattr(_lib(), "alpha_rt_" + fn)(*args, ctypes.byref(v)))
    return v.value


def _out_int(fn, *args):
    v = _I(0)
    _ck(getattr(_lib(), "alpha_rt_" + fn)(*args, ctypes.byref(v)))
    return v.value


def _longs(values):
    return (_L * max(1, len(values)))(*values)


def _arr(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a, a.ctypes.data_as(_P)


def _staging(buf_address):
    return _P(buf_address) if buf_address else None


class Cuda:
    """Runtime natives (Cuda.java)."""

    # ---- memory ----
    malloc = staticmethod(lambda size: _out_long("malloc", size))
    mallocHost = staticmethod(lambda size: _out_long("mallocHost", size))
    free = staticmethod(lambda address: _ck(_lib().alpha_rt_free(address)))
    freeHost = staticmethod(lambda address: _ck(_lib().alpha_rt_freeHost(address)))
    memsetAsync = staticmethod(lambda stream, address, value, size: _ck(_lib().alpha_rt_memsetAsync(stream, address, value, size)))
    memcpyAsyncHostToDevice = staticmethod(lambda s, dst, src, n: _ck(_lib().alpha_rt_memcpyAsyncHostToDevice(s, dst, src, n)))
    memcpyAsyncHostToHost = staticmethod(lambda s, dst, src, n: _ck(_lib().alpha_rt_memcpyAsyncHostToHost(s, dst, src, n)))
    memcpyAsyncDeviceToHost = staticmethod(lambda s, dst, src, n: _ck(_lib().alpha_rt_memcpyAsyncDeviceToHost(s, dst, src, n)))
    memcpyAsyncDeviceToDevice = staticmethod(lambda s, dst, src, n: _ck(_lib().alpha_rt_memcpyAsyncDeviceToDevice(s, dst, src, n)))
    memcpyAsyncDefault = staticmethod(lambda s, dst, src, n: _ck(_lib().alpha_rt_memcpyAsyncDefault(s, dst, src, n)))

    # ---- device ----
    getDeviceId = staticmethod(lambda: _out_int("getDeviceId"))
    getDeviceCount = staticmethod(lambda: _out_int("getDeviceCount"))
    setDevice = staticmethod(lambda dev: _ck(_lib().alpha_rt_setDevice(dev)))
    deviceSynchronize = staticmethod(lambda: _ck(_lib().alpha_rt_deviceSynchronize()))
    isDeviceP2PAccessEnabled = staticmethod(lambda d1, d2: bool(_out_int("isDeviceP2PAccessEnabled", d1, d2)))

    # ---- streams ----
    @staticmethod
    def getStreamPriorityRange():
        lo, hi = _I(0), _I(0)
        _ck(_lib().alpha_rt_getStreamPriorityRange(ctypes.byref(lo), ctypes.byref(hi)))
        return [lo.value, hi.value]

    @staticmethod
    def newStream_Blocking(priority=None):
        return _out_long("newStream_Blocking") if priority is None else _out_long("newStream_Blocking_priority", priority)

    @staticmethod
    def newStream_NonBlocking(priority=None):
        return _out_long("newStream_NonBlocking") if priority is None else _out_long("newStream_NonBlocking_priority", priority)

    @staticmethod
    def deleteStream(streams, length=None):
        if length is None:
            _ck(_lib().alpha_rt_deleteStream(streams))
        else:
            _ck(_lib().alpha_rt_deleteStreams(_longs(streams), length))

    streamQuery = staticmethod(lambda stream: bool(_out_int("streamQuery", stream)))

    @staticmethod
    def streamSynchronize(streams, length=None):
        if length is None:
            _ck(_lib().alpha_rt_streamSynchronize(streams))
        else:
            _ck(_lib().alpha_rt_streamsSynchronize(_longs(streams), length))

    # ---- events ----
    newEvent_Default = staticmethod(lambda: _out_long("newEvent_Default"))
    newEvent_BlockingSync = staticmethod(lambda: _out_long("newEvent_BlockingSync"))
    newEvent_DisableTiming = staticmethod(lambda: _out_long("newEvent_DisableTiming"))
    newEvent_Interprocess = staticmethod(lambda: _out_long("newEvent_Interprocess"))
    deleteEvent = staticmethod(lambda event: _ck(_lib().alpha_rt_deleteEvent(event)))

    @staticmethod
    def eventRecord(event, streams, length=None):
        if length is None:
            _ck(_lib().alpha_rt_eventRecord(event, streams))
        else:
            _ck(_lib().alpha_rt_eventRecord_streams(event, _longs(streams), length))

    eventSynchronize = staticmethod(lambda event: _ck(_lib().alpha_rt_eventSynchronize(event)))

    @staticmethod
    def eventElapsedTime(start, stop):
        ms = _F(0)
        _ck(_lib().alpha_rt_eventElapsedTime(start, stop, ctypes.byref(ms)))
        return ms.value

    streamWaitEvent_default = staticmethod(lambda stream, event: _ck(_lib().alpha_rt_streamWaitEvent_default(stream, event)))
    streamWaitEvent_external = staticmethod(lambda stream, event: _ck(_lib().alpha_rt_streamWaitEvent_external(stream, event)))
    streamsWaitEvent_default = staticmethod(
        lambda streams, length, event: _ck(_lib().alpha_rt_streamsWaitEvent_default(_longs(streams), length, event)))
    streamsWaitEvent_external = staticmethod(
        lambda streams, length, event: _ck(_lib().alpha_rt_streamsWaitEvent_external(_longs(streams), length, event)))

    # ---- error text ----
    getExceptionName = staticmethod(lambda t: _lib().alpha_rt_getExceptionName(t).decode())
    getExceptionInfo = staticmethod(lambda t: _lib().alpha_rt_getExceptionInfo(t).decode())
    getLastExceptionType = staticmethod(lambda: _lib().alpha_rt_getLastExceptionType())

    # ---- tensors: `value` arrays are filled in place by the get natives, as the Java arrays are ----
    @staticmethod
    def _get(stream, address, value, dims, buf):
        assert value.flags["C_CONTIGUOUS"] and value.dtype.itemsize in (1, 4)
        p = value.ctypes.data_as(_P)
        if len(dims) == 1:
            _ck(_lib().alpha_rt_get1D(stream, address, p, dims[0], value.dtype.itemsize, _staging(buf)))
        else:
            _ck(_lib().alpha_rt_get2D(stream, address, p, dims[0], dims[1], dims[2], value.dtype.itemsize, _staging(buf)))

    @staticmethod
    def _set(stream, address, value, dtype, dims, buf):
        a, p = _arr(value, dtype)
        if len(dims) == 1:
            _ck(_lib().alpha_rt_set1D(stream, address, p, dims[0], a.dtype.itemsize, _staging(buf)))
        else:
            _ck(_lib().alpha_rt_set2D(stream, address, p, dims[0], dims[1], dims[2], a.dtype.itemsize, _staging(buf)))

    get1D = staticmethod(lambda s, a, value, length: Cuda._get(s, a, value, (length,), 0))
    get2D = staticmethod(lambda s, a, value, h, w, st: Cuda._get(s, a, value, (h, w, st), 0))
    get1D_v2 = staticmethod(lambda s, a, value, buf, length: Cuda._get(s, a, value, (length,), buf))
    get2D_v2 = staticmethod(lambda s, a, value, buf, h, w, st: Cuda._get(s, a, value, (h, w, st), buf))
    get1D_int, get2D_int, get1D_v2_int, get2D_v2_int = get1D, get2D, get1D_v2, get2D_v2
    get1D_char, get2D_char, get1D_v2_char, get2D_v2_char = get1D, get2D, get1D_v2, get2D_v2

    @staticmethod
    def set1D(stream, address, value, length):
        """set1D(float value) fills; set1D(byte[]) converts each byte to float; set1D(float[]) copies."""
        if np.isscalar(value):
            _ck(_lib().alpha_rt_set1D_value(stream, address, float(value), length))
        elif np.asarray(value).dtype == np.int8:
            a, p = _arr(value, np.int8)
            _ck(_lib().alpha_rt_set1D_bytes(stream, address, p, length, None))
        else:
            Cuda._set(stream, address, value, np.float32, (length,), 0)

    @staticmethod
    def set2D(stream, address, value, height, width, stride):
        if np.isscalar(value):
            _ck(_lib().alpha_rt_set2D_value(stream, address, float(value), height, width, stride))
        elif np.asarray(value).dtype == np.int8:
            a, p = _arr(value, np.int8)
            _ck(_lib().alpha_rt_set2D_bytes(stream, address, p, height, width, stride, None))
        else:
            Cuda._set(stream, address, value, np.float32, (height, width, stride), 0)

    @staticmethod
    def set1D_v2(stream, address, value, buf, length):
        if np.asarray(value).dtype == np.int8:
            a, p = _arr(value, np.int8)
            _ck(_lib().alpha_rt_set1D_bytes(stream, address, p, length, _staging(buf)))
        else:
            Cuda._set(stream, address, value, np.float32, (length,), buf)

    @staticmethod
    def set2D_v2(stream, address, value, buf, height, width, stride):
        if np.asarray(value).dtype == np.int8:
            a, p = _arr(value, np.int8)
            _ck(_lib().alpha_rt_set2D_bytes(stream, address, p, height, width, stride, _staging(buf)))
        else:
            Cuda._set(stream, address, value, np.float32, (height, width, stride), buf)

    set1D_int = staticmethod(lambda s, a, value, length: Cuda._set(s, a, value, np.int32, (length,), 0))
    set2D_int = staticmethod(lambda s, a, value, h, w, st: Cuda._set(s, a, value, np.int32, (h, w, st), 0))
    set1D_v2_int = staticmethod(lambda s, a, value, buf, length: Cuda._set(s, a, value, np.int32, (length,), buf))
    set2D_v2_int = staticmethod(lambda s, a, value, buf, h, w, st: Cuda._set(s, a, value, np.int32, (h, w, st), buf))
    set1D_char = staticmethod(lambda s, a, value, length: Cuda._set(s, a, value, np.int8, (length,), 0))
    set2D_char = staticmethod(lambda s, a, value, h, w, st: Cuda._set(s, a, value, np.int8, (h, w, st), 0))
    set1D_v2_char = staticmethod(lambda s, a, value, buf, length: Cuda._set(s, a, value, np.int8, (length,), buf))
    set2D_v2_char = staticmethod(lambda s, a, value, buf, h, w, st: Cuda._set(s, a, value, np.int8, (h, w, st), buf))

    @staticmethod
    def set2D_v2_char_W3S4(stream, address, value, buf1, buf2, height):
        a, p = _arr(value, np.int8)
        _ck(_lib().alpha_rt_set2D_char_W3S4(stream, address, p, _P(buf1), _P(buf2), height))

    setFrom1Dto2D = staticmethod(lambda s, src, n, dst, h, w, st: _ck(_lib().alpha_rt_setFrom1Dto2D(s, src, n, dst, h, w, st)))
    setFrom2Dto1D = staticmethod(lambda s, src, h, w, st, dst, n: _ck(_lib().alpha_rt_setFrom2Dto1D(s, src, h, w, st, dst, n)))
    setFrom2Dto2D = staticmethod(
        lambda s, src, h, w, st, dst, dh, dw, dst_stride: _ck(_lib().alpha_rt_setFrom2Dto2D(s, src, h, w, st, dst, dh, dw, dst_stride)))


class DeviceProperties(ctypes.Structure):
    """alpha_device_properties of include/alpha_rt.h (member for member)."""
    _I3, _I2 = ctypes.c_int * 3, ctypes.c_int * 2
    _fields_ = (
        [("name", ctypes.c_char * 256), ("uuid", ctypes.c_ubyte * 16), ("luid", ctypes.c_ubyte * 8)]
        + [(n, _I) for n in ("luidDeviceNodeMask", "major", "minor", "pciBusID", "pciDeviceID", "pciDomainID", "multiGpuBoardGroupID",
                             "computeMode", "deviceOverlap", "integrated", "kernelExecTimeoutEnabled", "unifiedAddressing",
                             "canMapHostMemory", "canUseHostPointerForRegisteredMem", "directManagedMemAccessFromHost",
                             "concurrentKernels", "ECCEnabled", "tccDriver", "streamPrioritiesSupported", "globalL1CacheSupported",
                             "localL1CacheSupported", "managedMemory", "multiGpuBoard", "hostNativeAtomicSupported",
                             "pageableMemoryAccess", "cooperativeLaunch", "concurrentManagedAccess", "computePreemptionSupported",
                             "clockRate", "memoryClockRate", "memoryBusWidth")]
        + [("totalGlobalMemory", _L), ("totalConstMemory", _L)]
        + [(n, _I) for n in ("l2CacheSize", "persistingL2CacheMaxSize", "multiProcessorCount", "asyncEngineCount")]
        + [("maxGridSize", _I3), ("singleToDoublePrecisionPerfRatio", _I), ("accessPolicyMaxWindowSize", _I), ("memoryPitch", _L),
           ("maxThreadsPerMultiProcessor", _I), ("sharedMemPerMultiprocessor", _L), ("regsPerMultiprocessor", _I),
           ("maxBlocksPerMultiProcessor", _I), ("sharedMemPerBlock", _L), ("reservedSharedMemPerBlock", _L),
           ("sharedMemPerBlockOptin", _L), ("regsPerBlock", _I), ("maxThreadsPerBlock", _I), ("maxThreadsDim", _I3), ("warpSize", _I),
           ("textureAlignment", _L), ("texturePitchAlignment", _L), ("maxTexture1D", _I), ("maxTexture1DMipmap", _I),
           ("maxTexture1DLinear", _I), ("maxTexture2D", _I2), ("maxTexture2DMipmap", _I2), ("maxTexture2DLinear", _I3),
           ("maxTexture2DGather", _I2), ("maxTexture3D", _I3), ("maxTexture3DAlt", _I3), ("maxTexture1DLayered", _I2),
           ("maxTexture2DLayered", _I3), ("maxTextureCubemapLayered", _I2), ("surfaceAlignment", _L), ("maxSurface1D", _I),
           ("maxSurface2D", _I2), ("maxSurface3D", _I3), ("maxSurface1DLayered", _I2), ("maxSurface2DLayered", _I3),
           ("maxSurfaceCubemap", _I), ("maxSurfaceCubemapLayered", _I2)])


class CudaDevice:
    """Mirror of z.dragon.engine.cuda.impl.CudaDevice (CudaDevice.java:16-215): constructing it runs the class's one native,
    setProperty(device_id); the properties are then attributes under the Java field names (arrays as lists, the name as str)."""

    def __init__(self, device_id=None):
        self.id = Cuda.getDeviceId() if device_id is None else int(device_id)
        props = DeviceProperties()
        L = _lib()
        L.alpha_rt_getDeviceProperties.argtypes = [_I, ctypes.POINTER(DeviceProperties)]
        _ck(L.alpha_rt_getDeviceProperties(self.id, ctypes.byref(props)))
        for name, ctype in DeviceProperties._fields_:
            v = getattr(props, name)
            if name == "name":
                v = v.decode()
            elif hasattr(v, "__len__"):
                v = list(v)
            setattr(self, name, v)

    @staticmethod
    def getDevices():
        return [CudaDevice(i) for i in range(Cuda.getDeviceCount())]
