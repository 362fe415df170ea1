"""The JNI layer: every `static native` method of the reference's three conv classes resolves to an
exported symbol with the JNI-mangled name, and the stubs drive the C ABI through a fake JNIEnv
(stream-array copy, error -> Java exception). There is no JVM in this environment, so this proves the
shim's self-consistency with the JNI specification's table layout, not execution inside a real JVM."""
import ctypes
import subprocess

import numpy as np
import pytest

from fake_jni import FakeEnv
from util import load_package

pkg = load_package()

# `static native` method names as declared in the reference's Java classes
NATIVES = {
    "Cuda_conv3D": ["conv3D", "conv3D_texture", "conv3DV2", "conv3D_np", "conv3D_W1", "kernel_remode", "conv3D_GemmR",
                    "conv3D_GemmR_texture", "conv3D_GemmV2R", "conv3D_GemmR_W1"],
    "Cuda_dconv3D_deltaX": ["dconv3D_deltaX_s1", "dconv3D_deltaX_s1_texture", "dconv3D_deltaX_V2_s1", "dconv3D_deltaX_W1",
                            "ks_remode", "ks_remodev2", "dconv3D_deltaX_kernelSplit", "dconv3D_deltaX_ksImsR",
                            "dconv3D_deltaX_ksImsR_texture", "dconv3D_deltaX_ksIms2R", "dconv3D_deltaX_ksIms2R_texture",
                            "dconv3D_deltaX_ksV2_Ims2R", "dconv3D_deltaX_crossAdd"],
    "Cuda_dconv3D_deltaW": ["dconv3D_deltaW", "dconv3D_deltaW_W1", "buf_summary", "dconv3D_deltaW_GemmSK",
                            "dconv3D_deltaW_GemmV2SK", "dconv3D_deltaW_GemmSK_W1"],
}


def mangle(cls, method):
    esc = lambda s: s.replace("_", "_1")
    return "Java_z_dragon_engine_cuda_impl_math_%s_%s" % (esc(cls), esc(method))


def test_all_29_jni_symbols_exported():
    out = subprocess.check_output(["nm", "-D", "--defined-only", pkg.lib_path()], text=True)
    exported = {l.split()[-1] for l in out.splitlines() if " T " in l}
    want = [mangle(c, m) for c, ms in NATIVES.items() for m in ms]
    assert len(want) == 29
    assert not [w for w in want if w not in exported]
    assert len([e for e in exported if e.startswith("Java_z_dragon_engine_cuda_impl_math_")]) == 29   # nothing extra either


def _jni(name):
    return getattr(pkg.lib(), name)


def test_error_becomes_java_exception_and_streams_are_copied():
    env = FakeEnv()
    fn = _jni(mangle("Cuda_conv3D", "conv3D"))
    fn.restype = None
    L, I, P = ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p
    fn.argtypes = [P, P, P, I, L, I, I, L, I, I, L, I, I, I, I, I, I, I, I, I]
    arr = env.long_array([0, 0, 0])
    # IC = 6 is not a multiple of 4 -> the C ABI refuses before touching the GPU -> ThrowNew(CudaException)
    fn(env.ptr, None, arr, 3, 256, 8, 8, 256, 3, 3, 256, 8, 8, 4, 6, 8, 1, 1, 1, 1)
    assert env.thrown and env.thrown[0][0] == "z/dragon/engine/cuda/impl/CudaException"
    assert "multiples of 4" in env.thrown[0][1]
    # class lookup falls back when the engine's class is absent
    env2 = FakeEnv(known_classes=("java/lang/RuntimeException",))
    fn(env2.ptr, None, env2.long_array([0]), 1, 256, 8, 8, 256, 3, 3, 256, 8, 8, 4, 6, 8, 1, 1, 1, 1)
    assert env2.find_calls == ["z/dragon/engine/cuda/impl/CudaException", "z/jcuda/exception/CudaException",
                               "java/lang/RuntimeException"]
    assert env2.cleared == 2 and env2.thrown[0][0] == "java/lang/RuntimeException"
    assert env2.calls_while_pending == []   # each failed FindClass is cleared before the next JNI call
    # an empty stream array is refused, not dereferenced
    env3 = FakeEnv()
    fn(env3.ptr, None, env3.long_array([]), 0, 256, 8, 8, 256, 3, 3, 256, 8, 8, 4, 4, 8, 1, 1, 1, 1)
    assert "stream" in env3.thrown[0][1]


@pytest.mark.gpu
def test_forward_through_jni_symbols_on_gpu():
    from oracle import oracle as O
    from util import Dev, he_normal, uniform
    dev = Dev()
    N, IH, IW, IC, OC, F_ = 4, 12, 12, 16, 40, 3
    X, W = uniform((N, IH, IW, IC), 5001), he_normal(OC, F_, F_, IC, 5002)
    x, w = dev.put(X), dev.put(W)
    cw = dev.empty(F_ * F_ * IC * OC, fill=float("nan"))
    y = dev.empty(N, IH, IW, OC, fill=float("nan"))
    env = FakeEnv()
    L, I, P, Z = ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p, ctypes.c_uint8
    remode = _jni(mangle("Cuda_conv3D", "kernel_remode"))
    remode.restype, remode.argtypes = None, [P, P, L, L, L, I, I, I, I]
    remode(env.ptr, None, dev.stream, w.data_ptr(), cw.data_ptr(), F_, F_, OC, IC)
    conv = _jni(mangle("Cuda_conv3D", "conv3D_GemmV2R"))
    conv.restype = None
    conv.argtypes = [P, P, Z, P, I, L, I, I, L, L, I, I, L, I, I, I, I, I, I, I, I, I]
    streams = env.long_array([dev.stream] * 3)
    conv(env.ptr, None, 1, streams, 3, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), F_, F_, y.data_ptr(), IH, IW,
         N, IC, OC, 1, 1, 1, 1)
    assert not env.thrown
    want = O.conv3D_f64(X, W, 1, 1, 1, 1)
    floor = 1e-5 * max(1.0, float(np.sqrt(np.mean(want * want))))
    assert O.max_err_ratio(dev.get(y), want, 1e-4, floor) <= 1.0


def test_runtime_class_stubs_that_need_no_device():
    """Natives of the runtime class (Cuda.java:19-182) whose answer does not depend on a GPU: argument validation throws
    the Java exception, error names and the priority range come back as a jstring and an int[2]."""
    env = FakeEnv()
    L, I, P = ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p
    lib = pkg.lib()

    def jni(name, restype, *argtypes):
        fn = getattr(lib, "Java_z_dragon_engine_cuda_impl_Cuda_" + name)
        fn.restype, fn.argtypes = restype, [P, P] + list(argtypes)
        return lambda *a: fn(env.ptr, None, *a)

    jni("memsetAsync", None, L, L, I, L)(0, 0, 0, -4)
    assert env.thrown == [("z/dragon/engine/cuda/impl/CudaException", "alpha-rt-hip error 1: alpha_rt_memsetAsync: negative size")]
    assert env.strings[jni("getExceptionName", P, I)(1)] == "hipErrorInvalidValue"
    assert env.strings[jni("getExceptionInfo", P, I)(2)] == "out of memory"
    assert env.arrays[jni("getStreamPriorityRange", P)()] == [0, 0]
    jni("deleteStream__J", None, L)(0)                      # a zero handle is skipped without touching the device
    jni("deleteStream___3JI", None, P, I)(env.long_array([0, 0]), 2)
    assert len(env.thrown) == 1


# ---- CudaDevice.setProperty -------------------------------------------------------------------------------------------
# the fields of the reference's class z.dragon.engine.cuda.impl.CudaDevice that its native fills (CudaDevice.java:31-215),
# with their JNI signatures
DEVICE_FIELDS = dict(
    [("name", "Ljava/lang/String;"), ("uuid", "[B"), ("luid", "[B")]
    + [(n, "I") for n in ("luidDeviceNodeMask", "major", "minor", "pciBusID", "pciDeviceID", "pciDomainID", "multiGpuBoardGroupID",
                          "computeMode", "clockRate", "memoryClockRate", "memoryBusWidth", "l2CacheSize", "persistingL2CacheMaxSize",
                          "multiProcessorCount", "asyncEngineCount", "singleToDoublePrecisionPerfRatio", "accessPolicyMaxWindowSize",
                          "maxThreadsPerMultiProcessor", "regsPerMultiprocessor", "maxBlocksPerMultiProcessor", "regsPerBlock",
                          "maxThreadsPerBlock", "warpSize", "maxTexture1D", "maxTexture1DMipmap", "maxTexture1DLinear", "maxSurface1D",
                          "maxSurfaceCubemap")]
    + [(n, "Z") for n in ("deviceOverlap", "integrated", "kernelExecTimeoutEnabled", "unifiedAddressing", "canMapHostMemory",
                          "canUseHostPointerForRegisteredMem", "directManagedMemAccessFromHost", "concurrentKernels", "ECCEnabled",
                          "tccDriver", "streamPrioritiesSupported", "globalL1CacheSupported", "localL1CacheSupported", "managedMemory",
                          "multiGpuBoard", "hostNativeAtomicSupported", "pageableMemoryAccess", "cooperativeLaunch",
                          "concurrentManagedAccess", "computePreemptionSupported")]
    + [(n, "J") for n in ("totalGlobalMemory", "totalConstMemory", "memoryPitch", "sharedMemPerMultiprocessor", "sharedMemPerBlock",
                          "reservedSharedMemPerBlock", "sharedMemPerBlockOptin", "textureAlignment", "texturePitchAlignment",
                          "surfaceAlignment")]
    + [(n, "[I") for n in ("maxGridSize", "maxThreadsDim", "maxTexture2D", "maxTexture2DMipmap", "maxTexture2DLinear",
                           "maxTexture2DGather", "maxTexture3D", "maxTexture3DAlt", "maxTexture1DLayered", "maxTexture2DLayered",
                           "maxTextureCubemapLayered", "maxSurface2D", "maxSurface3D", "maxSurface1DLayered", "maxSurface2DLayered",
                           "maxSurfaceCubemapLayered")])


def _known_properties():
    """A struct in which every member holds a different value."""
    P = pkg.runtime.DeviceProperties
    props, want = P(), {}
    k = 100
    for name, ctype in P._fields_:
        if name == "name":
            props.name = b"fake device gfx950"
            want[name] = "fake device gfx950"
        elif name in ("uuid", "luid"):
            vals = [(k + 7 * i) % 127 for i in range(len(getattr(props, name)))]
            for i, v in enumerate(vals):
                getattr(props, name)[i] = v
            want[name] = vals
        elif hasattr(getattr(props, name), "__len__"):
            vals = [k + i for i in range(len(getattr(props, name)))]
            for i, v in enumerate(vals):
                getattr(props, name)[i] = v
            want[name] = vals
        elif DEVICE_FIELDS[name] == "Z":
            setattr(props, name, k % 2)
            want[name] = bool(k % 2)
        elif DEVICE_FIELDS[name] == "J":
            setattr(props, name, (k << 33) + 5)     # needs all 64 bits
            want[name] = (k << 33) + 5
        else:
            setattr(props, name, k)
            want[name] = k
        k += 3
    return props, want


def test_device_native_is_exported_and_the_struct_has_the_java_fields():
    out = subprocess.check_output(["nm", "-D", "--defined-only", pkg.lib_path()], text=True)
    assert "Java_z_dragon_engine_cuda_impl_CudaDevice_setProperty" in out
    assert sorted(n for n, _ in pkg.runtime.DeviceProperties._fields_) == sorted(DEVICE_FIELDS)
    assert len(DEVICE_FIELDS) == 77


def test_device_properties_reach_every_java_field_with_its_type():
    env = FakeEnv()
    obj = env.new_object(DEVICE_FIELDS)
    props, want = _known_properties()
    fn = pkg.lib().alpha_rt_selfcheck_fillDeviceObject
    fn.restype = None
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(pkg.runtime.DeviceProperties)]
    fn(env.ptr, obj, ctypes.byref(props))
    got = env.objects[obj]
    assert sorted(got) == sorted(DEVICE_FIELDS)                      # every field set ...
    assert len(env.set_calls) == len(DEVICE_FIELDS)                  # ... exactly once
    for name in DEVICE_FIELDS:
        assert got[name] == want[name], name
    # a Java class that lacks a field (an older CudaDevice): the others are still filled
    fewer = {k: v for k, v in DEVICE_FIELDS.items() if k != "maxTexture1DLinear"}
    obj2 = env.new_object(fewer)
    fn(env.ptr, obj2, ctypes.byref(props))
    assert sorted(env.objects[obj2]) == sorted(fewer)
    # the NoSuchFieldError that GetFieldID leaves pending is cleared before the next JNI call
    assert env.calls_while_pending == [] and not env.pending


@pytest.mark.gpu
def test_device_properties_of_the_real_device_through_the_jni_symbol():
    import torch
    assert torch.cuda.is_available()
    env = FakeEnv()
    obj = env.new_object(DEVICE_FIELDS)
    fn = _jni("Java_z_dragon_engine_cuda_impl_CudaDevice_setProperty")
    fn.restype = None
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32]
    fn(env.ptr, obj, 0)
    assert not env.thrown
    got = env.objects[obj]
    assert sorted(got) == sorted(DEVICE_FIELDS)
    tp = torch.cuda.get_device_properties(0)
    assert got["name"] == tp.name
    assert got["multiProcessorCount"] == tp.multi_processor_count == pkg.device_info()[0]
    assert got["totalGlobalMemory"] == tp.total_memory
    assert got["warpSize"] == 64 and (got["major"], got["minor"]) == (tp.major, tp.minor)
    assert got["maxThreadsPerBlock"] == 1024 and got["maxThreadsDim"][0] == 1024
    assert got["clockRate"] == pkg.device_info()[1]
    # the ctypes mirror of the Java class reads the same struct
    d = pkg.CudaDevice(0)
    assert (d.name, d.multiProcessorCount, d.l2CacheSize) == (got["name"], got["multiProcessorCount"], got["l2CacheSize"])
    assert len(pkg.CudaDevice.getDevices()) == pkg.Cuda.getDeviceCount()
    # an invalid device id becomes a Java exception, not a crash
    env2 = FakeEnv()
    fn(env2.ptr, env2.new_object(DEVICE_FIELDS), 99)
    assert env2.thrown and env2.thrown[0][0] == "z/dragon/engine/cuda/impl/CudaException"
