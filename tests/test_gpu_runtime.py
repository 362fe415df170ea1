"""GPU: the runtime natives (include/alpha_rt.h; the reference's class Cuda, Cuda.java:19-182) through the C ABI and,
for a sample, through their JNI symbols with a fake JNIEnv. Expected values are the definitions of the natives themselves
(copies, fills, row compaction/expansion), computed with numpy. The last test runs a convolution in which every device
address and stream handle comes from these natives, none from PyTorch."""
import ctypes

import numpy as np
import pytest

from fake_jni import FakeEnv
from oracle import oracle as O
from util import load_package

pytestmark = pytest.mark.gpu
pkg = load_package()
C = pkg.Cuda


@pytest.fixture(scope="module")
def stream():
    import torch   # only to have the process hold one HIP runtime before the library initialises it
    torch.cuda.init()
    s = C.newStream_NonBlocking()
    yield s
    C.deleteStream(s)


def test_device_stream_and_event_natives(stream):
    assert C.getDeviceCount() >= 1 and C.getDeviceId() == 0
    C.setDevice(0)
    assert C.getStreamPriorityRange() == [0, 0]
    s2 = C.newStream_Blocking(0)
    e0, e1 = C.newEvent_Default(), C.newEvent_Default()
    d = C.malloc(1 << 24)
    C.eventRecord(e0, stream)
    C.memsetAsync(stream, d, 7, 1 << 24)
    C.eventRecord(e1, stream)
    C.streamWaitEvent_default(s2, e1)
    C.streamsWaitEvent_external([s2, stream], 2, e1)
    C.eventSynchronize(e1)
    assert C.eventElapsedTime(e0, e1) >= 0.0
    C.streamSynchronize([stream, s2], 2)
    assert C.streamQuery(stream)
    assert C.streamQuery(s2) in (True, False)   # a stream that only ever waited on events: HIP may answer either
    C.eventRecord(e0, [stream, s2], 2)          # the array form synchronises the streams (reference behaviour)
    for e in (e0, e1, C.newEvent_BlockingSync(), C.newEvent_DisableTiming(), C.newEvent_Interprocess()):
        C.deleteEvent(e)
    C.deleteStream([s2, 0], 2)                  # a zero handle is skipped
    C.free(d)
    assert C.getExceptionName(0) == "hipSuccess" and "memory" in C.getExceptionInfo(2).lower()
    assert C.getLastExceptionType() == 0
    with pytest.raises(pkg.AlphaConvError):
        C.memsetAsync(stream, d, 0, -1)


def test_memcpy_and_memset_natives(stream):
    n = 1000
    src = np.arange(n, dtype=np.float32)
    pin, pin2 = C.mallocHost(4 * n), C.mallocHost(4 * n)
    d0, d1 = C.malloc(4 * n), C.malloc(4 * n + 3)
    ctypes.memmove(pin, src.ctypes.data, 4 * n)
    C.memcpyAsyncHostToDevice(stream, d0, pin, 4 * n)
    C.memcpyAsyncDeviceToDevice(stream, d1, d0, 4 * n)
    C.memsetAsync(stream, d0, 0, 4 * n)                     # word path
    C.memsetAsync(stream, d1 + 4 * n, 0x5A, 3)              # byte path (3 trailing bytes)
    C.memcpyAsyncDeviceToHost(stream, pin2, d1, 4 * n)
    C.streamSynchronize(stream)
    back = np.empty(n, np.float32)
    ctypes.memmove(back.ctypes.data, pin2, 4 * n)
    assert np.array_equal(back, src)
    C.memcpyAsyncDefault(stream, pin2, d0, 4 * n)
    C.memcpyAsyncHostToHost(stream, pin, pin2, 4 * n)
    C.streamSynchronize(stream)
    ctypes.memmove(back.ctypes.data, pin, 4 * n)
    assert not back.any()
    tail = np.empty(3, np.int8)
    C.get1D_char(stream, d1 + 4 * n, tail, 3)
    assert (tail == 0x5A).all()
    for p in (pin, pin2):
        C.freeHost(p)
    for p in (d0, d1):
        C.free(p)


@pytest.mark.parametrize("dtype,setter1,setter2,getter1,getter2", [
    (np.float32, "set1D", "set2D", "get1D", "get2D"),
    (np.int32, "set1D_int", "set2D_int", "get1D_int", "get2D_int"),
    (np.int8, "set1D_char", "set2D_char", "get1D_char", "get2D_char"),
])
@pytest.mark.parametrize("v2", [False, True])
def test_array_natives_1D_and_2D(stream, dtype, setter1, setter2, getter1, getter2, v2):
    rng = np.random.default_rng(7)
    h, w, st = 37, 3, 4                       # 3 logical channels stored with stride 4, as the engine stores them
    item = np.dtype(dtype).itemsize
    dense = rng.integers(-100, 100, (h, w)).astype(dtype)
    dev = C.malloc(h * st * item)
    buf = C.mallocHost(h * st * item) if v2 else 0
    sfx = "_v2" if v2 else ""

    def call(name, *args):
        base, _, kind = name.partition("_")          # get2D_int -> get2D_v2_int
        full = base + sfx + ("_" + kind if kind else "")
        a = list(args)
        if v2:
            a.insert(3, buf)
        getattr(C, full)(*a)

    call(setter2, stream, dev, dense, h, w, st)
    raw = np.empty(h * st, dtype)
    call(getter1, stream, dev, raw, h * st)
    want = np.zeros((h, st), dtype)
    want[:, :w] = dense
    assert np.array_equal(raw.reshape(h, st), want), "set2D expands rows and zeroes the padding"
    out = np.empty((h, w), dtype)
    call(getter2, stream, dev, out, h, w, st)
    assert np.array_equal(out, dense), "get2D compacts rows"
    flat = rng.integers(-100, 100, h * st).astype(dtype)
    call(setter1, stream, dev, flat, h * st)
    call(getter1, stream, dev, raw, h * st)
    assert np.array_equal(raw, flat)
    C.free(dev)
    if buf:
        C.freeHost(buf)


def test_fills_byte_conversion_and_restrides(stream):
    h, w, st = 50, 6, 8
    dev, dev2, dev1d = C.malloc(4 * h * st), C.malloc(4 * h * 12), C.malloc(4 * h * w)
    raw = np.empty(h * st, np.float32)
    C.set1D(stream, dev, 2.5, h * st)
    C.get1D(stream, dev, raw, h * st)
    assert (raw == 2.5).all()
    C.set2D(stream, dev, -1.25, h, w, st)
    C.get1D(stream, dev, raw, h * st)
    want = np.zeros((h, st), np.float32)
    want[:, :w] = -1.25
    assert np.array_equal(raw.reshape(h, st), want), "set2D(value): value in the data columns, zero in the padding"
    b = np.random.default_rng(3).integers(-128, 128, (h, w)).astype(np.int8)
    C.set2D(stream, dev, b, h, w, st)            # byte[] -> float tensor
    out = np.empty((h, w), np.float32)
    C.get2D(stream, dev, out, h, w, st)
    assert np.array_equal(out, b.astype(np.float32))
    pin = C.mallocHost(4 * h * w)
    C.set1D_v2(stream, dev1d, b.reshape(-1), pin, h * w)
    flat = np.empty(h * w, np.float32)
    C.get1D(stream, dev1d, flat, h * w)
    assert np.array_equal(flat, b.reshape(-1).astype(np.float32))
    # device-side re-strides: dense -> (w, st) -> (w2 = 10, st2 = 12) -> dense, with h*w = h2*w2
    C.set1D(stream, dev, 0.0, h * st)
    C.setFrom1Dto2D(stream, dev1d, h * w, dev, h, w, st)
    C.get2D(stream, dev, out, h, w, st)
    assert np.array_equal(out.reshape(-1), flat)
    h2, w2, st2 = h * w // 10, 10, 12
    C.setFrom2Dto2D(stream, dev, h, w, st, dev2, h2, w2, st2)
    out2 = np.empty((h2, w2), np.float32)
    C.get2D(stream, dev2, out2, h2, w2, st2)
    assert np.array_equal(out2.reshape(-1), flat)
    C.set1D(stream, dev1d, 0.0, h * w)
    C.setFrom2Dto1D(stream, dev2, h2, w2, st2, dev1d, h * w)
    back = np.empty(h * w, np.float32)
    C.get1D(stream, dev1d, back, h * w)
    assert np.array_equal(back, flat)
    # pictures: rows of 3 bytes stored with stride 4
    px = np.random.default_rng(4).integers(-128, 128, (h, 3)).astype(np.int8)
    b1, b2, dpx = C.mallocHost(h * 3), C.mallocHost(h * 4), C.malloc(h * 4)
    C.set2D_v2_char_W3S4(stream, dpx, px, b1, b2, h)
    got = np.empty(h * 4, np.int8)
    C.get1D_char(stream, dpx, got, h * 4)
    wantpx = np.zeros((h, 4), np.int8)
    wantpx[:, :3] = px
    assert np.array_equal(got.reshape(h, 4), wantpx)
    for p in (pin, b1, b2):
        C.freeHost(p)
    for p in (dev, dev2, dev1d, dpx):
        C.free(p)


def test_jni_symbols_of_the_runtime_class(stream):
    env = FakeEnv()
    L, I, P, F = ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p, ctypes.c_float
    lib = pkg.lib()

    def jni(name, restype, *argtypes):
        fn = getattr(lib, "Java_z_dragon_engine_cuda_impl_Cuda_" + name)
        fn.restype, fn.argtypes = restype, [P, P] + list(argtypes)
        return lambda *a: fn(env.ptr, None, *a)

    n = 19
    dev = jni("malloc", L, L)(4 * n * 4)
    assert dev != 0 and not env.thrown
    vals = [float(i) - 3.5 for i in range(n * 3)]
    arr = env.array(vals)
    jni("set2D__JJ_3FIII", None, L, L, P, I, I, I)(stream, dev, arr, n, 3, 4)      # float[] -> rows of stride 4
    out = env.array([0.0] * (n * 4))
    jni("get1D", None, L, L, P, I)(stream, dev, out, n * 4)
    got = np.array(env.arrays[out.value]).reshape(n, 4)
    assert np.array_equal(got[:, :3].reshape(-1), np.array(vals)) and not got[:, 3].any()
    ints = env.array(list(range(-5, 7)))
    jni("set1D_1int", None, L, L, P, I)(stream, dev, ints, 12)
    iout = env.array([0] * 12)
    jni("get1D_1int", None, L, L, P, I)(stream, dev, iout, 12)
    assert env.arrays[iout.value] == list(range(-5, 7))
    rng = jni("getStreamPriorityRange", P)()
    assert env.arrays[rng] == [0, 0]
    name = jni("getExceptionName", P, I)(1)
    assert env.strings[name] == "hipErrorInvalidValue"
    s2 = jni("newStream_1Blocking__I", L, I)(0)
    jni("streamSynchronize___3JI", None, P, I)(env.long_array([stream, s2]), 2)
    jni("deleteStream__J", None, L)(s2)
    assert not env.thrown
    jni("memsetAsync", None, L, L, I, L)(stream, dev, 0, -4)                         # negative size -> Java exception
    assert env.thrown and env.thrown[0][0] == "z/dragon/engine/cuda/impl/CudaException" and "negative" in env.thrown[0][1]
    jni("free", None, L)(dev)


def test_convolution_with_addresses_and_streams_from_these_natives(stream):
    """BASELINE config 1 geometry (3 channels stored as 4) end to end through this library alone."""
    N, IH, IW, ICl, IC, OC = 4, 32, 32, 3, 4, 64
    rng = np.random.default_rng(11)
    X3 = rng.uniform(-1, 1, (N * IH * IW, ICl)).astype(np.float32)
    W3 = rng.uniform(-1, 1, (OC * 9, ICl)).astype(np.float32)
    dX, dW, dY = C.malloc(4 * N * IH * IW * IC), C.malloc(4 * OC * 9 * IC), C.malloc(4 * N * IH * IW * OC)
    C.set2D(stream, dX, X3, N * IH * IW, ICl, IC)       # the engine's own way of padding channels: width 3, stride 4
    C.set2D(stream, dW, W3, OC * 9, ICl, IC)
    pkg.Cuda_conv3D.conv3D([stream], 1, dX, IH, IW, dW, 3, 3, dY, IH, IW, N, IC, OC, 1, 1, 1, 1)
    Y = np.empty((N * IH * IW, OC), np.float32)
    C.get2D(stream, dY, Y, N * IH * IW, OC, OC)
    X4 = np.zeros((N, IH, IW, IC), np.float32)
    X4[..., :ICl] = X3.reshape(N, IH, IW, ICl)
    W4 = np.zeros((OC, 3, 3, IC), np.float32)
    W4[..., :ICl] = W3.reshape(OC, 3, 3, ICl)
    want = O.conv3D_f64(X4, W4, 1, 1, 1, 1)
    r = O.max_err_ratio(Y.reshape(N, IH, IW, OC), want, 1e-4, 1e-5 * max(1.0, float(np.sqrt(np.mean(want * want)))))
    assert r <= 1.0, "err/allowed = %.3f" % r
    for p in (dX, dW, dY):
        C.free(p)
