"""CPU-side checks of the drop-in boundary: the shared library loads and exports every symbol that
include/alpha_conv.h declares, the JNI symbols of the three reference classes are present, and
argument validation rejects bad calls without touching a GPU."""
import ctypes
import os
import re
import subprocess

import pytest

from util import ROOT, load_package

pkg = load_package()


def _header_functions():
    hdr = open(os.path.join(ROOT, "include", "alpha_conv.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    return sorted(set(re.findall(r"\b(alpha_\w+)\s*\(", hdr)))


def _exported():
    out = subprocess.check_output(["nm", "-D", "--defined-only", pkg.lib_path()], text=True)
    return {l.split()[-1] for l in out.splitlines() if " T " in l}


def test_library_is_built_and_loads():
    assert os.path.exists(pkg.lib_path()), "run __graft_entry__.build() first"
    assert pkg.lib().alpha_conv_version().decode().startswith("alpha-conv-hip")


def test_every_declared_symbol_is_exported():
    declared = _header_functions()
    assert len(declared) >= 35
    exported = _exported()
    missing = [f for f in declared if f not in exported]
    assert not missing, missing
    assert sorted(pkg.exported_symbols()) == declared  # the ctypes mirror binds exactly the header


def test_runtime_header_symbols_and_jni_names():
    """include/alpha_rt.h: every declared function is exported, and so is every native of the reference's runtime class
    Cuda under its JNI long name (overloads carry their signature, as in the reference's Cuda_Stream.cuh / Cuda_float.cuh)."""
    hdr = open(os.path.join(ROOT, "include", "alpha_rt.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = sorted(set(re.findall(r"\b(alpha_rt_\w+)\s*\(", hdr)))
    assert len(declared) >= 55
    exported = _exported()
    assert not [f for f in declared if f not in exported]
    P = "Java_z_dragon_engine_cuda_impl_Cuda_"
    natives = ["malloc", "free", "mallocHost", "freeHost", "memsetAsync", "memcpyAsyncHostToDevice", "memcpyAsyncHostToHost",
               "memcpyAsyncDeviceToHost", "memcpyAsyncDeviceToDevice", "memcpyAsyncDefault", "getDeviceId", "getDeviceCount",
               "setDevice", "resetDevice", "deviceSynchronize", "isDeviceP2PAccessEnabled", "enableDeviceP2PAccess",
               "disableDeviceP2PAccess", "getStreamPriorityRange", "newStream_1Blocking__", "newStream_1Blocking__I",
               "newStream_1NonBlocking__", "newStream_1NonBlocking__I", "deleteStream__J", "deleteStream___3JI", "streamQuery",
               "streamSynchronize__J", "streamSynchronize___3JI", "newEvent_1Default", "newEvent_1BlockingSync",
               "newEvent_1DisableTiming", "newEvent_1Interprocess", "deleteEvent", "eventRecord__JJ", "eventRecord__J_3JI",
               "eventSynchronize", "eventElapsedTime", "streamWaitEvent_1default", "streamWaitEvent_1external",
               "streamsWaitEvent_1default", "streamsWaitEvent_1external", "getExceptionName", "getExceptionInfo",
               "getLastExceptionType", "get1D", "get2D", "get1D_1v2", "get2D_1v2", "set1D__JJFI", "set2D__JJFIII",
               "set1D__JJ_3BI", "set1D__JJ_3FI", "set1D_1v2__JJ_3BJI", "set1D_1v2__JJ_3FJI", "set2D__JJ_3BIII", "set2D__JJ_3FIII",
               "set2D_1v2__JJ_3BJIII", "set2D_1v2__JJ_3FJIII", "setFrom1Dto2D", "setFrom2Dto1D", "setFrom2Dto2D",
               "get1D_1int", "get2D_1int", "get1D_1v2_1int", "get2D_1v2_1int", "set1D_1int", "set2D_1int", "set1D_1v2_1int",
               "set2D_1v2_1int", "get1D_1char", "get2D_1char", "get1D_1v2_1char", "get2D_1v2_1char", "set1D_1char", "set2D_1char",
               "set1D_1v2_1char", "set2D_1v2_1char", "set2D_1v2_1char_1W3S4"]
    assert len(natives) == 78
    assert not [n for n in natives if P + n not in exported]


def test_argument_validation_without_gpu():
    L = pkg.lib()
    one = (ctypes.c_int64 * 1)(0)
    p = ctypes.c_void_p(256)
    # IC not a multiple of 4
    rc = L.alpha_conv3D(one, 1, p, 8, 8, p, 3, 3, p, 8, 8, 4, 6, 8, 1, 1, 1, 1)
    assert rc == 10001 and b"multiples of 4" in L.alpha_conv_last_error()
    # empty stream array
    rc = L.alpha_conv3D(one, 0, p, 8, 8, p, 3, 3, p, 8, 8, 4, 4, 8, 1, 1, 1, 1)
    assert rc == 10001 and b"stream" in L.alpha_conv_last_error()
    # null / misaligned pointer
    rc = L.alpha_conv3D(one, 1, ctypes.c_void_p(4), 8, 8, p, 3, 3, p, 8, 8, 4, 4, 8, 1, 1, 1, 1)
    assert rc == 10001
    rc = L.alpha_dconv3D_deltaW_GemmSK(one, 1, 4, p, 8, 8, p, 8, 8, p, None, 3, 3, 4, 4, 8, 1, 1, 1, 1)
    assert rc == 10001 and b"deltaW_buf" in L.alpha_conv_last_error()
    with pytest.raises(pkg.AlphaConvError):
        pkg.Cuda_conv3D.kernel_remode(0, 0, 0, 3, 3, 8, 4)
    # an output whose windows leave the padded input is refused at the C ABI too; a smaller one than the formula's is not
    # a size error (the call then fails later, on the null stream array of this test, not on the sizes)
    rc = L.alpha_conv3D(one, 1, p, 8, 8, p, 3, 3, p, 9, 8, 4, 4, 8, 1, 1, 1, 1)
    assert rc == 10001 and b"does not fit" in L.alpha_conv_last_error()
    rc = L.alpha_dconv3D_deltaX_s1(one, 1, p, 8, 12, p, 3, 3, p, 8, 8, 4, 4, 8, 1, 1)
    assert rc == 10001 and b"does not fit" in L.alpha_conv_last_error()
    rc = L.alpha_dconv3D_deltaW_GemmSK(one, 1, 2, p, 8, 8, p, 5, 5, p, p, 3, 3, 4, 4, 8, 2, 2, 1, 1)
    assert rc == 10001 and b"does not fit" in L.alpha_conv_last_error()


def _tap_filter_extent(AC, CO, TH, TW, b_off, b_sth, b_stw, b_sc):
    L = pkg.lib()
    fn = L.alpha_selfcheck_tap_filter_extent
    fn.argtypes = [ctypes.c_int] * 8 + [ctypes.POINTER(ctypes.c_long)] * 2
    fn.restype = ctypes.c_int
    lo, hi = ctypes.c_long(), ctypes.c_long()
    assert fn(AC, CO, TH, TW, b_off, b_sth, b_stw, b_sc, ctypes.byref(lo), ctypes.byref(hi)) == 0
    return lo.value, hi.value


@pytest.mark.parametrize("AC", [32, 36, 64, 68, 80, 92, 96, 100, 128, 160, 196])
@pytest.mark.parametrize("CO", [4, 20, 64, 100])
@pytest.mark.parametrize("TH,TW", [(3, 3), (5, 3), (2, 2), (7, 7), (1, 1)])
def test_tap_conv_filter_loads_stay_inside_the_filter(AC, CO, TH, TW):
    """The library walks the filter addresses of the LDS-halo kernel with the kernel's own address functions
    (same loop structure: the second half tap of every tap and the prefetch of the next). Every element index must lie
    inside the filter for both layouts the kernel is given: CW[TH,TW,AC,CO] (forward) and W[AC,TH,TW,CO] read in place
    with rotated taps (backward-data: reduced channel = OC of W, produced channel = IC of W). Channel counts with
    AC % 64 in [4, 32] are the ones whose last pass has an all-masked second half tap."""
    size = TH * TW * AC * CO
    lo, hi = _tap_filter_extent(AC, CO, TH, TW, 0, TW * AC * CO, AC * CO, CO)
    assert 0 <= lo and hi < size, ("CW", lo, hi, size)
    lo, hi = _tap_filter_extent(AC, CO, TH, TW, ((TH - 1) * TW + (TW - 1)) * CO, -TW * CO, -CO, TH * TW * CO)
    assert 0 <= lo and hi < size, ("W rotated", lo, hi, size)
    if AC % 64 == 0 and CO % 64 == 0:   # nothing is masked or clamped: the walk touches the first and the last element
        assert (lo, hi) == (0, size - 1)
