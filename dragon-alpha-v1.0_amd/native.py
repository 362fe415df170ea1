"""ctypes mirror of the reference's JNI native classes over the C ABI (include/alpha_conv.h).

Class and method names, argument order and meaning follow
  src/alpha_src/z/dragon/engine/cuda/impl/math/Cuda_conv3D.java           (natives at :240-766)
  src/alpha_src/z/dragon/engine/cuda/impl/math/Cuda_dconv3D_deltaX.java   (natives at :311-980)
  src/alpha_src/z/dragon/engine/cuda/impl/math/Cuda_dconv3D_deltaW.java   (natives at :243-472)
Addresses are plain integers (device pointers / hipStream_t handles), exactly like the jlong
arguments of the Java side. Where the Java natives return void and throw on error, these raise
AlphaConvError.
"""
import ctypes
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_NAME = "libalpha_conv_hip.so"
_lib = None

_I = ctypes.c_int
_L = ctypes.c_int64
_P = ctypes.c_void_p
_S = ctypes.POINTER(ctypes.c_int64)

# signature strings: S = stream array, i = int, p = device pointer, l = int64 handle
_SIGS = {
    "alpha_conv3D": "sipiipiipiiiiiiiii",
    "alpha_conv3D_texture": "sipiipiipiiiiiiiii",
    "alpha_conv3DV2": "isipiipiipiiiiiiiii",
    "alpha_conv3D_np": "sipiipiipiiiiiii",
    "alpha_conv3D_W1": "sipiippiii",
    "alpha_kernel_remode": "lppiiii",
    "alpha_conv3D_GemmR": "sipiippiipiiiiiiiii",
    "alpha_conv3D_GemmR_texture": "sipiippiipiiiiiiiii",
    "alpha_conv3D_GemmV2R": "isipiippiipiiiiiiiii",
    "alpha_conv3D_GemmR_W1": "sipiipppiii",
    "alpha_dconv3D_deltaX_s1": "sipiipiipiiiiiii",
    "alpha_dconv3D_deltaX_s1_texture": "sipiipiipiiiiiii",
    "alpha_dconv3D_deltaX_V2_s1": "isipiipiipiiiiiii",
    "alpha_dconv3D_deltaX_W1": "sipppiiiii",
    "alpha_ks_remode": "lpiipiiiiii",
    "alpha_ks_remodev2": "lpiipiiiiii",
    "alpha_dconv3D_deltaX_kernelSplit": "sipiipiipiiiiiiiii",
    "alpha_dconv3D_deltaX_ksImsR": "sipiipiipiiiiiiiii",
    "alpha_dconv3D_deltaX_ksImsR_texture": "sipiipiipiiiiiiiii",
    "alpha_dconv3D_deltaX_ksIms2R": "sipiipiipiiiiiii",
    "alpha_dconv3D_deltaX_ksIms2R_texture": "sipiipiipiiiiiii",
    "alpha_dconv3D_deltaX_ksV2_Ims2R": "isipiipiipiiiiiii",
    "alpha_dconv3D_deltaX_crossAdd": "sipiipiipiiiiiiiii",
    "alpha_dconv3D_deltaW": "sipiipiipiiiiiiiii",
    "alpha_dconv3D_deltaW_W1": "sipiippiii",
    "alpha_buf_summary": "lppii",
    "alpha_dconv3D_deltaW_GemmSK": "siipiipiippiiiiiiiii",
    "alpha_dconv3D_deltaW_GemmV2SK": "siipiipiippiiiiiiiii",
    "alpha_dconv3D_deltaW_GemmSK_W1": "siipiipppiii",
    "alpha_dconv3D_deltaW_GemmSK_static": "siipiipiipiiiiiiiii",
    "alpha_winograd_filter_transform": "lppii",
    "alpha_conv3D_winograd": "sipiippiiiiiii",
    "alpha_winograd_filter_transform_deltaX": "lppii",
    "alpha_dconv3D_deltaW_GemmSK_winograd": "siipiipiippiiiii",
    "alpha_dconv3D_deltaX_winograd": "sipiippiiiiiii",
    "alpha_dconv3D_deltaW_GemmSK_deltaB": "siipiipiippppiiiiiiiii",
    "alpha_conv3D_biased": "sipiipiippiiiiiiiii",
    "alpha_conv3D_GemmR_biased": "sipiippiippiiiiiiiii",
    "alpha_conv3D_winograd_biased": "sipiipppiiiiiii",
    "alpha_conv3D_fused": "sipiipiiepiiiiiiiii",
    "alpha_conv3D_GemmR_fused": "sipiippiiepiiiiiiiii",
    "alpha_conv3D_winograd_fused": "sipiipepiiiiiii",
    "alpha_dconv3D_deltaX_s1_leakyRelu": "sipiipiipfpiiiiiii",
    "alpha_dconv3D_deltaX_kernelSplit_leakyRelu": "sipiipiipfpiiiiiiiii",
    "alpha_leakyRelu2D": "lpfpiii",
    "alpha_leakyRelu2D_deltaX_v1": "lpppfiii",
    "alpha_batchNorm2D_row": "lpppfipiii",
    "alpha_batchNorm_affined2D_row": "lpppfppipiii",
    "alpha_field_affine_deltaAB_v1": "llppppiippppiiin",
    "alpha_field_affine_deltaAB_v2": "llppiippppiiin",
    "alpha_field_batchNorm_deltaAB_v2": "llppppfiippppiiin",
    "alpha_batchNorm2D_row_deltaX_v1": "lpppfppipiii",
    "alpha_batchNorm2D_row_deltaX_v2": "lppppfppipiii",
    "alpha_batchNorm_affined2D_row_deltaX_v1": "lpppfppppipiii",
    "alpha_batchNorm_affined2D_row_deltaX_v2": "lppppfpppipiii",
}


class Epilogue(ctypes.Structure):
    """alpha_conv_epilogue of include/alpha_conv.h: device addresses as integers (0 = absent), eps and k as floats."""
    _fields_ = [("Bias", _P), ("X_mean", _P), ("X_var", _P), ("eps", ctypes.c_float), ("A", _P), ("B", _P), ("k", ctypes.c_float)]

    def __init__(self, Bias=0, X_mean=0, X_var=0, eps=1e-5, A=0, B=0, k=1.0):
        super().__init__(Bias or None, X_mean or None, X_var or None, eps, A or None, B or None, k)


_CT = {"s": _S, "i": _I, "p": _P, "l": _L, "f": ctypes.c_float, "e": ctypes.POINTER(Epilogue), "n": ctypes.POINTER(ctypes.c_int)}


class AlphaConvError(RuntimeError):
    """Raised where the Java natives would throw CudaException."""


def lib_path():
    return os.path.join(_HERE, _LIB_NAME)


def exported_symbols():
    """Names the C ABI must export (every function include/alpha_conv.h declares)."""
    return sorted(list(_SIGS) + ["alpha_conv_version", "alpha_conv_last_error", "alpha_conv_device_info", "alpha_conv_set_fwd_algo",
                                 "alpha_conv_get_fwd_algo", "alpha_conv_set_pointwise_algo", "alpha_conv_set_kernel_split_sharing", "alpha_conv_set_deltaW_units", "alpha_conv_bind_workspace", "alpha_conv_bind_tickets", "alpha_winograd_filter_size", "alpha_dconv3D_deltaW_least_GridZ"])


def _preload_hip_runtime():
    """A process must hold exactly ONE HIP runtime. PyTorch wheels bundle their own libamdhip64.so
    (same SONAME as /opt/rocm's, different file); a second copy in the process finds no device.
    When torch is installed, map its copy first so that this library's NEEDED libamdhip64.so.7
    binds to it; a later `import torch` then re-uses the same file. Without torch the loader
    takes the system runtime as usual."""
    import importlib.util
    if "torch" in sys.modules:
        return
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        spec = None
    if spec is None or not spec.origin:
        return
    cand = os.path.join(os.path.dirname(spec.origin), "lib", "libamdhip64.so")
    if os.path.exists(cand):
        ctypes.CDLL(cand, mode=ctypes.RTLD_GLOBAL)


def lib():
    """Loads the HIP library; raises if it has not been built (there is no fallback path)."""
    global _lib
    if _lib is None:
        path = lib_path()
        if not os.path.exists(path):
            raise AlphaConvError("%s is not built: run `python %s`" % (path, os.path.join(_HERE, "build.py")))
        _preload_hip_runtime()
        L = ctypes.CDLL(path)
        for name, sig in _SIGS.items():
            fn = getattr(L, name)
            fn.argtypes = [_CT[c] for c in sig]
            fn.restype = _I
        L.alpha_conv_version.restype = ctypes.c_char_p
        L.alpha_conv_last_error.restype = ctypes.c_char_p
        L.alpha_conv_set_fwd_algo.argtypes = [_I]
        L.alpha_conv_get_fwd_algo.restype = _I
        L.alpha_conv_set_pointwise_algo.argtypes = [_I]
        L.alpha_conv_set_kernel_split_sharing.argtypes = [_I]
        L.alpha_conv_set_deltaW_units.argtypes = [_I]
        L.alpha_conv_bind_workspace.argtypes = [_P, ctypes.c_long]
        L.alpha_conv_bind_tickets.argtypes = [_P, ctypes.c_int]
        L.alpha_winograd_filter_size.argtypes = [_I, _I]
        L.alpha_winograd_filter_size.restype = ctypes.c_long
        L.alpha_dconv3D_deltaW_least_GridZ.argtypes = [_I] * 9
        L.alpha_dconv3D_deltaW_least_GridZ.restype = _I
        _lib = L
    return _lib


def _call(name, *args):
    L = lib()
    sig = _SIGS[name]
    conv = []
    keep = []
    it = iter(args)
    for c in sig:
        a = next(it)
        if c == "s":
            arr = (ctypes.c_int64 * max(1, len(a)))(*a)
            keep.append(arr)
            conv.append(arr)
        elif c == "p":
            conv.append(ctypes.c_void_p(int(a)))
        elif c == "l":
            conv.append(ctypes.c_int64(int(a)))
        elif c == "f":
            conv.append(ctypes.c_float(float(a)))
        elif c == "e":
            keep.append(a)
            conv.append(ctypes.byref(a))
        elif c == "n":
            conv.append(a)   # a ctypes.byref(c_int), or None
        else:
            conv.append(int(a))
    rc = getattr(L, name)(*conv)
    if rc != 0:
        raise AlphaConvError("%s failed (%d): %s" % (name, rc, L.alpha_conv_last_error().decode()))


def device_info():
    """(compute units, peak clock in kHz) of the current device."""
    cu, clk = ctypes.c_int(0), ctypes.c_int(0)
    rc = lib().alpha_conv_device_info(ctypes.byref(cu), ctypes.byref(clk))
    if rc != 0:
        raise AlphaConvError("alpha_conv_device_info failed (%d): %s" % (rc, lib().alpha_conv_last_error().decode()))
    return cu.value, clk.value


class Cuda_conv3D:
    """Forward natives (Cuda_conv3D.java)."""

    @staticmethod
    def outputTensorDim(IH, IW, FH, FW, N, OC, sh, sw, ph, pw):
        return [N, (IH + (ph << 1) - FH) // sh + 1, (IW + (pw << 1) - FW) // sw + 1, OC]

    @staticmethod
    def conv3D(streamArray, length, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_conv3D", streamArray, length, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def conv3D_texture(streamArray, length, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_conv3D_texture", streamArray, length, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def conv3DV2(useTexture, streamArray, length, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_conv3DV2", useTexture, streamArray, length, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def conv3D_np(streamArray, length, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw):
        _call("alpha_conv3D_np", streamArray, length, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw)

    @staticmethod
    def conv3D_W1(streamArray, length, X, IH, IW, W, Y, N, IC, OC):
        _call("alpha_conv3D_W1", streamArray, length, X, IH, IW, W, Y, N, IC, OC)

    @staticmethod
    def kernel_remode(stream, W, CW, FH, FW, OC, IC):
        _call("alpha_kernel_remode", stream, W, CW, FH, FW, OC, IC)

    @staticmethod
    def conv3D_GemmR(streamArray, length, X, IH, IW, W, CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_conv3D_GemmR", streamArray, length, X, IH, IW, W, CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def conv3D_GemmR_texture(streamArray, length, X, IH, IW, W, CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_conv3D_GemmR_texture", streamArray, length, X, IH, IW, W, CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def conv3D_GemmV2R(useTexture, streamArray, length, X, IH, IW, W, CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_conv3D_GemmV2R", useTexture, streamArray, length, X, IH, IW, W, CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def conv3D_GemmR_W1(streamArray, length, X, IH, IW, W, CW, Y, N, IC, OC):
        _call("alpha_conv3D_GemmR_W1", streamArray, length, X, IH, IW, W, CW, Y, N, IC, OC)

    # additional algorithm of this build (no Java counterpart)
    @staticmethod
    def winograd_filter_size(IC, OC):
        return int(lib().alpha_winograd_filter_size(IC, OC))

    @staticmethod
    def winograd_filter_transform(stream, W, U, IC, OC):
        _call("alpha_winograd_filter_transform", stream, W, U, IC, OC)

    @staticmethod
    def conv3D_winograd(streamArray, length, X, IH, IW, U, Y, OH, OW, N, IC, OC, ph, pw):
        _call("alpha_conv3D_winograd", streamArray, length, X, IH, IW, U, Y, OH, OW, N, IC, OC, ph, pw)

    # forward with the bias added in the kernel epilogue (the reference composes conv3D + linear_dual2D_row)
    @staticmethod
    def conv3D_biased(streamArray, length, X, IH, IW, W, FH, FW, Bias, Y, OH, OW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_conv3D_biased", streamArray, length, X, IH, IW, W, FH, FW, Bias, Y, OH, OW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def conv3D_GemmR_biased(streamArray, length, X, IH, IW, W, CW, FH, FW, Bias, Y, OH, OW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_conv3D_GemmR_biased", streamArray, length, X, IH, IW, W, CW, FH, FW, Bias, Y, OH, OW, N, IC, OC,
              sh, sw, ph, pw)

    @staticmethod
    def conv3D_winograd_biased(streamArray, length, X, IH, IW, U, Bias, Y, OH, OW, N, IC, OC, ph, pw):
        _call("alpha_conv3D_winograd_biased", streamArray, length, X, IH, IW, U, Bias, Y, OH, OW, N, IC, OC, ph, pw)

    # forward with bias, batch normalisation (given statistics) and leaky ReLU in the kernel epilogue; `epilogue` is an Epilogue
    @staticmethod
    def conv3D_fused(streamArray, length, X, IH, IW, W, FH, FW, epilogue, Y, OH, OW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_conv3D_fused", streamArray, length, X, IH, IW, W, FH, FW, epilogue, Y, OH, OW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def conv3D_GemmR_fused(streamArray, length, X, IH, IW, W, CW, FH, FW, epilogue, Y, OH, OW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_conv3D_GemmR_fused", streamArray, length, X, IH, IW, W, CW, FH, FW, epilogue, Y, OH, OW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def conv3D_winograd_fused(streamArray, length, X, IH, IW, U, epilogue, Y, OH, OW, N, IC, OC, ph, pw):
        _call("alpha_conv3D_winograd_fused", streamArray, length, X, IH, IW, U, epilogue, Y, OH, OW, N, IC, OC, ph, pw)


class Cuda_dconv3D_deltaX:
    """Backward-data natives (Cuda_dconv3D_deltaX.java)."""

    @staticmethod
    def dconv3D_deltaX_s1(streamArray, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw):
        _call("alpha_dconv3D_deltaX_s1", streamArray, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw)

    @staticmethod
    def winograd_filter_transform_deltaX(stream, W, U, IC, OC):
        """This build's Winograd path for backward-data (no reference counterpart): U as for the forward transform."""
        _call("alpha_winograd_filter_transform_deltaX", stream, W, U, IC, OC)

    @staticmethod
    def dconv3D_deltaX_winograd(streamArray, length, deltaY, OH, OW, U, deltaX, IH, IW, N, IC, OC, ph, pw):
        _call("alpha_dconv3D_deltaX_winograd", streamArray, length, deltaY, OH, OW, U, deltaX, IH, IW, N, IC, OC, ph, pw)

    @staticmethod
    def dconv3D_deltaX_s1_leakyRelu(streamArray, length, deltaY, OH, OW, W, FH, FW, Xf, k, deltaX, IH, IW, N, IC, OC, ph, pw):
        """Backward-data times the derivative of the leaky ReLU whose output Xf is this layer's input (fused epilogue)."""
        _call("alpha_dconv3D_deltaX_s1_leakyRelu", streamArray, length, deltaY, OH, OW, W, FH, FW, Xf, k, deltaX, IH, IW, N, IC, OC, ph, pw)

    @staticmethod
    def dconv3D_deltaX_kernelSplit_leakyRelu(streamArray, length, deltaY, OH, OW, CW, FH, FW, Xf, k, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_dconv3D_deltaX_kernelSplit_leakyRelu", streamArray, length, deltaY, OH, OW, CW, FH, FW, Xf, k, deltaX, IH, IW,
              N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def dconv3D_deltaX_s1_texture(streamArray, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw):
        _call("alpha_dconv3D_deltaX_s1_texture", streamArray, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw)

    @staticmethod
    def dconv3D_deltaX_V2_s1(useTexture, streamArray, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw):
        _call("alpha_dconv3D_deltaX_V2_s1", useTexture, streamArray, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw)

    @staticmethod
    def dconv3D_deltaX_W1(streamArray, length, deltaY, W, deltaX, IH, IW, N, IC, OC):
        _call("alpha_dconv3D_deltaX_W1", streamArray, length, deltaY, W, deltaX, IH, IW, N, IC, OC)

    @staticmethod
    def ks_remode(stream, W, FH, FW, CW, CFH, CFW, OC, IC, sh, sw):
        _call("alpha_ks_remode", stream, W, FH, FW, CW, CFH, CFW, OC, IC, sh, sw)

    @staticmethod
    def ks_remodev2(stream, W, FH, FW, CW, CFH, CFW, OC, IC, sh, sw):
        _call("alpha_ks_remodev2", stream, W, FH, FW, CW, CFH, CFW, OC, IC, sh, sw)

    @staticmethod
    def dconv3D_deltaX_kernelSplit(streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_dconv3D_deltaX_kernelSplit", streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def dconv3D_deltaX_ksImsR(streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_dconv3D_deltaX_ksImsR", streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def dconv3D_deltaX_ksImsR_texture(streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_dconv3D_deltaX_ksImsR_texture", streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def dconv3D_deltaX_ksIms2R(streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw):
        _call("alpha_dconv3D_deltaX_ksIms2R", streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw)

    @staticmethod
    def dconv3D_deltaX_ksIms2R_texture(streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw):
        _call("alpha_dconv3D_deltaX_ksIms2R_texture", streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw)

    @staticmethod
    def dconv3D_deltaX_ksV2_Ims2R(useTexture, streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw):
        _call("alpha_dconv3D_deltaX_ksV2_Ims2R", useTexture, streamArray, length, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw)

    @staticmethod
    def dconv3D_deltaX_crossAdd(streamArray, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_dconv3D_deltaX_crossAdd", streamArray, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw)


class Cuda_dconv3D_deltaW:
    """Backward-filter natives (Cuda_dconv3D_deltaW.java)."""

    @staticmethod
    def dconv3D_deltaW(streamArray, length, X, IH, IW, deltaY, OH, OW, deltaW, FH, FW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_dconv3D_deltaW", streamArray, length, X, IH, IW, deltaY, OH, OW, deltaW, FH, FW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def dconv3D_deltaW_W1(streamArray, length, X, IH, IW, deltaY, deltaW, N, IC, OC):
        _call("alpha_dconv3D_deltaW_W1", streamArray, length, X, IH, IW, deltaY, deltaW, N, IC, OC)

    @staticmethod
    def buf_summary(stream, deltaW_buf, deltaW, part, sizeW):
        _call("alpha_buf_summary", stream, deltaW_buf, deltaW, part, sizeW)

    @staticmethod
    def dconv3D_deltaW_GemmSK(streamArray, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, deltaW_buf, FH, FW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_dconv3D_deltaW_GemmSK", streamArray, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, deltaW_buf, FH, FW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def dconv3D_deltaW_GemmSK_winograd(streamArray, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, deltaW_buf, N, IC, OC, ph, pw):
        """This build's Winograd F(3x3,2x2) backward-filter for 3x3 stride-1 layers (no reference counterpart)."""
        _call("alpha_dconv3D_deltaW_GemmSK_winograd", streamArray, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, deltaW_buf, N, IC, OC, ph, pw)

    @staticmethod
    def dconv3D_deltaW_GemmV2SK(streamArray, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, deltaW_buf, FH, FW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_dconv3D_deltaW_GemmV2SK", streamArray, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, deltaW_buf, FH, FW, N, IC, OC, sh, sw, ph, pw)

    @staticmethod
    def dconv3D_deltaW_GemmSK_W1(streamArray, length, GridZ, X, IH, IW, deltaY, deltaW, deltaW_buf, N, IC, OC):
        _call("alpha_dconv3D_deltaW_GemmSK_W1", streamArray, length, GridZ, X, IH, IW, deltaY, deltaW, deltaW_buf, N, IC, OC)

    @staticmethod
    def dconv3D_deltaW_GemmSK_static(streamArray, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, FH, FW, N, IC, OC, sh, sw, ph, pw):
        """Split-K backward-filter plus the sum of its partial results, with the partials in the library's static device
        array: allocates nothing, takes no deltaW_buf (no reference counterpart)."""
        _call("alpha_dconv3D_deltaW_GemmSK_static", streamArray, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, FH, FW, N, IC, OC, sh, sw, ph, pw)

    # backward-filter plus the bias gradient (the reference: dconv3D_deltaW, then field_sum over deltaY)
    @staticmethod
    def dconv3D_deltaW_GemmSK_deltaB(streamArray, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, deltaW_buf,
                                     deltaB, deltaB_buf, FH, FW, N, IC, OC, sh, sw, ph, pw):
        _call("alpha_dconv3D_deltaW_GemmSK_deltaB", streamArray, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, deltaW_buf,
              deltaB, deltaB_buf, FH, FW, N, IC, OC, sh, sw, ph, pw)


class Cuda_reduce:
    """The field sums of batch normalisation's backward (Cuda_reduce.java:697, 746, 939), same argument order; they return
    the number of rows left after the last stage, as the reference's natives do. Only these three of the class."""

    @staticmethod
    def _run(name, *args):
        n = ctypes.c_int(0)
        _call(name, *args, ctypes.byref(n))
        return n.value

    @staticmethod
    def field_affine_deltaAB_v1(stream1, stream2, deltaY, Y, A, B, N, M, deltaA_buf, deltaA, deltaB_buf, deltaB, mem_width, mem_stride, partNum):
        return Cuda_reduce._run("alpha_field_affine_deltaAB_v1", stream1, stream2, deltaY, Y, A, B, N, M, deltaA_buf, deltaA, deltaB_buf, deltaB,
                                mem_width, mem_stride, partNum)

    @staticmethod
    def field_affine_deltaAB_v2(stream1, stream2, deltaY, X_norm, N, M, deltaA_buf, deltaA, deltaB_buf, deltaB, mem_width, mem_stride, partNum):
        return Cuda_reduce._run("alpha_field_affine_deltaAB_v2", stream1, stream2, deltaY, X_norm, N, M, deltaA_buf, deltaA, deltaB_buf, deltaB,
                                mem_width, mem_stride, partNum)

    @staticmethod
    def field_batchNorm_deltaAB_v2(stream1, stream2, deltaY, X, X_mean, X_var, eps, N, M, deltaA_buf, deltaA, deltaB_buf, deltaB,
                                   mem_width, mem_stride, partNum):
        return Cuda_reduce._run("alpha_field_batchNorm_deltaAB_v2", stream1, stream2, deltaY, X, X_mean, X_var, eps, N, M, deltaA_buf, deltaA,
                                deltaB_buf, deltaB, mem_width, mem_stride, partNum)

    @staticmethod
    def field_nextN(N, M):
        """Cuda_reduce.field_nextN (Cuda_reduce.java:35-45): rows of the buffers the Java engine allocates for these sums."""
        if M > 15:
            if N > 63:
                return N >> 6
            if N > 15:
                return 1
        if M > 7:
            if N > 127:
                return N >> 7
            if N > 31:
                return 1
        return (N + 63) >> 6


class Cuda_function:
    """The row functions the reference applies around a convolution (Cuda_function.java:1607, 1640, 3829, 3862 forward;
    3890, 3923, 3958, 3992 backward of batch normalisation), same argument order; one HBM-bound pass each. Only these:
    the class's other natives are outside this library."""

    @staticmethod
    def batchNorm2D_row_deltaX_v1(stream, deltaY, Y, X_var, eps, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv, mem_width, mem_stride):
        _call("alpha_batchNorm2D_row_deltaX_v1", stream, deltaY, Y, X_var, eps, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv, mem_width, mem_stride)

    @staticmethod
    def batchNorm2D_row_deltaX_v2(stream, deltaY, X, X_mean, X_var, eps, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv, mem_width, mem_stride):
        _call("alpha_batchNorm2D_row_deltaX_v2", stream, deltaY, X, X_mean, X_var, eps, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv,
              mem_width, mem_stride)

    @staticmethod
    def batchNorm_affined2D_row_deltaX_v1(stream, deltaY, Y, X_var, eps, A, B, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv, mem_width, mem_stride):
        _call("alpha_batchNorm_affined2D_row_deltaX_v1", stream, deltaY, Y, X_var, eps, A, B, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv,
              mem_width, mem_stride)

    @staticmethod
    def batchNorm_affined2D_row_deltaX_v2(stream, deltaY, X, X_mean, X_var, eps, A, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv,
                                          mem_width, mem_stride):
        _call("alpha_batchNorm_affined2D_row_deltaX_v2", stream, deltaY, X, X_mean, X_var, eps, A, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv,
              mem_width, mem_stride)

    @staticmethod
    def leakyRelu2D(stream, X, k, Y, lengthv, mem_width, mem_stride):
        _call("alpha_leakyRelu2D", stream, X, k, Y, lengthv, mem_width, mem_stride)

    @staticmethod
    def leakyRelu2D_deltaX_v1(stream, deltaX, deltaY, Y, k, lengthv, mem_width, mem_stride):
        _call("alpha_leakyRelu2D_deltaX_v1", stream, deltaX, deltaY, Y, k, lengthv, mem_width, mem_stride)

    @staticmethod
    def batchNorm2D_row(stream, X, X_mean, X_var, eps, row_lengthv, Y, lengthv, mem_width, mem_stride):
        _call("alpha_batchNorm2D_row", stream, X, X_mean, X_var, eps, row_lengthv, Y, lengthv, mem_width, mem_stride)

    @staticmethod
    def batchNorm_affined2D_row(stream, X, X_mean, X_var, eps, A, B, row_lengthv, Y, lengthv, mem_width, mem_stride):
        _call("alpha_batchNorm_affined2D_row", stream, X, X_mean, X_var, eps, A, B, row_lengthv, Y, lengthv, mem_width, mem_stride)
