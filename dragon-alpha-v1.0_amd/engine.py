"""ctypes access to the C++ host layer of include/alpha_engine.h: the counterpart of the reference's
CudaFloat32EngineBase convolution section (algorithm selection, split-K factor, scratch ownership).
Method names and argument order of `Engine` follow the reference's EngineBase operator API
(src/alpha_src/z/dragon/engine/EngineBase.java:171-199): output address first."""
import ctypes

from . import native

ENTRY_NAMES = [None,
               "conv3D", "conv3D_texture", "conv3DV2", "conv3D_np", "conv3D_W1",
               "conv3D_GemmR", "conv3D_GemmR_texture", "conv3D_GemmV2R", "conv3D_GemmR_W1",
               "dconv3D_deltaX_s1", "dconv3D_deltaX_s1_texture", "dconv3D_deltaX_V2_s1", "dconv3D_deltaX_W1",
               "dconv3D_deltaX_kernelSplit", "dconv3D_deltaX_ksImsR", "dconv3D_deltaX_ksImsR_texture",
               "dconv3D_deltaX_ksIms2R", "dconv3D_deltaX_ksIms2R_texture", "dconv3D_deltaX_ksV2_Ims2R",
               "dconv3D_deltaX_crossAdd",
               "dconv3D_deltaW", "dconv3D_deltaW_W1", "dconv3D_deltaW_GemmSK", "dconv3D_deltaW_GemmV2SK",
               "dconv3D_deltaW_GemmSK_W1", "conv3D_winograd", "dconv3D_deltaX_winograd", "dconv3D_deltaW_GemmSK_winograd"]


class Config(ctypes.Structure):
    _fields_ = [("conv3D_useTexture", ctypes.c_int), ("conv3D_remode", ctypes.c_int),
                ("conv3D_remode_V2_Q", ctypes.c_float), ("conv3D_V2_Q", ctypes.c_float),
                ("deltaW_SplitKThreshold", ctypes.c_int), ("deltaW_SK_MaxPartNum", ctypes.c_int),
                ("deltaW_SK_V2_Q", ctypes.c_float),
                ("deltaX_s1_useTexture", ctypes.c_int), ("deltaX_ks_useTexture", ctypes.c_int),
                ("deltaX_s1_V2_Q", ctypes.c_float), ("deltaX_ks_V2_Q", ctypes.c_float),
                ("conv3D_winograd", ctypes.c_int), ("deltaW_SK_fillUnits", ctypes.c_int),
                ("cache_filter_transforms", ctypes.c_int), ("deltaX_winograd", ctypes.c_int), ("deltaW_winograd", ctypes.c_int),
                ("deltaW_SK_leastUnits", ctypes.c_int), ("conv_workspace", ctypes.c_int)]


class Plan(ctypes.Structure):
    _fields_ = [("entry", ctypes.c_int), ("streams", ctypes.c_int), ("remode", ctypes.c_int), ("V2", ctypes.c_int),
                ("useTexture", ctypes.c_int), ("GridZ", ctypes.c_int), ("scratch_floats", ctypes.c_long),
                ("Q", ctypes.c_double)]

    @property
    def entry_name(self):
        return ENTRY_NAMES[self.entry]


_I, _P = ctypes.c_int, ctypes.c_void_p
_bound = False


def _lib():
    global _bound
    L = native.lib()
    if not _bound:
        L.alpha_blockNum.argtypes = [_I, _I]
        L.alpha_streamSize.argtypes = [_I, _I, _I]
        L.alpha_paddingScaleUp.argtypes = [_I] * 8
        L.alpha_paddingScaleUp.restype = ctypes.c_double
        L.alpha_engine_config_default.argtypes = [ctypes.POINTER(Config), _I]
        L.alpha_engine_config_default.restype = None
        L.alpha_plan_conv3D.argtypes = [ctypes.POINTER(Config)] + [_I] * 13 + [ctypes.POINTER(Plan)]
        L.alpha_plan_conv3D.restype = None
        for n in ("alpha_plan_deltaW", "alpha_plan_deltaX"):
            getattr(L, n).argtypes = [ctypes.POINTER(Config)] + [_I] * 11 + [ctypes.POINTER(Plan)]
            getattr(L, n).restype = None
        L.alpha_engine_param_check.argtypes = [_I] * 13
        L.alpha_engine_param_check.restype = ctypes.c_char_p
        L.alpha_engine_create.argtypes = [ctypes.c_int64]
        L.alpha_engine_create.restype = _P
        L.alpha_engine_destroy.argtypes = [_P]
        L.alpha_engine_destroy.restype = None
        L.alpha_engine_get_config.argtypes = [_P]
        L.alpha_engine_get_config.restype = ctypes.POINTER(Config)
        L.alpha_engine_last_error.argtypes = [_P]
        L.alpha_engine_last_error.restype = ctypes.c_char_p
        L.alpha_engine_sync.argtypes = [_P]
        L.alpha_engine_filter_changed.argtypes = [_P, _P]
        L.alpha_engine_filter_changed.restype = None
        L.alpha_engine_conv3D.argtypes = [_P, _P, _I, _I, _P, _I, _I, _P, _I, _I] + [_I] * 7 + [ctypes.POINTER(Plan)]
        L.alpha_engine_conv3D_biased.argtypes = ([_P, _P, _I, _I, _P, _I, _I, _P, _I, _I] + [_I] * 7 + [_P, _I, _I]
                                                 + [ctypes.POINTER(Plan)])
        L.alpha_engine_dconv3D_deltaW.argtypes = [_P, _P, _I, _I, _P, _I, _I, _P, _I, _I] + [_I] * 7 + [ctypes.POINTER(Plan)]
        L.alpha_engine_dconv3D_deltaW_deltaB.argtypes = ([_P, _P, _P, _I, _I, _P, _I, _I, _P, _I, _I] + [_I] * 7
                                                         + [ctypes.POINTER(Plan)])
        L.alpha_engine_dconv3D_deltaX.argtypes = [_P, _P, _I, _I, _P, _I, _I, _P, _I, _I] + [_I] * 7 + [ctypes.POINTER(Plan)]
        L.alpha_engine_conv3D_fused.argtypes = ([_P, _P, _I, _I, _P, _I, _I, _P, _I, _I] + [_I] * 7
                                                + [ctypes.POINTER(native.Epilogue), ctypes.POINTER(Plan)])
        L.alpha_engine_dconv3D_deltaX_leakyRelu.argtypes = ([_P, _P, _I, _I, _P, _I, _I, _P, _I, _I] + [_I] * 7
                                                            + [_P, ctypes.c_float, ctypes.POINTER(Plan)])
        F = ctypes.c_float
        L.alpha_engine_batchNorm2D_deltaX_v1.argtypes = [_P, _P, _P, _P, _P, F, _P, _P, _P, _P] + [_I] * 5
        L.alpha_engine_batchNorm2D_deltaX_v2.argtypes = [_P, _P, _P, _P, _P, _P, F, _P, _P, _P] + [_I] * 5
        _bound = True
    return L


def default_config(compute_units=256):
    c = Config()
    _lib().alpha_engine_config_default(ctypes.byref(c), compute_units)
    return c


def blockNum(GN, GM):
    return _lib().alpha_blockNum(GN, GM)


def streamSize(GN, GM, cap=10):
    return _lib().alpha_streamSize(GN, GM, cap)


def paddingScaleUp(IH, IW, OH, OW, FH, FW, sh, sw):
    return _lib().alpha_paddingScaleUp(IH, IW, OH, OW, FH, FW, sh, sw)


def param_check(OH, OW, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw):
    """None when the sizes are consistent, else the reason the engine refuses them."""
    r = _lib().alpha_engine_param_check(OH, OW, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw)
    return None if r is None else r.decode()


def plan_conv3D(cfg, IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, ph, pw):
    p = Plan()
    _lib().alpha_plan_conv3D(ctypes.byref(cfg), IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, ph, pw, ctypes.byref(p))
    return p


def plan_deltaW(cfg, IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw):
    p = Plan()
    _lib().alpha_plan_deltaW(ctypes.byref(cfg), IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, ctypes.byref(p))
    return p


def plan_deltaX(cfg, IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw):
    p = Plan()
    _lib().alpha_plan_deltaX(ctypes.byref(cfg), IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, ctypes.byref(p))
    return p


class Engine:
    """Owns scratch, chooses entries, enqueues on one stream; sync() releases scratch for reuse."""

    def __init__(self, stream):
        self._L = _lib()
        self._h = self._L.alpha_engine_create(int(stream))
        if not self._h:
            raise native.AlphaConvError("alpha_engine_create failed")

    @property
    def config(self):
        return self._L.alpha_engine_get_config(self._h).contents

    def _check(self, rc):
        if rc != 0:
            raise native.AlphaConvError("engine call failed (%d): %s" % (rc, self._L.alpha_engine_last_error(self._h).decode()))

    def conv3D(self, Y, OH, OW, X, IH, IW, W, FH, FW, N, IC, OC, sh, sw, ph, pw):
        p = Plan()
        self._check(self._L.alpha_engine_conv3D(self._h, Y, OH, OW, X, IH, IW, W, FH, FW, N, IC, OC, sh, sw, ph, pw, ctypes.byref(p)))
        return p

    def filter_changed(self, W=None):
        self._L.alpha_engine_filter_changed(self._h, W)

    def conv3D_biased(self, Y, OH, OW, X, IH, IW, W, FH, FW, N, IC, OC, sh, sw, ph, pw, Bias, lengthv, width):
        p = Plan()
        self._check(self._L.alpha_engine_conv3D_biased(self._h, Y, OH, OW, X, IH, IW, W, FH, FW, N, IC, OC, sh, sw, ph, pw,
                                                       Bias, lengthv, width, ctypes.byref(p)))
        return p

    def conv3D_fused(self, Y, OH, OW, X, IH, IW, W, FH, FW, N, IC, OC, sh, sw, ph, pw, epilogue):
        """conv3D + batch normalisation (given statistics) + leaky ReLU as one operator; `epilogue` is a native.Epilogue."""
        p = Plan()
        self._check(self._L.alpha_engine_conv3D_fused(self._h, Y, OH, OW, X, IH, IW, W, FH, FW, N, IC, OC, sh, sw, ph, pw,
                                                      ctypes.byref(epilogue), ctypes.byref(p)))
        return p

    def dconv3D_deltaX_leakyRelu(self, deltaX, IH, IW, deltaY, OH, OW, W, FH, FW, N, IC, OC, sh, sw, ph, pw, Xf, k):
        p = Plan()
        self._check(self._L.alpha_engine_dconv3D_deltaX_leakyRelu(self._h, deltaX, IH, IW, deltaY, OH, OW, W, FH, FW, N, IC, OC,
                                                                  sh, sw, ph, pw, Xf, k, ctypes.byref(p)))
        return p

    def batchNorm2D_deltaX_v1(self, deltaX, deltaY, Y, X_var, eps, field_length, row_lengthv, lengthv, width, stride,
                              A=None, B=None, deltaA=None, deltaB=None):
        """EngineBase.batchNorm2D_deltaX_v1 (A is None: not affine); with deltaA / deltaB: batchNorm2D_gradients_v1."""
        self._check(self._L.alpha_engine_batchNorm2D_deltaX_v1(self._h, deltaX, deltaY, Y, X_var, eps, A, B, deltaA, deltaB,
                                                               field_length, row_lengthv, lengthv, width, stride))

    def batchNorm2D_deltaX_v2(self, deltaX, deltaY, X, X_mean, X_var, eps, field_length, row_lengthv, lengthv, width, stride,
                              A=None, deltaA=None, deltaB=None):
        """EngineBase.batchNorm2D_deltaX_v2 (A is None: not affine); with deltaA / deltaB: batchNorm2D_gradients_v2."""
        self._check(self._L.alpha_engine_batchNorm2D_deltaX_v2(self._h, deltaX, deltaY, X, X_mean, X_var, eps, A, deltaA, deltaB,
                                                               field_length, row_lengthv, lengthv, width, stride))

    def dconv3D_deltaW(self, deltaW, FH, FW, X, IH, IW, deltaY, OH, OW, N, IC, OC, sh, sw, ph, pw):
        p = Plan()
        self._check(self._L.alpha_engine_dconv3D_deltaW(self._h, deltaW, FH, FW, X, IH, IW, deltaY, OH, OW, N, IC, OC,
                                                        sh, sw, ph, pw, ctypes.byref(p)))
        return p

    def dconv3D_deltaW_deltaB(self, deltaW, deltaB, FH, FW, X, IH, IW, deltaY, OH, OW, N, IC, OC, sh, sw, ph, pw):
        p = Plan()
        self._check(self._L.alpha_engine_dconv3D_deltaW_deltaB(self._h, deltaW, deltaB, FH, FW, X, IH, IW, deltaY, OH, OW,
                                                               N, IC, OC, sh, sw, ph, pw, ctypes.byref(p)))
        return p

    def dconv3D_deltaX(self, deltaX, IH, IW, deltaY, OH, OW, W, FH, FW, N, IC, OC, sh, sw, ph, pw):
        p = Plan()
        self._check(self._L.alpha_engine_dconv3D_deltaX(self._h, deltaX, IH, IW, deltaY, OH, OW, W, FH, FW, N, IC, OC,
                                                        sh, sw, ph, pw, ctypes.byref(p)))
        return p

    def sync(self):
        self._check(self._L.alpha_engine_sync(self._h))

    def close(self):
        if self._h:
            self._L.alpha_engine_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
