"""ctypes loader for the CPU oracle (liboracle.so, built from conv_oracle.c by the Makefile here).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's
cpu_baseline leg. The product package never imports this module.

All arrays are C-contiguous numpy arrays; layouts are the reference's
(X[N,IH,IW,IC], W[OC,FH,FW,IC], Y[N,OH,OW,OC]).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i = ctypes.c_int


def build(force=False):
    """Compile liboracle.so with gcc (always when force=True, else only if it is absent)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_samePercentRelative.restype = ctypes.c_float
        _lib.oracle_max_err_ratio.restype = ctypes.c_double
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def _p32(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_f32p)


def _p64(a):
    assert a.dtype == np.float64 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_f64p)


def out_dim(IH, IW, FH, FW, sh, sw, ph, pw):
    """Cuda_conv3D.outputTensorDim (J/math/Cuda_conv3D.java:148-157)."""
    return (IH + 2 * ph - FH) // sh + 1, (IW + 2 * pw - FW) // sw + 1


def num_threads():
    return lib().oracle_num_threads()


def set_num_threads(n):
    lib().oracle_set_num_threads(_i(n))


def _fwd(fn, X, W, sh, sw, ph, pw, out_dtype):
    N, IH, IW, IC = X.shape
    OC, FH, FW, IC2 = W.shape
    assert IC == IC2
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    Y = np.empty((N, OH, OW, OC), dtype=out_dtype)
    fn(_p32(X), _i(IH), _i(IW), _p32(W), _i(FH), _i(FW),
       _p64(Y) if out_dtype == np.float64 else _p32(Y), _i(OH), _i(OW),
       _i(N), _i(IC), _i(OC), _i(sh), _i(sw), _i(ph), _i(pw))
    return Y


def conv3D_naive(X, W, sh, sw, ph, pw):
    return _fwd(lib().oracle_conv3D_naive, X, W, sh, sw, ph, pw, np.float32)


def conv3D_f64(X, W, sh, sw, ph, pw):
    return _fwd(lib().oracle_conv3D_f64, X, W, sh, sw, ph, pw, np.float64)


def conv3D_f32acc(X, W, sh, sw, ph, pw):
    return _fwd(lib().oracle_conv3D_f32acc, X, W, sh, sw, ph, pw, np.float32)


def _dx(fn, dY, W, IH, IW, sh, sw, ph, pw, out_dtype):
    N, OH, OW, OC = dY.shape
    OC2, FH, FW, IC = W.shape
    assert OC == OC2
    dX = np.empty((N, IH, IW, IC), dtype=out_dtype)
    fn(_p32(dY), _i(OH), _i(OW), _p32(W), _i(FH), _i(FW),
       _p64(dX) if out_dtype == np.float64 else _p32(dX), _i(IH), _i(IW),
       _i(N), _i(IC), _i(OC), _i(sh), _i(sw), _i(ph), _i(pw))
    return dX


def deltaX_img2col(dY, W, IH, IW, sh, sw, ph, pw):
    return _dx(lib().oracle_deltaX_img2col, dY, W, IH, IW, sh, sw, ph, pw, np.float32)


def deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw):
    return _dx(lib().oracle_deltaX_f64, dY, W, IH, IW, sh, sw, ph, pw, np.float64)


def _dw(fn, X, dY, FH, FW, sh, sw, ph, pw, out_dtype, extra=()):
    N, IH, IW, IC = X.shape
    N2, OH, OW, OC = dY.shape
    assert N == N2
    dW = np.empty((OC, FH, FW, IC), dtype=out_dtype)
    fn(_p32(X), _i(IH), _i(IW), _p32(dY), _i(OH), _i(OW),
       _p64(dW) if out_dtype == np.float64 else _p32(dW), _i(FH), _i(FW),
       _i(N), _i(IC), _i(OC), _i(sh), _i(sw), _i(ph), _i(pw), *extra)
    return dW


def deltaW_naive(X, dY, FH, FW, sh, sw, ph, pw):
    return _dw(lib().oracle_deltaW_naive, X, dY, FH, FW, sh, sw, ph, pw, np.float32)


def deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw):
    return _dw(lib().oracle_deltaW_f64, X, dY, FH, FW, sh, sw, ph, pw, np.float64)


def deltaW_f32acc(X, dY, FH, FW, sh, sw, ph, pw):
    return _dw(lib().oracle_deltaW_f32acc, X, dY, FH, FW, sh, sw, ph, pw, np.float32)


def deltaW_slice_f64(X, dY, FH, FW, sh, sw, ph, pw, GZ, z):
    return _dw(lib().oracle_deltaW_slice_f64, X, dY, FH, FW, sh, sw, ph, pw, np.float64,
               extra=(_i(GZ), _i(z)))


def buf_summary(deltaW_buf, deltaW):
    """Returns the Kahan-summed deltaW (input arrays untouched). deltaW_buf: [part, sizeW]."""
    part = deltaW_buf.shape[0] if deltaW_buf.size else 0
    out = np.ascontiguousarray(deltaW, dtype=np.float32).copy()
    buf = np.ascontiguousarray(deltaW_buf, dtype=np.float32)
    lib().oracle_buf_summary(_p32(buf) if part else None, _p32(out), _i(part), _i(out.size))
    return out


def kernel_remode(W):
    OC, FH, FW, IC = W.shape
    CW = np.empty((FH, FW, IC, OC), dtype=np.float32)
    lib().oracle_kernel_remode(_p32(W), _p32(CW), _i(FH), _i(FW), _i(OC), _i(IC))
    return CW


def ks_dims(FH, FW, sh, sw):
    return (FH + sh - 1) // sh, (FW + sw - 1) // sw


def _ks(fn, W, sh, sw, fill):
    OC, FH, FW, IC = W.shape
    CFH, CFW = ks_dims(FH, FW, sh, sw)
    CW = np.full((sh * sw * OC * CFH * CFW * IC,), fill, dtype=np.float32)
    fn(_p32(W), _i(FH), _i(FW), _p32(CW), _i(CFH), _i(CFW), _i(OC), _i(IC), _i(sh), _i(sw))
    return CW


def ks_remode(W, sh, sw, fill=0.0):
    return _ks(lib().oracle_ks_remode, W, sh, sw, fill)


def ks_remodev2(W, sh, sw, fill=0.0):
    return _ks(lib().oracle_ks_remodev2, W, sh, sw, fill)


def deltaX_kernelSplit_f64(dY, CW, FH, FW, IH, IW, IC, sh, sw, ph, pw):
    N, OH, OW, OC = dY.shape
    dX = np.empty((N, IH, IW, IC), dtype=np.float64)
    lib().oracle_deltaX_kernelSplit_f64(_p32(dY), _i(OH), _i(OW), _p32(CW), _i(FH), _i(FW),
                                        _p64(dX), _i(IH), _i(IW), _i(N), _i(IC), _i(OC),
                                        _i(sh), _i(sw), _i(ph), _i(pw))
    return dX


def samePercentRelative(A, B, threshold):
    A = np.ascontiguousarray(A, dtype=np.float32).ravel()
    B = np.ascontiguousarray(B, dtype=np.float32).ravel()
    assert A.size == B.size
    return float(lib().oracle_samePercentRelative(_p32(A), _p32(B), ctypes.c_long(A.size),
                                                  ctypes.c_float(threshold)))


def max_err_ratio(got, want, rel=1e-4, floor_abs=1e-5):
    """Worst err/allowed with allowed = max(rel*|want|, floor_abs); <= 1.0 passes."""
    got = np.ascontiguousarray(got, dtype=np.float32).ravel()
    want = np.ascontiguousarray(want, dtype=np.float64).ravel()
    assert got.size == want.size
    return float(lib().oracle_max_err_ratio(_p32(got), _p64(want), ctypes.c_long(got.size),
                                            ctypes.c_double(rel), ctypes.c_double(floor_abs)))


# ---- backward of batch normalisation (numpy, fp64): restates the reference's kernels operation by operation -------------
def batchNorm_xnorm(form, S, X_mean=None, X_var=None, eps=0.0, A=None, B=None):
    """X_norm as the reference's backward kernels recover it. form "given": S itself (batchNorm2D_row_deltaX_v1,
    function/extra_batchNorm2D_row_deltaX_v1.cuh:57, 76); "from_y_affine": (S - B) / A
    (extra_batchNorm_affined2D_row_deltaX_v1.cuh:56, 91-95); "from_x": (S - X_mean) * rsqrt(X_var + eps)
    (extra_batchNorm2D_row_deltaX_v2.cuh:53-54, 86-90). S is [N, M]; the per-column vectors are [M]."""
    S = np.asarray(S, dtype=np.float64)
    if form == "given":
        return S
    if form == "from_y_affine":
        return (S - np.asarray(B, dtype=np.float64)) / np.asarray(A, dtype=np.float64)
    if form == "from_x":
        return (S - np.asarray(X_mean, dtype=np.float64)) / np.sqrt(np.asarray(X_var, dtype=np.float64) + float(eps))
    raise ValueError(form)


def batchNorm_deltaAB(deltaY, X_norm):
    """(deltaA, deltaB) = (sum over rows of deltaY * X_norm, sum over rows of deltaY) per column
    (reduce/field_batchNorm_deltaAB_v2.cuh:13-14, 40-45; deltaA is the row function's deltaXp2, deltaB its deltaXp1)."""
    dY = np.asarray(deltaY, dtype=np.float64)
    return (dY * np.asarray(X_norm, dtype=np.float64)).sum(axis=0), dY.sum(axis=0)


def batchNorm_deltaX(deltaY, X_norm, X_var, eps, deltaXp1, deltaXp2, A=None):
    """deltaX = scale * (deltaY - (deltaXp1 + deltaXp2 * X_norm) / N), scale = rsqrt(X_var + eps), times A when affine
    (function/extra_batchNorm2D_row_deltaX_v1.cuh:50-58, 86-90; extra_batchNorm_affined2D_row_deltaX_v2.cuh:52-60, 99-103).
    N is the number of rows."""
    dY = np.asarray(deltaY, dtype=np.float64)
    N = dY.shape[0]
    scale = 1.0 / np.sqrt(np.asarray(X_var, dtype=np.float64) + float(eps))
    if A is not None:
        scale = scale * np.asarray(A, dtype=np.float64)
    return scale * (dY - (np.asarray(deltaXp1, dtype=np.float64) + np.asarray(deltaXp2, dtype=np.float64) * np.asarray(X_norm, dtype=np.float64)) / N)
