"""GPU: batch normalisation (given statistics), bias and leaky ReLU fused into the convolution, and the backward of the leaky
ReLU fused into backward-data, against oracle = the fp64 convolution oracle followed by the closed-form row functions in
fp64 (Cuda_function.java:1607, 1640, 3829, 3862 define them: y = x > 0 ? x : k*x; deltaX = deltaY * (Y > 0 ? 1 : k);
y = (x - mean) * rsqrt(var + eps); y = A*y + B). Bar: rel 1e-4, abs 1e-5 * max(1, rms(expected)), as for the plain operators.
Shapes are chosen so that every kernel with a fused epilogue, and both kernels that are followed by a separate pass, run."""
import numpy as np
import pytest

from oracle import oracle as O
from util import Dev, he_normal, load_package, normal, out_dim, rng, uniform

pytestmark = pytest.mark.gpu
pkg = load_package()
C3, DX, FN = pkg.Cuda_conv3D, pkg.Cuda_dconv3D_deltaX, pkg.Cuda_function


@pytest.fixture(scope="module")
def dev():
    return Dev()


def check(got, want, what):
    floor = 1e-5 * max(1.0, float(np.sqrt(np.mean(want * want))))
    r = O.max_err_ratio(got, want, 1e-4, floor)
    assert r <= 1.0, "%s: err/allowed = %.3f (rel 1e-4, abs %.3g)" % (what, r, floor)


def leaky(y, k):
    return np.where(y > 0, y, k * y)


def params(OC, seed):
    r = rng(seed)
    return dict(Bias=r.standard_normal(OC).astype(np.float32), mean=r.standard_normal(OC).astype(np.float32),
                var=r.uniform(0.5, 2.0, OC).astype(np.float32), A=r.uniform(0.5, 1.5, OC).astype(np.float32),
                B=r.standard_normal(OC).astype(np.float32))


def closed_form(conv64, P, use, eps, k):
    y = conv64.copy()
    if "Bias" in use:
        y = y + P["Bias"].astype(np.float64)
    if "bn" in use:
        y = (y - P["mean"].astype(np.float64)) / np.sqrt(P["var"].astype(np.float64) + eps)
    if "affine" in use:
        y = y * P["A"].astype(np.float64) + P["B"].astype(np.float64)
    return leaky(y, k)


def make_epilogue(dev, P, use, eps, k):
    keep = {n: dev.put(v) for n, v in P.items()}
    ep = pkg.Epilogue(Bias=keep["Bias"].data_ptr() if "Bias" in use else 0,
                      X_mean=keep["mean"].data_ptr() if "bn" in use else 0, X_var=keep["var"].data_ptr() if "bn" in use else 0,
                      eps=eps, A=keep["A"].data_ptr() if "affine" in use else 0, B=keep["B"].data_ptr() if "affine" in use else 0, k=k)
    return ep, keep


FUSED_SHAPES = [
    # N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, kernel that serves it
    (4, 14, 14, 64, 64, 3, 3, 1, 1, 1, 1, "3x3 stride-1 kernel with the prefetched halo"),
    (4, 8, 8, 128, 132, 3, 3, 1, 1, 1, 1, "the same, narrow rows, ragged block of output channels"),
    (4, 13, 13, 20, 36, 3, 3, 1, 1, 1, 1, "ragged channel counts: generic kernel"),
    (4, 14, 14, 64, 128, 3, 3, 2, 2, 1, 1, "strided: the kernel without LDS from CW, the LDS-halo kernel from W"),
    (4, 12, 12, 96, 64, 5, 5, 1, 1, 2, 2, "LDS-halo kernel, 5x5"),
    (4, 30, 30, 4, 64, 7, 7, 2, 2, 3, 3, "stem kernel"),
    (4, 14, 14, 64, 128, 1, 1, 1, 1, 0, 0, "1x1 streaming kernel + a separate pass"),
    (4, 9, 11, 12, 20, 5, 4, 2, 3, 2, 1, "generic kernel"),
    (4, 12, 12, 64, 96, 3, 3, 2, 2, 1, 1, "the kernel without LDS, two blocks of 48 output channels (3 per lane)"),
    (4, 12, 12, 32, 32, 3, 3, 2, 2, 1, 1, "the same, 2 per lane"),
    (4, 12, 12, 32, 16, 5, 5, 1, 1, 2, 2, "the same, 1 per lane"),
    (4, 10, 10, 48, 36, 3, 3, 1, 1, 1, 1, "the same, 36 of a block of 48"),
    (128, 24, 24, 48, 64, 3, 3, 1, 1, 1, 1, "the same, 27 steps and 18 items per workgroup: whole items with an empty step"),
]


@pytest.mark.parametrize("shape", FUSED_SHAPES)
@pytest.mark.parametrize("use,k", [(("bn", "affine"), 0.1), (("Bias",), 0.01), (("Bias", "bn"), 1.0), ((), 0.25)])
def test_forward_with_batchnorm_and_leaky_relu_in_the_epilogue(dev, shape, use, k):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, what = shape
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    X, W = normal((N, IH, IW, IC), 8101), he_normal(OC, FH, FW, IC, 8102)
    if IC == 4:
        X[..., 3] = 0
        W[..., 3] = 0
    P, eps = params(OC, 8103), 1e-5
    want = closed_form(O.conv3D_f64(X, W, sh, sw, ph, pw), P, use, eps, k)
    ep, keep = make_epilogue(dev, P, use, eps, k)
    x, w = dev.put(X), dev.put(W)
    cw = dev.empty(FH * FW * IC * OC)
    C3.kernel_remode(dev.stream, w.data_ptr(), cw.data_ptr(), FH, FW, OC, IC)
    y1, y2 = dev.guarded(N, OH, OW, OC), dev.guarded(N, OH, OW, OC)
    C3.conv3D_fused(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), FH, FW, ep, y1.data_ptr(), OH, OW, N, IC, OC, sh, sw, ph, pw)
    C3.conv3D_GemmR_fused(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), FH, FW, ep, y2.data_ptr(), OH, OW,
                          N, IC, OC, sh, sw, ph, pw)
    check(dev.get(y1), want, "conv3D_fused %s %s k=%g (%s)" % (shape[:11], use, k, what))
    check(dev.get(y2), want, "conv3D_GemmR_fused %s %s k=%g (%s)" % (shape[:11], use, k, what))
    L = pkg.lib()
    try:   # the generic kernel has the fused form too
        L.alpha_conv_set_fwd_algo(3)
        y3 = dev.guarded(N, OH, OW, OC)
        C3.conv3D_GemmR_fused(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), FH, FW, ep, y3.data_ptr(), OH, OW,
                              N, IC, OC, sh, sw, ph, pw)
        check(dev.get(y3), want, "generic kernel, fused %s %s" % (shape[:11], use))
    finally:
        L.alpha_conv_set_fwd_algo(0)


@pytest.mark.parametrize("IC,OC", [(64, 64), (20, 36)])   # persistent Winograd kernel + a pass / fused in the other kernel
def test_winograd_forward_with_fused_epilogue(dev, IC, OC):
    N, IH, IW = 4, 14, 13
    X, W = normal((N, IH, IW, IC), 8201), he_normal(OC, 3, 3, IC, 8202)
    P, eps, k, use = params(OC, 8203), 1e-3, 0.2, ("Bias", "bn", "affine")
    want = closed_form(O.conv3D_f64(X, W, 1, 1, 1, 1), P, use, eps, k)
    ep, keep = make_epilogue(dev, P, use, eps, k)
    x, w = dev.put(X), dev.put(W)
    u = dev.empty(C3.winograd_filter_size(IC, OC))
    C3.winograd_filter_transform(dev.stream, w.data_ptr(), u.data_ptr(), IC, OC)
    y = dev.guarded(N, IH, IW, OC)
    C3.conv3D_winograd_fused(dev.streams, 1, x.data_ptr(), IH, IW, u.data_ptr(), ep, y.data_ptr(), IH, IW, N, IC, OC, 1, 1)
    check(dev.get(y), want, "conv3D_winograd_fused IC=%d OC=%d" % (IC, OC))


DX_SHAPES = [
    # N, IH, IW, IC, OC, F, p
    (4, 14, 14, 64, 64, 3, 1),      # prefetching kernel
    (4, 13, 11, 36, 44, 3, 1),      # generic kernel (ragged channels)
    (4, 12, 12, 64, 96, 5, 2),      # LDS-halo kernel
    (4, 14, 14, 128, 64, 1, 0),     # 1x1 streaming kernel + a separate pass
    (4, 12, 12, 96, 64, 3, 1),      # the kernel without LDS, two blocks of 48 produced channels (3 per lane)
    (4, 12, 12, 32, 64, 5, 2),      # the same, 2 per lane
    (4, 10, 10, 16, 32, 3, 1),      # the same, 1 per lane
    (4, 10, 10, 36, 64, 3, 1),      # the same, 36 of a block of 48
    (128, 24, 24, 64, 48, 3, 1),    # the same, 27 steps and 18 items per workgroup: whole items with an empty step
]


@pytest.mark.parametrize("shape", DX_SHAPES)
def test_backward_data_with_the_leaky_relu_derivative_in_the_epilogue(dev, shape):
    N, IH, IW, IC, OC, F_, p = shape
    OH, OW = out_dim(IH, IW, F_, F_, 1, 1, p, p)
    dY, W = normal((N, OH, OW, OC), 8301), he_normal(OC, F_, F_, IC, 8302)
    k = 0.1
    Xf = leaky(normal((N, IH, IW, IC), 8303).astype(np.float64), k).astype(np.float32)   # an activated tensor: output of a leaky ReLU
    Xf[0, 0, 0, :4] = 0.0   # zero counts as "not positive" (Y' = 1 + (0 >= Y)*(k - 1))
    want = O.deltaX_f64(dY, W, IH, IW, 1, 1, p, p) * np.where(Xf > 0, 1.0, k)
    dy, w, xf = dev.put(dY), dev.put(W), dev.put(Xf)
    dx = dev.guarded(N, IH, IW, IC)
    DX.dconv3D_deltaX_s1_leakyRelu(dev.streams, 1, dy.data_ptr(), OH, OW, w.data_ptr(), F_, F_, xf.data_ptr(), k, dx.data_ptr(), IH, IW,
                                   N, IC, OC, p, p)
    check(dev.get(dx), want, "deltaX_s1_leakyRelu %s" % (shape,))


@pytest.mark.parametrize("shape", [(4, 16, 16, 64, 128, 3, 3, 2, 2, 1, 1),     # four phases in one launch of the kernel without LDS
                                   (6, 14, 18, 132, 96, 3, 3, 2, 2, 1, 1),     # the same, three blocks of produced channels (the last ragged), ragged last tile
                                   (4, 14, 14, 128, 256, 1, 1, 2, 2, 0, 0),    # 1x1 stride 2: three phases without taps, whose zeros pass the gate too
                                   (4, 13, 11, 16, 16, 5, 4, 3, 2, 2, 1)])     # one launch of the generic kernel per phase
def test_strided_backward_data_with_the_leaky_relu_derivative_in_the_epilogue(dev, shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    dY, W = normal((N, OH, OW, OC), 8311), he_normal(OC, FH, FW, IC, 8312)
    k = 0.2
    Xf = leaky(normal((N, IH, IW, IC), 8313).astype(np.float64), k).astype(np.float32)
    want = O.deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw) * np.where(Xf > 0, 1.0, k)
    CFH, CFW = O.ks_dims(FH, FW, sh, sw)
    dy, w, xf = dev.put(dY), dev.put(W), dev.put(Xf)
    cw = dev.empty(sh * sw * OC * CFH * CFW * IC, fill=0.0)
    DX.ks_remodev2(dev.stream, w.data_ptr(), FH, FW, cw.data_ptr(), CFH, CFW, OC, IC, sh, sw)
    L = pkg.lib()
    try:
        for sharing in (0, 1, -1):   # the kernel without LDS: wavefronts with items of their own / sharing every group / by shape
            L.alpha_conv_set_kernel_split_sharing(sharing)
            dx = dev.guarded(N, IH, IW, IC)
            DX.dconv3D_deltaX_kernelSplit_leakyRelu(dev.streams, 1, dy.data_ptr(), OH, OW, cw.data_ptr(), FH, FW, xf.data_ptr(), k, dx.data_ptr(),
                                                    IH, IW, N, IC, OC, sh, sw, ph, pw)
            check(dev.get(dx), want, "deltaX_kernelSplit_leakyRelu sharing %d %s" % (sharing, shape))
    finally:
        L.alpha_conv_set_kernel_split_sharing(-1)


def test_row_functions_keep_pad_columns_zero_and_match_their_definitions(dev):
    height, width, stride = 37, 10, 12     # two pad columns per row
    X = normal((height, stride), 8401)
    X[:, width:] = 0
    dYv = normal((height, stride), 8402)
    P, eps, k = params(stride, 8403), 1e-4, 0.3
    x, dy = dev.put(X), dev.put(dYv)
    m, v, a, b = (dev.put(P[n]) for n in ("mean", "var", "A", "B"))
    pad = np.zeros((height, stride - width))
    y = dev.empty(height, stride, fill=float("nan"))
    FN.leakyRelu2D(dev.stream, x.data_ptr(), k, y.data_ptr(), height * stride, width, stride)
    got = dev.get(y)
    assert np.array_equal(got[:, :width], leaky(X[:, :width], np.float32(k)).astype(np.float32)) and np.array_equal(got[:, width:], pad)
    FN.leakyRelu2D_deltaX_v1(dev.stream, y.data_ptr(), dy.data_ptr(), x.data_ptr(), k, height * stride, width, stride)
    got = dev.get(y)
    assert np.array_equal(got[:, :width], (dYv * np.where(X > 0, np.float32(1), np.float32(k)))[:, :width]) and np.array_equal(got[:, width:], pad)
    X64 = X.astype(np.float64)
    norm = (X64 - P["mean"]) / np.sqrt(P["var"].astype(np.float64) + eps)
    FN.batchNorm2D_row(dev.stream, x.data_ptr(), m.data_ptr(), v.data_ptr(), eps, stride, y.data_ptr(), height * stride, width, stride)
    got = dev.get(y)
    check(np.ascontiguousarray(got[:, :width]), np.ascontiguousarray(norm[:, :width]), "batchNorm2D_row")
    assert np.array_equal(got[:, width:], pad)
    FN.batchNorm_affined2D_row(dev.stream, x.data_ptr(), m.data_ptr(), v.data_ptr(), eps, a.data_ptr(), b.data_ptr(), stride, x.data_ptr(),
                               height * stride, width, stride)     # in place
    got = dev.get(x)
    check(np.ascontiguousarray(got[:, :width]), np.ascontiguousarray((norm * P["A"] + P["B"])[:, :width]), "batchNorm_affined2D_row in place")
    assert np.array_equal(got[:, width:], pad)
    with pytest.raises(pkg.AlphaConvError):
        FN.leakyRelu2D(dev.stream, x.data_ptr(), k, y.data_ptr(), height * stride + 4, width, stride)   # lengthv not rows * stride


def test_engine_operators_with_fused_epilogues(dev):
    """conv -> bn -> leakyRelu forward and leakyRelu' -> deltaX backward through the host layer, stride 1 and stride 2."""
    eng = pkg.engine.Engine(dev.stream)
    try:
        for (N, IH, IW, IC, OC, F_, s, p) in [(8, 14, 14, 64, 64, 3, 1, 1), (8, 14, 14, 64, 128, 3, 2, 1), (8, 14, 14, 64, 128, 1, 1, 0)]:
            OH, OW = out_dim(IH, IW, F_, F_, s, s, p, p)
            X, W, dY = normal((N, IH, IW, IC), 8501), he_normal(OC, F_, F_, IC, 8502), normal((N, OH, OW, OC), 8503)
            P, eps, k, use = params(OC, 8504), 1e-5, 0.1, ("bn", "affine")
            ep, keep = make_epilogue(dev, P, use, eps, k)
            x, w, dy = dev.put(X), dev.put(W), dev.put(dY)
            y, dx = dev.guarded(N, OH, OW, OC), dev.guarded(N, IH, IW, IC)
            eng.conv3D_fused(y.data_ptr(), OH, OW, x.data_ptr(), IH, IW, w.data_ptr(), F_, F_, N, IC, OC, s, s, p, p, ep)
            Xf = leaky(X.astype(np.float64), k).astype(np.float32)
            xf = dev.put(Xf)
            eng.dconv3D_deltaX_leakyRelu(dx.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, w.data_ptr(), F_, F_, N, IC, OC, s, s, p, p,
                                         xf.data_ptr(), k)
            eng.sync()
            check(dev.get(y), closed_form(O.conv3D_f64(X, W, s, s, p, p), P, use, eps, k), "engine conv3D_fused s=%d F=%d" % (s, F_))
            check(dev.get(dx), O.deltaX_f64(dY, W, IH, IW, s, s, p, p) * np.where(Xf > 0, 1.0, k), "engine deltaX_leakyRelu s=%d F=%d" % (s, F_))
    finally:
        eng.close()
