"""GPU parity tests: every C-ABI entry of the conv3D hot path against the CPU oracle.

Bar (stated per test): max relative error 1e-4 with an absolute floor near zero of
1e-5 * max(1, rms(expected)), measured against the fp64 oracle (ratio err/allowed <= 1). For the
forward configs (He-normal filters, unit-scale inputs) rms is about 1 and the floor is the plain
1e-5; the K-long gradient sums of backward-filter have outputs of magnitude sqrt(K), and an fp32
accumulation cannot resolve 1e-5 next to partial sums that large, so the floor follows the scale of
the output tensor. The reference's own pass criterion (Vector.samePercentRelative with the thresholds of
experiments/test_cuda/Cuda_conv3D_test.java:86-97, Cuda_dconv3D_dX_test.java:93-100,
Cuda_dconv3D_dW_test.java:98-105) is applied the way the reference applies it: on uniform [0,1) data
(test_reference_style_criterion_*). Index-only work (filter re-layouts) and the Kahan buffer summation
must be bit-exact.
"""
import numpy as np
import pytest

from oracle import oracle as O
from util import Dev, he_normal, load_package, normal, out_dim, uniform

pytestmark = pytest.mark.gpu

pkg = load_package()
C3 = pkg.Cuda_conv3D
DX = pkg.Cuda_dconv3D_deltaX
DW = pkg.Cuda_dconv3D_deltaW

REL, ABS = 1e-4, 1e-5


@pytest.fixture(scope="module")
def dev():
    return Dev()


def tolerance_floor(want64):
    return ABS * max(1.0, float(np.sqrt(np.mean(np.square(want64)))))


def check(got, want64, what):
    floor = tolerance_floor(want64)
    ratio = O.max_err_ratio(got, want64, REL, floor)
    assert ratio <= 1.0, "%s: err/allowed = %.3f (rel %g, abs floor %.3g)" % (what, ratio, REL, floor)


def check_reference_style(got, cpu_float, what, thr, min_fraction):
    """The reference's test: fraction of elements with |a-b|/|a+b| < thr against its float CPU result."""
    sp = O.samePercentRelative(cpu_float, got, thr)
    assert sp >= min_fraction, "%s: samePercentRelative(%g) = %.5f < %g" % (what, thr, sp, min_fraction)


# ----------------------------------------------------------------------------------------------
# forward
# ----------------------------------------------------------------------------------------------
FWD_SHAPES = [
    # N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw
    (4, 32, 32, 4, 64, 3, 3, 1, 1, 1, 1),      # BASELINE config 1 (IC=3 stored as 4)
    (8, 33, 33, 64, 128, 4, 4, 1, 1, 1, 1),    # the reference's logged shape (Cuda_conv3D.java:185)
    (4, 32, 32, 64, 252, 3, 3, 2, 2, 1, 1),    # ragged OC (Cuda_conv3D.java:191)
    (4, 16, 16, 128, 128, 3, 3, 1, 1, 1, 1),
    (4, 8, 8, 256, 256, 3, 3, 1, 1, 1, 1),
    (4, 7, 7, 512, 512, 3, 3, 1, 1, 1, 1),
    (4, 30, 30, 4, 64, 7, 7, 2, 2, 3, 3),      # stem-like
    (4, 14, 14, 64, 128, 3, 3, 2, 2, 1, 1),
    (4, 14, 14, 64, 128, 1, 1, 2, 2, 0, 0),    # 1x1 stride 2 through the general entry
    (4, 9, 11, 12, 20, 5, 5, 2, 2, 2, 2),
    (4, 10, 9, 8, 36, 2, 2, 1, 1, 0, 0),
    (4, 9, 9, 4, 4, 3, 2, 3, 2, 0, 1),
    (4, 5, 5, 4, 8, 3, 3, 1, 1, 2, 2),
    (4, 13, 13, 20, 132, 3, 3, 1, 1, 1, 1),
]


def _run_fwd(dev, entry, X, W, sh, sw, ph, pw):
    N, IH, IW, IC = X.shape
    OC, FH, FW, _ = W.shape
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    dXd, dWd = dev.put(X), dev.put(W)
    Y = dev.guarded(N, OH, OW, OC)
    S, L = dev.streams, 1
    x, w, y = dXd.data_ptr(), dWd.data_ptr(), Y.data_ptr()
    if entry in ("conv3D", "conv3D_texture"):
        getattr(C3, entry)(S, L, x, IH, IW, w, FH, FW, y, OH, OW, N, IC, OC, sh, sw, ph, pw)
    elif entry == "conv3DV2":
        C3.conv3DV2(True, S, L, x, IH, IW, w, FH, FW, y, OH, OW, N, IC, OC, sh, sw, ph, pw)
    elif entry == "conv3D_np":
        assert ph == 0 and pw == 0
        C3.conv3D_np(S, L, x, IH, IW, w, FH, FW, y, OH, OW, N, IC, OC, sh, sw)
    elif entry == "conv3D_W1":
        C3.conv3D_W1(S, L, x, IH, IW, w, y, N, IC, OC)
    else:
        CW = dev.empty(FH, FW, IC, OC, fill=float("nan"))
        C3.kernel_remode(dev.stream, w, CW.data_ptr(), FH, FW, OC, IC)
        cw = CW.data_ptr()
        if entry in ("conv3D_GemmR", "conv3D_GemmR_texture"):
            getattr(C3, entry)(S, L, x, IH, IW, w, cw, FH, FW, y, OH, OW, N, IC, OC, sh, sw, ph, pw)
        elif entry == "conv3D_GemmV2R":
            C3.conv3D_GemmV2R(False, S, L, x, IH, IW, w, cw, FH, FW, y, OH, OW, N, IC, OC, sh, sw, ph, pw)
        elif entry == "conv3D_GemmR_W1":
            C3.conv3D_GemmR_W1(S, L, x, IH, IW, w, cw, y, N, IC, OC)
        else:
            raise AssertionError(entry)
    return dev.get(Y)


@pytest.mark.parametrize("shape", FWD_SHAPES)
@pytest.mark.parametrize("entry", ["conv3D", "conv3D_GemmR"])
def test_forward_general_entries(dev, shape, entry):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    X = uniform((N, IH, IW, IC), 1001)
    W = he_normal(OC, FH, FW, IC, 1002)
    want = O.conv3D_f64(X, W, sh, sw, ph, pw)
    check(_run_fwd(dev, entry, X, W, sh, sw, ph, pw), want, "%s %s" % (entry, shape))


@pytest.mark.parametrize("entry", ["conv3D", "conv3D_GemmR"])
def test_forward_three_channels_stored_as_four(dev, entry):
    """The kernel for 4 stored channels leaves out the MFMA step of channel 3 for every block of 64 output channels whose
    weights of that channel are all zero (a 3-channel layer as the engine pads it). Here the first 64 output channels are
    padded like that and the other 64 use all four channels, so one launch runs both paths; the pad channel of X holds
    data on purpose: it must not reach the first 64 outputs and must reach the others."""
    N, IH, IW, OC, F_, s_, p_ = 4, 30, 30, 128, 7, 2, 3
    X = uniform((N, IH, IW, 4), 1011)
    W = he_normal(OC, F_, F_, 4, 1012)
    W[:64, :, :, 3] = 0.0
    check(_run_fwd(dev, entry, X, W, s_, s_, p_, p_), O.conv3D_f64(X, W, s_, s_, p_, p_), entry)


@pytest.mark.parametrize("entry", ["conv3D_texture", "conv3DV2", "conv3D_GemmR_texture", "conv3D_GemmV2R"])
def test_forward_hint_variants_give_same_result(dev, entry):
    shape = (8, 12, 12, 32, 96, 3, 3, 1, 1, 1, 1)
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    X, W = normal((N, IH, IW, IC), 1003), he_normal(OC, FH, FW, IC, 1004)
    check(_run_fwd(dev, entry, X, W, sh, sw, ph, pw), O.conv3D_f64(X, W, sh, sw, ph, pw), entry)


def test_forward_np_and_w1_entries(dev):
    X, W = normal((4, 11, 10, 16), 1005), he_normal(40, 3, 3, 16, 1006)
    check(_run_fwd(dev, "conv3D_np", X, W, 2, 1, 0, 0), O.conv3D_f64(X, W, 2, 1, 0, 0), "conv3D_np")
    X, W = normal((4, 14, 14, 256), 1007), he_normal(1024, 1, 1, 256, 1008)
    want = O.conv3D_f64(X, W, 1, 1, 0, 0)
    check(_run_fwd(dev, "conv3D_W1", X, W, 1, 1, 0, 0), want, "conv3D_W1")
    check(_run_fwd(dev, "conv3D_GemmR_W1", X, W, 1, 1, 0, 0), want, "conv3D_GemmR_W1")


TAP_SHAPES = [
    # stride-1 layers served by the LDS-halo kernel: N, IH, IW, IC, OC, FH, FW, ph, pw
    (4, 56, 56, 64, 64, 3, 3, 1, 1),      # c3a / c5b geometry (units of 2 rows)
    (8, 32, 32, 64, 64, 3, 3, 1, 1),      # c2a geometry
    (8, 28, 28, 128, 128, 3, 3, 1, 1),    # c3b: two channel passes, two oc slices
    (16, 14, 14, 256, 256, 3, 3, 1, 1),   # c3c: units cross image borders
    (36, 7, 7, 512, 512, 3, 3, 1, 1),     # c3d: a unit spans several images
    (20, 8, 8, 256, 256, 3, 3, 1, 1),     # c2c
    (4, 13, 11, 36, 44, 3, 3, 1, 1),      # ragged IC / OC (zero-filled channel tails)
    (4, 12, 17, 100, 132, 5, 5, 2, 2),
    (4, 10, 10, 64, 64, 3, 3, 0, 0),      # no padding
    (4, 9, 14, 96, 72, 2, 4, 1, 3),       # non-square filter, asymmetric pad
    (4, 6, 5, 32, 64, 3, 3, 2, 2),        # pad larger than usual
    (3, 5, 5, 64, 64, 3, 3, 1, 1),        # fewer pixels than one unit
    (5, 17, 19, 32, 48, 3, 3, 1, 1),      # halo-prefetching kernel: one pass, ragged OC, last unit partial
    (2, 30, 62, 96, 80, 3, 3, 1, 1),      # ... widest row it takes (64 padded pixels), three passes, two oc slices
    (3, 18, 18, 64, 64, 3, 3, 0, 0),      # ... no padding
    (7, 40, 24, 64, 64, 3, 3, 2, 2),      # ... pad 2
    (180, 20, 20, 32, 64, 3, 3, 1, 1),    # ... more units than workgroup slots: several units per workgroup, 2-tile pieces
]


@pytest.mark.parametrize("shape", TAP_SHAPES)
def test_forward_lds_halo_kernel_vs_oracle_and_generic(dev, shape):
    N, IH, IW, IC, OC, FH, FW, ph, pw = shape
    X, W = normal((N, IH, IW, IC), 1101), he_normal(OC, FH, FW, IC, 1102)
    want = O.conv3D_f64(X, W, 1, 1, ph, pw)
    L = pkg.lib()
    try:
        L.alpha_conv_set_fwd_algo(0)
        fast = _run_fwd(dev, "conv3D_GemmR", X, W, 1, 1, ph, pw)
        fast_w = _run_fwd(dev, "conv3D", X, W, 1, 1, ph, pw)   # W[OC,FH,FW,IC] as it is (3x3: 128-bit filter fragment loads)
        L.alpha_conv_set_fwd_algo(3)
        generic = _run_fwd(dev, "conv3D_GemmR", X, W, 1, 1, ph, pw)
        L.alpha_conv_set_fwd_algo(1)
        halo = _run_fwd(dev, "conv3D_GemmR", X, W, 1, 1, ph, pw)
        L.alpha_conv_set_fwd_algo(6)
        direct = _run_fwd(dev, "conv3D_GemmR", X, W, 1, 1, ph, pw)
    finally:
        L.alpha_conv_set_fwd_algo(0)
    check(halo, want, "lds-halo fwd (forced) %s" % (shape,))
    check(direct, want, "fwd without LDS (forced) %s" % (shape,))
    check(fast, want, "lds-halo fwd %s" % (shape,))
    check(fast_w, want, "lds-halo fwd from W %s" % (shape,))
    check(generic, want, "generic fwd %s" % (shape,))


@pytest.mark.parametrize("shape", TAP_SHAPES)
def test_deltaX_lds_halo_kernel_vs_oracle(dev, shape):
    N, IH, IW, IC, OC, FH, FW, ph, pw = shape
    if ph > FH - 1 or pw > FW - 1:
        pytest.skip("backward-data needs ph <= FH-1")
    OH, OW = out_dim(IH, IW, FH, FW, 1, 1, ph, pw)
    dY, W = normal((N, OH, OW, OC), 1103), he_normal(OC, FH, FW, IC, 1104)
    dy, w = dev.put(dY), dev.put(W)
    want = O.deltaX_f64(dY, W, IH, IW, 1, 1, ph, pw)
    L = pkg.lib()
    try:
        for algo in (0, 1, 6, 3):   # the library's choice, the LDS-halo kernels, the kernel without LDS, the generic kernel
            L.alpha_conv_set_fwd_algo(algo)
            dXo = dev.guarded(N, IH, IW, IC)
            DX.dconv3D_deltaX_s1(dev.streams, 1, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, dXo.data_ptr(), IH, IW, N, IC, OC, ph, pw)
            check(dev.get(dXo), want, "dX algo %d %s" % (algo, shape))
    finally:
        L.alpha_conv_set_fwd_algo(0)


WINO_SHAPES = [
    # N, IH, IW, IC, OC, ph, pw   (3x3, stride 1)
    (4, 56, 56, 64, 64, 1, 1),
    (8, 28, 28, 128, 128, 1, 1),
    (16, 14, 14, 256, 256, 1, 1),
    (36, 7, 7, 512, 512, 1, 1),      # odd output size: partial tiles on the right / bottom
    (4, 13, 11, 36, 44, 1, 1),       # ragged channels, odd sizes
    (4, 10, 12, 16, 32, 0, 0),       # no padding
    (4, 6, 9, 32, 64, 2, 2),         # padding 2
    (3, 5, 5, 64, 64, 1, 1),         # fewer tiles than one workgroup
    (4, 32, 32, 4, 64, 1, 1),        # BASELINE config 1 geometry (IC = 3 stored as 4)
    # persistent kernel (IC % 16 == 0), 512 workgroups on 256 compute units:
    (25, 56, 56, 16, 16, 1, 1),      # 613 items: one whole item each, 101 left over -> 202 half items, ragged last group
    (40, 56, 56, 16, 20, 1, 1),      # 980 items: 468 left over -> whole extra items; 20 of 64 output channels
    (16, 56, 56, 32, 128, 1, 1),     # 784 items in two blocks of output channels, two chunks
    (66, 55, 53, 16, 16, 1, 1),      # 1560 items: three whole items each, 24 left over -> 48 half items; odd sizes
    (2, 9, 9, 48, 72, 1, 1),         # fewer items than workgroups, ragged block of output channels
]


@pytest.mark.parametrize("shape", WINO_SHAPES)
def test_forward_winograd_f2x2_vs_direct_oracle(dev, shape):
    """Winograd F(2x2,3x3) against the same fp64 direct convolution; tolerance as for the direct kernels
    (rel 1e-4, abs floor 1e-5 * max(1, rms)): the transforms only add a few ulps on unit-scale data."""
    N, IH, IW, IC, OC, ph, pw = shape
    OH, OW = out_dim(IH, IW, 3, 3, 1, 1, ph, pw)
    X, W = normal((N, IH, IW, IC), 1201), he_normal(OC, 3, 3, IC, 1202)
    x, w = dev.put(X), dev.put(W)
    U = dev.empty(C3.winograd_filter_size(IC, OC), fill=float("nan"))
    y = dev.guarded(N, OH, OW, OC)
    C3.winograd_filter_transform(dev.stream, w.data_ptr(), U.data_ptr(), IC, OC)
    C3.conv3D_winograd(dev.streams, 1, x.data_ptr(), IH, IW, U.data_ptr(), y.data_ptr(), OH, OW, N, IC, OC, ph, pw)
    check(dev.get(y), O.conv3D_f64(X, W, 1, 1, ph, pw), "winograd %s" % (shape,))


@pytest.mark.parametrize("shape", WINO_SHAPES)
def test_deltaX_winograd_vs_oracle(dev, shape):
    """Backward-data of a 3x3 stride-1 layer as a Winograd convolution of deltaY (rotated filter, padding 2 - p);
    same bar as the direct kernels. The table's layers read as (N, IH, IW, IC, OC) of the layer whose deltaX is wanted."""
    N, IH, IW, IC, OC, ph, pw = shape
    OH, OW = out_dim(IH, IW, 3, 3, 1, 1, ph, pw)
    dY, W = normal((N, OH, OW, OC), 1211), he_normal(OC, 3, 3, IC, 1212)
    dy, w = dev.put(dY), dev.put(W)
    U = dev.empty(C3.winograd_filter_size(IC, OC), fill=float("nan"))
    dXo = dev.guarded(N, IH, IW, IC)
    DX.winograd_filter_transform_deltaX(dev.stream, w.data_ptr(), U.data_ptr(), IC, OC)
    DX.dconv3D_deltaX_winograd(dev.streams, 1, dy.data_ptr(), OH, OW, U.data_ptr(), dXo.data_ptr(), IH, IW, N, IC, OC, ph, pw)
    check(dev.get(dXo), O.deltaX_f64(dY, W, IH, IW, 1, 1, ph, pw), "winograd dX %s" % (shape,))


def test_winograd_filter_transform_matches_G_g_Gt(dev):
    IC, OC = 8, 12
    W = he_normal(OC, 3, 3, IC, 1203)
    w = dev.put(W)
    U = dev.empty(16 * IC * OC, fill=float("nan"))
    C3.winograd_filter_transform(dev.stream, w.data_ptr(), U.data_ptr(), IC, OC)
    G = np.array([[1, 0, 0], [.5, .5, .5], [.5, -.5, .5], [0, 0, 1]], np.float64)
    g = W.astype(np.float64).transpose(0, 3, 1, 2)              # [oc][ic][3][3]
    want = np.einsum("ai,ocij,bj->aboc", G, g, G)               # [4][4][oc][ic] -> U[xi][ic][oc]
    want = want.transpose(0, 1, 3, 2).reshape(16, IC, OC)
    np.testing.assert_allclose(dev.get(U).reshape(16, IC, OC), want, rtol=1e-6, atol=1e-7)


def test_forward_oc_sweep_covers_every_ragged_width(dev):
    # the reference's "for OC from 1 to 128: correct" sweep (Cuda_conv3D_test.java:155-156), in steps of 4
    X = uniform((4, 9, 9, 8), 1009)
    for OC in range(4, 136, 4):
        W = he_normal(OC, 3, 3, 8, 1010 + OC)
        want = O.conv3D_f64(X, W, 1, 1, 1, 1)
        check(_run_fwd(dev, "conv3D_GemmR", X, W, 1, 1, 1, 1), want, "GemmR OC=%d" % OC)
        check(_run_fwd(dev, "conv3D", X, W, 1, 1, 1, 1), want, "conv3D OC=%d" % OC)


def test_forward_exact_small_integers(dev):
    # all-ones tensors: every partial sum is a small integer, so the result must be bit-exact
    X, W = np.ones((4, 7, 6, 8), np.float32), np.ones((12, 3, 3, 8), np.float32)
    want = O.conv3D_naive(X, W, 1, 1, 1, 1)
    assert np.array_equal(_run_fwd(dev, "conv3D_GemmR", X, W, 1, 1, 1, 1), want)
    assert np.array_equal(_run_fwd(dev, "conv3D", X, W, 1, 1, 1, 1), want)


def test_kernel_remode_bit_exact(dev):
    for (OC, FH, FW, IC) in [(64, 3, 3, 64), (8, 1, 1, 4), (252, 4, 4, 12), (4, 7, 7, 4), (132, 3, 5, 20)]:
        W = uniform((OC, FH, FW, IC), 1011)
        CW = dev.empty(FH, FW, IC, OC, fill=float("nan"))
        w = dev.put(W)
        C3.kernel_remode(dev.stream, w.data_ptr(), CW.data_ptr(), FH, FW, OC, IC)
        assert np.array_equal(dev.get(CW), O.kernel_remode(W))


# ----------------------------------------------------------------------------------------------
# backward-data
# ----------------------------------------------------------------------------------------------
DX_S1_SHAPES = [
    (4, 32, 32, 64, 64, 3, 3, 1, 1),     # N, IH, IW, IC, OC, FH, FW, ph, pw
    (4, 31, 31, 128, 32, 4, 4, 1, 1),    # Cuda_dconv3D_deltaX.java:259 (OH=31-ish)
    (4, 16, 16, 256, 64, 3, 3, 1, 1),
    (4, 8, 8, 256, 256, 3, 3, 1, 1),
    (4, 9, 10, 12, 20, 5, 5, 2, 2),
    (4, 9, 9, 8, 8, 3, 3, 0, 0),
    (4, 7, 9, 4, 36, 3, 2, 2, 1),
    (4, 12, 12, 132, 44, 3, 3, 1, 1),
    (16, 14, 14, 128, 256, 3, 3, 1, 1),  # 392 items of 144 steps on 256 workgroups: one or two each, all shared by the wavefronts
    (40, 7, 7, 192, 512, 3, 3, 1, 1),    # 369 items (the last tile ragged), three blocks of produced channels, 288 steps
    (48, 20, 20, 64, 48, 3, 3, 1, 1),    # 48 reduced channels: 27 steps, an odd number (the filter, rotated in place, is read with a negative tap stride)
    (32, 12, 12, 96, 80, 5, 5, 2, 2),    # 125 steps
]


@pytest.mark.parametrize("shape", DX_S1_SHAPES)
def test_deltaX_s1_entries(dev, shape):
    N, IH, IW, IC, OC, FH, FW, ph, pw = shape
    OH, OW = out_dim(IH, IW, FH, FW, 1, 1, ph, pw)
    dY, W = normal((N, OH, OW, OC), 2001), he_normal(OC, FH, FW, IC, 2002)
    want = O.deltaX_f64(dY, W, IH, IW, 1, 1, ph, pw)
    dy, w = dev.put(dY), dev.put(W)
    for entry in ("dconv3D_deltaX_s1", "dconv3D_deltaX_s1_texture", "dconv3D_deltaX_V2_s1"):
        dXo = dev.guarded(N, IH, IW, IC)
        args = (dev.streams, 1, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, dXo.data_ptr(), IH, IW, N, IC, OC, ph, pw)
        if entry == "dconv3D_deltaX_V2_s1":
            DX.dconv3D_deltaX_V2_s1(True, *args)
        else:
            getattr(DX, entry)(*args)
        check(dev.get(dXo), want, "%s %s" % (entry, shape))


def test_deltaX_W1(dev):
    for (N, IH, IW, IC, OC) in [(4, 14, 14, 256, 64), (4, 9, 7, 64, 256), (4, 5, 5, 12, 20)]:
        dY, W = normal((N, IH, IW, OC), 2003), he_normal(OC, 1, 1, IC, 2004)
        dXo = dev.guarded(N, IH, IW, IC)
        dy, w = dev.put(dY), dev.put(W)  # keep the device buffers alive across the call
        DX.dconv3D_deltaX_W1(dev.streams, 1, dy.data_ptr(), w.data_ptr(), dXo.data_ptr(), IH, IW, N, IC, OC)
        check(dev.get(dXo), O.deltaX_f64(dY, W, IH, IW, 1, 1, 0, 0), "deltaX_W1")


POINTWISE_SHAPES = [
    # N, IH, IW, IC, OC: 1x1 stride-1 layers served by the streaming GEMM kernel (reduced side a multiple of 64,
    # produced side 64/128/256, filter fits in LDS), forward in both filter layouts and backward-data
    (4, 14, 14, 256, 64),     # c5a geometry: K = 256 forward, K = 64 backward
    (4, 9, 7, 64, 256),       # c5c geometry; 252 pixels: the last 16-pixel tile is ragged
    (3, 5, 5, 128, 128),      # 75 pixels: fewer tiles than wavefronts
    (2, 33, 31, 64, 64),      # 2046 pixels
    (1, 1, 3, 192, 64),       # 3 pixels: a single ragged tile; K = 192 = 3 blocks forward (backward falls to another kernel)
    # the kernel without LDS (both operands from memory): any K that is a multiple of 32, N in blocks of 64
    (8, 56, 56, 64, 64),      # 25088 pixels = 1568 tiles: shares of 0 or 1 tile
    (37, 28, 28, 96, 36),     # 29008 pixels = 1813 tiles; K = 96 forward, a ragged block of 36 produced channels (K = 36 backward: other kernel)
    (64, 28, 30, 32, 200),    # 53760 pixels = 3360 tiles over 2048 wavefronts: shares of 1 and 2 tiles; 200 = 3 blocks + 8 channels
    (32, 56, 56, 64, 32),     # 100352 pixels = 6272 tiles: shares of 3 and 4 tiles (c5 geometry with fewer channels)
    (64, 60, 64, 32, 32),     # 245760 pixels = 15360 tiles: shares of 7 and 8 tiles (4 + 3 and 4 + 4)
    # what the library chooses by shape for narrow 1x1 layers with 64 pixels or more per compute unit
    (64, 28, 28, 192, 16),    # forward: 16 produced channels, blocks of 16 in the kernel of direct_conv; backward: 16 reduced channels = one step and an empty one per whole item
    (64, 28, 28, 192, 32),    # forward: blocks of 32; backward: 32 reduced into 192, the kernel without LDS of the 1x1 family
    (64, 28, 28, 192, 48),    # forward: a block of 48; backward: 48 reduced channels = 3 steps and an empty one
    (32, 28, 28, 192, 96),    # backward: 96 reduced into 192
    (96, 24, 24, 16, 64),     # forward: 16 reduced channels, 13 or 14 items per workgroup (no whole items: the generic kernel by shape)
    (192, 24, 24, 16, 64),    # the same with 27 items per workgroup: whole items, one step and an empty one
]


@pytest.mark.parametrize("shape", POINTWISE_SHAPES)
def test_pointwise_kernel_forward_and_deltaX(dev, shape):
    N, IH, IW, IC, OC = shape
    X, W, dY = normal((N, IH, IW, IC), 2101), he_normal(OC, 1, 1, IC, 2102), normal((N, IH, IW, OC), 2103)
    want_y, want_dx = O.conv3D_f64(X, W, 1, 1, 0, 0), O.deltaX_f64(dY, W, IH, IW, 1, 1, 0, 0)
    L = pkg.lib()
    outs = {}
    import os
    VARIANTS = (0, 3, "resident", "direct")
    try:
        # 0: the 1x1 kernels as the library chooses between them, 3: generic kernel, "resident" / "direct": algo 0 with
        # the kernel without LDS switched off / on wherever it applies, so that both stay tested on every shape
        for algo in VARIANTS:
            L.alpha_conv_set_fwd_algo(algo if isinstance(algo, int) else 0)
            if not isinstance(algo, int):
                L.alpha_conv_set_pointwise_algo(0 if algo == "resident" else 1)
            outs[algo] = (_run_fwd(dev, "conv3D_W1", X, W, 1, 1, 0, 0), _run_fwd(dev, "conv3D_GemmR_W1", X, W, 1, 1, 0, 0))
            dXo = dev.guarded(N, IH, IW, IC)
            dy, w = dev.put(dY), dev.put(W)
            DX.dconv3D_deltaX_W1(dev.streams, 1, dy.data_ptr(), w.data_ptr(), dXo.data_ptr(), IH, IW, N, IC, OC)
            outs[algo] += (dev.get(dXo),)
    finally:
        L.alpha_conv_set_pointwise_algo(-1)
        L.alpha_conv_set_fwd_algo(0)
    for algo in VARIANTS:
        check(outs[algo][0], want_y, "conv3D_W1 algo %s %s" % (algo, shape))
        check(outs[algo][1], want_y, "conv3D_GemmR_W1 algo %s %s" % (algo, shape))
        check(outs[algo][2], want_dx, "deltaX_W1 algo %s %s" % (algo, shape))


@pytest.mark.parametrize("shape", [
    # N, IH, IW, IC, OC, sh, sw: strided 1x1 layers (c4c geometry and ragged ones) through the general entries
    (8, 28, 28, 64, 128, 2, 2),
    (4, 9, 7, 128, 192, 2, 3),
    (2, 15, 15, 256, 320, 3, 1),
])
def test_pointwise_kernel_strided(dev, shape):
    N, IH, IW, IC, OC, sh, sw = shape
    X, W = normal((N, IH, IW, IC), 2111), he_normal(OC, 1, 1, IC, 2112)
    want = O.conv3D_f64(X, W, sh, sw, 0, 0)
    for entry in ("conv3D", "conv3D_GemmR", "conv3D_np"):
        check(_run_fwd(dev, entry, X, W, sh, sw, 0, 0), want, "%s strided 1x1 %s" % (entry, shape))


def _run_fwd_biased(dev, X, W, B, sh, sw, ph, pw):
    N, IH, IW, IC = X.shape
    OC, FH, FW, _ = W.shape
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    x, w, b = dev.put(X), dev.put(W), dev.put(B)
    cw = dev.empty(FH * FW * IC * OC, fill=float("nan"))
    C3.kernel_remode(dev.stream, w.data_ptr(), cw.data_ptr(), FH, FW, OC, IC)
    y = dev.guarded(N, OH, OW, OC)
    C3.conv3D_GemmR_biased(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), FH, FW, b.data_ptr(), y.data_ptr(),
                           OH, OW, N, IC, OC, sh, sw, ph, pw)
    return dev.get(y)


DIRECT_CONV_SHAPES = [
    # N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw: the kernel without LDS (both operands from memory), forward from CW
    (4, 28, 28, 64, 128, 3, 3, 2, 2, 1, 1),     # c4b geometry (56 -> 28 there): two blocks of produced channels
    (16, 56, 56, 64, 128, 3, 3, 2, 2, 1, 1),    # 12544 pixels = 784 tiles x 2 blocks: shares of 1 and 2 items
    (4, 15, 13, 64, 64, 3, 3, 2, 2, 1, 1),      # odd sizes: tiles straddle rows and images, last tile ragged
    (4, 17, 19, 32, 96, 5, 3, 2, 3, 2, 1),      # mixed strides, non-square filter, 96 = one and a half blocks
    (2, 16, 16, 96, 64, 2, 2, 2, 2, 0, 0),      # no overlap, no padding
    (3, 9, 30, 64, 36, 3, 3, 1, 2, 1, 1),       # stride only along the width; a ragged block of 36 produced channels
    (2, 12, 12, 32, 64, 3, 3, 1, 1, 1, 1),      # stride 1 (forced): every tap of a border pixel's window in the padding
    (1, 5, 5, 16, 8, 7, 6, 1, 1, 3, 3),         # window larger than the image, 16 channels (42 steps), 8 produced channels
    (40, 20, 20, 32, 64, 3, 3, 2, 2, 1, 1),     # 4000 pixels = 250 tiles: fewer items than wavefronts
    (64, 30, 34, 48, 64, 3, 3, 2, 2, 1, 1),     # 16320 pixels = 1020 tiles, 48 channels: 27 steps, an odd number -> one empty step is added
    # items left over in a workgroup are shared by its eight wavefronts (reduction cut in eight, partial sums through LDS):
    (8, 24, 24, 32, 192, 3, 3, 1, 1, 1, 1),     # 864 items on 256 workgroups: 3 or 4 each, all shared, 18 steps in parts of 2 and 3; a pair meets the end of a block
    (4, 10, 10, 32, 64, 1, 1, 1, 1, 0, 0),      # 2 steps: six of the eight wavefronts have none
    (32, 40, 40, 32, 64, 3, 3, 1, 1, 1, 1),     # 3200 items: 12 or 13 per workgroup, all shared in groups of 4, 4, 4 (, 1)
    (44, 40, 40, 32, 64, 3, 3, 1, 1, 1, 1),     # 4400 items: 17 or 18 per workgroup = 4 whole per SIMD + 1 or 2 shared
    (2, 56, 56, 64, 64, 3, 3, 1, 1, 1, 1),      # 392 items: 1 or 2 per workgroup, 36 steps in parts of 4 and 5
    # long reductions
    (16, 14, 14, 256, 128, 3, 3, 1, 1, 1, 1),   # 392 items of 144 steps on 256 workgroups: one or two each
    (36, 7, 7, 512, 192, 3, 3, 1, 1, 1, 1),     # 333 items of 288 steps (ragged last tile), three blocks of produced channels
    (4, 9, 9, 256, 64, 5, 5, 2, 2, 2, 2),       # strided 5x5: 7 items of 400 steps on 7 workgroups
    # short reductions (4 or 8 steps)
    (48, 56, 56, 64, 128, 1, 1, 2, 2, 0, 0),    # c4c geometry: 4704 items of 4 steps = 18 or 19 per workgroup: 4 whole per SIMD + 2 or 3 shared
    (24, 56, 56, 128, 64, 1, 1, 1, 1, 0, 0),    # 1x1 stride 1, 8 steps, 4704 items
    (64, 64, 64, 16, 64, 2, 2, 2, 2, 0, 0),     # 2x2 taps x 16 channels = 4 steps, 4096 items = 16 per workgroup, all whole
    # an odd number of steps (tap, 16 channels): an empty step is added to every group
    (64, 28, 28, 48, 96, 3, 3, 1, 1, 1, 1),     # 27 steps; 6272 items = 24 or 25 per workgroup: whole items and a shared one
    (24, 14, 14, 80, 128, 5, 5, 1, 1, 2, 2),    # 125 steps; 588 items: 2 or 3 per workgroup, all shared (parts of 15 and 16 steps)
    (40, 20, 20, 16, 64, 3, 3, 1, 1, 1, 1),     # 9 steps; 1000 items: 3 or 4 per workgroup, the eighth part of 10 steps is 1 or 2
    (96, 24, 24, 16, 64, 1, 1, 1, 1, 0, 0),     # a single step per item (1x1, 16 channels)
    # one to three produced channels per lane: blocks of 16, 32 or 48 produced channels instead of 64
    (8, 20, 20, 32, 48, 3, 3, 1, 1, 1, 1),      # one block of 48
    (8, 14, 14, 64, 144, 3, 3, 1, 1, 1, 1),     # three blocks of 48
    (8, 20, 20, 64, 32, 3, 3, 2, 2, 1, 1),      # one block of 32, strided
    (8, 17, 15, 32, 16, 5, 5, 1, 1, 2, 2),      # one block of 16, ragged last tile
    (8, 14, 14, 48, 24, 3, 3, 1, 1, 1, 1),      # 24 of a block of 32 (12 lanes of 2), an odd number of steps
    (8, 14, 14, 32, 20, 3, 3, 2, 2, 1, 1),      # 20 of a block of 32
    (8, 14, 14, 32, 12, 1, 1, 1, 1, 0, 0),      # 12 of a block of 16, 1x1
    (8, 14, 14, 32, 40, 3, 3, 1, 1, 1, 1),      # 40 = 3 per lane would split a lane's group at the end: four per lane
    # an odd number of steps and 16 or more items per workgroup: whole items, each followed by an empty step
    (128, 28, 28, 48, 192, 1, 1, 1, 1, 0, 0),   # 1x1, 48 channels: 3 steps + 1; 18816 items = 73 or 74 per workgroup
    (128, 28, 28, 16, 64, 3, 3, 1, 1, 1, 1),    # 9 steps + 1; 6272 items = 24 or 25 per workgroup
    (192, 24, 24, 16, 64, 1, 1, 1, 1, 0, 0),    # a single step + 1; 27 items per workgroup
    (96, 30, 30, 48, 48, 3, 3, 2, 2, 1, 1),     # 27 steps + 1, strided, one block of 48 produced channels; 5400 items = 21 or 22 per workgroup
    (64, 33, 31, 16, 20, 5, 5, 1, 1, 2, 2),     # 25 steps + 1, 20 of a block of 32, ragged last tile; 4092 items
    (50, 14, 14, 48, 256, 3, 3, 1, 1, 1, 1),    # 27 steps, 2452 items: 9 or 10 per workgroup - a group of two tiles per SIMD, steps 14 + 14
]


@pytest.mark.parametrize("shape", DIRECT_CONV_SHAPES)
def test_forward_direct_conv_kernel(dev, shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    X, W = normal((N, IH, IW, IC), 2401), he_normal(OC, FH, FW, IC, 2402)
    bias = normal((OC,), 2403)
    want = O.conv3D_f64(X, W, sh, sw, ph, pw)
    L = pkg.lib()
    try:
        for algo in (6, 1, 3):      # the kernel without LDS, the LDS-halo kernel, the generic kernel
            L.alpha_conv_set_fwd_algo(algo)
            for entry in ("conv3D_GemmR", "conv3D_GemmR_texture", "conv3D_GemmV2R"):
                check(_run_fwd(dev, entry, X, W, sh, sw, ph, pw), want, "%s algo %d %s" % (entry, algo, shape))
            check(_run_fwd_biased(dev, X, W, bias, sh, sw, ph, pw), want + bias.astype(np.float64), "GemmR_biased algo %d %s" % (algo, shape))
    finally:
        L.alpha_conv_set_fwd_algo(0)


STEM_FWD_SHAPES = [
    # N, IH, IW, OC, F, s, p: 4 stored input channels, 7x7 or 3x3 -> the stem kernels (without LDS, with LDS), forward
    (4, 30, 30, 64, 7, 2, 3),       # 900 pixels: ragged last tile, tiles straddle rows and images
    (16, 64, 64, 64, 7, 2, 3),      # 16384 pixels = 1024 tiles: shares of one tile, single-tile groups only
    (64, 64, 64, 64, 7, 2, 3),      # 4096 tiles: 4 per SIMD = 2 per wavefront
    (40, 96, 96, 64, 7, 2, 3),      # 92160 pixels = 5760 tiles: 5 or 6 per SIMD, groups of four tiles
    (150, 96, 96, 64, 7, 2, 3),     # 21600 tiles: 21 or 22 per SIMD, two or three groups of four in a row (the register sets swap)
    (8, 33, 29, 36, 7, 1, 3),       # stride 1, 36 output channels (a ragged block)
    (8, 21, 23, 136, 7, 2, 0),      # no padding, three blocks of output channels (the last with 8)
    (4, 32, 32, 64, 3, 1, 1),       # c1 geometry: 3x3 = three tap groups (taps 9..11 are padding)
    (32, 17, 19, 20, 3, 2, 1),      # 3x3 stride 2, 20 output channels
    (3, 34, 32, 64, 3, 1, 1),       # rows are whole tiles (groups = 16 columns x 4 rows), 102 rows: the last group has two
    (5, 38, 64, 64, 7, 2, 3),       # 7x7 stride 2, rows of 32 pixels, 19 rows per image: groups straddle images, 95 rows in all
    (3, 9, 9, 64, 5, 1, 2),         # 5x5: not taken by the kernel without LDS -> the LDS one
]


@pytest.mark.parametrize("shape", STEM_FWD_SHAPES)
@pytest.mark.parametrize("rgb", [True, False])
def test_forward_stem_kernels(dev, shape, rgb):
    """rgb: the fourth stored channel is zero in X and W (three logical channels; its MFMA step is left out)."""
    N, IH, IW, OC, F_, s_, p_ = shape
    X, W = normal((N, IH, IW, 4), 2501), he_normal(OC, F_, F_, 4, 2502)
    bias = normal((OC,), 2503)
    if rgb:
        X[..., 3] = 0.0
        W[..., 3] = 0.0
    want = O.conv3D_f64(X, W, s_, s_, p_, p_)
    L = pkg.lib()
    try:
        for algo in (0, 1, 3):      # the kernel without LDS, the kernel with the window in LDS, the generic kernel
            L.alpha_conv_set_fwd_algo(algo)
            for entry in ("conv3D", "conv3D_GemmR", "conv3D_GemmV2R"):
                check(_run_fwd(dev, entry, X, W, s_, s_, p_, p_), want, "%s algo %d %s" % (entry, algo, shape))
            check(_run_fwd_biased(dev, X, W, bias, s_, s_, p_, p_), want + bias.astype(np.float64), "GemmR_biased algo %d %s" % (algo, shape))
    finally:
        L.alpha_conv_set_fwd_algo(0)


STRIDED_TAP_SHAPES = [
    # N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw: strided layers with >= 32 input channels through the LDS-halo kernel
    # (columns of the halo de-interleaved by ow parity class), remode entries
    (4, 28, 28, 64, 128, 3, 3, 2, 2, 1, 1),     # c4b geometry (56 -> 28 there)
    (4, 15, 13, 64, 64, 3, 3, 2, 2, 1, 1),      # odd sizes: units cross rows and images
    (4, 17, 19, 32, 96, 5, 3, 2, 3, 2, 1),      # mixed strides, non-square filter
    (2, 16, 16, 96, 64, 2, 2, 2, 2, 0, 0),      # 2x2 stride 2 (no overlap), ragged channel pass
    (3, 9, 30, 64, 64, 3, 3, 1, 2, 1, 1),       # stride only along the width
]


@pytest.mark.parametrize("shape", STRIDED_TAP_SHAPES)
def test_strided_forward_through_the_halo_kernel(dev, shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    X, W, B = normal((N, IH, IW, IC), 2301), he_normal(OC, FH, FW, IC, 2302), normal((OC,), 2303)
    want = O.conv3D_f64(X, W, sh, sw, ph, pw)
    L = pkg.lib()
    try:
        for algo in (0, 1, 3):   # 0: the library's choice, 1: LDS-halo kernel, 3: generic kernel
            L.alpha_conv_set_fwd_algo(algo)
            for entry in ("conv3D_GemmR", "conv3D_GemmV2R"):
                check(_run_fwd(dev, entry, X, W, sh, sw, ph, pw), want, "%s algo %d %s" % (entry, algo, shape))
    finally:
        L.alpha_conv_set_fwd_algo(0)
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    x, w, b = dev.put(X), dev.put(W), dev.put(B)
    cw = dev.empty(FH * FW * IC * OC, fill=float("nan"))
    C3.kernel_remode(dev.stream, w.data_ptr(), cw.data_ptr(), FH, FW, OC, IC)
    y = dev.empty(N, OH, OW, OC, fill=float("nan"))
    C3.conv3D_GemmR_biased(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), FH, FW, b.data_ptr(), y.data_ptr(),
                           OH, OW, N, IC, OC, sh, sw, ph, pw)
    check(dev.get(y), want + B.astype(np.float64)[None, None, None, :], "strided biased %s" % (shape,))


BIAS_SHAPES = [
    # N, IH, IW, IC, OC, F, s, p: one layer per forward kernel (the bias rides in each kernel's epilogue)
    (4, 14, 14, 64, 64, 3, 1, 1),      # LDS-halo kernel
    (4, 9, 9, 64, 128, 1, 1, 0),       # streaming 1x1 GEMM
    (4, 16, 16, 4, 64, 7, 2, 3),       # stem kernel
    (4, 13, 11, 32, 48, 3, 2, 1),      # generic kernel (strided)
    (4, 6, 5, 12, 20, 3, 1, 1),        # generic kernel, ragged channels
    (25, 40, 40, 16, 72, 3, 1, 1),     # persistent Winograd kernel: 626 items in two blocks of output channels (the second
                                       # with 8 of 64), whole and half items
]


@pytest.mark.parametrize("shape", BIAS_SHAPES)
def test_forward_with_bias_in_the_epilogue(dev, shape):
    """Y = conv(X, W) + Bias[oc] (the reference: conv3D then linear_dual2D_row(Y, Bias), CudaFloat32EngineBase.java:1548-1557)."""
    N, IH, IW, IC, OC, F_, s_, p_ = shape
    OH, OW = out_dim(IH, IW, F_, F_, s_, s_, p_, p_)
    X, W, B = normal((N, IH, IW, IC), 2201), he_normal(OC, F_, F_, IC, 2202), normal((OC,), 2203)
    want = O.conv3D_f64(X, W, s_, s_, p_, p_) + B.astype(np.float64)[None, None, None, :]
    x, w, b = dev.put(X), dev.put(W), dev.put(B)
    cw = dev.empty(F_ * F_ * IC * OC, fill=float("nan"))
    C3.kernel_remode(dev.stream, w.data_ptr(), cw.data_ptr(), F_, F_, OC, IC)
    y = dev.empty(N, OH, OW, OC, fill=float("nan"))
    C3.conv3D_biased(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), F_, F_, b.data_ptr(), y.data_ptr(), OH, OW, N, IC, OC,
                     s_, s_, p_, p_)
    check(dev.get(y), want, "conv3D_biased %s" % (shape,))
    y = dev.empty(N, OH, OW, OC, fill=float("nan"))
    C3.conv3D_GemmR_biased(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), F_, F_, b.data_ptr(), y.data_ptr(),
                           OH, OW, N, IC, OC, s_, s_, p_, p_)
    check(dev.get(y), want, "conv3D_GemmR_biased %s" % (shape,))
    if F_ == 3 and s_ == 1:
        U = dev.empty(16 * IC * OC, fill=float("nan"))
        C3.winograd_filter_transform(dev.stream, w.data_ptr(), U.data_ptr(), IC, OC)
        y = dev.empty(N, OH, OW, OC, fill=float("nan"))
        C3.conv3D_winograd_biased(dev.streams, 1, x.data_ptr(), IH, IW, U.data_ptr(), b.data_ptr(), y.data_ptr(), OH, OW, N, IC, OC,
                                  p_, p_)
        check(dev.get(y), want, "conv3D_winograd_biased %s" % (shape,))


KS_SHAPES = [
    # N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw
    (4, 16, 16, 64, 128, 3, 3, 2, 2, 1, 1),
    (4, 32, 32, 64, 32, 4, 4, 2, 2, 1, 1),
    (4, 14, 14, 32, 64, 1, 1, 2, 2, 0, 0),
    (4, 16, 12, 16, 24, 5, 5, 2, 2, 2, 2),
    (4, 12, 12, 20, 16, 7, 7, 2, 2, 3, 3),
    (4, 12, 9, 16, 16, 3, 3, 3, 3, 1, 1),     # Ims: IH % sh == 0
    (4, 13, 11, 16, 16, 5, 4, 3, 2, 2, 1),    # general kernel split (IH % sh != 0)
    (4, 9, 9, 12, 8, 2, 2, 2, 2, 0, 0),       # odd IH with stride 2
    # deltaY channel counts the LDS-halo kernel takes (>= 32): every phase in one launch
    (4, 28, 28, 64, 128, 3, 3, 2, 2, 1, 1),   # c4b geometry
    (4, 15, 13, 20, 96, 5, 5, 2, 2, 2, 2),    # odd sizes: the phases have different numbers of pixels; 96 = 64 + 32 channels
    (4, 12, 12, 36, 68, 7, 7, 2, 2, 3, 3),    # ragged channel counts on both sides
    (4, 12, 9, 64, 32, 3, 3, 3, 3, 1, 1),     # nine phases of one tap each
    (4, 13, 11, 32, 64, 5, 4, 3, 2, 2, 1),    # six phases, rectangular filter
    (4, 20, 20, 64, 64, 2, 2, 2, 2, 0, 0),    # one tap per phase, no padding
    (4, 11, 11, 64, 48, 3, 3, 2, 2, 0, 0),    # no padding, odd size
    # the kernel without LDS: phases of one size (IH % sh == 0, IW % sw == 0), deltaY channels a multiple of 32
    (16, 56, 56, 64, 128, 3, 3, 2, 2, 1, 1),  # 12544 coarse pixels = 784 tiles: shares of 0 and 1 item
    (6, 30, 34, 36, 64, 3, 3, 2, 2, 1, 1),    # 1530 coarse pixels (last tile ragged), a ragged block of 36 produced channels
    (40, 56, 56, 32, 64, 3, 3, 2, 2, 1, 1),   # 1960 tiles: shares of several items per SIMD
    (24, 60, 52, 36, 32, 5, 5, 2, 2, 2, 2),   # the same with phases of 9, 6, 6 and 4 taps, ragged channels and a ragged last tile
    (6, 14, 18, 132, 96, 3, 3, 2, 2, 1, 1),   # small map, 96 channels of deltaY (6 steps per tap: parts of 0 and 2 steps), three blocks of produced channels
    (10, 8, 8, 64, 256, 3, 3, 2, 2, 1, 1),    # 4x4 coarse pixels per image, 256 channels of deltaY
    (4, 12, 16, 64, 32, 3, 3, 1, 2, 1, 1),    # two phases (stride along the width only)
    (4, 16, 12, 68, 96, 3, 5, 2, 1, 1, 2),    # two phases (stride along the height only), two blocks of produced channels
    (4, 14, 14, 64, 64, 1, 1, 2, 2, 0, 0),    # 1x1 stride 2: three phases without taps write zeros
    (4, 16, 16, 32, 32, 2, 3, 2, 2, 0, 1),    # filter rows = stride: every phase one tap row
    # 1x1 filters under a larger stride: one scattered matrix product with zeros in between (its own kernel where IH = sh * OH)
    (8, 28, 28, 64, 128, 1, 1, 2, 2, 0, 0),   # c4c geometry (56 -> 28 there) at N = 8
    (3, 9, 12, 132, 96, 1, 1, 3, 2, 0, 0),    # blocks of 3 x 2 pixels, 54 pixels of deltaY (ragged tile), 132 produced channels (ragged block)
    (2, 6, 20, 8, 32, 1, 1, 1, 4, 0, 0),      # stride along the width only, 8 produced channels
    (2, 15, 15, 64, 64, 1, 1, 2, 2, 0, 0),    # odd size: the last row and column of deltaX belong to no block -> the phase kernels
    (4, 14, 14, 128, 256, 1, 1, 2, 2, 0, 0),  # more than 20 FLOP per byte moved: the phases (one with the tap, three of zeros) instead of the scattered product
]


@pytest.mark.parametrize("shape", KS_SHAPES)
def test_deltaX_kernel_split_family(dev, shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    dY, W = normal((N, OH, OW, OC), 2005), he_normal(OC, FH, FW, IC, 2006)
    want = O.deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw)
    CFH, CFW = O.ks_dims(FH, FW, sh, sw)
    dy, w = dev.put(dY), dev.put(W)
    CW = dev.empty(sh * sw * OC * CFH * CFW * IC, fill=0.0)
    DX.ks_remodev2(dev.stream, w.data_ptr(), FH, FW, CW.data_ptr(), CFH, CFW, OC, IC, sh, sw)
    assert np.array_equal(dev.get(CW), O.ks_remodev2(W, sh, sw)), "ks_remodev2 layout"
    CW1 = dev.empty(sh * sw * OC * CFH * CFW * IC, fill=0.0)
    DX.ks_remode(dev.stream, w.data_ptr(), FH, FW, CW1.data_ptr(), CFH, CFW, OC, IC, sh, sw)
    assert np.array_equal(dev.get(CW1), O.ks_remode(W, sh, sw)), "ks_remode layout"

    entries = ["dconv3D_deltaX_kernelSplit"]
    if IH % sh == 0 and IW % sw == 0:
        entries += ["dconv3D_deltaX_ksImsR", "dconv3D_deltaX_ksImsR_texture"]
    if sh == 2 and sw == 2 and IH % 2 == 0 and IW % 2 == 0:
        entries += ["dconv3D_deltaX_ksIms2R", "dconv3D_deltaX_ksIms2R_texture", "dconv3D_deltaX_ksV2_Ims2R"]
    for entry in entries:
        dXo = dev.guarded(N, IH, IW, IC)
        base = (dev.streams, 1, dy.data_ptr(), OH, OW, CW.data_ptr(), FH, FW, dXo.data_ptr(), IH, IW, N, IC, OC)
        if entry == "dconv3D_deltaX_ksV2_Ims2R":
            DX.dconv3D_deltaX_ksV2_Ims2R(False, *base, ph, pw)
        elif "Ims2R" in entry:
            getattr(DX, entry)(*base, ph, pw)
        else:
            getattr(DX, entry)(*base, sh, sw, ph, pw)
        check(dev.get(dXo), want, "%s %s" % (entry, shape))
    # the other paths - 1: all phases in one launch of the LDS-halo kernel (stride 2 x 2, even sizes) else as 3; 3: one
    # launch of the generic kernel per phase; 6: as 0 (the kernel without LDS where the phases have one size) - and the
    # tiny-IC entry, which reads W in place
    L = pkg.lib()
    try:
        # the kernel without LDS with every wavefront on items of its own, and with the workgroup's wavefronts sharing
        # every group (by shape above: the small layers share)
        for sharing in (0, 1):
            L.alpha_conv_set_kernel_split_sharing(sharing)
            dXo = dev.guarded(N, IH, IW, IC)
            DX.dconv3D_deltaX_kernelSplit(dev.streams, 1, dy.data_ptr(), OH, OW, CW.data_ptr(), FH, FW, dXo.data_ptr(), IH, IW, N, IC, OC,
                                          sh, sw, ph, pw)
            check(dev.get(dXo), want, "kernelSplit sharing %d %s" % (sharing, shape))
            dXo = dev.guarded(N, IH, IW, IC)
            DX.dconv3D_deltaX_crossAdd(dev.streams, 1, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, dXo.data_ptr(), IH, IW, N, IC, OC,
                                       sh, sw, ph, pw)
            check(dev.get(dXo), want, "crossAdd (filter in place) sharing %d %s" % (sharing, shape))
    finally:
        L.alpha_conv_set_kernel_split_sharing(-1)
    try:
        for algo in (1, 3, 6):
            L.alpha_conv_set_fwd_algo(algo)
            dXo = dev.guarded(N, IH, IW, IC)
            DX.dconv3D_deltaX_kernelSplit(dev.streams, 1, dy.data_ptr(), OH, OW, CW.data_ptr(), FH, FW, dXo.data_ptr(), IH, IW, N, IC, OC,
                                          sh, sw, ph, pw)
            check(dev.get(dXo), want, "kernelSplit algo %d %s" % (algo, shape))
            dXo = dev.guarded(N, IH, IW, IC)
            DX.dconv3D_deltaX_crossAdd(dev.streams, 1, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, dXo.data_ptr(), IH, IW, N, IC, OC,
                                       sh, sw, ph, pw)
            check(dev.get(dXo), want, "crossAdd (filter in place) algo %d %s" % (algo, shape))
    finally:
        L.alpha_conv_set_fwd_algo(0)
    dXo = dev.guarded(N, IH, IW, IC)
    DX.dconv3D_deltaX_crossAdd(dev.streams, 1, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, dXo.data_ptr(), IH, IW, N, IC, OC, sh, sw, ph, pw)
    check(dev.get(dXo), want, "crossAdd (filter in place) %s" % (shape,))


@pytest.mark.parametrize("shape", [
    (4, 16, 16, 4, 64, 7, 7, 2, 2, 3, 3),      # stem backward (IC = 3 stored as 4)
    (4, 12, 12, 8, 32, 3, 3, 1, 1, 1, 1),
    (4, 12, 12, 16, 32, 4, 4, 2, 2, 1, 1),
    (4, 11, 13, 8, 12, 3, 3, 3, 2, 1, 0),
])
def test_deltaX_crossAdd_is_deterministic_gather(dev, shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    dY, W = normal((N, OH, OW, OC), 2007), he_normal(OC, FH, FW, IC, 2008)
    dy, w = dev.put(dY), dev.put(W)
    outs = []
    for _ in range(2):
        dXo = dev.guarded(N, IH, IW, IC)
        DX.dconv3D_deltaX_crossAdd(dev.streams, 1, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, dXo.data_ptr(), IH, IW,
                                   N, IC, OC, sh, sw, ph, pw)
        outs.append(dev.get(dXo))
    check(outs[0], O.deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw), "crossAdd %s" % (shape,))
    assert np.array_equal(outs[0], outs[1])


DX_STEM_SHAPES = [
    # N, IH, IW, OC, FH, FW, sh, sw, ph, pw: 4 stored input channels, strides 1 or 2 -> the stem backward-data kernel
    (4, 32, 32, 64, 7, 7, 2, 2, 3, 3),      # c4a geometry: window 4 x 4, one block of 16 x 16 coarse pixels per image... and a row of blocks
    (2, 46, 70, 64, 7, 7, 2, 2, 3, 3),      # several blocks per image, ragged in both directions (23 x 35 coarse pixels)
    (3, 21, 19, 64, 7, 7, 2, 2, 3, 3),      # odd sizes: the last coarse row and column have one phase only
    (5, 16, 16, 32, 7, 7, 2, 2, 3, 3),      # 32 output channels: two wavefronts' share of the reduction is empty
    (2, 18, 18, 20, 5, 5, 2, 2, 2, 2),      # window 3 x 3 inside the 4 x 4 kernel, ragged channel count
    (4, 16, 20, 64, 3, 3, 2, 2, 1, 1),      # window 2 x 2 (the small instantiation)
    (4, 17, 15, 48, 4, 4, 2, 2, 1, 1),      # 4 x 4 stride 2 padding 1: window 3 x 3
    (4, 14, 14, 64, 2, 2, 2, 2, 0, 0),      # one tap per phase
    (3, 12, 18, 64, 3, 3, 1, 1, 1, 1),      # stride 1: one phase, window 3 x 3
    (3, 12, 18, 16, 3, 5, 1, 2, 1, 2),      # mixed strides: two phases
    (3, 19, 12, 64, 6, 3, 2, 1, 2, 1),      # stride along the height only, no padding symmetry
    (2, 20, 20, 64, 7, 7, 2, 2, 0, 0),      # no padding: window 4 x 4 from offset -3
    (140, 16, 16, 64, 7, 7, 2, 2, 3, 3),    # 140 blocks over 512 workgroups: most get none
    (9, 64, 64, 64, 7, 7, 2, 2, 3, 3),      # 72 blocks per... 9 x 4 x 2 blocks: every XCD's range holds several
]


@pytest.mark.parametrize("shape", DX_STEM_SHAPES)
def test_deltaX_stem_kernel(dev, shape):
    N, IH, IW, OC, FH, FW, sh, sw, ph, pw = shape
    IC = 4
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    dY, W = normal((N, OH, OW, OC), 2301), he_normal(OC, FH, FW, IC, 2302)
    W[..., 3] = 0      # three logical channels stored as four
    want = O.deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw)
    dy, w = dev.put(dY), dev.put(W)
    L = pkg.lib()
    outs = {}
    try:
        for algo in (0, 0, 3):          # twice through the stem kernel (bit-identical), once through the generic one
            L.alpha_conv_set_fwd_algo(algo)
            dXo = dev.guarded(N, IH, IW, IC)
            DX.dconv3D_deltaX_crossAdd(dev.streams, 1, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, dXo.data_ptr(), IH, IW,
                                       N, IC, OC, sh, sw, ph, pw)
            outs.setdefault(algo, []).append(dev.get(dXo))
    finally:
        L.alpha_conv_set_fwd_algo(0)
    check(outs[0][0], want, "stem deltaX %s" % (shape,))
    check(outs[3][0], want, "generic deltaX %s" % (shape,))
    assert np.array_equal(outs[0][0], outs[0][1])
    assert not np.any(outs[0][0][..., 3])     # the pad channel's gradient is exactly zero


# ----------------------------------------------------------------------------------------------
# backward-filter
# ----------------------------------------------------------------------------------------------
DW_SHAPES = [
    # N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw
    (4, 32, 32, 64, 64, 3, 3, 1, 1, 1, 1),
    (4, 32, 32, 64, 256, 4, 4, 2, 2, 1, 1),    # Cuda_dconv3D_deltaW.java:327
    (8, 8, 8, 256, 256, 3, 3, 1, 1, 1, 1),
    (4, 16, 16, 4, 64, 7, 7, 2, 2, 3, 3),
    (4, 13, 11, 12, 20, 5, 3, 2, 1, 2, 1),
    (4, 9, 9, 132, 36, 3, 3, 1, 1, 1, 1),
]


def _sum_partials(dev, dWo, buf, GridZ):
    DW.buf_summary(dev.stream, buf.data_ptr(), dWo.data_ptr(), GridZ - 1, dWo.numel())
    return dev.get(dWo)


@pytest.mark.parametrize("shape", DW_SHAPES)
def test_deltaW_entries(dev, shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    X, dY = normal((N, IH, IW, IC), 3001), normal((N, OH, OW, OC), 3002)
    want = O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw)
    x, dy = dev.put(X), dev.put(dY)
    dWo = dev.guarded(OC, FH, FW, IC)
    DW.dconv3D_deltaW(dev.streams, 1, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(), FH, FW, N, IC, OC, sh, sw, ph, pw)
    check(dev.get(dWo), want, "dconv3D_deltaW %s" % (shape,))
    sizeW = OC * FH * FW * IC
    for entry in ("dconv3D_deltaW_GemmSK", "dconv3D_deltaW_GemmV2SK"):
        for GridZ in (2, 5, 16):
            dWo = dev.guarded(OC, FH, FW, IC)
            buf = dev.empty(GridZ - 1, sizeW, fill=float("nan"))
            getattr(DW, entry)(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(), buf.data_ptr(),
                               FH, FW, N, IC, OC, sh, sw, ph, pw)
            check(_sum_partials(dev, dWo, buf, GridZ), want, "%s GridZ=%d %s" % (entry, GridZ, shape))


def test_deltaW_split_k_slices_follow_the_reference_partition(dev):
    # slice z must hold exactly k in [z*GK_slice, ...) with GK_slice = (GK/GZ)>>3<<3, the last slice the rest
    N, IH, IW, IC, OC, F_, s, p = 4, 9, 9, 8, 8, 3, 1, 1
    OH, OW = out_dim(IH, IW, F_, F_, s, s, p, p)
    X, dY = normal((N, IH, IW, IC), 3003), normal((N, OH, OW, OC), 3004)
    x, dy = dev.put(X), dev.put(dY)
    GridZ, sizeW = 5, OC * F_ * F_ * IC
    dWo = dev.guarded(OC, F_, F_, IC)
    buf = dev.empty(GridZ - 1, sizeW, fill=float("nan"))
    DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(), buf.data_ptr(),
                             F_, F_, N, IC, OC, s, s, p, p)
    parts = [dev.get(dWo)] + [b.reshape(OC, F_, F_, IC) for b in dev.get(buf)]
    for z in range(GridZ):
        check(parts[z], O.deltaW_slice_f64(X, dY, F_, F_, s, s, p, p, GridZ, z), "slice %d" % z)


DW_STREAM_SHAPES = [
    # N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, GridZ, R: the persistent backward-filter kernel (one workgroup per compute
    # unit; its own partition of the pixels among deltaW and the buffers, so only the sum is compared). On 256 compute units
    # (R: pieces per item where every item is cut into equal pieces - partial sums R .. GridZ - 1 are then zeros - else None):
    (128, 8, 8, 256, 256, 3, 3, 1, 1, 1, 1, 3, None),      # c2c: 144 items in a line cut into 256 shares, 2 or 3 pieces per item
    (32, 56, 56, 64, 64, 3, 3, 1, 1, 1, 1, 128, 28),     # c5b: 9 items x 28 pieces, buffers 28 .. 127 filled with zeros
    (40, 30, 30, 64, 128, 3, 3, 2, 2, 1, 1, 16, 14),     # stride 2, rows of 15 pixels (ragged last group): 18 items x 14 pieces
    (24, 21, 23, 64, 176, 3, 3, 1, 1, 1, 1, 12, None),     # 27 items (third block of output channels 48 of 64) in a line, rows of 23 pixels
    (8, 32, 32, 256, 64, 1, 1, 1, 1, 0, 0, 128, 64),     # 1x1: 4 items x 64 pieces
    (128, 9, 9, 256, 256, 4, 4, 1, 1, 1, 1, 2, 1),      # 256 items, one piece each; the one buffer is all zeros
    (16, 40, 36, 128, 64, 5, 3, 1, 2, 2, 1, 64, None),  # 5x3 filter, stride 1 x 2: 30 items in a line (8 equal pieces each would use 240 workgroups)
    (16, 7, 7, 128, 192, 3, 3, 1, 1, 1, 1, 8, None),    # 7x7 maps: rows of two pixel groups (the second ragged), 54 items of 224 groups in a line, 47 groups per workgroup
    (32, 14, 14, 128, 128, 3, 3, 2, 2, 1, 1, 8, 7),     # stride 2 onto 7x7 maps: 36 items x 7 pieces of 64 groups
    (8, 14, 14, 96, 208, 3, 3, 1, 1, 1, 1, 8, None),    # blocks filled to 61 % (96 of 128 input, 208 of 256 output channels): 72 items in a line
    (16, 14, 14, 16, 48, 5, 5, 1, 1, 2, 2, 16, 10),     # 5x5, one block filled to 19 %: 25 items x 10 pieces
    (128, 4, 4, 96, 208, 3, 3, 1, 1, 1, 1, 2, 2),       # 72 items would meet up to 5 shares of a line, GridZ is 2: 2 pieces each on 144 workgroups
    # short rows: pixel groups of four consecutive pixels of the image
    (64, 2, 2, 128, 128, 3, 3, 1, 1, 1, 1, 8, 7),       # 2x2 maps: a group is an image (two rows on per group)
    (32, 5, 5, 128, 64, 3, 3, 1, 1, 1, 1, 16, 14),      # rows of 5: 7 groups per image, the last with one pixel
    (48, 6, 6, 64, 128, 3, 3, 2, 2, 1, 1, 16, 14),      # stride 2 onto 3x3 maps: a row and a column on per group
    (16, 9, 9, 64, 64, 5, 5, 1, 1, 2, 2, 12, 10),       # rows of 9, 5x5 filter
    (2048, 1, 1, 128, 64, 1, 1, 1, 1, 0, 0, 128, 128),  # 1x1 maps: one pixel per group (a fully connected layer's shape)
    (16, 13, 13, 128, 192, 3, 3, 1, 1, 1, 1, 6, None),   # rows of 13 (AlexNet's later layers): 43 groups per image, the last with one pixel; 54 items in a line
]


@pytest.mark.parametrize("shape", DW_STREAM_SHAPES)
def test_deltaW_persistent_kernel_sum_and_reproducibility(dev, shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, GridZ, R = shape
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    X, dY = normal((N, IH, IW, IC), 3401), normal((N, OH, OW, OC), 3402)
    want = O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw)
    x, dy = dev.put(X), dev.put(dY)
    sizeW = OC * FH * FW * IC
    runs = []
    for _ in range(2):
        dWo = dev.guarded(OC, FH, FW, IC)
        buf = dev.empty(GridZ - 1, sizeW, fill=float("nan"))
        DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(), buf.data_ptr(),
                                 FH, FW, N, IC, OC, sh, sw, ph, pw)
        parts = np.concatenate([dev.get(dWo).reshape(1, -1), dev.get(buf)])
        runs.append(parts)
        check(_sum_partials(dev, dWo, buf, GridZ), want, "persistent dW GridZ=%d %s" % (GridZ, shape))
    assert np.array_equal(runs[0].view(np.uint32), runs[1].view(np.uint32)), "partial sums differ between two runs %s" % (shape,)
    if R is not None and pkg.device_info()[0] == 256:
        # this kernel, not another one, served the call: the partial sums beyond an item's pieces are zeros, the last piece is not
        assert not runs[0][R:].any() and runs[0][R - 1].any(), "partial sums %d .. %d are not all zeros %s" % (R, GridZ - 1, shape)
    # the same layer through the tap-per-workgroup kernel (the reference's partition): the totals agree within tolerance
    L = pkg.lib()
    try:
        L.alpha_conv_set_fwd_algo(4)
        dWo = dev.guarded(OC, FH, FW, IC)
        buf = dev.empty(GridZ - 1, sizeW, fill=float("nan"))
        DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(), buf.data_ptr(),
                                 FH, FW, N, IC, OC, sh, sw, ph, pw)
        check(_sum_partials(dev, dWo, buf, GridZ), want, "tap kernel GridZ=%d %s" % (GridZ, shape))
    finally:
        L.alpha_conv_set_fwd_algo(0)


@pytest.mark.parametrize("IC,OC", [(16, 64), (32, 64), (48, 128), (64, 16), (64, 32), (128, 48), (16, 16), (16, 32), (32, 16), (32, 32),
                                   (48, 16), (16, 48), (48, 32), (32, 48), (48, 48), (96, 96), (36, 44), (144, 96), (20, 208)])
@pytest.mark.parametrize("geom", [(16, 12, 12, 3, 3, 1, 1, 1, 1, 8), (12, 15, 13, 5, 5, 2, 2, 2, 2, 5)])
def test_deltaW_persistent_kernel_channels_per_lane(dev, IC, OC, geom):
    """Channel counts that the persistent backward-filter kernel holds in blocks of 16 x (1, 2 or 3) channels per lane on
    either side (16, 32, 48, 96 = 2 x 48, 144 = 3 x 48; 36 of 48; 20 = 20 of 32; 44 and 208 stay at 4 per lane): every
    pair of per-lane counts, the sum of deltaW and the buffers against the oracle, bit-identical from run to run."""
    N, IH, IW, FH, FW, sh, sw, ph, pw, GridZ = geom
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    X, dY = normal((N, IH, IW, IC), 3601), normal((N, OH, OW, OC), 3602)
    want = O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw)
    x, dy = dev.put(X), dev.put(dY)
    sizeW = OC * FH * FW * IC
    runs = []
    for _ in range(2):
        dWo = dev.guarded(OC, FH, FW, IC)
        buf = dev.empty(GridZ - 1, sizeW, fill=float("nan"))
        DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(), buf.data_ptr(),
                                 FH, FW, N, IC, OC, sh, sw, ph, pw)
        runs.append(np.concatenate([dev.get(dWo).reshape(1, -1), dev.get(buf)]))
        assert np.isfinite(runs[-1]).all(), "an element of deltaW or of a buffer was not written (%d, %d) %s" % (IC, OC, geom)
        check(_sum_partials(dev, dWo, buf, GridZ), want, "dW %d -> %d channels %s" % (IC, OC, geom))
    assert np.array_equal(runs[0].view(np.uint32), runs[1].view(np.uint32)), "partial sums differ between two runs (%d, %d) %s" % (IC, OC, geom)


DW_UNITS_SHAPES = [
    # N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, GridZ: the persistent kernel's other cut - every item in P equal pieces, the
    # P x items units dealt out whole - forced on small layers (by shape only tensors beyond 56 MB get it)
    (16, 16, 16, 256, 512, 3, 3, 1, 1, 1, 1, 8),    # 288 items of 1024 groups on 256 workgroups: P = 4, 4 or 5 units per workgroup
    (32, 16, 16, 96, 128, 5, 5, 1, 1, 2, 2, 6),     # 100 items (blocks of 48 x 64): P = 5, 1 or 2 units per workgroup
    (512, 2, 2, 256, 512, 3, 3, 1, 1, 1, 1, 4),     # pixel groups by image, 288 items of 512 groups: P = 2, 2 or 3 units
    (24, 19, 13, 64, 192, 3, 3, 2, 2, 1, 1, 12),    # 27 items, rows of 7 pixels: P = 9, 243 units on 256 workgroups (13 idle, spread out)
    (8, 12, 12, 64, 64, 3, 3, 1, 1, 1, 1, 3),       # 9 items, 3 buffers: 27 units
]


@pytest.mark.parametrize("shape", DW_UNITS_SHAPES)
def test_deltaW_persistent_kernel_whole_units_against_the_line_of_items(dev, shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, GridZ = shape
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    X, dY = normal((N, IH, IW, IC), 3701), normal((N, OH, OW, OC), 3702)
    want = O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw)
    x, dy = dev.put(X), dev.put(dY)
    sizeW = OC * FH * FW * IC
    L = pkg.lib()
    try:
        for units in (1, 0, -1):
            assert L.alpha_conv_set_deltaW_units(units) == 0
            runs = []
            for _ in range(2):
                dWo = dev.guarded(OC, FH, FW, IC)
                buf = dev.empty(GridZ - 1, sizeW, fill=float("nan"))
                DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(), buf.data_ptr(),
                                         FH, FW, N, IC, OC, sh, sw, ph, pw)
                runs.append(np.concatenate([dev.get(dWo).reshape(1, -1), dev.get(buf)]))
                assert np.isfinite(runs[-1]).all(), "an element of deltaW or of a buffer was not written, units %d %s" % (units, shape)
                check(_sum_partials(dev, dWo, buf, GridZ), want, "dW units %d %s" % (units, shape))
            assert np.array_equal(runs[0].view(np.uint32), runs[1].view(np.uint32)), "partial sums differ between two runs, units %d %s" % (units, shape)
    finally:
        L.alpha_conv_set_deltaW_units(-1)
    assert L.alpha_conv_set_deltaW_units(2) != 0


DW_STEM_SHAPES = [
    # N, IH, IW, OC, FH, FW, sh, sw, ph, pw, GridZ: 4 stored input channels (all four carry data here), the kernel whose MFMA
    # columns are 16 taps; its own equal cut of the pixels into GridZ slices, so the sum is compared
    (8, 32, 32, 64, 3, 3, 1, 1, 1, 1, 16),      # a VGG's first layer: 9 of a tap group's 16 taps, eight parts of a slice per workgroup
    (4, 40, 36, 64, 7, 7, 2, 2, 3, 3, 8),       # a ResNet's stem: four tap groups (the last with one tap), rows of 18 pixels (ragged last group)
    (6, 32, 32, 96, 6, 6, 2, 2, 2, 2, 4),       # the reference's AlexNet on CIFAR: three tap groups, two blocks of output channels (the second half full)
    (4, 32, 32, 64, 5, 5, 1, 1, 2, 2, 128),     # GridZ 128: eight pixel groups a slice, one tap group per workgroup
    (2, 23, 29, 20, 11, 11, 4, 4, 2, 2, 3),     # 121 taps: eight tap groups in a workgroup, 20 output channels, odd sizes
    (4, 9, 9, 8, 1, 1, 1, 1, 0, 0, 2),          # a single tap
    (3, 12, 12, 32, 3, 5, 2, 1, 1, 2, 5),       # 3x5 filter, stride 2 x 1
    (5, 10, 10, 16, 3, 3, 1, 1, 1, 1, 64),      # more slices than pixel groups a part: empty parts and empty slices
]


@pytest.mark.parametrize("shape", DW_STEM_SHAPES)
def test_deltaW_stem_kernel_sum_and_reproducibility(dev, shape):
    N, IH, IW, OC, FH, FW, sh, sw, ph, pw, GridZ = shape
    IC = 4
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    X, dY = normal((N, IH, IW, IC), 3501), normal((N, OH, OW, OC), 3502)
    want = O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw)
    x, dy = dev.put(X), dev.put(dY)
    sizeW = OC * FH * FW * IC
    runs = []
    for _ in range(2):
        dWo = dev.guarded(OC, FH, FW, IC)
        buf = dev.empty(GridZ - 1, sizeW, fill=float("nan"))
        DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(), buf.data_ptr(),
                                 FH, FW, N, IC, OC, sh, sw, ph, pw)
        runs.append(np.concatenate([dev.get(dWo).reshape(1, -1), dev.get(buf)]))
        assert np.isfinite(runs[-1]).all(), "an element of deltaW or of a buffer was not written %s" % (shape,)
        check(_sum_partials(dev, dWo, buf, GridZ), want, "stem dW GridZ=%d %s" % (GridZ, shape))
    assert np.array_equal(runs[0].view(np.uint32), runs[1].view(np.uint32)), "partial sums differ between two runs %s" % (shape,)
    # the same layer through the generic kernel (the reference's slices): the totals agree within tolerance
    L = pkg.lib()
    try:
        L.alpha_conv_set_fwd_algo(3)
        dWo = dev.guarded(OC, FH, FW, IC)
        buf = dev.empty(GridZ - 1, sizeW, fill=float("nan"))
        DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(), buf.data_ptr(),
                                 FH, FW, N, IC, OC, sh, sw, ph, pw)
        check(_sum_partials(dev, dWo, buf, GridZ), want, "generic kernel GridZ=%d %s" % (GridZ, shape))
    finally:
        L.alpha_conv_set_fwd_algo(0)


DW_ROWS_SHAPES = [
    # stride-1 layers served by the row-streaming kernel: N, IH, IW, IC, OC, F, p, GridZ
    (4, 56, 56, 64, 64, 3, 1, 16),     # c5b geometry
    (8, 32, 32, 64, 64, 3, 1, 8),      # c2a geometry
    (16, 16, 16, 128, 128, 3, 1, 7),   # c2b: slices end inside rows and inside images
    (32, 8, 8, 256, 256, 3, 1, 3),     # c2c with the split-K factor the Java engine would pass
    (4, 9, 9, 16, 16, 3, 1, 5),        # GK = 324, slices of 64 pixels: boundaries in the middle of rows
    (4, 13, 11, 36, 44, 3, 1, 3),      # ragged channel counts, OW not a multiple of 4
    (4, 10, 12, 32, 48, 3, 0, 2),      # no padding
    (4, 6, 7, 64, 32, 3, 2, 2),        # padding 2
    (8, 56, 56, 256, 64, 1, 0, 16),    # c5a geometry (1x1)
    (8, 56, 56, 64, 256, 1, 0, 16),    # c5c geometry (1x1)
    (4, 7, 9, 20, 36, 1, 0, 2),        # 1x1 ragged
    # 1x1 with channel counts multiples of 64: the register kernel (64x64 output blocks, slice pixels split in parts)
    (4, 14, 14, 128, 64, 1, 0, 3),     # 2 blocks, one per workgroup, 8 parts each
    (8, 16, 16, 256, 128, 1, 0, 40),   # 8 blocks; slices of 48 pixels = 12 groups over 8 parts (1 or 2 groups each)
    (4, 3, 3, 64, 192, 1, 0, 1),       # single slice of 36 pixels
    (4, 8, 8, 256, 256, 1, 0, 32),     # 16 blocks, two per workgroup, 4 parts; slices of 8 pixels: parts may be empty
    (4, 8, 8, 512, 512, 1, 0, 32),     # 64 blocks, eight per workgroup, no pixel split
    (8, 12, 12, 128, 256, 3, 1, 13),   # enough workgroups for the 32-output-channel variant, 4 rows per step
    (3, 14, 14, 64, 64, 3, 1, 2),      # c2c-sized rows: 3 rows per step, last step of an image has 2
    (2, 5, 20, 32, 32, 3, 1, 1),       # single slice; 2 rows per step with OH odd
    (5, 3, 40, 16, 48, 3, 1, 2),       # wide and short: one row per step, window spans the whole image
]


@pytest.mark.parametrize("shape", DW_ROWS_SHAPES)
def test_deltaW_row_streaming_kernel_slices_and_sum(dev, shape):
    N, IH, IW, IC, OC, F_, p, GridZ = shape
    OH, OW = out_dim(IH, IW, F_, F_, 1, 1, p, p)
    X, dY = normal((N, IH, IW, IC), 3101), normal((N, OH, OW, OC), 3102)
    x, dy = dev.put(X), dev.put(dY)
    sizeW = OC * F_ * F_ * IC
    outs = {}
    L = pkg.lib()
    try:
        for algo in (5, 3):   # 5: row-streaming kernel where eligible, 3: generic kernel
            L.alpha_conv_set_fwd_algo(algo)
            dWo = dev.guarded(OC, F_, F_, IC)
            buf = dev.empty(max(GridZ - 1, 1), sizeW, fill=float("nan"))
            if F_ == 1:
                DW.dconv3D_deltaW_GemmSK_W1(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), dWo.data_ptr(), buf.data_ptr(),
                                            N, IC, OC)
            else:
                DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(),
                                         buf.data_ptr(), F_, F_, N, IC, OC, 1, 1, p, p)
            outs[algo] = [dev.get(dWo)] + [b.reshape(OC, F_, F_, IC) for b in dev.get(buf)[:GridZ - 1]]
    finally:
        L.alpha_conv_set_fwd_algo(0)
    total = np.zeros((OC, F_, F_, IC))
    for z in range(GridZ):
        want = O.deltaW_slice_f64(X, dY, F_, F_, 1, 1, p, p, GridZ, z)
        total += want
        floor = tolerance_floor(total if z else want)
        for algo in (5, 3):
            r = O.max_err_ratio(outs[algo][z], want, REL, max(floor, tolerance_floor(want)))
            assert r <= 1.0, "slice %d algo %d %s: err/allowed %.3f" % (z, algo, shape, r)
    dWs = dev.put(outs[5][0])
    if GridZ > 1:
        bufs = dev.put(np.stack([o.reshape(-1) for o in outs[5][1:]]))
        DW.buf_summary(dev.stream, bufs.data_ptr(), dWs.data_ptr(), GridZ - 1, sizeW)
    check(dev.get(dWs), O.deltaW_f64(X, dY, F_, F_, 1, 1, p, p), "row-streaming dW total %s" % (shape,))


DW_TAPS_SHAPES = [
    # the tap-per-workgroup kernel takes any geometry: N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, GridZ
    (32, 8, 8, 256, 256, 3, 3, 1, 1, 1, 1, 3),      # c2c with the Java engine's split-K factor (slices end inside rows)
    (16, 16, 16, 128, 128, 3, 3, 1, 1, 1, 1, 7),    # c2b geometry: 14 sharing groups, linear block order
    (8, 32, 32, 64, 64, 3, 3, 1, 1, 1, 1, 8),       # c2a geometry: 8 sharing groups, one per XCD
    (4, 56, 56, 64, 64, 3, 3, 1, 1, 1, 1, 16),      # c5b geometry
    (4, 9, 9, 16, 16, 3, 3, 1, 1, 1, 1, 5),         # slices of 64 pixels: boundaries in the middle of rows, channels < 64
    (4, 13, 11, 36, 44, 3, 3, 1, 1, 1, 1, 3),       # ragged channel counts, OW not a multiple of 4
    (4, 10, 12, 32, 48, 3, 3, 1, 1, 0, 0, 2),       # no padding
    (4, 6, 7, 64, 32, 3, 3, 1, 1, 2, 2, 2),         # padding 2
    (4, 14, 14, 64, 128, 3, 3, 2, 2, 1, 1, 4),      # c4b geometry: stride 2
    (4, 15, 13, 68, 132, 3, 3, 2, 2, 1, 1, 3),      # stride 2, odd sizes, ragged channels over several blocks
    (4, 30, 30, 4, 64, 7, 7, 2, 2, 3, 3, 6),        # stem-like: 4 stored input channels, 49 taps
    (4, 9, 11, 12, 20, 5, 4, 2, 3, 2, 1, 2),        # rectangular filter, different strides
    (4, 14, 14, 64, 128, 1, 1, 2, 2, 0, 0, 5),      # 1x1 stride 2 (c4c geometry)
    (8, 14, 14, 128, 64, 1, 1, 1, 1, 0, 0, 3),      # 1x1 stride 1
    (4, 8, 8, 64, 64, 3, 3, 1, 1, 1, 1, 1),         # a single slice
    (4, 4, 4, 64, 64, 3, 3, 1, 1, 1, 1, 16),        # GK = 64 < 8 * GridZ: GK_slice = 0, every slice but the last is empty
    (4, 5, 6, 8, 8, 3, 3, 1, 1, 1, 1, 9),           # fewer rows in a slice than wavefronts in a workgroup
]


@pytest.mark.parametrize("shape", DW_TAPS_SHAPES)
def test_deltaW_tap_per_workgroup_kernel_slices_and_sum(dev, shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, GridZ = shape
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    X, dY = normal((N, IH, IW, IC), 3301), normal((N, OH, OW, OC), 3302)
    x, dy = dev.put(X), dev.put(dY)
    sizeW = OC * FH * FW * IC
    L = pkg.lib()
    runs = []
    try:
        L.alpha_conv_set_fwd_algo(4)   # the tap-per-workgroup kernel wherever it fits (it fits everything here)
        for _ in range(2):
            dWo = dev.guarded(OC, FH, FW, IC)
            buf = dev.empty(max(GridZ - 1, 1), sizeW, fill=float("nan"))
            DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(),
                                     buf.data_ptr(), FH, FW, N, IC, OC, sh, sw, ph, pw)
            runs.append([dev.get(dWo)] + [b.reshape(OC, FH, FW, IC) for b in dev.get(buf)[:GridZ - 1]])
    finally:
        L.alpha_conv_set_fwd_algo(0)
    for z in range(GridZ):
        want = O.deltaW_slice_f64(X, dY, FH, FW, sh, sw, ph, pw, GridZ, z)
        check(runs[0][z], want, "tap kernel slice %d %s" % (z, shape))
        assert np.array_equal(runs[0][z].view(np.uint32), runs[1][z].view(np.uint32)), "slice %d differs between two runs" % z
    dWs = dev.put(runs[0][0])
    if GridZ > 1:
        bufs = dev.put(np.stack([o.reshape(-1) for o in runs[0][1:]]))
        DW.buf_summary(dev.stream, bufs.data_ptr(), dWs.data_ptr(), GridZ - 1, sizeW)
    check(dev.get(dWs), O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw), "tap kernel dW total %s" % (shape,))


DW_WINO_SHAPES = [
    # N, IH, IW, IC, OC, ph, pw, GridZ   (3x3, stride 1)
    (4, 56, 56, 64, 64, 1, 1, 16),
    (8, 32, 32, 64, 64, 1, 1, 5),       # slices that end inside an image
    (16, 16, 16, 128, 128, 1, 1, 7),    # four blocks of input channels, two of output channels
    (36, 7, 7, 64, 96, 1, 1, 3),        # odd sizes: partial tiles on the right / bottom; ragged block of output channels
    (4, 13, 11, 36, 44, 1, 1, 4),       # ragged channels
    (4, 10, 12, 32, 64, 0, 0, 2),       # no padding
    (4, 6, 9, 32, 64, 2, 2, 1),         # padding 2, one slice (no partial buffers)
    (2, 5, 5, 64, 64, 1, 1, 9),         # more slices than chunks of tiles: empty slices must write zeros
]


@pytest.mark.parametrize("shape", DW_WINO_SHAPES)
def test_deltaW_winograd_slices_sum_to_the_oracle(dev, shape):
    """Winograd F(3x3,2x2) backward-filter: the slices are ranges of 2x2 tiles (not the reference's pixel ranges), so only
    their Kahan sum (buf_summary, as after the GemmSK entry) is compared with the fp64 oracle; same bar as the direct
    kernels. Two runs must agree bit for bit (no atomics)."""
    N, IH, IW, IC, OC, ph, pw, GridZ = shape
    OH, OW = out_dim(IH, IW, 3, 3, 1, 1, ph, pw)
    X, dY = normal((N, IH, IW, IC), 3201), normal((N, OH, OW, OC), 3202)
    x, dy = dev.put(X), dev.put(dY)
    sizeW = OC * 9 * IC
    runs = []
    for _ in range(2):
        dWo = dev.guarded(OC, 3, 3, IC)
        buf = dev.empty(max(GridZ - 1, 1), sizeW, fill=float("nan"))
        DW.dconv3D_deltaW_GemmSK_winograd(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(),
                                          buf.data_ptr(), N, IC, OC, ph, pw)
        if GridZ > 1:
            DW.buf_summary(dev.stream, buf.data_ptr(), dWo.data_ptr(), GridZ - 1, sizeW)
        runs.append(dev.get(dWo))
    assert np.array_equal(runs[0], runs[1]), "two runs differ"
    check(runs[0], O.deltaW_f64(X, dY, 3, 3, 1, 1, ph, pw), "winograd dW %s" % (shape,))


def test_deltaW_W1_entries(dev):
    for (N, IH, IW, IC, OC) in [(4, 14, 14, 256, 64), (4, 12, 12, 64, 256), (4, 7, 9, 12, 20)]:
        X, dY = normal((N, IH, IW, IC), 3005), normal((N, IH, IW, OC), 3006)
        want = O.deltaW_f64(X, dY, 1, 1, 1, 1, 0, 0)
        x, dy = dev.put(X), dev.put(dY)
        dWo = dev.guarded(OC, 1, 1, IC)
        DW.dconv3D_deltaW_W1(dev.streams, 1, x.data_ptr(), IH, IW, dy.data_ptr(), dWo.data_ptr(), N, IC, OC)
        check(dev.get(dWo), want, "deltaW_W1")
        GridZ = 3
        dWo = dev.guarded(OC, 1, 1, IC)
        buf = dev.empty(GridZ - 1, OC * IC, fill=float("nan"))
        DW.dconv3D_deltaW_GemmSK_W1(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), dWo.data_ptr(), buf.data_ptr(), N, IC, OC)
        check(_sum_partials(dev, dWo, buf, GridZ), want, "deltaW_GemmSK_W1")


def test_buf_summary_bit_exact_kahan(dev):
    r = np.random.Generator(np.random.PCG64(3007))
    for part, sizeW in [(1, 64), (15, 36864), (127, 2308), (3, 8)]:
        buf = (r.standard_normal((part, sizeW)) * 10.0 ** r.integers(-3, 4, (part, sizeW))).astype(np.float32)
        dw = r.standard_normal(sizeW).astype(np.float32)
        d, b = dev.put(dw), dev.put(buf)
        DW.buf_summary(dev.stream, b.data_ptr(), d.data_ptr(), part, sizeW)
        assert np.array_equal(dev.get(d), O.buf_summary(buf, dw)), (part, sizeW)


def test_deltaW_bit_reproducible_run_to_run(dev):
    # BASELINE config 5 requirement at reduced N: identical bits for identical (shape, GridZ)
    N, IH, IW, IC, OC = 4, 56, 56, 64, 64
    X, dY = normal((N, IH, IW, IC), 3008), normal((N, IH, IW, OC), 3009)
    x, dy = dev.put(X), dev.put(dY)
    GridZ, sizeW = 16, OC * 9 * IC
    outs = []
    for _ in range(3):
        dWo = dev.guarded(OC, 3, 3, IC)
        buf = dev.empty(GridZ - 1, sizeW, fill=float("nan"))
        DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), IH, IW, dWo.data_ptr(), buf.data_ptr(),
                                 3, 3, N, IC, OC, 1, 1, 1, 1)
        outs.append(_sum_partials(dev, dWo, buf, GridZ))
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    check(outs[0], O.deltaW_f64(X, dY, 3, 3, 1, 1, 1, 1), "config-5b dW (N=4)")


# ----------------------------------------------------------------------------------------------
# the reference's own acceptance test, on its own data distribution (uniform [0,1), unseeded there)
# ----------------------------------------------------------------------------------------------
def test_reference_style_criterion_forward(dev):
    # Cuda_conv3D_test.java:86-97: thr 1e-5, >= 99.9 % vs Tense.conv3D_naive; shape of :185 (IH=33, 4x4, OC ragged)
    for (N, IH, IW, IC, OC, F_, s, p) in [(8, 33, 33, 64, 128, 4, 1, 1), (4, 32, 32, 64, 252, 3, 2, 1)]:
        X, W = uniform((N, IH, IW, IC), 4001, 0, 1), uniform((OC, F_, F_, IC), 4002, 0, 1)
        cpu = O.conv3D_naive(X, W, s, s, p, p)
        for entry in ("conv3D", "conv3D_GemmR"):
            check_reference_style(_run_fwd(dev, entry, X, W, s, s, p, p), cpu, entry, 1e-5, 0.999)


def test_reference_style_criterion_deltaX(dev):
    # Cuda_dconv3D_dX_test.java:93-100: thr 1e-4, >= 99.9 % vs Tense.deconv3D_deltaX_img2col
    N, IH, IW, IC, OC, F_, p = 4, 31, 31, 128, 32, 4, 1
    OH, OW = out_dim(IH, IW, F_, F_, 1, 1, p, p)
    dY, W = uniform((N, OH, OW, OC), 4003, 0, 1), uniform((OC, F_, F_, IC), 4004, 0, 1)
    dXo = dev.guarded(N, IH, IW, IC)
    dy, w = dev.put(dY), dev.put(W)
    DX.dconv3D_deltaX_s1(dev.streams, 1, dy.data_ptr(), OH, OW, w.data_ptr(), F_, F_, dXo.data_ptr(), IH, IW,
                         N, IC, OC, p, p)
    check_reference_style(dev.get(dXo), O.deltaX_img2col(dY, W, IH, IW, 1, 1, p, p), "deltaX_s1", 1e-4, 0.999)


def test_reference_style_criterion_deltaW(dev):
    # Cuda_dconv3D_dW_test.java:98-105: thr 1e-5, 100 % vs Tense.deconv3d_deltaW_naive; shape of Cuda_dconv3D_deltaW.java:327
    N, IH, IW, IC, OC, F_, s, p = 4, 32, 32, 64, 256, 4, 2, 1
    OH, OW = out_dim(IH, IW, F_, F_, s, s, p, p)
    X, dY = uniform((N, IH, IW, IC), 4005, 0, 1), uniform((N, OH, OW, OC), 4006, 0, 1)
    cpu = O.deltaW_naive(X, dY, F_, F_, s, s, p, p)
    x, dy = dev.put(X), dev.put(dY)
    GridZ, sizeW = 4, OC * F_ * F_ * IC
    dWo = dev.guarded(OC, F_, F_, IC)
    buf = dev.empty(GridZ - 1, sizeW, fill=float("nan"))
    DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dWo.data_ptr(), buf.data_ptr(),
                             F_, F_, N, IC, OC, s, s, p, p)
    check_reference_style(_sum_partials(dev, dWo, buf, GridZ), cpu, "deltaW_GemmSK", 1e-5, 1.0)


# ----------------------------------------------------------------------------------------------
# the kernel without LDS with scratch lent by the caller (alpha_conv_bind_workspace): equal shares of whole items, the items
# left over cut along the reduction and added by a second kernel
# ----------------------------------------------------------------------------------------------
WORKSPACE_SHAPES = [
    # N, IH, IW, IC, OC, F, p, (items left over, pieces per item) on 256 compute units
    (24, 7, 7, 256, 512, 3, 1, (80, 3)),     # 1176 pixels = 74 tiles (the last one half empty) x 8 blocks = 592 = 2 x 256 + 80
    (16, 14, 14, 256, 256, 3, 1, (16, 8)),   # 196 tiles x 4 blocks = 784 = 3 x 256 + 16: 16 pieces possible, 8 used
    (64, 8, 8, 128, 320, 3, 1, (0, 0)),      # 256 tiles x 5 blocks = 5 x 256: nothing left over, the workspace stays untouched
]


@pytest.mark.parametrize("shape", WORKSPACE_SHAPES)
def test_forward_and_deltaX_with_bound_workspace(dev, shape):
    N, IH, IW, IC, OC, F_, p_, (left, split) = shape
    torch = dev.torch
    L = pkg.lib()
    X, W, dY = normal((N, IH, IW, IC), 5301), he_normal(OC, F_, F_, IC, 5302), normal((N, IH, IW, OC), 5303)
    B = normal((OC,), 5304)
    want_y = O.conv3D_f64(X, W, 1, 1, p_, p_)
    want_dx = O.deltaX_f64(dY, W, IH, IW, 1, 1, p_, p_)
    x, w, dy, b = dev.put(X), dev.put(W), dev.put(dY), dev.put(B)
    cw = dev.empty(F_ * F_ * IC * OC, fill=float("nan"))
    C3.kernel_remode(dev.stream, w.data_ptr(), cw.data_ptr(), F_, F_, OC, IC)
    ws_floats = 1 << 18
    ws = dev.guarded(ws_floats)

    def forward(bias):
        y = dev.guarded(N, IH, IW, OC)
        if bias:
            C3.conv3D_GemmR_biased(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), F_, F_, b.data_ptr(), y.data_ptr(),
                                   IH, IW, N, IC, OC, 1, 1, p_, p_)
        else:
            C3.conv3D_GemmR(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), F_, F_, y.data_ptr(), IH, IW, N, IC, OC, 1, 1, p_, p_)
        return dev.get(y)

    def backward():
        dx = dev.guarded(N, IH, IW, IC)
        DX.dconv3D_deltaX_s1(dev.streams, 1, dy.data_ptr(), IH, IW, w.data_ptr(), F_, F_, dx.data_ptr(), IH, IW, N, IC, OC, p_, p_)
        return dev.get(dx)

    plain_y, plain_dx = forward(False), backward()
    try:
        assert L.alpha_conv_bind_workspace(ws.data_ptr(), ws_floats * 4) == 0
        ws.fill_(float("nan"))
        got_y = forward(False)
        used = ws[:max(1, left * split * 1024)].clone()
        got_y2 = forward(False)
        got_yb = forward(True)
        ws.fill_(float("nan"))
        got_dx = backward()
        # with ticket words the workgroup that delivers an item's last piece adds the pieces (no second kernel): the
        # same order of addition, so the same bits; the words are zero again after every launch
        tickets = torch.zeros(128, dtype=torch.int32, device=ws.device)
        assert L.alpha_conv_bind_tickets(tickets.data_ptr(), 128) == 0
        ws.fill_(float("nan"))
        ticket_y = [forward(False) for _ in range(3)]
        ticket_used = ws[:max(1, left * split * 1024)].clone()
        ticket_yb = forward(True)
        ticket_dx = [backward() for _ in range(2)]
        dev.sync()
        assert int(tickets.abs().sum().item()) == 0, "ticket words not left zero"
    finally:
        L.alpha_conv_bind_tickets(None, 0)
        L.alpha_conv_bind_workspace(None, 0)
    dev.check_guards(ws)
    for k, ty in enumerate(ticket_y):
        assert np.array_equal(ty.view(np.uint32), got_y.view(np.uint32)), "forward with tickets, run %d: bits differ from the second kernel's" % k
    assert np.array_equal(ticket_yb.view(np.uint32), got_yb.view(np.uint32)), "forward with tickets and bias"
    for k, tdx in enumerate(ticket_dx):
        assert np.array_equal(tdx.view(np.uint32), got_dx.view(np.uint32)), "backward-data with tickets, run %d" % k
    if pkg.device_info()[0] == 256 and left:
        assert not bool(torch.isnan(ticket_used).any())
    check(got_y, want_y, "forward with workspace %s" % (shape,))
    check(got_yb, want_y + B.astype(np.float64), "forward with workspace and bias %s" % (shape,))
    check(got_dx, want_dx, "backward-data with workspace %s" % (shape,))
    assert np.array_equal(got_y.view(np.uint32), got_y2.view(np.uint32)), "two runs differ"
    if pkg.device_info()[0] == 256:
        if left:
            # the path ran: every partial sum was written (without the workspace such a layer may go to another kernel
            # altogether, so the two results are only compared through the oracle)
            assert not bool(torch.isnan(used).any()), "partial sums missing in the workspace"
        else:
            assert bool(torch.isnan(used).all()) and np.array_equal(got_y.view(np.uint32), plain_y.view(np.uint32))
    # after unbinding the plain path is back
    assert np.array_equal(forward(False).view(np.uint32), plain_y.view(np.uint32))
    assert np.array_equal(backward().view(np.uint32), plain_dx.view(np.uint32))
