"""Pins the CPU oracle (oracle/conv_oracle.c) with evidence that is independent of it.

The reference ships no golden vectors for the conv path (its tests draw unseeded random data),
so each oracle function is checked against: a library routine (torch conv2d and its gradients
in fp64 on the CPU), closed forms, invariants, and a pure-Python brute force on tiny shapes.
Each check is chosen so that a plausible slip (dropped tap, wrong pad sign, transposed filter
axis, un-rotated filter in deltaX, wrong stride lattice) fails it.
"""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as O

SHAPES = [
    # N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw
    (2, 8, 8, 4, 8, 3, 3, 1, 1, 1, 1),
    (2, 9, 7, 8, 4, 3, 3, 2, 2, 1, 1),
    (1, 10, 11, 4, 12, 5, 5, 2, 2, 2, 2),
    (2, 7, 7, 12, 8, 1, 1, 1, 1, 0, 0),
    (2, 12, 10, 4, 8, 7, 7, 2, 2, 3, 3),
    (3, 6, 9, 8, 8, 4, 4, 1, 1, 1, 1),
    (2, 9, 9, 4, 4, 3, 2, 3, 2, 0, 1),
    (2, 8, 8, 4, 8, 2, 2, 2, 2, 0, 0),
    (1, 5, 5, 4, 4, 3, 3, 1, 1, 2, 2),
    (2, 8, 6, 8, 8, 1, 1, 2, 2, 0, 0),
]


def _rand(shape, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.uniform(-1, 1, size=shape).astype(np.float32)


def _torch_fwd(X, W, sh, sw, ph, pw):
    x = torch.from_numpy(X.astype(np.float64)).permute(0, 3, 1, 2)
    w = torch.from_numpy(W.astype(np.float64)).permute(0, 3, 1, 2)
    return F.conv2d(x, w, stride=(sh, sw), padding=(ph, pw)).permute(0, 2, 3, 1).contiguous().numpy()


def _torch_dx(dY, W, IH, IW, IC, sh, sw, ph, pw):
    N = dY.shape[0]
    g = torch.from_numpy(dY.astype(np.float64)).permute(0, 3, 1, 2)
    w = torch.from_numpy(W.astype(np.float64)).permute(0, 3, 1, 2)
    dx = torch.nn.grad.conv2d_input((N, IC, IH, IW), w, g, stride=(sh, sw), padding=(ph, pw))
    return dx.permute(0, 2, 3, 1).contiguous().numpy()


def _torch_dw(X, dY, FH, FW, sh, sw, ph, pw):
    OC, IC = dY.shape[3], X.shape[3]
    x = torch.from_numpy(X.astype(np.float64)).permute(0, 3, 1, 2)
    g = torch.from_numpy(dY.astype(np.float64)).permute(0, 3, 1, 2)
    dw = torch.nn.grad.conv2d_weight(x, (OC, IC, FH, FW), g, stride=(sh, sw), padding=(ph, pw))
    return dw.permute(0, 2, 3, 1).contiguous().numpy()


@pytest.mark.parametrize("shape", SHAPES)
def test_forward_vs_torch_fp64(shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    X, W = _rand((N, IH, IW, IC), 1), _rand((OC, FH, FW, IC), 2)
    want = _torch_fwd(X, W, sh, sw, ph, pw)
    got64 = O.conv3D_f64(X, W, sh, sw, ph, pw)
    assert got64.shape == want.shape
    np.testing.assert_allclose(got64, want, rtol=1e-12, atol=1e-12)
    # double accumulator over FLOAT products (Tense.java:168), float out: each term carries one float rounding
    np.testing.assert_allclose(O.conv3D_naive(X, W, sh, sw, ph, pw), want, rtol=2e-6, atol=2e-6)
    np.testing.assert_allclose(O.conv3D_f32acc(X, W, sh, sw, ph, pw), want, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("shape", SHAPES)
def test_deltaX_vs_torch_fp64(shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    OH, OW = O.out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    dY, W = _rand((N, OH, OW, OC), 3), _rand((OC, FH, FW, IC), 4)
    want = _torch_dx(dY, W, IH, IW, IC, sh, sw, ph, pw)
    np.testing.assert_allclose(O.deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw), want, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(O.deltaX_img2col(dY, W, IH, IW, sh, sw, ph, pw), want, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("shape", SHAPES)
def test_deltaW_vs_torch_fp64(shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    OH, OW = O.out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    X, dY = _rand((N, IH, IW, IC), 5), _rand((N, OH, OW, OC), 6)
    want = _torch_dw(X, dY, FH, FW, sh, sw, ph, pw)
    np.testing.assert_allclose(O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw), want, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(O.deltaW_naive(X, dY, FH, FW, sh, sw, ph, pw), want, rtol=2e-6, atol=2e-6)
    np.testing.assert_allclose(O.deltaW_f32acc(X, dY, FH, FW, sh, sw, ph, pw), want, rtol=1e-4, atol=1e-5)


def _brute_forward(X, W, sh, sw, ph, pw):
    N, IH, IW, IC = X.shape
    OC, FH, FW, _ = W.shape
    OH, OW = (IH + 2 * ph - FH) // sh + 1, (IW + 2 * pw - FW) // sw + 1
    Y = np.zeros((N, OH, OW, OC))
    for n, oh, ow, oc, fh, fw, ic in itertools.product(range(N), range(OH), range(OW), range(OC),
                                                       range(FH), range(FW), range(IC)):
        ih, iw = oh * sh - ph + fh, ow * sw - pw + fw
        if 0 <= ih < IH and 0 <= iw < IW:
            Y[n, oh, ow, oc] += float(X[n, ih, iw, ic]) * float(W[oc, fh, fw, ic])
    return Y


def test_forward_brute_force_tiny():
    for (IH, IW, FH, FW, sh, sw, ph, pw) in [(4, 5, 3, 3, 1, 1, 1, 1), (5, 4, 2, 3, 2, 1, 1, 2), (3, 3, 3, 3, 2, 2, 1, 1)]:
        X, W = _rand((1, IH, IW, 2), 7), _rand((3, FH, FW, 2), 8)
        np.testing.assert_allclose(O.conv3D_f64(X, W, sh, sw, ph, pw), _brute_forward(X, W, sh, sw, ph, pw),
                                   rtol=1e-13, atol=1e-13)


def test_naive_variants_add_float_products_to_a_double_accumulator():
    """Tense.conv3D_naive (Tense.java:168) computes `v += X[..] * W[..]` with float operands and a double v: Java rounds the
    product to float first. Emulated term by term with numpy scalars in the reference's (fh, fw, ic) order; a product taken
    in double instead gives different bits in some outputs, which the last assertion shows for this data."""
    IH, IW, IC, OC, F_, p = 5, 4, 4, 4, 3, 1
    X, W = _rand((1, IH, IW, IC), 21), _rand((OC, F_, F_, IC), 22)
    want = np.zeros((1, IH, IW, OC), np.float32)
    dbl = np.zeros((1, IH, IW, OC), np.float32)
    for oh, ow, oc in itertools.product(range(IH), range(IW), range(OC)):
        v, vd = np.float64(0), np.float64(0)
        for fh, fw, ic in itertools.product(range(F_), range(F_), range(IC)):
            ih, iw = oh - p + fh, ow - p + fw
            if 0 <= ih < IH and 0 <= iw < IW:
                v = v + np.float64(np.float32(X[0, ih, iw, ic] * W[oc, fh, fw, ic]))
                vd = vd + np.float64(X[0, ih, iw, ic]) * np.float64(W[oc, fh, fw, ic])
        want[0, oh, ow, oc], dbl[0, oh, ow, oc] = np.float32(v), np.float32(vd)
    got = O.conv3D_naive(X, W, 1, 1, p, p)
    assert np.array_equal(got, want)
    assert not np.array_equal(want, dbl)
    # deltaW_naive is the same routine with deltaY as the filter (Tense.java:1277-1320): sum over (oh, ow, n)
    dY = _rand((1, IH, IW, OC), 23)
    wantW = np.zeros((OC, F_, F_, IC), np.float32)
    for oc, fh, fw, ic in itertools.product(range(OC), range(F_), range(F_), range(IC)):
        v = np.float64(0)
        for oh, ow in itertools.product(range(IH), range(IW)):
            ih, iw = oh - p + fh, ow - p + fw
            if 0 <= ih < IH and 0 <= iw < IW:
                v = v + np.float64(np.float32(X[0, ih, iw, ic] * dY[0, oh, ow, oc]))
        wantW[oc, fh, fw, ic] = np.float32(v)
    assert np.array_equal(O.deltaW_naive(X, dY, F_, F_, 1, 1, p, p), wantW)


def test_all_ones_counts_in_bounds_taps():
    # X = W = 1  =>  Y = IC * (#taps inside the image): exact small integers, pins the padding logic.
    N, IH, IW, IC, OC, F_, s, p = 1, 7, 6, 4, 4, 3, 1, 1
    X, W = np.ones((N, IH, IW, IC), np.float32), np.ones((OC, F_, F_, IC), np.float32)
    Y = O.conv3D_naive(X, W, s, s, p, p)
    rows = np.array([min(oh - p + F_, IH) - max(oh - p, 0) for oh in range(IH)])
    cols = np.array([min(ow - p + F_, IW) - max(ow - p, 0) for ow in range(IW)])
    want = IC * rows[:, None] * cols[None, :]
    assert np.array_equal(Y[0, :, :, 0], want.astype(np.float32))
    assert np.array_equal(O.conv3D_f32acc(X, W, s, s, p, p)[0, :, :, 3], want.astype(np.float32))


def test_impulse_gives_flipped_filter():
    # A unit impulse at (c,c), channel ic0: Y[oh,ow,oc] = W[oc, c+p-oh, c+p-ow, ic0].
    IH = IW = 7
    F_, p, ic0 = 3, 1, 2
    X = np.zeros((1, IH, IW, 4), np.float32)
    X[0, 3, 3, ic0] = 1.0
    W = _rand((4, F_, F_, 4), 9)
    Y = O.conv3D_naive(X, W, 1, 1, p, p)
    for oh, ow in itertools.product(range(IH), range(IW)):
        fh, fw = 3 + p - oh, 3 + p - ow
        want = W[:, fh, fw, ic0] if (0 <= fh < F_ and 0 <= fw < F_) else np.zeros(4, np.float32)
        assert np.array_equal(Y[0, oh, ow, :], want)


def test_1x1_is_matrix_product_and_identity():
    X, W = _rand((2, 5, 6, 8), 10), _rand((12, 1, 1, 8), 11)
    want = X.reshape(-1, 8).astype(np.float64) @ W.reshape(12, 8).astype(np.float64).T
    np.testing.assert_allclose(O.conv3D_f64(X, W, 1, 1, 0, 0).reshape(-1, 12), want, rtol=1e-13, atol=1e-13)
    eye = np.eye(8, dtype=np.float32).reshape(8, 1, 1, 8)
    assert np.array_equal(O.conv3D_naive(X, eye, 1, 1, 0, 0), X)


def test_stride_is_subsampled_stride1():
    X, W = _rand((2, 9, 11, 4), 12), _rand((8, 3, 3, 4), 13)
    full = O.conv3D_f64(X, W, 1, 1, 1, 1)
    np.testing.assert_array_equal(O.conv3D_f64(X, W, 2, 3, 1, 1), full[:, ::2, ::3, :])


def test_channel_pad_invariance():
    # IC=3 stored as 4 with a zero channel gives the same Y (how the engine pads channels).
    X3, W3 = _rand((2, 6, 6, 3), 14), _rand((4, 3, 3, 3), 15)
    X4 = np.concatenate([X3, np.zeros((2, 6, 6, 1), np.float32)], axis=3)
    W4 = np.concatenate([W3, np.zeros((4, 3, 3, 1), np.float32)], axis=3)
    np.testing.assert_array_equal(O.conv3D_f64(np.ascontiguousarray(X4), np.ascontiguousarray(W4), 1, 1, 1, 1),
                                  O.conv3D_f64(X3, W3, 1, 1, 1, 1))


@pytest.mark.parametrize("shape", SHAPES)
def test_adjointness_ties_the_three_operators(shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    OH, OW = O.out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    X, W, dY = _rand((N, IH, IW, IC), 16), _rand((OC, FH, FW, IC), 17), _rand((N, OH, OW, OC), 18)
    a = np.sum(O.conv3D_f64(X, W, sh, sw, ph, pw) * dY)
    b = np.sum(X * O.deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw))
    c = np.sum(W * O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw))
    assert abs(a - b) <= 1e-10 * max(1.0, abs(a))
    assert abs(a - c) <= 1e-10 * max(1.0, abs(a))


def test_kernel_remode_is_axis_permutation():
    W = _rand((8, 3, 5, 4), 19)
    assert np.array_equal(O.kernel_remode(W), np.transpose(W, (1, 2, 3, 0)))


@pytest.mark.parametrize("FH,FW,sh,sw", [(3, 3, 2, 2), (4, 4, 2, 2), (5, 5, 2, 2), (3, 3, 3, 3), (5, 4, 3, 2), (1, 1, 2, 2), (7, 7, 2, 2)])
def test_ks_remode_layouts(FH, FW, sh, sw):
    OC, IC = 8, 4
    W = _rand((OC, FH, FW, IC), 20)
    CFH, CFW = O.ks_dims(FH, FW, sh, sw)
    v1 = O.ks_remode(W, sh, sw, fill=np.nan).reshape(sh * sw, -1)
    v2 = O.ks_remodev2(W, sh, sw, fill=np.nan).reshape(sh * sw, -1)
    seen = np.zeros_like(W, dtype=np.int32)
    for y in range(sh):
        for x in range(sw):
            cfh, cfw = len(range(y, FH, sh)), len(range(x, FW, sw))  # independent count of taps of this phase
            n = OC * cfh * cfw * IC
            b1 = v1[y * sw + x][:n].reshape(OC, cfh, cfw, IC)
            b2 = v2[y * sw + x][:n].reshape(cfh, cfw, OC, IC)
            assert np.all(np.isnan(v1[y * sw + x][n:])) and np.all(np.isnan(v2[y * sw + x][n:]))
            for fhr in range(cfh):
                for fwr in range(cfw):
                    fh, fw = y + (cfh - 1 - fhr) * sh, x + (cfw - 1 - fwr) * sw
                    assert np.array_equal(b1[:, fhr, fwr, :], W[:, fh, fw, :])
                    assert np.array_equal(b2[fhr, fwr, :, :], W[:, fh, fw, :])
                    seen[:, fh, fw, :] += 1
    assert np.all(seen == 1)  # every tap lands in exactly one phase block


@pytest.mark.parametrize("shape", [s for s in SHAPES if s[7] > 1 or s[8] > 1] + [(2, 8, 8, 4, 8, 3, 3, 2, 2, 1, 1), (1, 9, 6, 4, 4, 5, 5, 3, 3, 2, 2)])
def test_kernel_split_decomposition_equals_deltaX(shape):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = shape
    OH, OW = O.out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    dY, W = _rand((N, OH, OW, OC), 21), _rand((OC, FH, FW, IC), 22)
    CW = O.ks_remodev2(W, sh, sw)
    got = O.deltaX_kernelSplit_f64(dY, CW, FH, FW, IH, IW, IC, sh, sw, ph, pw)
    np.testing.assert_allclose(got, _torch_dx(dY, W, IH, IW, IC, sh, sw, ph, pw), rtol=1e-12, atol=1e-12)


def test_split_k_slices_sum_to_full_and_partition_k():
    N, IH, IW, IC, OC, F_, s, p = 4, 9, 9, 4, 8, 3, 1, 1
    OH, OW = O.out_dim(IH, IW, F_, F_, s, s, p, p)
    X, dY = _rand((N, IH, IW, IC), 23), _rand((N, OH, OW, OC), 24)
    full = O.deltaW_f64(X, dY, F_, F_, s, s, p, p)
    for GZ in (1, 2, 3, 5):
        parts = [O.deltaW_slice_f64(X, dY, F_, F_, s, s, p, p, GZ, z) for z in range(GZ)]
        np.testing.assert_allclose(sum(parts), full, rtol=1e-12, atol=1e-12)
    # slice boundaries: GK=324, GZ=5 -> GK_slice = (324//5)>>3<<3 = 64; last slice takes 324-256=68.
    # With dY = 1 on exactly one k and X = 1, only the slice owning that k is non-zero.
    GK, GZ = N * OH * OW, 5
    assert GK == 324
    Xo = np.ones_like(X)
    for k, owner in [(0, 0), (63, 0), (64, 1), (255, 3), (256, 4), (323, 4)]:
        d = np.zeros((GK, OC), np.float32)
        d[k, :] = 1
        d = d.reshape(N, OH, OW, OC)
        nz = [bool(np.any(O.deltaW_slice_f64(Xo, d, F_, F_, s, s, p, p, GZ, z))) for z in range(GZ)]
        assert nz == [z == owner for z in range(GZ)]


def test_buf_summary_is_fp32_kahan_in_fixed_order():
    rng = np.random.Generator(np.random.PCG64(25))
    part, sizeW = 37, 64
    buf = (rng.standard_normal((part, sizeW)) * 10.0 ** rng.integers(-3, 4, (part, sizeW))).astype(np.float32)
    dW = rng.standard_normal(sizeW).astype(np.float32)
    got = O.buf_summary(buf, dW)
    # independent restatement with numpy float32 scalars (IEEE single ops, no contraction)
    want = dW.copy()
    c = np.zeros(sizeW, np.float32)
    for p in range(part):
        b = buf[p] - c
        t = want + b
        c = (t - want) - b
        want = t
    assert np.array_equal(got, want)
    # compensated sum is closer to the exact sum than naive fp32 accumulation, and part=0 is the identity
    exact = dW.astype(np.float64) + buf.astype(np.float64).sum(0)
    naive = dW.copy()
    for p in range(part):
        naive = naive + buf[p]
    assert np.abs(got - exact).max() <= np.abs(naive - exact).max()
    assert np.array_equal(O.buf_summary(np.zeros((0, sizeW), np.float32), dW), dW)


def test_samePercentRelative_matches_definition():
    A = np.array([1.0, 2.0, 0.0, 1.0, np.nan, 1.0], np.float32)
    B = np.array([1.0, 2.00001, 0.0, 1.1, np.nan, -1.0], np.float32)
    # elementwise: equal, |d|/|s| = 2.5e-6 < 1e-5, equal, 0.1/2.1 fails, both NaN pass, 2/eps fails
    assert O.samePercentRelative(A, B, 1e-5) == pytest.approx(4 / 6)
    assert O.samePercentRelative(A, B, 1e-7) == pytest.approx(3 / 6)


def test_max_err_ratio():
    want = np.array([1.0, 0.0, -2.0])
    got = np.array([1.00005, 5e-6, -2.0], np.float32)
    r = O.max_err_ratio(got, want, 1e-4, 1e-5)
    assert 0.49 < r < 0.52


# ---- backward of batch normalisation: the oracle's closed forms against automatic differentiation ----------------------
@pytest.mark.parametrize("N,M,affine", [(37, 8, True), (64, 12, False), (200, 4, True)])
def test_batchNorm_backward_oracle_equals_autograd(N, M, affine):
    """The reference's formulas are the gradient of Y = A * (X - mean(X)) / sqrt(var(X) + eps) + B when mean / var are the
    batch statistics of X (biased variance): torch's automatic differentiation of exactly that expression, in fp64, pins
    deltaA, deltaB and deltaX of all four forms (X_norm taken from Y, from (Y - B) / A and from X); a dropped 1/N, a sign
    or a swapped deltaXp1 / deltaXp2 changes deltaX by orders of magnitude more than the 1e-10 allowed."""
    import torch
    g = torch.Generator().manual_seed(77 + N)
    X = torch.randn((N, M), generator=g, dtype=torch.float64) * 1.7 + 0.3
    dY = torch.randn((N, M), generator=g, dtype=torch.float64)
    A = (torch.rand((M,), generator=g, dtype=torch.float64) + 0.5) if affine else torch.ones(M, dtype=torch.float64)
    B = torch.randn((M,), generator=g, dtype=torch.float64) if affine else torch.zeros(M, dtype=torch.float64)
    eps = 1e-5
    Xr, Ar, Br = X.clone().requires_grad_(True), A.clone().requires_grad_(True), B.clone().requires_grad_(True)
    mean, var = Xr.mean(0), Xr.var(0, unbiased=False)
    Y = Ar * (Xr - mean) / torch.sqrt(var + eps) + Br
    (Y * dY).sum().backward()
    mean_n, var_n, Yn = mean.detach().numpy(), var.detach().numpy(), Y.detach().numpy()
    forms = [("from_x", X.numpy())]
    forms.append(("from_y_affine", Yn) if affine else ("given", Yn))
    for form, S in forms:
        xn = O.batchNorm_xnorm(form, S, X_mean=mean_n, X_var=var_n, eps=eps, A=A.numpy(), B=B.numpy())
        dA, dB = O.batchNorm_deltaAB(dY.numpy(), xn)
        dX = O.batchNorm_deltaX(dY.numpy(), xn, var_n, eps, dB, dA, A=A.numpy() if affine else None)
        assert np.allclose(dA, Ar.grad.numpy(), rtol=1e-10, atol=1e-10), form
        assert np.allclose(dB, Br.grad.numpy(), rtol=1e-10, atol=1e-10), form
        assert np.allclose(dX, Xr.grad.numpy(), rtol=1e-9, atol=1e-10), form
