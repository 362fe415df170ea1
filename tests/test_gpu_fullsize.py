"""GPU: every layer of BASELINE.json's five configs at FULL size, through the C++ host layer.

The CPU oracle cannot finish these sizes in seconds, so each layer is checked by
  (1) the oracle on a few whole images of the batch (a convolution treats images independently, so image n of the
      full-batch result must equal the oracle's result for image n alone) — forward (implicit GEMM and Winograd) and
      backward-data;
  (2) the adjoint identity  <conv(X,W), dY> = <X, deltaX(dY,W)> = <W, deltaW(X,dY)>  evaluated in fp64 on the device,
      which ties the full-size backward-filter (a sum over the whole batch) to the forward result;
  (3) for config 5: backward-filter twice, bit-identical;
  (4) backward-filter element by element: deltaW[oc] depends on deltaY[..., oc] only, so the oracle run on the FULL batch
      with deltaY restricted to a few output channels (first, middle, last) must give those channels' whole filters - for
      the direct kernels and for the Winograd backward-filter.
Tolerance: rel 1e-4 with abs floor 1e-5 * max(1, rms(expected)) for (1); 2e-5 relative for the inner products of (2).
"""
import numpy as np
import pytest

from oracle import oracle as O
from util import Dev, load_package, out_dim

pytestmark = pytest.mark.gpu
pkg = load_package()

# id: N, IH, IW, IC(stored), OC, F, s, p, logical IC, input distribution
LAYERS = {
    "c1": (4, 32, 32, 4, 64, 3, 1, 1, 3, "uniform"),
    "c2a": (128, 32, 32, 64, 64, 3, 1, 1, 64, "normal"),
    "c2b": (128, 16, 16, 128, 128, 3, 1, 1, 128, "normal"),
    "c2c": (128, 8, 8, 256, 256, 3, 1, 1, 256, "normal"),
    "c3a": (64, 56, 56, 64, 64, 3, 1, 1, 64, "normal"),
    "c3b": (64, 28, 28, 128, 128, 3, 1, 1, 128, "normal"),
    "c3c": (64, 14, 14, 256, 256, 3, 1, 1, 256, "normal"),
    "c3d": (64, 7, 7, 512, 512, 3, 1, 1, 512, "normal"),
    "c4a": (64, 224, 224, 4, 64, 7, 2, 3, 3, "uniform"),
    "c4b": (64, 56, 56, 64, 128, 3, 2, 1, 64, "uniform"),
    "c4c": (64, 56, 56, 64, 128, 1, 2, 0, 64, "uniform"),
    "c4d": (64, 14, 14, 256, 1024, 1, 1, 0, 256, "uniform"),
    "c5a": (32, 56, 56, 256, 64, 1, 1, 0, 256, "normal"),
    "c5b": (32, 56, 56, 64, 64, 3, 1, 1, 64, "normal"),
    "c5c": (32, 56, 56, 64, 256, 1, 1, 0, 64, "normal"),
}


@pytest.fixture(scope="module")
def dev():
    return Dev()


def _tensors(dev, layer, seed):
    torch = dev.torch
    N, IH, IW, IC, OC, F, s, p, ICl, dist = LAYERS[layer]
    OH, OW = out_dim(IH, IW, F, F, s, s, p, p)
    g = torch.Generator(device="cpu").manual_seed(seed)
    X = torch.randn((N, IH, IW, IC), generator=g) if dist == "normal" else torch.rand((N, IH, IW, IC), generator=g) * 2 - 1
    W = torch.randn((OC, F, F, IC), generator=g) * float(np.sqrt(2.0 / (F * F * ICl)))   # He-normal
    if ICl < IC:
        X[..., ICl:] = 0
        W[..., ICl:] = 0
    dY = torch.randn((N, OH, OW, OC), generator=g)
    return X, W, dY, OH, OW


def _check(got, want, what):
    floor = 1e-5 * max(1.0, float(np.sqrt(np.mean(want * want))))
    r = O.max_err_ratio(np.ascontiguousarray(got), want, 1e-4, floor)
    assert r <= 1.0, "%s: err/allowed = %.3f (rel 1e-4, abs floor %.3g)" % (what, r, floor)


@pytest.mark.parametrize("layer", sorted(LAYERS))
def test_full_size_layer(dev, layer):
    torch = dev.torch
    N, IH, IW, IC, OC, F, s, p, ICl, _ = LAYERS[layer]
    X, W, dY, OH, OW = _tensors(dev, layer, 7000 + sorted(LAYERS).index(layer))
    x, w, dy = X.to(dev.dev), W.to(dev.dev), dY.to(dev.dev)
    y = torch.full((N, OH, OW, OC), float("nan"), device=dev.dev)
    dx = torch.full((N, IH, IW, IC), float("nan"), device=dev.dev)
    dw = torch.full((OC, F, F, IC), float("nan"), device=dev.dev)
    eng = pkg.engine.Engine(dev.stream)
    try:
        eng.conv3D(y.data_ptr(), OH, OW, x.data_ptr(), IH, IW, w.data_ptr(), F, F, N, IC, OC, s, s, p, p)
        eng.dconv3D_deltaX(dx.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, w.data_ptr(), F, F, N, IC, OC, s, s, p, p)
        eng.dconv3D_deltaW(dw.data_ptr(), F, F, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC, s, s, p, p)
        eng.sync()
        yw = None
        if F == 3 and s == 1 and IC >= 16:
            yw = torch.full((N, OH, OW, OC), float("nan"), device=dev.dev)
            eng.config.conv3D_winograd = 1
            plan = eng.conv3D(yw.data_ptr(), OH, OW, x.data_ptr(), IH, IW, w.data_ptr(), F, F, N, IC, OC, s, s, p, p)
            eng.config.conv3D_winograd = 0
            eng.sync()
            assert plan.entry_name == "conv3D_winograd"
        dxw = dww = dww2 = None
        if F == 3 and s == 1 and IC >= 16:   # the same layer through the Winograd backward paths of this build
            dxw = torch.full((N, IH, IW, IC), float("nan"), device=dev.dev)
            dww = torch.full((OC, F, F, IC), float("nan"), device=dev.dev)
            dww2 = torch.full((OC, F, F, IC), float("nan"), device=dev.dev)
            eng.config.deltaX_winograd = 1
            eng.config.deltaW_winograd = pkg.device_info()[0]
            px = eng.dconv3D_deltaX(dxw.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, w.data_ptr(), F, F, N, IC, OC, s, s, p, p)
            pw_ = eng.dconv3D_deltaW(dww.data_ptr(), F, F, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC, s, s, p, p)
            eng.dconv3D_deltaW(dww2.data_ptr(), F, F, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC, s, s, p, p)
            eng.config.deltaX_winograd = 0
            eng.config.deltaW_winograd = 0
            eng.sync()
            assert px.entry_name == "dconv3D_deltaX_winograd" and pw_.entry_name == "dconv3D_deltaW_GemmSK_winograd"
        dw2 = None
        if layer.startswith("c5"):
            dw2 = torch.full((OC, F, F, IC), float("nan"), device=dev.dev)
            eng.dconv3D_deltaW(dw2.data_ptr(), F, F, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC, s, s, p, p)
            eng.sync()
    finally:
        eng.close()

    # (1) whole images against the oracle
    Xn, Wn, dYn = X.numpy(), W.numpy(), dY.numpy()
    for n in sorted({0, N // 2, N - 1}):
        want = O.conv3D_f64(np.ascontiguousarray(Xn[n:n + 1]), Wn, s, s, p, p)
        _check(y[n:n + 1].cpu().numpy(), want, "%s forward image %d" % (layer, n))
        if yw is not None:
            _check(yw[n:n + 1].cpu().numpy(), want, "%s Winograd forward image %d" % (layer, n))
        wantx = O.deltaX_f64(np.ascontiguousarray(dYn[n:n + 1]), Wn, IH, IW, s, s, p, p)
        _check(dx[n:n + 1].cpu().numpy(), wantx, "%s deltaX image %d" % (layer, n))
        if dxw is not None:
            _check(dxw[n:n + 1].cpu().numpy(), wantx, "%s Winograd deltaX image %d" % (layer, n))

    # (2) adjointness in fp64 on the device
    a = float((y.double() * dy.double()).sum())
    b = float((x.double() * dx.double()).sum())
    c = float((w.double() * dw.double()).sum())
    scale = float((y.double().abs() * dy.double().abs()).sum())   # size of the terms being summed
    assert abs(a - b) <= 2e-5 * scale, "%s: <Y,dY> = %r vs <X,dX> = %r" % (layer, a, b)
    assert abs(a - c) <= 2e-5 * scale, "%s: <Y,dY> = %r vs <W,dW> = %r" % (layer, a, c)
    assert bool(torch.isfinite(dw).all()) and bool(torch.isfinite(dx).all())
    if dww is not None:
        cw = float((w.double() * dww.double()).sum())
        assert abs(a - cw) <= 2e-5 * scale, "%s: <Y,dY> = %r vs <W,dW Winograd> = %r" % (layer, a, cw)
        # element-wise against the direct kernel's result (both within the bar of the oracle: twice the bar between them)
        ref = dw.double()
        floor = 1e-5 * max(1.0, float(ref.pow(2).mean().sqrt()))
        err = (dww.double() - ref).abs() - 2 * torch.clamp(1e-4 * ref.abs(), min=floor)
        assert float(err.max()) <= 0.0, "%s: Winograd deltaW differs from the direct kernel's beyond twice the bar" % layer
        assert torch.equal(dww, dww2), "%s: Winograd deltaW differs between two runs" % layer

    # (4) backward-filter element by element on the full batch, for a few output channels (Tense.java:1277-1320 restated)
    ocs = sorted({0, 1, OC // 2 + 1, OC - 2, OC - 1})
    wantw = O.deltaW_f64(Xn, np.ascontiguousarray(dYn[..., ocs]), F, F, s, s, p, p)
    _check(dw[ocs].cpu().numpy(), wantw, "%s deltaW, output channels %s, all %d images" % (layer, ocs, N))
    if dww is not None:
        _check(dww[ocs].cpu().numpy(), wantw, "%s Winograd deltaW, output channels %s, all %d images" % (layer, ocs, N))

    # (3) run-to-run bit reproducibility of backward-filter (config 5)
    if dw2 is not None:
        assert torch.equal(dw, dw2), "%s: deltaW differs between two runs" % layer


# ----------------------------------------------------------------------------------------------
# The reference's own acceptance criterion on the kernels that serve the BASELINE layers, at full size and on the
# reference's own data distribution: uniform [0,1) operands, Vector.samePercentRelative (|a-b| / |a+b| below the
# threshold) against the CPU loops that add float products into a double (Tense.conv3D_naive,
# deconv3D_deltaX_img2col, deconv3d_deltaW_naive):
#   forward         threshold 1e-5, at least 99.9 % of the elements   (experiments/test_cuda/Cuda_conv3D_test.java:86-97)
#   backward-data   threshold 1e-4, at least 99.9 %                   (Cuda_dconv3D_dX_test.java:93-100)
#   backward-filter threshold 1e-5, 100 %                             (Cuda_dconv3D_dW_test.java:98-105)
# The CPU side runs on whole images of the batch (forward, backward-data) and on the whole batch for a few output
# channels (backward-filter: deltaW[oc] depends on deltaY[..., oc] only).
# ----------------------------------------------------------------------------------------------
def _uniform01(dev, shape, seed):
    g = dev.torch.Generator(device="cpu").manual_seed(seed)
    return dev.torch.rand(shape, generator=g)


def _same_percent(got, want, thr, need, what):
    pct = O.samePercentRelative(np.ascontiguousarray(want, dtype=np.float32), np.ascontiguousarray(got, dtype=np.float32), thr)
    assert np.isfinite(got).all(), what
    assert pct >= need, "%s: samePercentRelative(%g) = %.6f, the reference's test asks for %.4f" % (what, thr, pct, need)
    return pct


@pytest.mark.parametrize("layer,winograd", [("c3a", False), ("c3a", True), ("c3d", False)])
def test_reference_criterion_forward_full_size(dev, layer, winograd):
    torch = dev.torch
    N, IH, IW, IC, OC, F, s, p, ICl, _ = LAYERS[layer]
    OH, OW = out_dim(IH, IW, F, F, s, s, p, p)
    X, W = _uniform01(dev, (N, IH, IW, IC), 8101), _uniform01(dev, (OC, F, F, IC), 8102)
    x, w = X.to(dev.dev), W.to(dev.dev)
    y = torch.full((N, OH, OW, OC), float("nan"), device=dev.dev)
    eng = pkg.engine.Engine(dev.stream)
    try:
        eng.config.conv3D_winograd = 1 if winograd else 0
        plan = eng.conv3D(y.data_ptr(), OH, OW, x.data_ptr(), IH, IW, w.data_ptr(), F, F, N, IC, OC, s, s, p, p)
        eng.sync()
    finally:
        eng.close()
    assert (plan.entry_name == "conv3D_winograd") == winograd
    imgs = sorted({0, N // 2, N - 1})
    want = O.conv3D_naive(np.ascontiguousarray(X.numpy()[imgs]), W.numpy(), s, s, p, p)
    _same_percent(y[imgs].cpu().numpy(), want, 1e-5, 0.999, "%s forward%s" % (layer, " (Winograd)" if winograd else ""))


@pytest.mark.parametrize("layer,winograd", [("c5b", False), ("c5b", True), ("c5a", False), ("c5c", False)])
def test_reference_criterion_deltaX_full_size(dev, layer, winograd):
    torch = dev.torch
    N, IH, IW, IC, OC, F, s, p, ICl, _ = LAYERS[layer]
    OH, OW = out_dim(IH, IW, F, F, s, s, p, p)
    dY, W = _uniform01(dev, (N, OH, OW, OC), 8103), _uniform01(dev, (OC, F, F, IC), 8104)
    dy, w = dY.to(dev.dev), W.to(dev.dev)
    dx = torch.full((N, IH, IW, IC), float("nan"), device=dev.dev)
    eng = pkg.engine.Engine(dev.stream)
    try:
        eng.config.deltaX_winograd = 1 if winograd else 0
        plan = eng.dconv3D_deltaX(dx.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, w.data_ptr(), F, F, N, IC, OC, s, s, p, p)
        eng.sync()
    finally:
        eng.close()
    assert (plan.entry_name == "dconv3D_deltaX_winograd") == winograd
    imgs = sorted({0, N - 1})
    want = O.deltaX_img2col(np.ascontiguousarray(dY.numpy()[imgs]), W.numpy(), IH, IW, s, s, p, p)
    _same_percent(dx[imgs].cpu().numpy(), want, 1e-4, 0.999, "%s deltaX%s" % (layer, " (Winograd)" if winograd else ""))


@pytest.mark.parametrize("layer,mode", [("c5a", "direct"), ("c5b", "direct"), ("c5c", "direct"), ("c2c", "direct"), ("c2a", "direct"),
                                        ("c5b", "least"), ("c5a", "least"), ("c5b", "winograd"), ("c2c", "winograd")])
def test_reference_criterion_deltaW_full_size(dev, layer, mode):
    torch = dev.torch
    N, IH, IW, IC, OC, F, s, p, ICl, _ = LAYERS[layer]
    OH, OW = out_dim(IH, IW, F, F, s, s, p, p)
    X, dY = _uniform01(dev, (N, IH, IW, IC), 8105), _uniform01(dev, (N, OH, OW, OC), 8106)
    x, dy = X.to(dev.dev), dY.to(dev.dev)
    dw = torch.full((OC, F, F, IC), float("nan"), device=dev.dev)
    eng = pkg.engine.Engine(dev.stream)
    try:
        cus = pkg.device_info()[0]
        eng.config.deltaW_winograd = cus if mode == "winograd" else 0
        eng.config.deltaW_SK_leastUnits = cus if mode == "least" else 0
        plan = eng.dconv3D_deltaW(dw.data_ptr(), F, F, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC, s, s, p, p)
        eng.sync()
    finally:
        eng.close()
    assert (plan.entry_name == "dconv3D_deltaW_GemmSK_winograd") == (mode == "winograd")
    ocs = sorted({0, 1, OC // 2 + 1, OC - 1})
    want = O.deltaW_naive(X.numpy(), np.ascontiguousarray(dY.numpy()[..., ocs]), F, F, s, s, p, p)
    _same_percent(dw[ocs].cpu().numpy(), want, 1e-5, 1.0, "%s deltaW (%s, GridZ %d)" % (layer, mode, plan.GridZ))


# ----------------------------------------------------------------------------------------------
# The items left over after equal shares (c3c: 64 items in 4 pieces, c3d: 32 in 8): added by a second kernel, or - with
# ticket words, what an engine object lends - by whichever workgroup delivers an item's last piece. Who adds must not
# show in the bits: the whole output is compared bit for bit, over several launches (the workgroup that comes last
# changes from launch to launch), and the ticket words are zero afterwards.
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("layer", ["c3c", "c3d"])
def test_pieces_added_by_last_workgroup_equal_second_kernel_full_size(dev, layer):
    torch = dev.torch
    L = pkg.lib()
    C3 = pkg.Cuda_conv3D
    N, IH, IW, IC, OC, F, s, p, _, _ = LAYERS[layer]
    X, W, _, OH, OW = _tensors(dev, layer, 8301)
    x, w = X.to(dev.dev), W.to(dev.dev)
    cw = torch.empty(F * F * IC * OC, device=dev.dev)
    C3.kernel_remode(dev.stream, w.data_ptr(), cw.data_ptr(), F, F, OC, IC)
    ws = torch.full((1 << 18,), float("nan"), device=dev.dev)
    tickets = torch.zeros(128, dtype=torch.int32, device=dev.dev)

    def forward():
        y = torch.full((N, OH, OW, OC), float("nan"), device=dev.dev)
        C3.conv3D_GemmR(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), F, F, y.data_ptr(), OH, OW, N, IC, OC, s, s, p, p)
        dev.sync()
        return y

    try:
        assert L.alpha_conv_bind_workspace(ws.data_ptr(), ws.numel() * 4) == 0
        second_kernel = forward()
        assert L.alpha_conv_bind_tickets(tickets.data_ptr(), tickets.numel()) == 0
        for k in range(6):
            ws.fill_(float("nan"))
            got = forward()
            assert torch.equal(got.view(torch.int32), second_kernel.view(torch.int32)), "%s launch %d: bits differ" % (layer, k)
            assert int(tickets.abs().sum().item()) == 0, "%s launch %d: ticket words not left zero" % (layer, k)
    finally:
        L.alpha_conv_bind_tickets(None, 0)
        L.alpha_conv_bind_workspace(None, 0)
    if pkg.device_info()[0] == 256:
        assert not bool(torch.isnan(ws[:32 * 8 * 1024]).any()), "the pieces were not written: the path did not run"
    imgs = [0, N - 1]
    want = O.conv3D_f64(np.ascontiguousarray(X.numpy()[imgs]), W.numpy(), s, s, p, p)
    _check(second_kernel[imgs].cpu().numpy(), want, "%s forward, equal shares" % layer)


# Kernel-split backward-data of a workgroup's wavefronts sharing every group of items (what small maps with many
# channels get by shape), at full size: the stride-2 3x3 layers that open the third and fourth stage of a ResNet
# (N = 64; the first has items enough for every wavefront and shares only when forced), the second stage's on 16x16
# maps at N = 128, c4b, and a 1x1 stride-2 layer with too many channels for the scattered product. Whole images against the oracle, <X, deltaX> = <Y, deltaY> in fp64 over the
# full batch, and the two distributions of the work against each other.
@pytest.mark.parametrize("case", [(64, 28, 28, 128, 256, 3, 1, False), (64, 14, 14, 256, 512, 3, 1, True), (128, 16, 16, 128, 256, 3, 1, True),
                                  (64, 56, 56, 64, 128, 3, 1, False),
                                  # a 1x1 shortcut of a ResNet-50 under stride 2: one phase with the tap (128 steps an item), three that write zeros
                                  (64, 14, 14, 1024, 2048, 1, 0, False)])
def test_kernel_split_shared_groups_full_size(dev, case):
    torch = dev.torch
    L = pkg.lib()
    DX = pkg.Cuda_dconv3D_deltaX
    N, IH, IW, IC, OC, F, p, shares_by_shape = case
    s = 2
    OH, OW = out_dim(IH, IW, F, F, s, s, p, p)
    g = torch.Generator(device="cpu").manual_seed(8400 + IH)
    X = torch.randn((N, IH, IW, IC), generator=g)
    W = torch.randn((OC, F, F, IC), generator=g) * float(np.sqrt(2.0 / (F * F * IC)))
    dY = torch.randn((N, OH, OW, OC), generator=g)
    x, w, dy = X.to(dev.dev), W.to(dev.dev), dY.to(dev.dev)

    def backward(sharing):
        assert L.alpha_conv_set_kernel_split_sharing(sharing) == 0
        dx = torch.full((N, IH, IW, IC), float("nan"), device=dev.dev)
        DX.dconv3D_deltaX_crossAdd(dev.streams, 1, dy.data_ptr(), OH, OW, w.data_ptr(), F, F, dx.data_ptr(), IH, IW, N, IC, OC, s, s, p, p)
        dev.sync()
        return dx

    try:
        own = backward(0)
        shared = backward(1)
        by_shape = backward(-1)
    finally:
        L.alpha_conv_set_kernel_split_sharing(-1)
    expect = shared if shares_by_shape else own
    assert torch.equal(by_shape.view(torch.int32), expect.view(torch.int32)), "the choice by shape is not the expected one"
    imgs = [0, N // 2, N - 1]
    want = O.deltaX_f64(np.ascontiguousarray(dY.numpy()[imgs]), W.numpy(), IH, IW, s, s, p, p)
    _check(own[imgs].cpu().numpy(), want, "deltaX, items of their own %s" % (case,))
    _check(shared[imgs].cpu().numpy(), want, "deltaX, shared groups %s" % (case,))
    y = torch.full((N, OH, OW, OC), float("nan"), device=dev.dev)
    eng = pkg.engine.Engine(dev.stream)
    try:
        eng.conv3D(y.data_ptr(), OH, OW, x.data_ptr(), IH, IW, w.data_ptr(), F, F, N, IC, OC, s, s, p, p)
        eng.sync()
    finally:
        eng.close()
    a = float((y.double() * dy.double()).sum())
    scale = float((y.double().abs() * dy.double().abs()).sum())
    for name, dx in (("own", own), ("shared", shared)):
        b = float((x.double() * dx.double()).sum())
        assert abs(a - b) <= 2e-5 * scale, "%s %s: <Y,dY> = %r vs <X,dX> = %r" % (case, name, a, b)
    ref = own.double()
    floor = 1e-5 * max(1.0, float(ref.pow(2).mean().sqrt()))
    err = (shared.double() - ref).abs() - 2 * torch.clamp(1e-4 * ref.abs(), min=floor)
    assert float(err.max()) <= 0.0, "%s: the two distributions differ beyond twice the bar" % (case,)


@pytest.mark.parametrize("case", [(64, 27, 27, 96, 256, 5, 2, 14, 5),      # AlexNet's second layer: 200 items, 65 MB: 5 pieces per item, 3 or 4 units per workgroup
                                  (512, 16, 16, 64, 192, 3, 1, 85, 9),     # 27 items, 134 MB: 9 pieces, one unit per workgroup on 243 of them
                                  (64, 32, 32, 128, 256, 3, 1, 42, 7)])    # 72 items, 101 MB: 7 pieces, 1 or 2 units per workgroup
def test_deltaW_whole_units_by_shape_full_size(dev, case):
    """Large tensors whose line of items would start every share at a different place of the pixel range get the cut into
    whole (piece, item) units by shape: the buffers beyond the P pieces are zeros, the sums under both cuts agree, and
    output channels of both are checked against the oracle."""
    torch = dev.torch
    L = pkg.lib()
    DW = pkg.Cuda_dconv3D_deltaW
    N, IH, IW, IC, OC, F, p, GridZ, P = case
    OH, OW = out_dim(IH, IW, F, F, 1, 1, p, p)
    g = torch.Generator(device="cpu").manual_seed(8500 + IH)
    X = torch.randn((N, IH, IW, IC), generator=g)
    dY = torch.randn((N, OH, OW, OC), generator=g)
    x, dy = X.to(dev.dev), dY.to(dev.dev)
    sizeW = OC * F * F * IC

    def run(units):
        assert L.alpha_conv_set_deltaW_units(units) == 0
        dw = torch.full((OC, F, F, IC), float("nan"), device=dev.dev)
        buf = torch.full((GridZ - 1, sizeW), float("nan"), device=dev.dev)
        DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dw.data_ptr(), buf.data_ptr(),
                                 F, F, N, IC, OC, 1, 1, p, p)
        dev.sync()
        return dw, buf

    try:
        line = run(0)
        by_shape = run(-1)
        units = run(1)
    finally:
        L.alpha_conv_set_deltaW_units(-1)
    assert torch.equal(by_shape[0].view(torch.int32), units[0].view(torch.int32)) and torch.equal(by_shape[1].view(torch.int32), units[1].view(torch.int32)), \
        "the choice by shape is not the cut into whole units"
    if pkg.device_info()[0] == 256:
        assert not bool(by_shape[1][P - 1:].any()) and bool(by_shape[1][P - 2].any()), "expected %d pieces per item" % P
    ocs = [0, OC // 2 + 1, OC - 1]
    want = O.deltaW_f64(X.numpy(), np.ascontiguousarray(dY.numpy()[..., ocs]), F, F, 1, 1, p, p)
    sums = {}
    for name, (dw, buf) in (("line", line), ("units", by_shape)):
        tot = (dw.double() + buf.double().sum(0).view(OC, F, F, IC))
        sums[name] = tot
        _check(tot[ocs].cpu().numpy(), want, "deltaW %s %s" % (name, case))
    ref = sums["line"]
    floor = 1e-5 * max(1.0, float(ref.pow(2).mean().sqrt()))
    err = (sums["units"] - ref).abs() - 2 * torch.clamp(1e-4 * ref.abs(), min=floor)
    assert float(err.max()) <= 0.0, "%s: the two cuts differ beyond twice the bar" % (case,)


# Tensors between 2 GB and the 2^31 elements the entries accept: the kernels that address through 2 GB buffer
# descriptors refuse them (nothing launched) and the layer goes to the kernels that index elements. X and deltaX are
# 2.2 GB here (44 x 512 x 512 x 48); first and last image against the oracle; backward-filter with deltaY zero outside
# those two images, so the two images are the whole sum.
# N = 38, 16 output channels: 1.9 GB, the largest the descriptor kernels take (byte offsets up to 2^31).
@pytest.mark.parametrize("N,OC", [(44, 8), (38, 16)])
def test_tensors_beyond_2GB(dev, N, OC):
    torch = dev.torch
    C3, DX, DW = pkg.Cuda_conv3D, pkg.Cuda_dconv3D_deltaX, pkg.Cuda_dconv3D_deltaW
    IH, IW, IC, F, s, p = 512, 512, 48, 3, 1, 1
    OH, OW = out_dim(IH, IW, F, F, s, s, p, p)
    assert N * IH * IW * IC < (1 << 31) and (N * IH * IW * IC * 4 > (1 << 31)) == (N == 44)
    g = torch.Generator(device=dev.dev).manual_seed(9100)
    x = torch.randn((N, IH, IW, IC), generator=g, device=dev.dev)
    w = torch.randn((OC, F, F, IC), generator=g, device=dev.dev) * float(np.sqrt(2.0 / (F * F * IC)))
    dy = torch.randn((N, OH, OW, OC), generator=g, device=dev.dev)
    imgs = [0, N - 1]
    Xs, Ws, dYs = x[imgs].cpu().numpy(), w.cpu().numpy(), dy[imgs].cpu().numpy()

    cw = torch.empty(F * F * IC * OC, device=dev.dev)
    C3.kernel_remode(dev.stream, w.data_ptr(), cw.data_ptr(), F, F, OC, IC)
    y = torch.full((N, OH, OW, OC), float("nan"), device=dev.dev)
    C3.conv3D_GemmR(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), F, F, y.data_ptr(), OH, OW, N, IC, OC, s, s, p, p)
    dev.sync()
    assert bool(torch.isfinite(y).all())
    _check(y[imgs].cpu().numpy(), O.conv3D_f64(Xs, Ws, s, s, p, p), "forward, X of %.1f GB" % (x.numel() * 4 / 1e9))
    del y

    dx = torch.full((N, IH, IW, IC), float("nan"), device=dev.dev)
    DX.dconv3D_deltaX_s1(dev.streams, 1, dy.data_ptr(), OH, OW, w.data_ptr(), F, F, dx.data_ptr(), IH, IW, N, IC, OC, p, p)
    dev.sync()
    assert bool(torch.isfinite(dx[N // 2]).all())
    _check(dx[imgs].cpu().numpy(), O.deltaX_f64(dYs, Ws, IH, IW, s, s, p, p), "deltaX of %.1f GB" % (x.numel() * 4 / 1e9))
    del dx

    dy[1:N - 1].zero_()
    GridZ, sizeW = 64, OC * F * F * IC    # the generic kernel: 7 x 1 blocks of the filter x GridZ workgroups
    dw = torch.full((OC, F, F, IC), float("nan"), device=dev.dev)
    buf = torch.full((GridZ - 1, sizeW), float("nan"), device=dev.dev)
    DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dw.data_ptr(), buf.data_ptr(),
                             F, F, N, IC, OC, s, s, p, p)
    DW.buf_summary(dev.stream, buf.data_ptr(), dw.data_ptr(), GridZ - 1, sizeW)
    dev.sync()
    # 180 224 products per slice and element in one fp32 accumulator (an image spans a slice and a half): the floor that
    # the other tests take for sums of a few thousand terms, 1e-5 rms, is below sqrt(180 224) rounding errors here - 4e-5
    want = O.deltaW_f64(Xs, dYs, F, F, s, s, p, p)
    floor = 4e-5 * float(np.sqrt(np.mean(want * want)))
    r = O.max_err_ratio(np.ascontiguousarray(dw.cpu().numpy()), want, 1e-4, floor)
    assert r <= 1.0, "deltaW, X of %.1f GB: err/allowed = %.3f (rel 1e-4, abs floor %.3g)" % (x.numel() * 4 / 1e9, r, floor)
