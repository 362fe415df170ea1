"""GPU: the natives of one training step of a layer - kernel_remode, conv3D_GemmR, dconv3D_deltaX_s1,
dconv3D_deltaW_GemmSK, buf_summary, and the backward-filter entry that takes no workspace - recorded into a HIP graph and
replayed. The natives only enqueue kernels on the
stream they are given (conv/A.cu:149-171 and twins take the stream handles from Java and launch on them), allocate nothing
and clear nothing with memset calls, so a caller may capture them; every replay, with fresh inputs copied into the same
buffers and eager work of the program between the replays, is compared with the fp64 oracle.
Two layers: a 3x3 one (forward and backward-data through the kernel without LDS, some of whose work items are shared by a
workgroup's wavefronts through dynamic LDS; backward-filter through the persistent kernel, which writes zeros into the
partial-sum buffers it does not need) and the 7x7 stride-2 stem with 4 stored channels."""
import numpy as np
import pytest

from oracle import oracle as O
from util import Dev, he_normal, load_package, normal, out_dim

pytestmark = pytest.mark.gpu
pkg = load_package()
C3, DX, DW = pkg.Cuda_conv3D, pkg.Cuda_dconv3D_deltaX, pkg.Cuda_dconv3D_deltaW


@pytest.fixture(scope="module")
def dev():
    return Dev()


def check(got, want, what):
    floor = 1e-5 * max(1.0, float(np.sqrt(np.mean(want * want))))
    r = O.max_err_ratio(got, want, 1e-4, floor)
    assert r <= 1.0, "%s: err/allowed = %.3f (rel 1e-4, abs %.3g)" % (what, r, floor)


GRAPH_SHAPES = [
    # N, IH, IW, IC, OC, F, s, p, GridZ, backward-data?, scratch and ticket words lent?
    (32, 28, 28, 64, 64, 3, 1, 1, 32, True, False),
    (8, 64, 64, 4, 64, 7, 2, 3, 8, False, False),
    # 784 work items on 256 compute units: with the scratch three each and 16 left over, whose pieces the workgroup that
    # delivers the last one adds - the ticket words must be zero again after every replay for the next one to be right
    (16, 14, 14, 256, 256, 3, 1, 1, 8, True, True),
]


@pytest.mark.parametrize("shape", GRAPH_SHAPES)
def test_natives_replayed_from_a_graph(dev, shape):
    torch = dev.torch
    N, IH, IW, IC, OC, F_, s_, p_, GridZ, with_dx, lend = shape
    OH, OW = out_dim(IH, IW, F_, F_, s_, s_, p_, p_)
    sizeW = OC * F_ * F_ * IC
    x = dev.empty(N, IH, IW, IC, fill=0.0)
    w = dev.empty(OC, F_, F_, IC, fill=0.0)
    dy = dev.empty(N, OH, OW, OC, fill=0.0)
    cw = dev.empty(sizeW, fill=float("nan"))
    y = dev.empty(N, OH, OW, OC, fill=float("nan"))
    dx = dev.empty(N, IH, IW, IC, fill=float("nan"))
    dw = dev.empty(OC, F_, F_, IC, fill=float("nan"))
    dw_static = dev.empty(OC, F_, F_, IC, fill=float("nan"))
    buf = dev.empty(GridZ - 1, sizeW, fill=float("nan"))

    def step(stream):
        S = [stream]
        C3.kernel_remode(stream, w.data_ptr(), cw.data_ptr(), F_, F_, OC, IC)
        C3.conv3D_GemmR(S, 1, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), F_, F_, y.data_ptr(), OH, OW, N, IC, OC, s_, s_, p_, p_)
        if with_dx:
            DX.dconv3D_deltaX_s1(S, 1, dy.data_ptr(), OH, OW, w.data_ptr(), F_, F_, dx.data_ptr(), IH, IW, N, IC, OC, p_, p_)
        DW.dconv3D_deltaW_GemmSK(S, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dw.data_ptr(), buf.data_ptr(),
                                 F_, F_, N, IC, OC, s_, s_, p_, p_)
        DW.buf_summary(stream, buf.data_ptr(), dw.data_ptr(), GridZ - 1, sizeW)
        # the entry that takes no workspace (partial sums in the library's static device array): capture refuses any
        # allocation, so recording it here tests that it makes none
        DW.dconv3D_deltaW_GemmSK_static(S, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dw_static.data_ptr(),
                                        F_, F_, N, IC, OC, s_, s_, p_, p_)

    def fresh(seed):
        X, W, dY = normal((N, IH, IW, IC), seed), he_normal(OC, F_, F_, IC, seed + 1), normal((N, OH, OW, OC), seed + 2)
        if IC == 4:   # three logical channels stored as four
            X[..., 3] = 0.0
            W[..., 3] = 0.0
        x.copy_(dev.put(X)); w.copy_(dev.put(W)); dy.copy_(dev.put(dY))
        for t in (cw, y, dx, dw, dw_static, buf):
            t.fill_(float("nan"))
        return X, W, dY

    def verify(X, W, dY, what):
        torch.cuda.synchronize()
        check(y.cpu().numpy(), O.conv3D_f64(X, W, s_, s_, p_, p_), "forward, %s %s" % (what, shape))
        if with_dx:
            check(dx.cpu().numpy(), O.deltaX_f64(dY, W, IH, IW, s_, s_, p_, p_), "backward-data, %s %s" % (what, shape))
        check(dw.cpu().numpy(), O.deltaW_f64(X, dY, F_, F_, s_, s_, p_, p_), "backward-filter, %s %s" % (what, shape))
        assert torch.equal(dw.view(torch.int32), dw_static.view(torch.int32)), "static-scratch backward-filter, %s %s" % (what, shape)

    ws = dev.empty(1 << 18, fill=float("nan"))
    tickets = torch.zeros(128, dtype=torch.int32, device=ws.device)
    torch.cuda.synchronize()
    L = pkg.lib()
    if lend:
        assert L.alpha_conv_bind_workspace(ws.data_ptr(), ws.numel() * 4) == 0
        assert L.alpha_conv_bind_tickets(tickets.data_ptr(), tickets.numel()) == 0
    try:
        _capture_and_replay(dev, torch, step, fresh, verify)
        if lend:
            torch.cuda.synchronize()
            assert int(tickets.abs().sum().item()) == 0, "ticket words not left zero"
            if pkg.device_info()[0] == 256:
                assert not bool(torch.isnan(ws[:16 * 8 * 1024]).any()), "the pieces were not written: the path did not run"
    finally:
        L.alpha_conv_bind_tickets(None, 0)
        L.alpha_conv_bind_workspace(None, 0)


def _capture_and_replay(dev, torch, step, fresh, verify):
    side = torch.cuda.Stream()
    # eager first, on the stream that will capture: per-kernel attributes (dynamic LDS limits) are set on a kernel's first launch
    data = fresh(4100)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        step(int(side.cuda_stream))
    verify(*data, "eager")

    graph = torch.cuda.CUDAGraph()
    data = fresh(4200)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        step(int(torch.cuda.current_stream().cuda_stream))
    for rep in range(3):
        data = fresh(4300 + 10 * rep)           # eager copies and fills of the program between the replays
        graph.replay()
        verify(*data, "replay %d" % rep)
