"""GPU: backward of batch normalisation around the convolution - the field sums (Cuda_reduce.field_affine_deltaAB_v1 / _v2,
field_batchNorm_deltaAB_v2) and the four row functions (Cuda_function.batchNorm2D_row_deltaX_v1 / _v2 and the affine twins)
through the C ABI, and the host layer's operators built from them - against the oracle's fp64 closed forms (which
tests/test_oracle.py pins by automatic differentiation).
Tolerance: |err| <= max(1e-4 * |want|, 1e-5 * max(1, rms(want))), the bar of the backward-filter sums; the field sums must
also be bit-identical from run to run, with the result aliasing the head of its buffer as the Java engine passes them."""
import numpy as np
import pytest

from oracle import oracle as O
from util import Dev, load_package, normal, uniform

pytestmark = pytest.mark.gpu
pkg = load_package()
R, F = pkg.Cuda_reduce, pkg.Cuda_function


@pytest.fixture(scope="module")
def dev():
    return Dev()


def check(got, want, what):
    floor = 1e-5 * max(1.0, float(np.sqrt(np.mean(want * want))))
    r = O.max_err_ratio(np.ascontiguousarray(got), want, 1e-4, floor)
    assert r <= 1.0, "%s: err/allowed = %.3f (rel 1e-4, abs %.3g)" % (what, r, floor)


def _data(N, M, width, seed):
    """deltaY, X, the batch statistics of X, affine parameters and Y = A * X_norm + B, pad columns zero."""
    X = normal((N, M), seed) * 1.3 + 0.4
    dY = normal((N, M), seed + 1)
    A = uniform((M,), seed + 2, 0.5, 1.5)
    B = normal((M,), seed + 3)
    for t in (X, dY):
        t[:, width:] = 0
    mean = X.astype(np.float64).mean(0).astype(np.float32)
    var = X.astype(np.float64).var(0).astype(np.float32)
    eps = np.float32(1e-5)
    xn = ((X - mean) / np.sqrt(var + eps)).astype(np.float32)
    Yaff = (A * xn + B).astype(np.float32)
    for t in (xn, Yaff):
        t[:, width:] = 0
    return X, dY, A, B, mean, var, float(eps), xn, Yaff


SHAPES = [
    # rows, row_lengthv (= mem_stride), mem_width
    (64 * 56 * 56, 64, 64),     # the headline layer's output: 200704 pixels x 64 channels
    (32 * 56 * 56, 256, 256),   # c5c's output
    (1000, 256, 256),
    (530, 12, 10),              # ragged: two pad columns, one chunk of rows cut short
    (37, 8, 7),                 # one stage only (field_nextN = 1)
    (9, 4, 4),
    (4100, 1024, 1024),
]


@pytest.mark.parametrize("N,M,width", SHAPES)
def test_field_sums_and_row_functions(dev, N, M, width):
    X, dY, A, B, mean, var, eps, xn, Yaff = _data(N, M, width, 6000 + N % 97)
    d = {k: dev.put(v) for k, v in dict(X=X, dY=dY, A=A, B=B, mean=mean, var=var, xn=xn, Yaff=Yaff).items()}
    nextN = R.field_nextN(N, M)
    want_next = nextN
    while want_next > 1:
        want_next = R.field_nextN(want_next, M)
    lengthv = N * M
    cases = [
        ("affine_v2 / row v1", lambda *a: R.field_affine_deltaAB_v2(dev.stream, dev.stream, d["dY"].data_ptr(), d["xn"].data_ptr(), N, M, *a),
         O.batchNorm_xnorm("given", xn), None,
         lambda p1, p2, dx: F.batchNorm2D_row_deltaX_v1(dev.stream, d["dY"].data_ptr(), d["xn"].data_ptr(), d["var"].data_ptr(), eps, p1, p2, M, dx,
                                                        lengthv, width, M)),
        ("affine_v1 / affined row v1", lambda *a: R.field_affine_deltaAB_v1(dev.stream, dev.stream, d["dY"].data_ptr(), d["Yaff"].data_ptr(),
                                                                            d["A"].data_ptr(), d["B"].data_ptr(), N, M, *a),
         O.batchNorm_xnorm("from_y_affine", Yaff, A=A, B=B), A,
         lambda p1, p2, dx: F.batchNorm_affined2D_row_deltaX_v1(dev.stream, d["dY"].data_ptr(), d["Yaff"].data_ptr(), d["var"].data_ptr(), eps,
                                                                d["A"].data_ptr(), d["B"].data_ptr(), p1, p2, M, dx, lengthv, width, M)),
        ("batchNorm_v2 / row v2", lambda *a: R.field_batchNorm_deltaAB_v2(dev.stream, dev.stream, d["dY"].data_ptr(), d["X"].data_ptr(),
                                                                          d["mean"].data_ptr(), d["var"].data_ptr(), eps, N, M, *a),
         O.batchNorm_xnorm("from_x", X, X_mean=mean, X_var=var, eps=eps), None,
         lambda p1, p2, dx: F.batchNorm2D_row_deltaX_v2(dev.stream, d["dY"].data_ptr(), d["X"].data_ptr(), d["mean"].data_ptr(), d["var"].data_ptr(),
                                                        eps, p1, p2, M, dx, lengthv, width, M)),
        ("batchNorm_v2 / affined row v2", lambda *a: R.field_batchNorm_deltaAB_v2(dev.stream, dev.stream, d["dY"].data_ptr(), d["X"].data_ptr(),
                                                                                  d["mean"].data_ptr(), d["var"].data_ptr(), eps, N, M, *a),
         O.batchNorm_xnorm("from_x", X, X_mean=mean, X_var=var, eps=eps), A,
         lambda p1, p2, dx: F.batchNorm_affined2D_row_deltaX_v2(dev.stream, d["dY"].data_ptr(), d["X"].data_ptr(), d["mean"].data_ptr(),
                                                                d["var"].data_ptr(), eps, d["A"].data_ptr(), p1, p2, M, dx, lengthv, width, M)),
    ]
    for name, sums, xn64, A_or_none, rowfn in cases:
        want_dA, want_dB = O.batchNorm_deltaAB(dY, xn64)
        want_dA[width:] = 0
        want_dB[width:] = 0
        outs = []
        for rep in range(2):
            # the buffers as the Java engine passes them: nextN x M floats, the result at the head of its own buffer
            bufA = dev.empty(nextN * M + 64, fill=float("nan"))
            bufB = dev.empty(nextN * M + 64, fill=float("nan"))
            got_next = sums(bufA.data_ptr(), bufA.data_ptr(), bufB.data_ptr(), bufB.data_ptr(), width, M, 1)
            dev.sync()
            assert got_next == want_next, name
            assert bool(dev.torch.isnan(bufA[nextN * M:]).all()) and bool(dev.torch.isnan(bufB[nextN * M:]).all()), "%s wrote past its buffers" % name
            outs.append((bufA[:M].cpu().numpy().copy(), bufB[:M].cpu().numpy().copy()))
        assert np.array_equal(outs[0][0].view(np.uint32), outs[1][0].view(np.uint32)) and \
            np.array_equal(outs[0][1].view(np.uint32), outs[1][1].view(np.uint32)), "%s: field sums differ between two runs" % name
        check(outs[0][0], want_dA, "%s deltaA %s" % (name, (N, M, width)))
        check(outs[0][1], want_dB, "%s deltaB %s" % (name, (N, M, width)))
        # separate result tensors give the same bits as the aliased ones
        dA, dB = dev.guarded(M), dev.guarded(M)
        bufA = dev.empty(max(nextN, 1) * M, fill=float("nan"))
        bufB = dev.empty(max(nextN, 1) * M, fill=float("nan"))
        sums(bufA.data_ptr(), dA.data_ptr(), bufB.data_ptr(), dB.data_ptr(), width, M, 1)
        assert np.array_equal(dev.get(dA).view(np.uint32), outs[0][0].view(np.uint32)), name
        assert np.array_equal(dev.get(dB).view(np.uint32), outs[0][1].view(np.uint32)), name
        # the row function with the sums just made (deltaXp1 = deltaB, deltaXp2 = deltaA)
        dx = dev.guarded(N, M)
        rowfn(dB.data_ptr(), dA.data_ptr(), dx.data_ptr())
        want_dx = O.batchNorm_deltaX(dY, xn64, var, eps, dev.get(dB), dev.get(dA), A=A_or_none)
        want_dx[:, width:] = 0
        got_dx = dev.get(dx)
        check(got_dx, want_dx, "%s deltaX %s" % (name, (N, M, width)))
        assert np.all(got_dx[:, width:] == 0), "%s: pad columns of deltaX must be zero" % name


def test_affine_row_function_zeroes_nan_results(dev):
    # A == 0 makes (Y - B) / A infinite or NaN; the reference writes zero there (within_width_zero_nan)
    N, M = 64, 8
    X, dY, A, B, mean, var, eps, xn, Yaff = _data(N, M, M, 6100)
    A[3] = 0.0
    Yaff = (A * xn + B).astype(np.float32)
    d = {k: dev.put(v) for k, v in dict(dY=dY, A=A, B=B, var=var, Yaff=Yaff).items()}
    p1, p2 = dev.put(normal((M,), 1)), dev.put(normal((M,), 2))
    dx = dev.guarded(N, M)
    F.batchNorm_affined2D_row_deltaX_v1(dev.stream, d["dY"].data_ptr(), d["Yaff"].data_ptr(), d["var"].data_ptr(), eps, d["A"].data_ptr(),
                                        d["B"].data_ptr(), p1.data_ptr(), p2.data_ptr(), M, dx.data_ptr(), N * M, M, M)
    got = dev.get(dx)
    assert np.isfinite(got).all() and np.all(got[:, 3] == 0)


@pytest.mark.parametrize("N,OH,OC", [(16, 28, 64), (4, 7, 132)])
def test_engine_operators(dev, N, OH, OC):
    """The host layer's operators: field sums into scratch (or into deltaA / deltaB for the gradients forms), then the row
    function, on one stream; deltaX in place of deltaY as a training step may do."""
    rows, M = N * OH * OH, OC
    X, dY, A, B, mean, var, eps, xn, Yaff = _data(rows, M, M, 6200 + OC)
    d = {k: dev.put(v) for k, v in dict(X=X, dY=dY, A=A, B=B, mean=mean, var=var, xn=xn, Yaff=Yaff).items()}
    eng = pkg.engine.Engine(dev.stream)
    try:
        xn64 = O.batchNorm_xnorm("from_x", X, X_mean=mean, X_var=var, eps=eps)
        dA64, dB64 = O.batchNorm_deltaAB(dY, xn64)
        # v2, not affine
        dx = dev.guarded(rows, M)
        eng.batchNorm2D_deltaX_v2(dx.data_ptr(), d["dY"].data_ptr(), d["X"].data_ptr(), d["mean"].data_ptr(), d["var"].data_ptr(), eps,
                                  rows, M, rows * M, M, M)
        check(dev.get(dx), O.batchNorm_deltaX(dY, xn64, var, eps, dB64, dA64), "engine batchNorm2D_deltaX_v2")
        # v2 gradients: deltaX, deltaA, deltaB
        dx, dA, dB = dev.guarded(rows, M), dev.guarded(M), dev.guarded(M)
        eng.batchNorm2D_deltaX_v2(dx.data_ptr(), d["dY"].data_ptr(), d["X"].data_ptr(), d["mean"].data_ptr(), d["var"].data_ptr(), eps,
                                  rows, M, rows * M, M, M, A=d["A"].data_ptr(), deltaA=dA.data_ptr(), deltaB=dB.data_ptr())
        check(dev.get(dx), O.batchNorm_deltaX(dY, xn64, var, eps, dB64, dA64, A=A), "engine batchNorm2D_gradients_v2 deltaX")
        check(dev.get(dA), dA64, "engine gradients_v2 deltaA")
        check(dev.get(dB), dB64, "engine gradients_v2 deltaB")
        # v1 from Y, not affine, and affine with gradients; the last one in place
        xg = O.batchNorm_xnorm("given", xn)
        gA, gB = O.batchNorm_deltaAB(dY, xg)
        dx = dev.guarded(rows, M)
        eng.batchNorm2D_deltaX_v1(dx.data_ptr(), d["dY"].data_ptr(), d["xn"].data_ptr(), d["var"].data_ptr(), eps, rows, M, rows * M, M, M)
        check(dev.get(dx), O.batchNorm_deltaX(dY, xg, var, eps, gB, gA), "engine batchNorm2D_deltaX_v1")
        xa = O.batchNorm_xnorm("from_y_affine", Yaff, A=A, B=B)
        aA, aB = O.batchNorm_deltaAB(dY, xa)
        inplace = dev.put(dY)
        dA, dB = dev.guarded(M), dev.guarded(M)
        eng.batchNorm2D_deltaX_v1(inplace.data_ptr(), inplace.data_ptr(), d["Yaff"].data_ptr(), d["var"].data_ptr(), eps, rows, M, rows * M, M, M,
                                  A=d["A"].data_ptr(), B=d["B"].data_ptr(), deltaA=dA.data_ptr(), deltaB=dB.data_ptr())
        eng.sync()
        check(inplace.cpu().numpy(), O.batchNorm_deltaX(dY, xa, var, eps, aB, aA, A=A), "engine batchNorm2D_gradients_v1 deltaX in place")
        check(dev.get(dA), aA, "engine gradients_v1 deltaA")
        check(dev.get(dB), aB, "engine gradients_v1 deltaB")
    finally:
        eng.close()


def test_argument_errors_are_reported():
    p = 256
    with pytest.raises(pkg.AlphaConvError, match="row_lengthv"):
        F.batchNorm2D_row_deltaX_v1(0, p, p, p, 1e-5, p, p, 8, p, 64, 8, 16)
    with pytest.raises(pkg.AlphaConvError, match="buffers are null"):
        R.field_affine_deltaAB_v2(0, 0, p, p, 4096, 64, 0, p, 0, p, 64, 64, 1)
