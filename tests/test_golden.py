"""Committed golden vectors (tests/golden/conv_golden.npz, written by tests/golden/make_fixtures.py): the CPU oracle must
still reproduce them exactly (CPU), and every operator of the HIP library must match them to the bar of the parity tests
(GPU; re-layouts and the Kahan sum bit for bit)."""
import os

import numpy as np
import pytest

from oracle import oracle as O
from util import ROOT, Dev, load_package

G = np.load(os.path.join(ROOT, "tests", "golden", "conv_golden.npz"))
CASES = sorted({k.split("/")[0] for k in G.files})
GRIDZ = 3


def _case(name):
    d = {k.split("/")[1]: G[k] for k in G.files if k.startswith(name + "/")}
    return d, [int(v) for v in d["dims"]]


@pytest.mark.parametrize("name", CASES)
def test_oracle_reproduces_the_golden_vectors(name):
    d, (N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw) = _case(name)
    X, W, dY = d["X"], d["W"], d["dY"]
    assert np.array_equal(O.conv3D_f64(X, W, sh, sw, ph, pw), d["Y"])
    assert np.array_equal(O.deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw), d["dX"])
    assert np.array_equal(O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw), d["dW"])
    assert np.array_equal(O.kernel_remode(W), d["CW"])
    assert np.array_equal(O.ks_remode(W, sh, sw), d["ksCW1"])
    assert np.array_equal(O.ks_remodev2(W, sh, sw), d["ksCW2"])
    parts = np.stack([O.deltaW_slice_f64(X, dY, FH, FW, sh, sw, ph, pw, GRIDZ, z).astype(np.float32) for z in range(GRIDZ)])
    assert np.array_equal(parts, d["dW_parts"])
    assert np.array_equal(O.buf_summary(parts[1:].reshape(GRIDZ - 1, -1), parts[0]).reshape(OC, FH, FW, IC), d["dW_kahan"])
    # the vectors are consistent with each other: the slices add up to the whole, the float variants agree with fp64
    np.testing.assert_allclose(d["dW_parts"].astype(np.float64).sum(0), d["dW"], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(O.conv3D_naive(X, W, sh, sw, ph, pw), d["Y"], rtol=2e-6, atol=2e-6)


def _ok(got, want, what):
    floor = 1e-5 * max(1.0, float(np.sqrt(np.mean(want * want))))
    r = O.max_err_ratio(got, want, 1e-4, floor)
    assert r <= 1.0, "%s: err/allowed = %.3f (rel 1e-4, abs %.3g)" % (what, r, floor)


@pytest.mark.gpu
@pytest.mark.parametrize("name", CASES)
def test_hip_library_matches_the_golden_vectors(name):
    pkg = load_package()
    C3, DX, DW = pkg.Cuda_conv3D, pkg.Cuda_dconv3D_deltaX, pkg.Cuda_dconv3D_deltaW
    dev = Dev()
    d, (N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw) = _case(name)
    OH, OW = d["Y"].shape[1:3]
    x, w, dy = dev.put(d["X"]), dev.put(d["W"]), dev.put(d["dY"])
    S = dev.streams
    # re-layouts: bit for bit
    cw = dev.guarded(FH, FW, IC, OC)
    C3.kernel_remode(dev.stream, w.data_ptr(), cw.data_ptr(), FH, FW, OC, IC)
    assert np.array_equal(dev.get(cw), d["CW"])
    CFH, CFW = O.ks_dims(FH, FW, sh, sw)
    for ver, key in ((DX.ks_remode, "ksCW1"), (DX.ks_remodev2, "ksCW2")):
        k = dev.empty(d[key].size, fill=0.0)
        ver(dev.stream, w.data_ptr(), FH, FW, k.data_ptr(), CFH, CFW, OC, IC, sh, sw)
        assert np.array_equal(dev.get(k), d[key]), key
    # forward from W and from CW
    y = dev.guarded(N, OH, OW, OC)
    C3.conv3D(S, 1, x.data_ptr(), IH, IW, w.data_ptr(), FH, FW, y.data_ptr(), OH, OW, N, IC, OC, sh, sw, ph, pw)
    _ok(dev.get(y), d["Y"], name + " conv3D")
    y = dev.guarded(N, OH, OW, OC)
    C3.conv3D_GemmR(S, 1, x.data_ptr(), IH, IW, w.data_ptr(), cw.data_ptr(), FH, FW, y.data_ptr(), OH, OW, N, IC, OC, sh, sw, ph, pw)
    _ok(dev.get(y), d["Y"], name + " conv3D_GemmR")
    # backward-data
    dx = dev.guarded(N, IH, IW, IC)
    if sh == 1 and sw == 1:
        DX.dconv3D_deltaX_s1(S, 1, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, dx.data_ptr(), IH, IW, N, IC, OC, ph, pw)
    else:
        k = dev.put(d["ksCW2"])
        DX.dconv3D_deltaX_kernelSplit(S, 1, dy.data_ptr(), OH, OW, k.data_ptr(), FH, FW, dx.data_ptr(), IH, IW, N, IC, OC, sh, sw, ph, pw)
    _ok(dev.get(dx), d["dX"], name + " deltaX")
    dx = dev.guarded(N, IH, IW, IC)
    DX.dconv3D_deltaX_crossAdd(S, 1, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, dx.data_ptr(), IH, IW, N, IC, OC, sh, sw, ph, pw)
    _ok(dev.get(dx), d["dX"], name + " deltaX crossAdd")
    # backward-filter: slices one by one through the kernels that keep the reference's slices (the default kernels for
    # 4 stored input channels and for large layers cut the pixels their own way: only their sum is the reference's), the
    # sum through the default path, then the Kahan sum of the golden partials bit for bit
    L = pkg.lib()
    for algo in (3, 4, 0):
        dw = dev.guarded(OC, FH, FW, IC)
        buf = dev.empty(GRIDZ - 1, OC * FH * FW * IC, fill=float("nan"))
        try:
            L.alpha_conv_set_fwd_algo(algo)
            DW.dconv3D_deltaW_GemmSK(S, 1, GRIDZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, dw.data_ptr(), buf.data_ptr(), FH, FW,
                                     N, IC, OC, sh, sw, ph, pw)
        finally:
            L.alpha_conv_set_fwd_algo(0)
        parts = [dev.get(dw)] + [b.reshape(OC, FH, FW, IC) for b in dev.get(buf)]
        if algo != 0:
            for z in range(GRIDZ):
                _ok(parts[z], d["dW_parts"][z].astype(np.float64), "%s deltaW slice %d (algo %d)" % (name, z, algo))
        DW.buf_summary(dev.stream, buf.data_ptr(), dw.data_ptr(), GRIDZ - 1, OC * FH * FW * IC)
        _ok(dev.get(dw), d["dW"], "%s deltaW after buf_summary (algo %d)" % (name, algo))
    gp = dev.put(d["dW_parts"])
    DW.buf_summary(dev.stream, gp[1:].data_ptr(), gp[0].data_ptr(), GRIDZ - 1, OC * FH * FW * IC)
    assert np.array_equal(dev.get(gp)[0], d["dW_kahan"])
