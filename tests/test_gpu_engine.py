"""GPU: the C++ host layer (alpha_engine_*) end to end — it picks the entry the Java engine would pick, owns the
scratch, and the result matches the oracle to the parity bar of test_gpu_parity.py."""
import numpy as np
import pytest

from oracle import oracle as O
from util import Dev, he_normal, load_package, normal, out_dim

pytestmark = pytest.mark.gpu
pkg = load_package()


@pytest.fixture(scope="module")
def dev():
    return Dev()


@pytest.fixture(scope="module")
def eng(dev):
    e = pkg.engine.Engine(dev.stream)
    yield e
    e.close()


def check(got, want, what):
    floor = 1e-5 * max(1.0, float(np.sqrt(np.mean(want * want))))
    r = O.max_err_ratio(got, want, 1e-4, floor)
    assert r <= 1.0, "%s: err/allowed = %.3f (rel 1e-4, abs floor %.3g)" % (what, r, floor)


CASES = [
    # N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, fwd entry, dX entry, dW entry
    (64, 14, 14, 64, 64, 3, 3, 1, 1, 1, 1, "conv3D_GemmV2R", "dconv3D_deltaX_V2_s1", "dconv3D_deltaW_GemmV2SK"),
    (8, 28, 28, 64, 64, 3, 3, 1, 1, 1, 1, "conv3D_GemmR_texture", "dconv3D_deltaX_s1_texture", "dconv3D_deltaW_GemmSK"),
    (8, 14, 14, 64, 128, 1, 1, 1, 1, 0, 0, "conv3D_GemmR_W1", "dconv3D_deltaX_W1", "dconv3D_deltaW_GemmSK_W1"),
    (8, 28, 28, 32, 64, 3, 3, 2, 2, 1, 1, "conv3D_GemmR_texture", "dconv3D_deltaX_ksIms2R", "dconv3D_deltaW_GemmSK"),
    (4, 32, 32, 4, 64, 7, 7, 2, 2, 3, 3, "conv3D_GemmR_texture", "dconv3D_deltaX_crossAdd", "dconv3D_deltaW_GemmSK"),
    (4, 12, 9, 32, 32, 3, 3, 3, 3, 1, 1, "conv3D_GemmR_texture", "dconv3D_deltaX_ksImsR", "dconv3D_deltaW"),
    (4, 13, 11, 32, 16, 5, 4, 3, 2, 2, 1, "conv3D_texture", "dconv3D_deltaX_kernelSplit", "dconv3D_deltaW"),
    (4, 9, 9, 16, 8, 3, 3, 1, 1, 0, 0, "conv3D_np", "dconv3D_deltaX_s1_texture", "dconv3D_deltaW"),
    # 1x1 stride 2 (BASELINE c4c geometry): must NOT go to the stride-less W1 natives
    (8, 28, 28, 64, 128, 1, 1, 2, 2, 0, 0, "conv3D_GemmR_texture", "dconv3D_deltaX_ksIms2R", "dconv3D_deltaW_GemmSK"),
]


def test_engine_refuses_inconsistent_sizes(dev, eng):
    x = dev.empty(4, 8, 8, 8, fill=0.0)
    w = dev.empty(8, 3, 3, 8, fill=0.0)
    y = dev.empty(4, 8, 8, 8, fill=0.0)
    with pytest.raises(pkg.AlphaConvError, match="illegal size"):
        eng.conv3D(y.data_ptr(), 16, 16, x.data_ptr(), 8, 8, w.data_ptr(), 3, 3, 4, 8, 8, 1, 1, 1, 1)   # OH larger than the input allows


@pytest.mark.parametrize("case", CASES)
def test_engine_runs_the_entry_java_would_pick(dev, eng, case):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, e_fwd, e_dx, e_dw = case
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    X, W, dY = normal((N, IH, IW, IC), 6001), he_normal(OC, FH, FW, IC, 6002), normal((N, OH, OW, OC), 6003)
    x, w, dy = dev.put(X), dev.put(W), dev.put(dY)
    y = dev.empty(N, OH, OW, OC, fill=float("nan"))
    dx = dev.empty(N, IH, IW, IC, fill=float("nan"))
    dw = dev.empty(OC, FH, FW, IC, fill=float("nan"))
    p1 = eng.conv3D(y.data_ptr(), OH, OW, x.data_ptr(), IH, IW, w.data_ptr(), FH, FW, N, IC, OC, sh, sw, ph, pw)
    p2 = eng.dconv3D_deltaX(dx.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, N, IC, OC, sh, sw, ph, pw)
    p3 = eng.dconv3D_deltaW(dw.data_ptr(), FH, FW, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC, sh, sw, ph, pw)
    eng.sync()
    assert (p1.entry_name, p2.entry_name, p3.entry_name) == (e_fwd, e_dx, e_dw)
    check(dev.get(y), O.conv3D_f64(X, W, sh, sw, ph, pw), "engine conv3D %s" % (case,))
    check(dev.get(dx), O.deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw), "engine deltaX %s" % (case,))
    check(dev.get(dw), O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw), "engine deltaW %s" % (case,))


def test_engine_deltaX_winograd_flag(dev, eng):
    """deltaX_winograd = 1 sends 3x3 stride-1 backward-data through the Winograd entry (scratch from the engine's pool);
    off, the plan is the reference's."""
    N, IH, IC, OC = 8, 14, 64, 32
    dY, W = normal((N, IH, IH, OC), 6211), he_normal(OC, 3, 3, IC, 6212)
    want = O.deltaX_f64(dY, W, IH, IH, 1, 1, 1, 1)
    dy, w = dev.put(dY), dev.put(W)
    for wino in (0, 1):
        eng.config.deltaX_winograd = wino
        try:
            dx = dev.empty(N, IH, IH, IC, fill=float("nan"))
            p = eng.dconv3D_deltaX(dx.data_ptr(), IH, IH, dy.data_ptr(), IH, IH, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, 1, 1)
            eng.sync()
        finally:
            eng.config.deltaX_winograd = 0
        assert p.entry_name == ("dconv3D_deltaX_winograd" if wino else "dconv3D_deltaX_s1_texture")
        check(dev.get(dx), want, "engine deltaX (winograd %d)" % wino)
    # a strided layer keeps the reference's plan with the flag set
    eng.config.deltaX_winograd = 1
    try:
        assert pkg.engine.plan_deltaX(eng.config, 14, 14, 7, 7, 3, 3, N, IC, OC, 2, 2).entry_name != "dconv3D_deltaX_winograd"
    finally:
        eng.config.deltaX_winograd = 0


def test_engine_deltaW_winograd_flag(dev, eng):
    """deltaW_winograd > 0 sends the split-K backward-filter of a 3x3 stride-1 layer through the Winograd F(3x3,2x2) entry
    (1: the reference's GridZ; > 1: GridZ sized for that many compute units); off, the plan is the reference's."""
    N, IH, IC, OC = 8, 16, 64, 64
    X, dY = normal((N, IH, IH, IC), 6221), normal((N, IH, IH, OC), 6222)
    want = O.deltaW_f64(X, dY, 3, 3, 1, 1, 1, 1)
    x, dy = dev.put(X), dev.put(dY)
    ref_plan = pkg.engine.plan_deltaW(eng.config, IH, IH, IH, IH, 3, 3, N, IC, OC, 1, 1)
    for flag in (0, 1, 64):
        eng.config.deltaW_winograd = flag
        try:
            dw = dev.empty(OC, 3, 3, IC, fill=float("nan"))
            p = eng.dconv3D_deltaW(dw.data_ptr(), 3, 3, x.data_ptr(), IH, IH, dy.data_ptr(), IH, IH, N, IC, OC, 1, 1, 1, 1)
            eng.sync()
        finally:
            eng.config.deltaW_winograd = 0
        if flag:
            assert p.entry_name == "dconv3D_deltaW_GemmSK_winograd"
            if flag == 1:
                assert p.GridZ == ref_plan.GridZ
            else:
                assert p.GridZ == min(64 // 2, N * 8 * 8 // 64)   # 2 channel blocks; slices of at least 64 tiles
        else:
            assert p.entry_name == ref_plan.entry_name
        check(dev.get(dw), want, "engine deltaW (winograd %d)" % flag)
    # strided and 1x1 layers keep the reference's plan with the flag set
    eng.config.deltaW_winograd = 1
    try:
        assert pkg.engine.plan_deltaW(eng.config, 16, 16, 8, 8, 3, 3, N, IC, OC, 2, 2).entry_name != "dconv3D_deltaW_GemmSK_winograd"
        assert pkg.engine.plan_deltaW(eng.config, 16, 16, 16, 16, 1, 1, N, IC, OC, 1, 1).entry_name != "dconv3D_deltaW_GemmSK_winograd"
    finally:
        eng.config.deltaW_winograd = 0


def test_engine_conv3D_biased(dev, eng):
    N, IH, IC, OC = 8, 14, 64, 64
    X, W, B = normal((N, IH, IH, IC), 6201), he_normal(OC, 3, 3, IC, 6202), normal((OC,), 6203)
    want = O.conv3D_f64(X, W, 1, 1, 1, 1) + B.astype(np.float64)[None, None, None, :]
    x, w, b = dev.put(X), dev.put(W), dev.put(B)
    for wino in (0, 1):
        eng.config.conv3D_winograd = wino
        try:
            y = dev.empty(N, IH, IH, OC, fill=float("nan"))
            p = eng.conv3D_biased(y.data_ptr(), IH, IH, x.data_ptr(), IH, IH, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, 1, 1,
                                  b.data_ptr(), N * IH * IH * OC, OC)
            eng.sync()
        finally:
            eng.config.conv3D_winograd = 0
        assert p.entry_name == ("conv3D_winograd" if wino else "conv3D_GemmR_texture")
        check(dev.get(y), want, "engine conv3D_biased (winograd %d)" % wino)
    with pytest.raises(pkg.AlphaConvError, match="lengthv"):
        eng.conv3D_biased(y.data_ptr(), IH, IH, x.data_ptr(), IH, IH, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, 1, 1,
                          b.data_ptr(), N * IH * IH * OC - 4, OC)


@pytest.mark.parametrize("shape", [
    # N, IH, IW, IC, OC, F, s, p: row-streaming kernel (32 and 16 channels per workgroup), register 1x1 kernel, 1x1 through
    # the row kernel (ragged channels), generic kernel (strided), single-pass entry (GK < 512)
    (16, 14, 14, 64, 128, 3, 1, 1),
    (32, 8, 8, 256, 256, 3, 1, 1),
    (8, 14, 14, 128, 64, 1, 1, 0),
    (8, 12, 12, 36, 44, 1, 1, 0),
    (8, 20, 20, 32, 48, 3, 2, 1),
    (4, 9, 9, 16, 24, 3, 1, 1),
    (16, 32, 32, 4, 64, 3, 1, 1),      # a first layer (4 stored input channels): its own kernel, the column sums as a pass
    (8, 40, 40, 4, 96, 7, 2, 3),
])
def test_engine_deltaW_with_bias_gradient(dev, eng, shape):
    """deltaB[oc] = sum over all pixels of deltaY (the reference: field_sum(deltaY, OC) after dconv3D_deltaW)."""
    N, IH, IW, IC, OC, F_, s_, p_ = shape
    OH, OW = out_dim(IH, IW, F_, F_, s_, s_, p_, p_)
    X, dY = normal((N, IH, IW, IC), 6401), normal((N, OH, OW, OC), 6402)
    x, dy = dev.put(X), dev.put(dY)
    got = []
    for _ in range(2):
        dw = dev.empty(OC, F_, F_, IC, fill=float("nan"))
        db = dev.empty(OC, fill=float("nan"))
        eng.dconv3D_deltaW_deltaB(dw.data_ptr(), db.data_ptr(), F_, F_, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC,
                                  s_, s_, p_, p_)
        eng.sync()
        got.append((dev.get(dw), dev.get(db)))
    check(got[0][0], O.deltaW_f64(X, dY, F_, F_, s_, s_, p_, p_), "deltaW with deltaB %s" % (shape,))
    check(got[0][1], dY.astype(np.float64).sum(axis=(0, 1, 2)), "deltaB %s" % (shape,))
    assert np.array_equal(got[0][0], got[1][0]) and np.array_equal(got[0][1], got[1][1]), "run-to-run bits differ"


def test_engine_filter_transform_cache(dev):
    """With cache_filter_transforms the re-layout runs once per filter; a weight update must be reported."""
    N, IH, IC, OC = 8, 12, 64, 64
    X, W1, W2 = normal((N, IH, IH, IC), 6301), he_normal(OC, 3, 3, IC, 6302), he_normal(OC, 3, 3, IC, 6303)
    dY = normal((N, 6, 6, OC), 6304)
    x, w, dy = dev.put(X), dev.put(W1), dev.put(dY)
    e = pkg.engine.Engine(dev.stream)
    try:
        e.config.cache_filter_transforms = 1
        for wino in (0, 1):
            e.config.conv3D_winograd = wino
            w.copy_(dev.put(W1))
            e.filter_changed(w.data_ptr())
            y = dev.empty(N, IH, IH, OC, fill=float("nan"))
            for _ in range(2):   # second call: transform taken from the cache
                e.conv3D(y.data_ptr(), IH, IH, x.data_ptr(), IH, IH, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, 1, 1)
            e.sync()
            check(dev.get(y), O.conv3D_f64(X, W1, 1, 1, 1, 1), "cached transform, first weights (winograd %d)" % wino)
            w.copy_(dev.put(W2))              # optimizer step: same address, new values
            e.conv3D(y.data_ptr(), IH, IH, x.data_ptr(), IH, IH, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, 1, 1)
            e.sync()
            stale = dev.get(y)
            check(stale, O.conv3D_f64(X, W1, 1, 1, 1, 1), "unreported update keeps the old transform (winograd %d)" % wino)
            e.filter_changed(w.data_ptr())
            e.conv3D(y.data_ptr(), IH, IH, x.data_ptr(), IH, IH, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, 1, 1)
            e.sync()
            check(dev.get(y), O.conv3D_f64(X, W2, 1, 1, 1, 1), "after filter_changed (winograd %d)" % wino)
        # kernel-split backward-data shares the cache (another kind under the same address)
        e.config.conv3D_winograd = 0
        dx = dev.empty(N, IH, IH, IC, fill=float("nan"))
        for _ in range(2):
            p = e.dconv3D_deltaX(dx.data_ptr(), IH, IH, dy.data_ptr(), 6, 6, w.data_ptr(), 3, 3, N, IC, OC, 2, 2, 1, 1)
        e.sync()
        assert p.remode == 1
        check(dev.get(dx), O.deltaX_f64(dY, W2, IH, IH, 2, 2, 1, 1), "cached kernel-split filter")
    finally:
        e.close()


def test_engine_winograd_flags_and_a_smaller_output_than_the_formula(dev):
    """The engine accepts an output smaller than (IH + 2p - F)/s + 1 (EngineCore.java:653-665); the Winograd kernels need the
    exact size, so with every Winograd flag on such a layer runs on its default entries and gives the leading block of
    the full result (forward) / the gradients of a deltaY that is zero outside that block (backward)."""
    N, IH, IW, IC, OC = 4, 12, 12, 32, 32
    OH, OW = 11, 10
    X, W, dY = normal((N, IH, IW, IC), 6401), he_normal(OC, 3, 3, IC, 6402), normal((N, OH, OW, OC), 6403)
    dYfull = np.zeros((N, IH, IW, OC), np.float32)
    dYfull[:, :OH, :OW] = dY
    x, w, dy = dev.put(X), dev.put(W), dev.put(dY)
    e = pkg.engine.Engine(dev.stream)
    try:
        e.config.conv3D_winograd = 1
        e.config.deltaX_winograd = 1
        e.config.deltaW_winograd = 1
        e.config.deltaW_SplitKThreshold = 64
        y = dev.guarded(N, OH, OW, OC)
        dx = dev.guarded(N, IH, IW, IC)
        dw = dev.guarded(OC, 3, 3, IC)
        p1 = e.conv3D(y.data_ptr(), OH, OW, x.data_ptr(), IH, IW, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, 1, 1)
        p2 = e.dconv3D_deltaX(dx.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, 1, 1)
        p3 = e.dconv3D_deltaW(dw.data_ptr(), 3, 3, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC, 1, 1, 1, 1)
        e.sync()
        assert "winograd" not in p1.entry_name + p2.entry_name + p3.entry_name
        check(dev.get(y), np.ascontiguousarray(O.conv3D_f64(X, W, 1, 1, 1, 1)[:, :OH, :OW]), "smaller output, forward")
        check(dev.get(dx), O.deltaX_f64(dYfull, W, IH, IW, 1, 1, 1, 1), "smaller output, deltaX")
        check(dev.get(dw), O.deltaW_f64(X, dYfull, 3, 3, 1, 1, 1, 1), "smaller output, deltaW")
    finally:
        e.close()


def test_engine_deltaW_with_fill_option(dev):
    """A larger split-K factor changes the summation order, not the result beyond the parity bar."""
    N, IH, IC, OC = 32, 14, 128, 128
    X, dY = normal((N, IH, IH, IC), 6101), normal((N, IH, IH, OC), 6102)
    x, dy = dev.put(X), dev.put(dY)
    want = O.deltaW_f64(X, dY, 3, 3, 1, 1, 1, 1)
    e = pkg.engine.Engine(dev.stream)
    try:
        gz = []
        e.config.deltaW_SK_leastUnits = 0     # engine objects lower GridZ to what the persistent kernel needs (7 here): not the subject
        for units in (0, 256):
            e.config.deltaW_SK_fillUnits = units
            dw = dev.empty(OC, 3, 3, IC, fill=float("nan"))
            p = e.dconv3D_deltaW(dw.data_ptr(), 3, 3, x.data_ptr(), IH, IH, dy.data_ptr(), IH, IH, N, IC, OC, 1, 1, 1, 1)
            e.sync()
            gz.append(p.GridZ)
            check(dev.get(dw), want, "engine deltaW fillUnits=%d (GridZ %d)" % (units, p.GridZ))
        assert gz[1] > gz[0] and gz[1] == 24      # GK = 6272: 512/8 tiles = 64, capped by GK>>8 = 24
    finally:
        e.close()


@pytest.mark.parametrize("shape,least", [((32, 28, 64, 64, 3), 28),      # 9 items of (tap, 64 x 64 block): 28 pieces each on 256 units (reference: 39)
                                         ((32, 28, 256, 64, 1), 64),     # 1x1: 4 items -> 64 pieces (reference: 98)
                                         ((32, 16, 128, 128, 3), 7)])    # 36 items -> 7 pieces (reference: 28)
def test_engine_deltaW_with_least_option(dev, shape, least):
    """The least split-K factor the persistent kernel needs: the same result to the parity bar from fewer partial sums,
    and bit-identical from run to run."""
    N, IH, IC, OC, F_ = shape
    p_ = F_ // 2
    X, dY = normal((N, IH, IH, IC), 6111), normal((N, IH, IH, OC), 6112)
    x, dy = dev.put(X), dev.put(dY)
    want = O.deltaW_f64(X, dY, F_, F_, 1, 1, p_, p_)
    units = pkg.device_info()[0]
    e = pkg.engine.Engine(dev.stream)
    try:
        gz, got = [], []
        for on in (0, units, units):
            e.config.deltaW_SK_leastUnits = on
            dw = dev.empty(OC, F_, F_, IC, fill=float("nan"))
            p = e.dconv3D_deltaW(dw.data_ptr(), F_, F_, x.data_ptr(), IH, IH, dy.data_ptr(), IH, IH, N, IC, OC, 1, 1, p_, p_)
            e.sync()
            gz.append(p.GridZ)
            got.append(dev.get(dw))
            check(got[-1], want, "engine deltaW leastUnits=%d (GridZ %d) %s" % (on, p.GridZ, shape))
        assert gz[1] <= gz[0] and gz[1] == gz[2]
        if units == 256:
            assert gz[1] == least, gz
        assert np.array_equal(got[1], got[2])
    finally:
        e.close()


def test_engine_scratch_is_recycled_after_sync(dev, eng):
    N, IH, IC, OC = 8, 16, 32, 64
    X, W = normal((N, IH, IH, IC), 6004), he_normal(OC, 3, 3, IC, 6005)
    x, w = dev.put(X), dev.put(W)
    want = O.conv3D_f64(X, W, 1, 1, 1, 1)
    for _ in range(3):
        y = dev.empty(N, IH, IH, OC, fill=float("nan"))
        for _ in range(4):   # several enqueues between syncs: each takes its own CW block
            eng.conv3D(y.data_ptr(), IH, IH, x.data_ptr(), IH, IH, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, 1, 1)
        eng.sync()
        check(dev.get(y), want, "repeat")


def _random_cases(count, seed):
    """Seeded random layer geometries inside what the Java engine accepts (EngineCore.java:630-678: sh <= FH, sw <= FW,
    pads below the filter size, N/IC/OC multiples of 4): the analogue of the reference's sweeps over ragged sizes
    (Cuda_conv3D_test.java:155-156), with image widths on both sides of the kernels' row-width classes (16/32/48
    padded columns), channel counts on both sides of 64 and all filter sizes the specialised kernels serve."""
    rng = np.random.Generator(np.random.PCG64(seed))
    cases = []
    while len(cases) < count:
        F_ = int(rng.choice([1, 2, 3, 3, 3, 4, 5, 7]))
        FW_ = F_ if rng.random() < 0.8 else int(rng.choice([1, 2, 3, 4, 5]))
        sh = int(rng.integers(1, min(F_, 3) + 1)) if rng.random() < 0.4 else 1
        sw = min(sh, FW_) if rng.random() < 0.8 else int(rng.integers(1, min(FW_, 3) + 1))
        ph, pw = int(rng.integers(0, F_)), int(rng.integers(0, FW_))
        IH, IW = int(rng.integers(F_, 41)), int(rng.integers(FW_, 61))
        IC = 4 * int(rng.choice([1, 2, 3, 8, 16, 17, 24, 32, 40]))
        OC = 4 * int(rng.choice([1, 2, 5, 8, 16, 16, 19, 32, 48]))
        N = int(rng.choice([4, 8]))
        OH, OW = out_dim(IH, IW, F_, FW_, sh, sw, ph, pw)
        if OH < 1 or OW < 1 or N * IH * IW * IC > 3_000_000 or N * OH * OW * OC > 3_000_000:
            continue
        cases.append((N, IH, IW, IC, OC, F_, FW_, sh, sw, ph, pw))
    return cases


@pytest.mark.parametrize("case", _random_cases(36, 20240611))
def test_engine_random_geometries(dev, eng, case):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = case
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    seed = 7000 + (hash(case) % 1000)
    X, W, dY = normal((N, IH, IW, IC), seed), he_normal(OC, FH, FW, IC, seed + 1), normal((N, OH, OW, OC), seed + 2)
    x, w, dy = dev.put(X), dev.put(W), dev.put(dY)
    y = dev.empty(N, OH, OW, OC, fill=float("nan"))
    dx = dev.empty(N, IH, IW, IC, fill=float("nan"))
    dw = dev.empty(OC, FH, FW, IC, fill=float("nan"))
    eng.conv3D(y.data_ptr(), OH, OW, x.data_ptr(), IH, IW, w.data_ptr(), FH, FW, N, IC, OC, sh, sw, ph, pw)
    eng.dconv3D_deltaX(dx.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, N, IC, OC, sh, sw, ph, pw)
    eng.dconv3D_deltaW(dw.data_ptr(), FH, FW, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC, sh, sw, ph, pw)
    eng.sync()
    check(dev.get(y), O.conv3D_f64(X, W, sh, sw, ph, pw), "conv3D %s" % (case,))
    check(dev.get(dx), O.deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw), "deltaX %s" % (case,))
    check(dev.get(dw), O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw), "deltaW %s" % (case,))


def _random_small_map_cases(count, seed):
    """Seeded random layers on small maps (2 to 14 pixels a side) at larger batches, channel counts on both sides of the 64-wide
    blocks and 4 stored input channels: the geometries of the reference's CIFAR-10 networks' later stages, where the work
    items per compute unit are few and the persistent backward-filter kernel's rows are short."""
    rng = np.random.Generator(np.random.PCG64(seed))
    cases = []
    while len(cases) < count:
        F_ = int(rng.choice([1, 3, 3, 5]))
        s_ = int(rng.choice([1, 1, 2]))
        p_ = int(rng.choice([0, F_ // 2]))
        IH, IW = int(rng.choice([2, 3, 4, 5, 6, 7, 8, 9, 13, 14])), int(rng.choice([2, 3, 4, 5, 6, 7, 8, 9, 13, 14]))
        IC = int(rng.choice([4, 16, 32, 48, 64, 96, 128, 256]))
        OC = int(rng.choice([8, 36, 64, 96, 128, 208, 256]))
        N = int(rng.choice([32, 64, 128]))
        if IH + 2 * p_ < F_ or IW + 2 * p_ < F_ or s_ > F_:
            continue
        OH, OW = out_dim(IH, IW, F_, F_, s_, s_, p_, p_)
        if OH < 1 or OW < 1 or N * OH * OW * OC * IC * F_ * F_ > 300_000_000:
            continue
        cases.append((N, IH, IW, IC, OC, F_, F_, s_, s_, p_, p_))
    return cases


@pytest.mark.parametrize("case", _random_small_map_cases(30, 20250217))
def test_engine_random_small_maps(dev, eng, case):
    N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw = case
    OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
    seed = 7500 + (hash(case) % 1000)
    X, W, dY = normal((N, IH, IW, IC), seed), he_normal(OC, FH, FW, IC, seed + 1), normal((N, OH, OW, OC), seed + 2)
    x, w, dy = dev.put(X), dev.put(W), dev.put(dY)
    y = dev.empty(N, OH, OW, OC, fill=float("nan"))
    dw = dev.empty(OC, FH, FW, IC, fill=float("nan"))
    eng.conv3D(y.data_ptr(), OH, OW, x.data_ptr(), IH, IW, w.data_ptr(), FH, FW, N, IC, OC, sh, sw, ph, pw)
    eng.dconv3D_deltaW(dw.data_ptr(), FH, FW, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC, sh, sw, ph, pw)
    eng.sync()
    check(dev.get(y), O.conv3D_f64(X, W, sh, sw, ph, pw), "conv3D %s" % (case,))
    check(dev.get(dw), O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw), "deltaW %s" % (case,))
    want = O.deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw)
    L = pkg.lib()
    try:
        for sharing in ((-1,) if sh == 1 else (-1, 0, 1)):   # strided: both distributions of the kernel-split kernel's work
            L.alpha_conv_set_kernel_split_sharing(sharing)
            dx = dev.empty(N, IH, IW, IC, fill=float("nan"))
            eng.dconv3D_deltaX(dx.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, w.data_ptr(), FH, FW, N, IC, OC, sh, sw, ph, pw)
            eng.sync()
            check(dev.get(dx), want, "deltaX sharing %d %s" % (sharing, case))
    finally:
        L.alpha_conv_set_kernel_split_sharing(-1)


def _random_3x3_cases(count, seed):
    """Seeded random 3x3 stride-1 layers with channel counts the LDS-halo kernels take: row widths from 3 to 62 (both
    row-width classes of the halo-prefetching kernel and its limits), batch sizes that give anything from a fraction of
    a unit to several units per workgroup plus left-over pieces, pads 0..2, ragged output channel counts."""
    rng = np.random.Generator(np.random.PCG64(seed))
    cases = []
    while len(cases) < count:
        IH, IW = int(rng.integers(3, 41)), int(rng.integers(3, 63))
        IC = int(rng.choice([32, 64, 96, 128]))
        OC = int(rng.choice([16, 48, 64, 80, 128]))
        ph, pw = int(rng.integers(0, 3)), int(rng.integers(0, 3))
        N = int(rng.choice([1, 3, 4, 8, 20, 60, 150]))
        OH, OW = out_dim(IH, IW, 3, 3, 1, 1, ph, pw)
        if OH < 1 or OW < 1 or N * OH * OW * OC * IC * 18 > 1.5e9 or N * IH * IW * IC > 6_000_000:
            continue
        cases.append((N, IH, IW, IC, OC, ph, pw))
    return cases


@pytest.mark.parametrize("case", _random_3x3_cases(20, 20241125))
def test_engine_random_3x3_stride1_layers(dev, eng, case):
    N, IH, IW, IC, OC, ph, pw = case
    OH, OW = out_dim(IH, IW, 3, 3, 1, 1, ph, pw)
    seed = 9000 + (hash(case) % 1000)
    X, W, dY = normal((N, IH, IW, IC), seed), he_normal(OC, 3, 3, IC, seed + 1), normal((N, OH, OW, OC), seed + 2)
    x, w, dy = dev.put(X), dev.put(W), dev.put(dY)
    y, y_w = dev.guarded(N, OH, OW, OC), dev.guarded(N, OH, OW, OC)
    dx = dev.guarded(N, IH, IW, IC)
    dw = dev.guarded(OC, 3, 3, IC)
    eng.conv3D(y.data_ptr(), OH, OW, x.data_ptr(), IH, IW, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, ph, pw)
    pkg.Cuda_conv3D.conv3D(dev.streams, 1, x.data_ptr(), IH, IW, w.data_ptr(), 3, 3, y_w.data_ptr(), OH, OW, N, IC, OC, 1, 1, ph, pw)
    eng.dconv3D_deltaX(dx.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, ph, pw)
    eng.dconv3D_deltaW(dw.data_ptr(), 3, 3, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC, 1, 1, ph, pw)
    eng.sync()
    want = O.conv3D_f64(X, W, 1, 1, ph, pw)
    check(dev.get(y), want, "conv3D %s" % (case,))
    check(dev.get(y_w), want, "conv3D from W %s" % (case,))
    check(dev.get(dx), O.deltaX_f64(dY, W, IH, IW, 1, 1, ph, pw), "deltaX %s" % (case,))
    check(dev.get(dw), O.deltaW_f64(X, dY, 3, 3, 1, 1, ph, pw), "deltaW %s" % (case,))
    # the same layer through this build's three Winograd paths
    y2, dx2, dw2 = dev.guarded(N, OH, OW, OC), dev.guarded(N, IH, IW, IC), dev.guarded(OC, 3, 3, IC)
    eng.config.conv3D_winograd, eng.config.deltaX_winograd, eng.config.deltaW_winograd = 1, 1, 40
    try:
        p1 = eng.conv3D(y2.data_ptr(), OH, OW, x.data_ptr(), IH, IW, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, ph, pw)
        p2 = eng.dconv3D_deltaX(dx2.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, w.data_ptr(), 3, 3, N, IC, OC, 1, 1, ph, pw)
        p3 = eng.dconv3D_deltaW(dw2.data_ptr(), 3, 3, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, N, IC, OC, 1, 1, ph, pw)
        eng.sync()
    finally:
        eng.config.conv3D_winograd, eng.config.deltaX_winograd, eng.config.deltaW_winograd = 0, 0, 0
    assert p1.entry_name == "conv3D_winograd" and p2.entry_name == "dconv3D_deltaX_winograd"
    check(dev.get(y2), want, "Winograd conv3D %s" % (case,))
    check(dev.get(dx2), O.deltaX_f64(dY, W, IH, IW, 1, 1, ph, pw), "Winograd deltaX %s" % (case,))
    if N * OH * OW >= 512:   # below the split-K threshold the plain entry stays
        assert p3.entry_name == "dconv3D_deltaW_GemmSK_winograd"
    check(dev.get(dw2), O.deltaW_f64(X, dY, 3, 3, 1, 1, ph, pw), "Winograd deltaW %s" % (case,))



DECONV_CASES = [
    # N, input H, W, input channels (= OC of the filter W[OC, FH, FW, IC]), produced channels (= IC), FH, FW, sh, sw, ph, pw
    (8, 14, 14, 64, 32, 4, 4, 2, 2, 1, 1),    # the usual 2x up-sampling: 14x14 -> 28x28
    (4, 16, 16, 32, 64, 3, 3, 1, 1, 1, 1),    # stride 1: a 3x3 convolution with the rotated, transposed filter
    (4, 9, 7, 32, 16, 3, 3, 2, 2, 0, 0),      # no padding, odd sizes: 9x7 -> 19x15
]


@pytest.mark.parametrize("case", DECONV_CASES)
def test_engine_transposed_convolution_unit(dev, eng, case):
    """The reference's Deconv3D unit is the same three operators with the roles swapped (nn/unit/simple/Deconv3D.java:141-176,
    Engine.java:1819-1852): forward = dconv3D_deltaX of its input, gradient of W = dconv3D_deltaW with the unit's deltaY as
    X and its input as deltaY, gradient of the input = conv3D of deltaY. Each against the oracle, and the pair
    (forward, input gradient) against each other: <forward(X), dY> = <X, backward(dY)> for any X, dY."""
    N, H, Wd, C_in, C_out, FH, FW, sh, sw, ph, pw = case
    OH, OW = (H - 1) * sh + FH - 2 * ph, (Wd - 1) * sw + FW - 2 * pw     # Deconv3D.java:144-145
    X, Wt, dYu = normal((N, H, Wd, C_in), 6101), he_normal(C_in, FH, FW, C_out, 6102), normal((N, OH, OW, C_out), 6103)
    x, w, dyu = dev.put(X), dev.put(Wt), dev.put(dYu)
    y = dev.empty(N, OH, OW, C_out, fill=float("nan"))
    dw = dev.empty(C_in, FH, FW, C_out, fill=float("nan"))
    dx = dev.empty(N, H, Wd, C_in, fill=float("nan"))
    # in the operators' own terms the convolution is [N, OH, OW, IC = C_out] -> [N, H, Wd, OC = C_in]
    eng.dconv3D_deltaX(y.data_ptr(), OH, OW, x.data_ptr(), H, Wd, w.data_ptr(), FH, FW, N, C_out, C_in, sh, sw, ph, pw)
    eng.dconv3D_deltaW(dw.data_ptr(), FH, FW, dyu.data_ptr(), OH, OW, x.data_ptr(), H, Wd, N, C_out, C_in, sh, sw, ph, pw)
    eng.conv3D(dx.data_ptr(), H, Wd, dyu.data_ptr(), OH, OW, w.data_ptr(), FH, FW, N, C_out, C_in, sh, sw, ph, pw)
    eng.sync()
    got_y, got_dw, got_dx = dev.get(y), dev.get(dw), dev.get(dx)
    check(got_y, O.deltaX_f64(X, Wt, OH, OW, sh, sw, ph, pw), "transposed convolution forward %s" % (case,))
    check(got_dw, O.deltaW_f64(dYu, X, FH, FW, sh, sw, ph, pw), "transposed convolution, gradient of W %s" % (case,))
    check(got_dx, O.conv3D_f64(dYu, Wt, sh, sw, ph, pw), "transposed convolution, gradient of the input %s" % (case,))
    lhs = float(np.sum(got_y.astype(np.float64) * dYu))
    rhs = float(np.sum(X.astype(np.float64) * got_dx))
    scale = float(np.sqrt(np.sum(got_y.astype(np.float64) ** 2) * np.sum(dYu.astype(np.float64) ** 2)))
    assert abs(lhs - rhs) <= 1e-5 * scale, "adjointness: %.9g against %.9g" % (lhs, rhs)
