"""The host-side selection logic (include/alpha_engine.h) against values computed by hand from the reference's Java
formulas (CudaFloat32EngineBase.java:1355-1474, 1666-1762, 1796-2005; Cuda_conv3D.java:19-135 and twins). Pure integer
functions: no GPU needed."""
import pytest

from util import load_package

pkg = load_package()
E = pkg.engine


def java_blockNum(GN, GM):
    """Independent restatement of the Java loop as arithmetic on the binary digits."""
    def side(g):
        return g // 128 + sum(1 for b in (64, 32, 16, 8, 4) if g % 128 & b)
    return side(GN) * side(GM)


def test_blockNum_and_streamSize_hand_values():
    assert E.blockNum(64, 100352) == 784              # 1 x 784 whole 128-tiles
    assert E.blockNum(64, 576) == 5                   # 576 = 4*128 + 64
    assert E.blockNum(252, 4096) == (1 + 5) * 32      # 252 = 128 + 64+32+16+8+4
    assert E.blockNum(4, 4) == 1
    for gn, gm in [(64, 200704), (132, 36), (1024, 12544), (20, 52), (255 // 4 * 4, 100)]:
        assert E.blockNum(gn, gm) == java_blockNum(gn, gm)
    assert E.streamSize(64, 4096) == 1                # both powers of two
    assert E.streamSize(252, 4096) == 6               # 128 + 64+32+16+8+4 -> 6 strips
    assert E.streamSize(252, 100) == 10               # 6 x 3 = 18, capped at 10   (100 = 64+32+4)
    assert E.streamSize(252, 100, 12) == 12
    assert E.streamSize(1024, 12544) == 1             # 12544 = 98*128: one strip


def test_forward_plans_of_the_baseline_configs():
    cfg = E.default_config(256)
    # c3a: N=64 > 63, OC=64 > 63, Q = 58*58/(56*56) = 1.0727 > 1.05  ->  V2 entry, one stream (64, 64 powers of two)
    p = E.plan_conv3D(cfg, 56, 56, 56, 56, 3, 3, 64, 64, 64, 1, 1, 1, 1)
    assert p.entry_name == "conv3D_GemmV2R" and p.remode == 1 and p.V2 == 1 and p.streams == 1
    assert p.Q == pytest.approx(3364 / 3136) and p.scratch_floats == 3 * 3 * 64 * 64
    # c1: N=4 -> not V2; texture flag on -> GemmR_texture
    p = E.plan_conv3D(cfg, 32, 32, 32, 32, 3, 3, 4, 4, 64, 1, 1, 1, 1)
    assert p.entry_name == "conv3D_GemmR_texture" and p.streams == 1
    # c4d: 1x1 -> GemmR_W1
    p = E.plan_conv3D(cfg, 14, 14, 14, 14, 1, 1, 64, 256, 1024, 1, 1, 0, 0)
    assert p.entry_name == "conv3D_GemmR_W1" and p.V2 == 0
    # c4a stem: N=64, OC=64, Q = (111*2+7)^2/224^2 = 1.045 < 1.05 -> GemmR_texture
    p = E.plan_conv3D(cfg, 224, 224, 112, 112, 7, 7, 64, 4, 64, 2, 2, 3, 3)
    assert p.entry_name == "conv3D_GemmR_texture" and p.Q == pytest.approx(229 * 229 / 224 / 224)
    # small problems take the non-remode entries
    assert E.plan_conv3D(cfg, 8, 8, 8, 8, 3, 3, 4, 8, 16, 1, 1, 1, 1).entry_name == "conv3D_texture"
    assert E.plan_conv3D(cfg, 8, 8, 8, 8, 3, 3, 4, 8, 8, 1, 1, 1, 1).entry_name == "conv3D"       # OC <= 15: no texture
    assert E.plan_conv3D(cfg, 8, 8, 6, 6, 3, 3, 4, 8, 16, 1, 1, 0, 0).entry_name == "conv3D_np"
    assert E.plan_conv3D(cfg, 8, 8, 8, 8, 1, 1, 4, 8, 16, 1, 1, 0, 0).entry_name == "conv3D_W1"
    cfg.conv3D_remode = 0
    assert E.plan_conv3D(cfg, 8, 8, 8, 8, 3, 3, 128, 128, 128, 1, 1, 1, 1).entry_name == "conv3DV2"  # Q=1.5625 >= 1.25
    cfg.conv3D_remode, cfg.conv3D_useTexture = 1, 0
    assert E.plan_conv3D(cfg, 32, 32, 32, 32, 3, 3, 4, 4, 64, 1, 1, 1, 1).entry_name == "conv3D_GemmR"


def test_deltaW_plans_and_split_k_factor():
    cfg = E.default_config(256)
    assert cfg.deltaW_SK_MaxPartNum == 128 and E.default_config(8).deltaW_SK_MaxPartNum == 16
    # c5b: GK = 100352; b1 = b2 = 784, b3 = 5 -> (784+784)/10 = 156 -> capped by MaxPartNum 128 (GK>>8 = 392)
    p = E.plan_deltaW(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1)
    assert p.entry_name == "dconv3D_deltaW_GemmSK" and p.GridZ == 128 and p.scratch_floats == 127 * 36864
    # c5a (1x1, 256 -> 64): b1 = 784, b2 = 2*784, b3 = 2 -> 588 -> 128
    p = E.plan_deltaW(cfg, 56, 56, 56, 56, 1, 1, 32, 256, 64, 1, 1)
    assert p.entry_name == "dconv3D_deltaW_GemmSK_W1" and p.GridZ == 128
    cfg.deltaW_SK_MaxPartNum = 1000
    assert E.plan_deltaW(cfg, 56, 56, 56, 56, 1, 1, 32, 256, 64, 1, 1).GridZ == 392    # min(588, 1000, GK>>8 = 392)
    cfg = E.default_config(256)
    # c2c: Q = 10*10/64 = 1.5625 >= 1.15, OC, IC > 63 -> V2; b1 = b2 = 2*1*64, b3 = 2*2*9 -> 256/72 = 3
    p = E.plan_deltaW(cfg, 8, 8, 8, 8, 3, 3, 128, 256, 256, 1, 1)
    assert p.entry_name == "dconv3D_deltaW_GemmV2SK" and p.GridZ == 3 and p.V2 == 1
    # c2b: Q = 18*18/256 = 1.266 -> V2; b1 = b2 = 256, b3 = 9 -> 512/18 = 28
    assert E.plan_deltaW(cfg, 16, 16, 16, 16, 3, 3, 128, 128, 128, 1, 1).GridZ == 28
    # GK < 512: single pass
    p = E.plan_deltaW(cfg, 8, 8, 8, 8, 3, 3, 4, 16, 16, 1, 1)
    assert p.entry_name == "dconv3D_deltaW" and p.GridZ == 1 and p.scratch_floats == 0
    assert E.plan_deltaW(cfg, 8, 8, 8, 8, 1, 1, 4, 16, 16, 1, 1).entry_name == "dconv3D_deltaW_W1"
    # GridZ floor of 2 and the GK>>8 cap: GK = 512 -> GridZ2 = 2
    assert E.plan_deltaW(cfg, 8, 8, 8, 8, 3, 3, 8, 16, 16, 1, 1).GridZ == 2


def test_deltaW_fill_option_only_raises_the_split_k_factor():
    """deltaW_SK_fillUnits is this build's option (no reference flag): two workgroups of 64 ic x 32 oc (64 oc for 1x1) per
    compute unit, slices of at least 256 pixels, never below the reference's GridZ."""
    cfg = E.default_config(256)
    assert cfg.deltaW_SK_fillUnits == 0
    cfg.deltaW_SK_fillUnits = 256
    # c2c: tiles = 4 x 8 = 32 -> 512/32 = 16 (reference: 3); GK>>8 = 32 does not bind
    p = E.plan_deltaW(cfg, 8, 8, 8, 8, 3, 3, 128, 256, 256, 1, 1)
    assert p.GridZ == 16 and p.scratch_floats == 15 * 256 * 9 * 256 and p.entry_name == "dconv3D_deltaW_GemmV2SK"
    # c2b: tiles = 2 x 4 -> 64 (reference: 28)
    assert E.plan_deltaW(cfg, 16, 16, 16, 16, 3, 3, 128, 128, 128, 1, 1).GridZ == 64
    # rows wider than 36 pixels: one workgroup per unit. c5b: tiles = 1 x 2 -> 128 = the reference's value; c5a (1x1):
    # tiles = 4 x 1 -> 64 < 128, unchanged; c2a (32-pixel rows): tiles = 2 -> 256 (reference: 128)
    assert E.plan_deltaW(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1).GridZ == 128
    assert E.plan_deltaW(cfg, 56, 56, 56, 56, 1, 1, 32, 256, 64, 1, 1).GridZ == 128
    assert E.plan_deltaW(cfg, 32, 32, 32, 32, 3, 3, 128, 64, 64, 1, 1).GridZ == 256
    # small GK: the 256-pixel floor binds (GK = 2048 -> at most 8 slices)
    assert E.plan_deltaW(cfg, 8, 8, 8, 8, 3, 3, 32, 64, 64, 1, 1).GridZ == 8
    # many tiles: want = 1 < reference value -> reference value kept
    big = E.plan_deltaW(cfg, 14, 14, 14, 14, 3, 3, 64, 1024, 1024, 1, 1).GridZ
    cfg.deltaW_SK_fillUnits = 0
    assert big == E.plan_deltaW(cfg, 14, 14, 14, 14, 3, 3, 64, 1024, 1024, 1, 1).GridZ


def test_deltaW_least_option_sets_the_split_k_factor_the_persistent_kernel_needs():
    """deltaW_SK_leastUnits is this build's option (no reference flag): the persistent backward-filter kernel cuts every
    (tap, 64 x 64 block) item into R = floor(units / items) pieces whatever GridZ is (or the line of items into one share per
    unit), so GridZ can come down to R (or to the most shares an item meets) without changing what the kernel does."""
    cfg = E.default_config(256)
    assert cfg.deltaW_SK_leastUnits == 0
    cfg.deltaW_SK_leastUnits = 256
    # c5b, c2a: 9 items -> 28 pieces each (reference: 128)
    p = E.plan_deltaW(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1)
    assert p.GridZ == 28 and p.scratch_floats == 27 * 64 * 9 * 64 and p.entry_name == "dconv3D_deltaW_GemmSK"
    assert E.plan_deltaW(cfg, 32, 32, 32, 32, 3, 3, 128, 64, 64, 1, 1).GridZ == 28
    # c2b: 36 items -> 7 pieces (reference: 28); c5a / c5c: 4 items -> 64 (reference: 128)
    assert E.plan_deltaW(cfg, 16, 16, 16, 16, 3, 3, 128, 128, 128, 1, 1).GridZ == 7
    assert E.plan_deltaW(cfg, 56, 56, 56, 56, 1, 1, 32, 256, 64, 1, 1).GridZ == 64
    assert E.plan_deltaW(cfg, 56, 56, 56, 56, 1, 1, 32, 64, 256, 1, 1).GridZ == 64
    # c2c: 144 items form a line cut into 256 shares, an item meets 2 or 3 of them: the reference's 3 stays
    assert E.plan_deltaW(cfg, 8, 8, 8, 8, 3, 3, 128, 256, 256, 1, 1).GridZ == 3
    # not raised beyond the reference's own cap GK >> 8: 9 items on 256 units want 28, the reference gives 2 (GK = 512)
    assert E.plan_deltaW(cfg, 8, 8, 8, 8, 3, 3, 8, 64, 64, 1, 1).GridZ == 2
    # raised within that cap where the reference's value has fewer buffers than the kernel's cut needs pieces: 4x4 maps at
    # N = 512 (GK = 8192, the reference gives 2), 96 -> 208 channels: 72 items in a line of 256 shares meet up to 5 of them;
    # 256 -> 384: 216 items, up to 3
    assert E.plan_deltaW(E.default_config(256), 4, 4, 4, 4, 3, 3, 512, 96, 208, 1, 1).GridZ == 2
    assert E.plan_deltaW(cfg, 4, 4, 4, 4, 3, 3, 512, 96, 208, 1, 1).GridZ == 5
    assert E.plan_deltaW(cfg, 4, 4, 4, 4, 3, 3, 512, 256, 384, 1, 1).GridZ == 3
    # a first layer (4 stored input channels): one workgroup per slice, group of 16 taps and block of 64 output channels
    assert E.plan_deltaW(E.default_config(256), 32, 32, 32, 32, 3, 3, 512, 4, 64, 1, 1).GridZ == 128
    assert E.plan_deltaW(cfg, 32, 32, 32, 32, 3, 3, 512, 4, 64, 1, 1).GridZ == 256      # 9 taps, 64 channels: a workgroup per slice
    assert E.plan_deltaW(cfg, 224, 224, 112, 112, 7, 7, 64, 4, 64, 2, 2).GridZ == 128   # 49 taps: four groups, 64 slices would do
    assert E.plan_deltaW(cfg, 32, 32, 32, 32, 3, 3, 4, 4, 64, 1, 1).GridZ == 16         # c1: GK / 256 = 16 caps it
    # channel counts that fill the kernel's blocks (16 x 1 to 4 channels per lane a side) to less than 40 % go to other
    # kernels: unchanged (8 of 16 and 12 of 16: 37.5 %); 36 x 44 channels are 36 of 48 and 44 of 64 (52 %): lowered
    cfg0 = E.default_config(256)
    for shape in [(28, 28, 28, 28, 3, 3, 32, 36, 44, 1, 1), (14, 14, 14, 14, 3, 3, 64, 1024, 1024, 1, 1)]:
        assert E.plan_deltaW(cfg, *shape).GridZ <= E.plan_deltaW(cfg0, *shape).GridZ
    assert E.plan_deltaW(cfg, 28, 28, 28, 28, 3, 3, 32, 8, 12, 1, 1).GridZ == E.plan_deltaW(cfg0, 28, 28, 28, 28, 3, 3, 32, 8, 12, 1, 1).GridZ
    assert E.plan_deltaW(cfg, 28, 28, 28, 28, 3, 3, 32, 36, 44, 1, 1).GridZ == 28 < E.plan_deltaW(cfg0, 28, 28, 28, 28, 3, 3, 32, 36, 44, 1, 1).GridZ
    # the same arithmetic behind the C ABI, for a caller that chooses GridZ itself (units, GridZ, OH, OW, FH, FW, N, IC, OC)
    L = pkg.lib()
    assert L.alpha_dconv3D_deltaW_least_GridZ(256, 128, 56, 56, 3, 3, 32, 64, 64) == 28
    assert L.alpha_dconv3D_deltaW_least_GridZ(256, 16, 56, 56, 3, 3, 32, 64, 64) == 16      # never raised
    assert L.alpha_dconv3D_deltaW_least_GridZ(304, 128, 56, 56, 3, 3, 32, 64, 64) == 33     # another device width
    assert L.alpha_dconv3D_deltaW_least_GridZ(256, 1, 56, 56, 3, 3, 32, 64, 64) == 1        # no split-K: nothing to lower
    # the Winograd option sets its own GridZ
    cfg.deltaW_winograd = 256
    assert E.plan_deltaW(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1).GridZ == 128


def test_deltaW_whole_units_for_large_tensors_with_few_items():
    """Tensors beyond 56 MB whose line of items would start its 256 shares at 32 or more different places of the pixel range
    (256 / gcd(items, 256)) are cut into whole units instead - every item in P equal pieces, P minimising
    ceil(P items / 256) x (ceil(groups / P) + 64) - and the helpers report P. (units, GridZ, OH, OW, FH, FW, N, IC, OC)"""
    L = pkg.lib()
    f = L.alpha_dconv3D_deltaW_least_GridZ
    # AlexNet's second layer at N = 64: 200 items (two blocks of 48 x four of 64 x 25 taps) of 12096 groups, 65 MB:
    # P = 5 -> 1000 units, 4 x (2420 + 64) = 9936 (P = 14: 11 x (864 + 64) = 10208; the line: 9450 + 128)
    assert f(256, 14, 27, 27, 5, 5, 64, 96, 256) == 5
    # 3x3 64 -> 192 on 512x16x16: 27 items, 134 MB: P = 9 (243 units, one each; P = 28 ties and the smaller wins)
    assert f(256, 85, 16, 16, 3, 3, 512, 64, 192) == 9
    assert f(256, 128, 56, 56, 3, 3, 64, 64, 192) == 28     # 206 MB, 50176 groups: 756 units, three each
    assert f(256, 42, 32, 32, 3, 3, 64, 128, 256) == 7      # 72 items, 101 MB: 504 units, two each
    # 144 items (pairs of shares over the same pixels), tensors of 46 MB, and either with the switch at "line": the line of items
    assert f(256, 43, 56, 56, 3, 3, 32, 256, 256) == 3
    assert f(256, 5, 8, 8, 5, 5, 512, 96, 256) == 3
    try:
        assert L.alpha_conv_set_deltaW_units(0) == 0
        assert f(256, 14, 27, 27, 5, 5, 64, 96, 256) == 3
        assert L.alpha_conv_set_deltaW_units(1) == 0
        assert f(256, 43, 56, 56, 3, 3, 32, 256, 256) == 7
    finally:
        L.alpha_conv_set_deltaW_units(-1)
    # what the reduced factor is, the launcher cuts the same way: the least factor of the least factor is itself
    for args in [(14, 27, 27, 5, 5, 64, 96, 256), (128, 56, 56, 3, 3, 64, 64, 192), (42, 32, 32, 3, 3, 64, 128, 256), (43, 56, 56, 3, 3, 32, 256, 256)]:
        g = f(256, *args)
        assert f(256, g, *args[1:]) == g
    # the engine's option lowers (or, within GK / 256, raises) GridZ to it
    cfg = E.default_config(256)
    cfg.deltaW_SK_leastUnits = 256
    assert E.plan_deltaW(cfg, 27, 27, 27, 27, 5, 5, 64, 96, 256, 1, 1).GridZ == 5
    assert E.plan_deltaW(cfg, 32, 32, 32, 32, 3, 3, 64, 128, 256, 1, 1).GridZ == 7


def test_deltaW_least_GridZ_is_idempotent_and_never_raises():
    """Over seeded random layers and each setting of the cut switch: the reduced factor is at most GridZ (and at least 2
    where GridZ is), and reducing it again changes nothing - a caller that passes it gets the cut it was computed for."""
    import random
    rnd = random.Random(20240611)
    L = pkg.lib()
    f = L.alpha_dconv3D_deltaW_least_GridZ
    try:
        for units in (-1, 0, 1):
            assert L.alpha_conv_set_deltaW_units(units) == 0
            for _ in range(400):
                OH = rnd.choice([1, 2, 4, 7, 8, 13, 14, 16, 27, 28, 32, 56, 112]); OW = rnd.choice([OH, OH, rnd.randint(1, 60)])
                F = rnd.choice([1, 3, 3, 5, 7]); N = rnd.choice([1, 8, 32, 64, 128, 512])
                IC = rnd.choice([4, 16, 32, 48, 64, 96, 128, 192, 256, 512, 1024]); OC = rnd.choice([16, 32, 64, 96, 128, 208, 256, 384, 512, 2048])
                GZ = rnd.choice([1, 2, 3, 5, 8, 14, 28, 64, 128, 392, 1000]); cus = rnd.choice([256, 304, 64])
                g = f(cus, GZ, OH, OW, F, F, N, IC, OC)
                assert g <= GZ and (g >= 2 or GZ < 2), (units, cus, GZ, OH, OW, F, N, IC, OC, g)
                assert f(cus, g, OH, OW, F, F, N, IC, OC) == g, (units, cus, GZ, OH, OW, F, N, IC, OC, g)
    finally:
        L.alpha_conv_set_deltaW_units(-1)


def test_deltaX_plans():
    cfg = E.default_config(256)
    assert E.plan_deltaX(cfg, 224, 224, 112, 112, 7, 7, 64, 4, 64, 2, 2).entry_name == "dconv3D_deltaX_crossAdd"   # IC <= 8
    assert E.plan_deltaX(cfg, 16, 16, 8, 8, 3, 3, 8, 16, 32, 2, 2).entry_name == "dconv3D_deltaX_crossAdd"        # IC <= 16, s*s >= 4
    assert E.plan_deltaX(cfg, 56, 56, 56, 56, 1, 1, 32, 256, 64, 1, 1).entry_name == "dconv3D_deltaX_W1"
    # c5b: N=32 -> not V2; texture on, IC > 15
    assert E.plan_deltaX(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1).entry_name == "dconv3D_deltaX_s1_texture"
    # c2a: N=128, IC=64, Q = 34*34/1024 = 1.129 > 1.1 -> V2
    p = E.plan_deltaX(cfg, 32, 32, 32, 32, 3, 3, 128, 64, 64, 1, 1)
    assert p.entry_name == "dconv3D_deltaX_V2_s1" and p.Q == pytest.approx(1156 / 1024)
    cfg.deltaX_s1_useTexture = 0
    assert E.plan_deltaX(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1).entry_name == "dconv3D_deltaX_s1"
    cfg = E.default_config(256)
    # stride 2, even input: Ims2 family. N=32 -> not V2, ks texture off
    p = E.plan_deltaX(cfg, 56, 56, 28, 28, 3, 3, 32, 64, 128, 2, 2)
    assert p.entry_name == "dconv3D_deltaX_ksIms2R" and p.remode == 1 and p.scratch_floats == 128 * 2 * 2 * 64 * 4
    # N=64, IC=64: Q = 0.25*((28+1)+(28+0))^2/(28*28) = 0.25*57*57/784 = 1.036 < 1.1 -> still not V2
    assert E.plan_deltaX(cfg, 56, 56, 28, 28, 3, 3, 64, 64, 128, 2, 2).entry_name == "dconv3D_deltaX_ksIms2R"
    # 8x8 input, 5x5: Q = 0.25*((4+2)+(4+1))^2/16 = 1.89 -> V2
    assert E.plan_deltaX(cfg, 8, 8, 4, 4, 5, 5, 64, 64, 64, 2, 2).entry_name == "dconv3D_deltaX_ksV2_Ims2R"
    assert E.plan_deltaX(cfg, 12, 9, 4, 3, 3, 3, 8, 32, 32, 3, 3).entry_name == "dconv3D_deltaX_ksImsR"          # IH%sh == 0
    assert E.plan_deltaX(cfg, 13, 11, 5, 5, 5, 4, 8, 32, 32, 3, 2).entry_name == "dconv3D_deltaX_kernelSplit"
    assert E.plan_deltaX(cfg, 9, 9, 4, 4, 3, 3, 8, 32, 32, 2, 2).entry_name == "dconv3D_deltaX_kernelSplit"      # odd IH, stride 2


def test_w1_entries_only_for_stride_one_and_sizes_are_checked():
    cfg = E.default_config(256)
    # 1x1 stride 2 (BASELINE c4c): the W1 natives carry no stride, so the general entries must be used
    assert E.plan_conv3D(cfg, 56, 56, 28, 28, 1, 1, 64, 64, 128, 2, 2, 0, 0).entry_name == "conv3D_GemmR_texture"
    assert E.plan_conv3D(cfg, 56, 56, 56, 56, 1, 1, 64, 64, 128, 1, 1, 0, 0).entry_name == "conv3D_GemmR_W1"
    assert E.plan_deltaW(cfg, 56, 56, 28, 28, 1, 1, 64, 64, 128, 2, 2).entry_name == "dconv3D_deltaW_GemmSK"
    assert E.plan_deltaX(cfg, 56, 56, 28, 28, 1, 1, 64, 64, 128, 2, 2).entry_name == "dconv3D_deltaX_ksIms2R"
    # EngineCore.conv3D_param_check conditions
    ok = (28, 28, 56, 56, 3, 3, 64, 64, 128, 2, 2, 1, 1)
    assert E.param_check(*ok) is None
    assert "(IH - FH + 2*ph) < (OH - 1)*sh" in E.param_check(56, 28, 56, 56, 3, 3, 64, 64, 128, 2, 2, 1, 1)   # OH too large
    assert "(IW - FW + 2*pw) < (OW - 1)*sw" in E.param_check(28, 56, 56, 56, 3, 3, 64, 64, 128, 2, 2, 1, 1)
    assert "padding" in E.param_check(28, 28, 56, 56, 3, 3, 64, 64, 128, 2, 2, 3, 1)                           # FH <= ph
    assert "multiples of 4" in E.param_check(28, 28, 56, 56, 3, 3, 64, 62, 128, 2, 2, 1, 1)
    assert "stride" in E.param_check(28, 28, 56, 56, 3, 3, 64, 64, 128, 0, 2, 1, 1)


def test_winograd_backward_flags_change_only_3x3_stride1_plans():
    """This build's options deltaX_winograd / deltaW_winograd (no reference counterpart): off by default; on, they take
    3x3 stride-1 layers only, with scratch 16*IC*OC for backward-data and a split-K factor sized for the device for
    backward-filter (values above 1 = compute units to fill; 32 x 64 channel blocks; slices of at least 64 tiles)."""
    cfg = E.default_config(256)
    assert cfg.deltaX_winograd == 0 and cfg.deltaW_winograd == 0
    ref_dx = E.plan_deltaX(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1).entry_name
    ref_dw = E.plan_deltaW(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1)
    cfg.deltaX_winograd = 1
    p = E.plan_deltaX(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1)
    assert p.entry_name == "dconv3D_deltaX_winograd" and p.scratch_floats == 16 * 64 * 64 and p.streams == 1
    assert E.plan_deltaX(cfg, 56, 56, 28, 28, 3, 3, 32, 64, 128, 2, 2).entry_name != "dconv3D_deltaX_winograd"   # stride 2
    assert E.plan_deltaX(cfg, 56, 56, 56, 56, 1, 1, 32, 256, 64, 1, 1).entry_name == "dconv3D_deltaX_W1"          # 1x1
    assert E.plan_deltaX(cfg, 32, 32, 32, 32, 3, 3, 4, 4, 64, 1, 1).entry_name == "dconv3D_deltaX_crossAdd"       # IC <= 8
    cfg.deltaX_winograd = 0
    assert E.plan_deltaX(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1).entry_name == ref_dx

    cfg.deltaW_winograd = 1   # the reference's GridZ
    p = E.plan_deltaW(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1)
    assert p.entry_name == "dconv3D_deltaW_GemmSK_winograd" and p.GridZ == ref_dw.GridZ
    assert p.scratch_floats == 64 * 9 * 64 * (p.GridZ - 1)
    cfg.deltaW_winograd = 256   # c5b: 2 x 1 channel blocks -> 128 slices of 196 tiles
    p = E.plan_deltaW(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1)
    assert p.GridZ == 128 and p.scratch_floats == 64 * 9 * 64 * 127
    # c2c: 8 x 4 channel blocks -> 8 slices; 2048 tiles / 64 = 32 would allow more
    assert E.plan_deltaW(cfg, 8, 8, 8, 8, 3, 3, 128, 256, 256, 1, 1).GridZ == 8
    # below the split-K threshold (N*OH*OW = 256 < 512) the reference's plain entry stays
    p = E.plan_deltaW(cfg, 8, 8, 8, 8, 3, 3, 4, 64, 64, 1, 1)
    assert p.entry_name == "dconv3D_deltaW" and p.GridZ == 1
    # 16 images of 8x8: 256 tiles, at most 4 slices of 64 tiles although 256 units / 2 channel blocks would ask for 128
    assert E.plan_deltaW(cfg, 8, 8, 8, 8, 3, 3, 16, 64, 64, 1, 1).GridZ == 4
    assert E.plan_deltaW(cfg, 56, 56, 28, 28, 3, 3, 32, 64, 128, 2, 2).entry_name != "dconv3D_deltaW_GemmSK_winograd"
    assert E.plan_deltaW(cfg, 56, 56, 56, 56, 1, 1, 32, 256, 64, 1, 1).entry_name == "dconv3D_deltaW_GemmSK_W1"
    cfg.deltaW_winograd = 0
    assert E.plan_deltaW(cfg, 56, 56, 56, 56, 3, 3, 32, 64, 64, 1, 1).entry_name == ref_dw.entry_name


def test_winograd_flags_leave_layers_beyond_32bit_offsets_on_the_default_entries():
    """The Winograd kernels address with 32-bit offsets that keep the top bits for "outside" marks: the persistent forward
    kernel needs the output within 1 GB (input and transformed filter within 2 GB), the backward-filter kernel X within
    1 GB. With the flags set, a layer beyond that keeps the plan it has without them instead of failing at the call."""
    cfg = E.default_config(256)
    big = (128, 128, 128, 128, 3, 3, 64, 256, 256, 1, 1)      # X = Y = 1 GiB exactly
    bigger = (128, 128, 128, 128, 3, 3, 64, 256, 512, 1, 1)   # Y = 2 GiB
    ref = {k: (E.plan_conv3D(cfg, *k[:11], 1, 1).entry_name, E.plan_deltaX(cfg, *k).entry_name, E.plan_deltaW(cfg, *k).entry_name)
           for k in (big, bigger)}
    cfg.conv3D_winograd, cfg.deltaX_winograd, cfg.deltaW_winograd = 1, 1, 256
    # 1 GiB output fits the forward kernel (limit inclusive); X + one pixel beyond 1 GiB does not fit backward-filter
    assert E.plan_conv3D(cfg, *big, 1, 1).entry_name == "conv3D_winograd"
    assert E.plan_deltaX(cfg, *big).entry_name == "dconv3D_deltaX_winograd"
    assert E.plan_deltaW(cfg, *big).entry_name == ref[big][2]
    # 2 GiB of Y: forward output too large, backward-data input too large, backward-filter deltaY too large
    assert E.plan_conv3D(cfg, *bigger, 1, 1).entry_name == ref[bigger][0]
    assert E.plan_deltaX(cfg, *bigger).entry_name == ref[bigger][1]
    assert E.plan_deltaW(cfg, *bigger).entry_name == ref[bigger][2]
    # just inside: half the images
    inside = (128, 128, 128, 128, 3, 3, 32, 256, 256, 1, 1)
    assert E.plan_deltaW(cfg, *inside).entry_name == "dconv3D_deltaW_GemmSK_winograd"


def test_winograd_forward_flag_leaves_layers_with_a_smaller_output_on_the_default_entry():
    """The engine's size check is not strict (EngineCore.java:653-665: the output may be smaller than the formula's); the
    Winograd kernels take exact-size layers only, so such a layer keeps the plan it has without the flag."""
    cfg = E.default_config(256)
    base = E.plan_conv3D(cfg, 12, 12, 11, 12, 3, 3, 8, 64, 64, 1, 1, 1, 1)
    cfg.conv3D_winograd = 1
    assert E.plan_conv3D(cfg, 12, 12, 12, 12, 3, 3, 8, 64, 64, 1, 1, 1, 1).entry_name == "conv3D_winograd"
    for OH, OW in ((11, 12), (12, 10), (9, 9)):
        p = E.plan_conv3D(cfg, 12, 12, OH, OW, 3, 3, 8, 64, 64, 1, 1, 1, 1)
        assert p.entry_name == base.entry_name and p.entry_name != "conv3D_winograd"
    assert E.param_check(11, 12, 12, 12, 3, 3, 8, 64, 64, 1, 1, 1, 1) is None
    assert E.param_check(13, 12, 12, 12, 3, 3, 8, 64, 64, 1, 1, 1, 1) is not None
