#!/usr/bin/env python3
"""Benchmark of the conv3D hot path on one MI355X.

Default run: the headline workload of BASELINE.json's north_star — fp32 NHWC 3x3 stride-1 pad-1
forward, N=64, 56x56x64 -> 64 (config "c3a") — called the way the reference's Java engine calls it
(kernel_remode then the GemmR entry, both per step; CudaFloat32EngineBase.java:1363-1420), inputs
resident in HBM. One "step" = one forward pass over that batch.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--layer c3a] [--op fwd|dx|dw] [--no-layers] [--no-parity]

Output: the LAST line of stdout is the result, one JSON object kept under 4 KB (headline figures, `roofline`, the
headline's parity, `winograd`, `parity_summary`, `cpu_baseline` and `layers_min`: one short entry per layer and operator).
Before it, every layer and operator of BASELINE.json's five configs is printed as a JSON line of its own, as soon as it
is measured (same step count as the headline): its time, its roofline fractions and its parity against the fp64 CPU
oracle on a subset of the same seeded tensors (images for forward / backward-data, output channels over the full batch
for backward-filter), with the tolerance it is held to. The same rows are also written to a file, as one array.
--no-layers leaves them out. `--sweep` measures the layers outside the configs (OTHER_LAYERS) the same way, one JSON line
each; `--layer <one of them>` measures that layer alone (for profiles).
The cpu_baseline leg times the CPU oracle's float-accumulate direct loops on a bounded sample on the host cores
(baseline only, never a target): the headline operator on all cores, backward-data and backward-filter of c5b on all
cores, and config 1 forward on one core.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_F32_TFLOPS = 157.3   # MI355X published dense fp32 matrix peak
PEAK_HBM_GBPS = 8000.0         # MI355X published HBM3E bandwidth

# id: (N, IH, IW, IC(stored), OC, F, s, p, logical IC, ops timed)
LAYERS = {
    "c1":  (4, 32, 32, 4, 64, 3, 1, 1, 3, ("fwd",)),
    "c2a": (128, 32, 32, 64, 64, 3, 1, 1, 64, ("fwd", "dx", "dw")),
    "c2b": (128, 16, 16, 128, 128, 3, 1, 1, 128, ("fwd", "dx", "dw")),
    "c2c": (128, 8, 8, 256, 256, 3, 1, 1, 256, ("fwd", "dx", "dw")),
    "c3a": (64, 56, 56, 64, 64, 3, 1, 1, 64, ("fwd",)),
    "c3b": (64, 28, 28, 128, 128, 3, 1, 1, 128, ("fwd",)),
    "c3c": (64, 14, 14, 256, 256, 3, 1, 1, 256, ("fwd",)),
    "c3d": (64, 7, 7, 512, 512, 3, 1, 1, 512, ("fwd",)),
    "c4a": (64, 224, 224, 4, 64, 7, 2, 3, 3, ("fwd", "dx")),   # dx rows of config 4: the strided backward-data family,
    "c4b": (64, 56, 56, 64, 128, 3, 2, 1, 64, ("fwd", "dx")),  # not asked for by BASELINE.json, measured all the same
    "c4c": (64, 56, 56, 64, 128, 1, 2, 0, 64, ("fwd", "dx")),
    "c4d": (64, 14, 14, 256, 1024, 1, 1, 0, 256, ("fwd",)),
    "c5a": (32, 56, 56, 256, 64, 1, 1, 0, 256, ("dx", "dw")),
    "c5b": (32, 56, 56, 64, 64, 3, 1, 1, 64, ("dx", "dw")),
    "c5c": (32, 56, 56, 64, 256, 1, 1, 0, 64, ("dx", "dw")),
}
# Layers outside BASELINE.json's five configs, for `--sweep`: the other layers of the networks the configs are taken from
# (ResNet-18/34/50 stages, VGG, AlexNet) and of the reference's own example networks (GoogLeNet modules, its AlexNet and
# CIFAR stems), small batches and ragged channel counts. Not part of the default line.
OTHER_LAYERS = {
    "vgg_112":    (32, 112, 112, 64, 128, 3, 1, 1, 64, ("fwd", "dx", "dw")),
    "r18_s2_28":  (64, 56, 56, 64, 128, 3, 2, 1, 64, ("fwd", "dx", "dw")),
    "r18_s2_14":  (64, 28, 28, 128, 256, 3, 2, 1, 128, ("fwd", "dx", "dw")),
    "r18_s2_7":   (64, 14, 14, 256, 512, 3, 2, 1, 256, ("fwd", "dx", "dw")),
    "r18_14":     (64, 14, 14, 256, 256, 3, 1, 1, 256, ("dx", "dw")),
    "r18_7":      (64, 7, 7, 512, 512, 3, 1, 1, 512, ("dx", "dw")),
    "r50_28_in":  (64, 28, 28, 512, 128, 1, 1, 0, 512, ("fwd", "dx", "dw")),
    "r50_28_out": (64, 28, 28, 128, 512, 1, 1, 0, 128, ("fwd", "dx", "dw")),
    "r50_14_in":  (64, 14, 14, 1024, 256, 1, 1, 0, 1024, ("fwd", "dx", "dw")),
    "r50_7_in":   (64, 7, 7, 2048, 512, 1, 1, 0, 2048, ("fwd", "dx", "dw")),
    "r50_7_out":  (64, 7, 7, 512, 2048, 1, 1, 0, 512, ("fwd", "dx", "dw")),
    "r50_sc_28":  (64, 56, 56, 256, 512, 1, 2, 0, 256, ("fwd", "dx", "dw")),
    "r50_sc_14":  (64, 28, 28, 512, 1024, 1, 2, 0, 512, ("fwd", "dx", "dw")),
    "r50_sc_7":   (64, 14, 14, 1024, 2048, 1, 2, 0, 1024, ("fwd", "dx", "dw")),
    "alex_c2":    (64, 27, 27, 96, 256, 5, 1, 2, 96, ("fwd", "dx", "dw")),
    "alex_c3":    (64, 13, 13, 256, 384, 3, 1, 1, 256, ("fwd", "dx", "dw")),
    "alex_c4":    (64, 13, 13, 384, 384, 3, 1, 1, 384, ("fwd", "dx", "dw")),
    "alex_stem":  (64, 224, 224, 4, 64, 11, 4, 2, 3, ("fwd", "dw")),
    "cifar_stem": (64, 32, 32, 4, 64, 5, 1, 2, 3, ("fwd", "dw")),
    "g3a_1x1":    (64, 28, 28, 192, 64, 1, 1, 0, 192, ("fwd", "dx", "dw")),
    "g3a_3x3r":   (64, 28, 28, 192, 96, 1, 1, 0, 192, ("fwd", "dx", "dw")),
    "g3a_3x3":    (64, 28, 28, 96, 128, 3, 1, 1, 96, ("fwd", "dx", "dw")),
    "g3a_5x5r":   (64, 28, 28, 192, 16, 1, 1, 0, 192, ("fwd", "dx", "dw")),
    "g3a_5x5":    (64, 28, 28, 16, 32, 5, 1, 2, 16, ("fwd", "dx", "dw")),
    "g4a_3x3":    (64, 14, 14, 96, 208, 3, 1, 1, 96, ("fwd", "dx", "dw")),
    "g4a_5x5":    (64, 14, 14, 16, 48, 5, 1, 2, 16, ("fwd", "dx", "dw")),
    "g5b_1x1":    (64, 7, 7, 832, 384, 1, 1, 0, 832, ("fwd", "dx", "dw")),
    "g5b_5x5":    (64, 7, 7, 48, 128, 5, 1, 2, 48, ("fwd", "dx", "dw")),
    "gan_4x4":    (64, 32, 32, 64, 128, 4, 2, 1, 64, ("fwd", "dx", "dw")),
    "patch_2x2":  (64, 56, 56, 64, 128, 2, 2, 0, 64, ("fwd", "dx", "dw")),
    "n8_14":      (8, 14, 14, 256, 256, 3, 1, 1, 256, ("fwd", "dx", "dw")),
    "n1_56":      (1, 56, 56, 64, 64, 3, 1, 1, 64, ("fwd", "dx", "dw")),
    "ic48_28":    (64, 28, 28, 48, 96, 3, 1, 1, 48, ("fwd", "dx", "dw")),
    "ic32_56":    (64, 56, 56, 32, 32, 3, 1, 1, 32, ("fwd", "dx", "dw")),
    # the reference's CIFAR-10 experiments (experiments/alpha_code/src/cifar10: VGG, ResNet, GoogLeNet, AlexNet) at their
    # training batch of 512, and first layers (3 channels stored as 4) in backward-filter
    "cf_vgg_32":  (512, 32, 32, 64, 64, 3, 1, 1, 64, ("fwd", "dx", "dw")),
    "cf_vgg_8":   (512, 8, 8, 256, 256, 3, 1, 1, 256, ("fwd", "dx", "dw")),
    "cf_vgg_4":   (512, 4, 4, 512, 512, 3, 1, 1, 512, ("fwd", "dx", "dw")),
    "cf_vgg_2":   (512, 2, 2, 512, 512, 3, 1, 1, 512, ("fwd", "dx", "dw")),
    "cf_res_s2":  (512, 8, 8, 256, 512, 3, 2, 1, 256, ("fwd", "dx", "dw")),
    "cf_res_sc":  (512, 8, 8, 256, 512, 1, 2, 0, 256, ("fwd", "dx", "dw")),
    "cf_goo_c2":  (512, 16, 16, 64, 192, 3, 1, 1, 64, ("fwd", "dx", "dw")),
    "cf_goo_4":   (512, 4, 4, 96, 208, 3, 1, 1, 96, ("fwd", "dx", "dw")),
    "cf_goo_2":   (512, 2, 2, 192, 384, 3, 1, 1, 192, ("fwd", "dx", "dw")),
    "cf_alex_c2": (512, 8, 8, 96, 256, 5, 1, 2, 96, ("fwd", "dx", "dw")),
    "cf_alex_c3": (512, 4, 4, 256, 384, 3, 1, 1, 256, ("fwd", "dx", "dw")),
    "cf_first":   (512, 32, 32, 4, 64, 3, 1, 1, 3, ("fwd", "dw")),
    "cf_first_5": (512, 32, 32, 4, 64, 5, 1, 2, 3, ("fwd", "dw")),
    "cf_first_a": (512, 32, 32, 4, 96, 6, 2, 2, 3, ("fwd", "dw")),
    "stem_7x7":   (64, 224, 224, 4, 64, 7, 2, 3, 3, ("dw",)),
}
RIDGE = PEAK_MFMA_F32_TFLOPS * 1e12 / (PEAK_HBM_GBPS * 1e9)   # FLOP per byte at which the two published peaks meet (19.7)
UNIFORM_INPUT = {"c1", "c4a", "c4b", "c4c", "c4d"}   # BASELINE.json: inputs uniform[-1,1] (the others N(0,1)); filters He-normal
REL_TOL, ABS_TOL = 1e-4, 1e-5


def out_dim(IH, F, s, p):
    return (IH + 2 * p - F) // s + 1


def flops(layer):
    N, IH, IW, IC, OC, F, s, p, ICl, _ = LAYERS[layer]
    return 2.0 * N * out_dim(IH, F, s, p) * out_dim(IW, F, s, p) * OC * F * F * ICl


def algorithmic_bytes(layer):
    """One read of each input tensor + one write of the output, at stored (x4-padded) size."""
    N, IH, IW, IC, OC, F, s, p, _, _ = LAYERS[layer]
    OH, OW = out_dim(IH, F, s, p), out_dim(IW, F, s, p)
    return 4.0 * (N * IH * IW * IC + OC * F * F * IC + N * OH * OW * OC)


def touched_bytes(layer):
    """As algorithmic_bytes, but of the input only the pixels a strided 1x1 filter reads (c4c: every second pixel of every
    second row, a quarter of X); None where every input pixel is read."""
    N, IH, IW, IC, OC, F, s, p, _, _ = LAYERS[layer]
    if s <= F:
        return None
    OH, OW = out_dim(IH, F, s, p), out_dim(IW, F, s, p)
    return 4.0 * (N * OH * OW * F * F * IC + OC * F * F * IC + N * OH * OW * OC)


class Workload:
    """Device tensors of one layer plus closures that enqueue each operator the way the Java engine does."""

    def __init__(self, pkg, torch, layer, seed):
        self.pkg, self.torch, self.layer = pkg, torch, layer
        N, IH, IW, IC, OC, F, s, p, ICl, _ = LAYERS[layer]
        self.dims = (N, IH, IW, IC, OC, F, s, p)
        OH, OW = out_dim(IH, F, s, p), out_dim(IW, F, s, p)
        self.OH, self.OW = OH, OW
        dev = torch.device("cuda:0")
        g = torch.Generator(device="cpu").manual_seed(seed)
        if layer in UNIFORM_INPUT:
            X = torch.rand((N, IH, IW, IC), generator=g) * 2 - 1
        else:
            X = torch.randn((N, IH, IW, IC), generator=g)
        W = torch.randn((OC, F, F, IC), generator=g) * float(np.sqrt(2.0 / (F * F * ICl)))
        if ICl < IC:
            X[..., ICl:] = 0
            W[..., ICl:] = 0
        dY = torch.randn((N, OH, OW, OC), generator=g)
        self.Xh, self.Wh, self.dYh = X, W, dY   # host copies: what the oracle is given
        self.X, self.W, self.dY = X.to(dev), W.to(dev), dY.to(dev)
        self.Y = torch.empty((N, OH, OW, OC), device=dev)
        self.dX = torch.empty((N, IH, IW, IC), device=dev)
        self.dW = torch.empty((OC, F, F, IC), device=dev)
        self.CW = torch.empty(F * F * IC * OC, device=dev)
        self.Bias = torch.randn((OC,), generator=g)
        self.Biash, self.Bias = self.Bias, self.Bias.to(dev)
        # batch-norm statistics and affine parameters of the fused-epilogue row
        self.bn_h = {"mean": torch.randn((OC,), generator=g), "var": torch.rand((OC,), generator=g) * 1.5 + 0.5,
                     "A": torch.rand((OC,), generator=g) + 0.5, "B": torch.randn((OC,), generator=g)}
        self.bn_d = {k: v.to(dev) for k, v in self.bn_h.items()}
        self.bn_eps, self.leaky_k = 1e-5, 0.1
        self.epilogue = pkg.Epilogue(X_mean=self.bn_d["mean"].data_ptr(), X_var=self.bn_d["var"].data_ptr(), eps=self.bn_eps,
                                     A=self.bn_d["A"].data_ptr(), B=self.bn_d["B"].data_ptr(), k=self.leaky_k)
        self.stream = int(torch.cuda.current_stream().cuda_stream)
        self.streams = [self.stream]
        self.engine = pkg.engine.Engine(self.stream)
        if NO_WORKSPACE:
            self.engine.config.conv_workspace = 0
        elif NO_TICKETS:
            self.engine.config.conv_workspace = 2
        self.dx_plan = pkg.engine.plan_deltaX(self.engine.config, IH, IW, OH, OW, F, F, N, IC, OC, s, s)
        if s > 1:
            cf = (F + s - 1) // s
            self.ksCW = torch.empty(s * s * OC * cf * cf * IC, device=dev)
        if F == 3 and s == 1:
            self.U = torch.empty(16 * IC * OC, device=dev)
        self.set_op("fwd")

    def set_op(self, op):
        """Engine options of one bench row (all of them this build's additions, off by default) and the split-K factor the
        host layer passes with them (CudaFloat32EngineBase.java:1707-1715)."""
        N, IH, IW, IC, OC, F, s, p = self.dims
        cfg = self.engine.config
        cus = self.pkg.device_info()[0]
        cfg.deltaW_SK_leastUnits = cus if op == "dw_least" else 0
        cfg.deltaW_winograd = cus if op == "dw_wino" else 0
        cfg.conv3D_winograd = 1 if op == "wino" else 0
        cfg.deltaX_winograd = 1 if op == "dx_wino" else 0
        cfg.cache_filter_transforms = 1 if op == "fwd_cached" else 0
        self.GridZ = max(1, self.pkg.engine.plan_deltaW(cfg, IH, IW, self.OH, self.OW, F, F, N, IC, OC, s, s).GridZ)
        need = max(1, self.GridZ - 1) * self.dW.numel()
        if getattr(self, "buf", None) is None or self.buf.numel() < need:
            self.buf = self.torch.empty(need, device=self.X.device)

    def close(self):
        self.engine.close()

    # forward: remode + GemmR entry (W1 entry for 1x1 stride 1), as CudaFloat32EngineBase.conv3D does
    def fwd_remode(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.pkg.Cuda_conv3D.kernel_remode(self.stream, self.W.data_ptr(), self.CW.data_ptr(), F, F, OC, IC)

    def fwd_conv(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        C = self.pkg.Cuda_conv3D
        if F == 1 and s == 1:
            C.conv3D_GemmR_W1(self.streams, 1, self.X.data_ptr(), IH, IW, self.W.data_ptr(), self.CW.data_ptr(),
                              self.Y.data_ptr(), N, IC, OC)
        else:
            C.conv3D_GemmV2R(True, self.streams, 1, self.X.data_ptr(), IH, IW, self.W.data_ptr(), self.CW.data_ptr(), F, F,
                             self.Y.data_ptr(), self.OH, self.OW, N, IC, OC, s, s, p, p)

    def wino_conv(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.pkg.Cuda_conv3D.conv3D_winograd(self.streams, 1, self.X.data_ptr(), IH, IW, self.U.data_ptr(), self.Y.data_ptr(),
                                             self.OH, self.OW, N, IC, OC, p, p)

    def fwd_bias(self):
        # conv3D_biased through the host layer: same plan as fwd, bias added in the kernel epilogue
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.engine.conv3D_biased(self.Y.data_ptr(), self.OH, self.OW, self.X.data_ptr(), IH, IW, self.W.data_ptr(), F, F,
                                  N, IC, OC, s, s, p, p, self.Bias.data_ptr(), N * self.OH * self.OW * OC, OC)

    def fwd_fused(self):
        # conv3D + batch normalisation (given statistics, affine) + leaky ReLU as one operator through the host layer
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.engine.conv3D_fused(self.Y.data_ptr(), self.OH, self.OW, self.X.data_ptr(), IH, IW, self.W.data_ptr(), F, F,
                                 N, IC, OC, s, s, p, p, self.epilogue)

    def fwd_fused_conv(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.pkg.Cuda_conv3D.conv3D_GemmR_fused(self.streams, 1, self.X.data_ptr(), IH, IW, self.W.data_ptr(), self.CW.data_ptr(), F, F,
                                                self.epilogue, self.Y.data_ptr(), self.OH, self.OW, N, IC, OC, s, s, p, p)

    def fwd(self):
        # whole operator through the C++ host layer: entry selection, CW scratch, kernel_remode, conv entry
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.engine.conv3D(self.Y.data_ptr(), self.OH, self.OW, self.X.data_ptr(), IH, IW, self.W.data_ptr(), F, F,
                           N, IC, OC, s, s, p, p)

    def dx(self):
        # the backward-data entry alone; strided layers: the entry the host layer picks, filter re-layout done beforehand
        N, IH, IW, IC, OC, F, s, p = self.dims
        D = self.pkg.Cuda_dconv3D_deltaX
        if F == 1 and s == 1:
            D.dconv3D_deltaX_W1(self.streams, 1, self.dY.data_ptr(), self.W.data_ptr(), self.dX.data_ptr(), IH, IW, N, IC, OC)
        elif s == 1:
            D.dconv3D_deltaX_V2_s1(True, self.streams, 1, self.dY.data_ptr(), self.OH, self.OW, self.W.data_ptr(), F, F,
                                   self.dX.data_ptr(), IH, IW, N, IC, OC, p, p)
        elif self.dx_plan.entry_name == "dconv3D_deltaX_crossAdd":
            D.dconv3D_deltaX_crossAdd(self.streams, 1, self.dY.data_ptr(), self.OH, self.OW, self.W.data_ptr(), F, F,
                                      self.dX.data_ptr(), IH, IW, N, IC, OC, s, s, p, p)
        else:
            D.dconv3D_deltaX_kernelSplit(self.streams, 1, self.dY.data_ptr(), self.OH, self.OW, self.ksCW.data_ptr(), F, F,
                                         self.dX.data_ptr(), IH, IW, N, IC, OC, s, s, p, p)

    def dx_prepare(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        if s > 1:
            cf = (F + s - 1) // s
            self.pkg.Cuda_dconv3D_deltaX.ks_remodev2(self.stream, self.W.data_ptr(), F, F, self.ksCW.data_ptr(), cf, cf, OC, IC, s, s)

    def dw_gemm(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        D = self.pkg.Cuda_dconv3D_deltaW
        if F == 1 and s == 1:   # the W1 natives carry no stride: 1x1 stride 1 only
            D.dconv3D_deltaW_GemmSK_W1(self.streams, 1, self.GridZ, self.X.data_ptr(), IH, IW, self.dY.data_ptr(),
                                       self.dW.data_ptr(), self.buf.data_ptr(), N, IC, OC)
        else:
            D.dconv3D_deltaW_GemmSK(self.streams, 1, self.GridZ, self.X.data_ptr(), IH, IW, self.dY.data_ptr(), self.OH, self.OW,
                                    self.dW.data_ptr(), self.buf.data_ptr(), F, F, N, IC, OC, s, s, p, p)

    def dw(self):
        # whole operator through the C++ host layer: GridZ, deltaW_buf scratch, split-K entry, buf_summary
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.engine.dconv3D_deltaW(self.dW.data_ptr(), F, F, self.X.data_ptr(), IH, IW, self.dY.data_ptr(), self.OH, self.OW,
                                   N, IC, OC, s, s, p, p)

    def dw_wino_gemm(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.pkg.Cuda_dconv3D_deltaW.dconv3D_deltaW_GemmSK_winograd(self.streams, 1, self.GridZ, self.X.data_ptr(), IH, IW,
                                                                    self.dY.data_ptr(), self.OH, self.OW, self.dW.data_ptr(),
                                                                    self.buf.data_ptr(), N, IC, OC, p, p)

    def dx_wino_conv(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.pkg.Cuda_dconv3D_deltaX.dconv3D_deltaX_winograd(self.streams, 1, self.dY.data_ptr(), self.OH, self.OW, self.U.data_ptr(),
                                                             self.dX.data_ptr(), IH, IW, N, IC, OC, p, p)

    def dx_op(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.engine.dconv3D_deltaX(self.dX.data_ptr(), IH, IW, self.dY.data_ptr(), self.OH, self.OW, self.W.data_ptr(), F, F,
                                   N, IC, OC, s, s, p, p)


NO_TICKETS = False     # --no-tickets: scratch lent, but the pieces of the items left over are added by a second kernel
NO_WORKSPACE = False   # --no-workspace: the conv entries as an unmodified Java engine calls them (no scratch lent)
CLOCK_RAMP_MS = 40.0   # untimed run-in before every measurement; reported in the JSON line


def time_loop(torch, fn, steps, warmup):
    """Wall-clock (sync'ed both sides) and HIP-event time of `steps` back-to-back calls, in ms per call.

    Before the `warmup` calls the same call is repeated, untimed, for CLOCK_RAMP_MS of wall time: the device raises its
    clock only after some tens of milliseconds of continuous work (the same kernel measures 0.123 ms in the first 60
    calls after an idle spell and 0.114 ms from about the 200th on), and between two rows of the default run the device
    idles while the host checks parity."""
    t_ramp = time.perf_counter()
    while (time.perf_counter() - t_ramp) * 1e3 < CLOCK_RAMP_MS:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return wall_ms, e0.elapsed_time(e1) / steps


def cpu_baseline(layer, op, budget_s=12.0, threads=None):
    """Times the oracle's float-accumulate direct loops (forward: conv3D_f32acc, backward-data: deltaX_img2col,
    backward-filter: deltaW_f32acc) on a batch subset sized for ~budget_s, on `threads` host threads (default: all)."""
    from oracle import oracle as O
    N, IH, IW, IC, OC, F, s, p, ICl, _ = LAYERS[layer]
    OH, OW = out_dim(IH, F, s, p), out_dim(IW, F, s, p)
    r = np.random.Generator(np.random.PCG64(7))
    all_cores = O.num_threads()
    cores = all_cores if threads is None else threads
    O.set_num_threads(cores)

    def run(n):
        X = r.standard_normal((n, IH, IW, IC)).astype(np.float32)
        W = r.standard_normal((OC, F, F, IC)).astype(np.float32)
        dY = r.standard_normal((n, OH, OW, OC)).astype(np.float32)
        t0 = time.perf_counter()
        if op == "fwd":
            O.conv3D_f32acc(X, W, s, s, p, p)
        elif op == "dx":
            O.deltaX_img2col(dY, W, IH, IW, s, s, p, p)
        else:
            O.deltaW_f32acc(X, dY, F, F, s, s, p, p)
        return time.perf_counter() - t0

    try:
        per_image = flops(layer) / N
        n0 = min(N, max(1, cores // 4))
        t_probe = run(n0)
        n = int(max(n0, min(N, n0 * budget_s / max(t_probe, 1e-6))))
        t1 = run(n) if n > n0 else t_probe
        n_used = n if n > n0 else n0
        reps = int(max(1, min(5000, budget_s / max(t1, 1e-6))))   # repeat the subset until ~budget_s of CPU work is timed
        t = sum(run(n_used) for _ in range(reps))
    finally:
        O.set_num_threads(all_cores)
    return {
        "value": round(per_image * n_used * reps / t / 1e12, 6), "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": "%s %s, %d of %d images x %d repeats, %.1f s; direct loops, fp32 accumulate, OpenMP" % (layer, op, n_used, N, reps, t),
    }


def load_traffic(layer, op):
    """HBM bytes per launch measured offline with rocprofv3 --pmc (FETCH_SIZE / WRITE_SIZE), if recorded."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(path):
        try:
            return json.load(open(path)).get("%s_%s" % (layer, op))
        except (ValueError, OSError):
            return None
    return None


ORACLE_MACS = 2.5e8   # multiply-adds of fp64 oracle work per bench row (a fraction of a second on the host cores)


def parity(wl, op, step):
    """Runs `step` once and compares part of its output with the fp64 oracle on the same tensors. Forward and backward-data:
    a subset of images (the first ones and the last one). Backward-filter: the full batch for four output channels (the
    first two and the last two), i.e. every element of deltaW[oc] for those oc. Reports the bar of the GPU tests
    (|err| <= max(1e-4*|want|, 1e-5*max(1, rms(want)))), the same with the literal absolute floor 1e-5, and the reference's
    own criterion (Vector.samePercentRelative, threshold 1e-4)."""
    from oracle import oracle as O
    torch = wl.torch
    N, IH, IW, IC, OC, F, s, p = wl.dims
    OH, OW = wl.OH, wl.OW
    out = {"fwd": wl.Y, "dx": wl.dX, "dw": wl.dW}[kind_of(op)]
    out.fill_(float("nan"))
    step()
    wl.engine.sync()
    torch.cuda.synchronize()
    extra = {}
    if kind_of(op) == "dw":
        ocs = sorted(set([0, 1, OC - 2, OC - 1]))
        dYs = np.ascontiguousarray(wl.dYh.numpy()[..., ocs])
        want = O.deltaW_f64(wl.Xh.numpy(), dYs, F, F, s, s, p, p)
        got = out[ocs].cpu().numpy()
        subset = "all %d images, output channels %s" % (N, ocs)
        first = out.clone()
        step()
        wl.engine.sync()
        torch.cuda.synchronize()
        extra["bit_reproducible_run_to_run"] = bool(torch.equal(first.view(torch.int32), out.view(torch.int32)))
    else:
        per_image = float(OH) * OW * OC * F * F * IC
        n = int(max(2, min(N, ORACLE_MACS // per_image)))
        imgs = list(range(n - 1)) + [N - 1]
        if kind_of(op) == "fwd":
            want = O.conv3D_f64(np.ascontiguousarray(wl.Xh.numpy()[imgs]), wl.Wh.numpy(), s, s, p, p)
            if op == "fwd_bias":
                want = want + wl.Biash.numpy().astype(np.float64)
            if op == "fwd_fused":   # closed form of the row functions in fp64
                b = {k: v.numpy().astype(np.float64) for k, v in wl.bn_h.items()}
                want = (want - b["mean"]) / np.sqrt(b["var"] + wl.bn_eps) * b["A"] + b["B"]
                want = np.where(want > 0, want, wl.leaky_k * want)
        else:
            want = O.deltaX_f64(np.ascontiguousarray(wl.dYh.numpy()[imgs]), wl.Wh.numpy(), IH, IW, s, s, p, p)
        got = out[imgs].cpu().numpy()
        subset = "images %s of %d, all channels" % (imgs, N)
    rms = float(np.sqrt(np.mean(want * want)))
    tol_abs = ABS_TOL * max(1.0, rms)
    r = {"vs": "fp64 CPU oracle", "subset": subset, "checked": int(want.size), "tol_rel": REL_TOL, "tol_abs": float("%.3g" % tol_abs),
         "max_err_ratio": round(O.max_err_ratio(got, want, REL_TOL, tol_abs), 4),
         "max_err_ratio_at_abs_1e-5": round(O.max_err_ratio(got, want, REL_TOL, ABS_TOL), 4),
         "max_abs_err": float("%.3g" % float(np.max(np.abs(got.astype(np.float64) - want)))), "rms_expected": float("%.4g" % rms),
         "samePercentRelative_1e-4": round(O.samePercentRelative(want.astype(np.float32), got, 1e-4), 6),
         "samePercentRelative_1e-5": round(O.samePercentRelative(want.astype(np.float32), got, 1e-5), 6)}
    r["ok"] = bool(r["max_err_ratio"] <= 1.0 and np.isfinite(got).all())
    r.update(extra)
    return r


def kind_of(op):
    return "fwd" if op in ("fwd", "fwd_bias", "fwd_cached", "fwd_fused", "wino") else "dx" if op in ("dx", "dx_wino") else "dw"


def measure(wl, op, steps, warmup, with_parity=True):
    pkg, torch, layer = wl.pkg, wl.torch, wl.layer
    wl.set_op(op)
    step = {"fwd": wl.fwd, "fwd_cached": wl.fwd, "fwd_bias": wl.fwd_bias, "fwd_fused": wl.fwd_fused, "dx": wl.dx_op, "dw": wl.dw, "dw_least": wl.dw, "wino": wl.fwd,
            "dx_wino": wl.dx_op, "dw_wino": wl.dw}[op]
    kernel = {"fwd": wl.fwd_conv, "fwd_cached": wl.fwd_conv, "fwd_bias": wl.fwd_conv, "fwd_fused": wl.fwd_fused_conv, "dx": wl.dx, "dw": wl.dw_gemm, "dw_least": wl.dw_gemm,
              "wino": wl.wino_conv, "dx_wino": wl.dx_wino_conv, "dw_wino": wl.dw_wino_gemm}[op]
    N_, IH_, IW_, IC_, OC_, F_, s_, p_ = wl.dims
    if op in ("fwd", "fwd_bias", "fwd_cached", "fwd_fused"):
        wl.fwd_remode()
    if op == "wino":
        pkg.Cuda_conv3D.winograd_filter_transform(wl.stream, wl.W.data_ptr(), wl.U.data_ptr(), IC_, OC_)
    if op == "dx_wino":
        pkg.Cuda_dconv3D_deltaX.winograd_filter_transform_deltaX(wl.stream, wl.W.data_ptr(), wl.U.data_ptr(), IC_, OC_)
    if op == "dx":
        wl.dx_prepare()
    wall_ms, ev_ms = time_loop(torch, step, steps, warmup)
    wl.engine.sync()
    # the conv entry alone (its dominant kernel; HIP events on its stream), with the scratch the host layer lends it
    if getattr(wl, "ws", None) is None:
        wl.ws = torch.empty(1 << 18, device=wl.X.device)
        wl.tickets = torch.zeros(128, dtype=torch.int32, device=wl.X.device)   # zero when bound; the kernels leave them zero
        torch.cuda.synchronize()
    if wl.engine.config.conv_workspace:
        pkg.lib().alpha_conv_bind_workspace(wl.ws.data_ptr(), wl.ws.numel() * 4)
        if not NO_TICKETS:
            pkg.lib().alpha_conv_bind_tickets(wl.tickets.data_ptr(), wl.tickets.numel())
    try:
        # The entry alone cannot take longer than the operator that contains it. Where it reads so - some devices of the
        # pool run a long row of identical back-to-back launches at a lower clock than the operator loop, whose small
        # kernels break the row - the timed region is repeated (at most twice) and the shortest one reported; every
        # region's figure is kept in `kernel_ms_regions`.
        k_regions = []
        for _ in range(3):
            k_regions.append(time_loop(torch, kernel, steps, max(1, warmup // 2))[1])
            if k_regions[-1] <= ev_ms * 1.02:
                break
        k_ms = min(k_regions)
    finally:
        pkg.lib().alpha_conv_bind_tickets(None, 0)
        pkg.lib().alpha_conv_bind_workspace(None, 0)
    fl, by = flops(layer), algorithmic_bytes(layer)
    hbm = fl / by < RIDGE   # below the ridge the HBM roofline binds (c1, c4c), above it the matrix pipes (the 1x1 layers of
    #                         config 5 sit just above: 25.6 FLOP/B against a ridge of 19.7)
    roof = {
        "bound": "hbm" if hbm else "mfma",
        "achieved": round(by / (k_ms * 1e-3) / 1e9, 2) if hbm else round(fl / (k_ms * 1e-3) / 1e12, 3),
        "peak": PEAK_HBM_GBPS if hbm else PEAK_MFMA_F32_TFLOPS,
        "unit": "GB/s" if hbm else "TFLOP/s",
        "kernel_ms": round(k_ms, 5),
        **({"kernel_ms_regions": [round(v, 5) for v in k_regions]} if len(k_regions) > 1 else {}),
        "traffic": load_traffic(layer, op),
    }
    roof["frac"] = round(roof["achieved"] / roof["peak"], 4)
    roof["flop_per_byte"] = round(fl / by, 2)
    # both fractions for every row, whichever roofline binds
    roof["mfma_frac"] = round(fl / (k_ms * 1e-3) / 1e12 / PEAK_MFMA_F32_TFLOPS, 4)
    roof["hbm_frac"] = round(by / (k_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4)
    if touched_bytes(layer) is not None and kind_of(op) == "fwd":
        # a stride beyond the filter: forward reads only the pixels under the filter; both figures are stated
        roof["touched_MB"] = round(touched_bytes(layer) / 1e6, 2)
        roof["hbm_frac_touched"] = round(touched_bytes(layer) / (k_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4)
    if op in ("wino", "dx_wino", "dw_wino"):
        roof["note"] = "Winograd: FLOPs credited are the direct convolution's (2.25x the multiplies executed); frac is not a roofline fraction"
        roof["executed_mfma_frac"] = round(roof["mfma_frac"] / 2.25, 4)
    row = {"layer": layer, "op": op, "ms_per_step": round(wall_ms, 5), "event_ms_per_step": round(ev_ms, 5),
           "tflops": round(fl / (wall_ms * 1e-3) / 1e12, 3), "gflop": round(fl / 1e9, 3),
           "algorithmic_MB": round(by / 1e6, 2), "GridZ": wl.GridZ if kind_of(op) == "dw" else None, "roofline": roof}
    if with_parity:
        row["parity"] = parity(wl, op, step)
    wl.set_op("fwd")
    return row


def measure_bn_backward(wl, steps, warmup, with_parity=True):
    """Backward of the batch normalisation that follows the layer's convolution (batchNorm2D_gradients_v2 through the host
    layer: field sums of deltaY and deltaY * X_norm over the layer's output, then the row function), an HBM-bound operator:
    algorithmic bytes = one read of deltaY and of the normalisation's input, one write of deltaX (the two passes read both
    inputs twice). `kernel_ms` is the row function alone, with the sums given."""
    from oracle import oracle as O
    pkg, torch = wl.pkg, wl.torch
    N, IH, IW, IC, OC, F, s, p = wl.dims
    rows, M = N * wl.OH * wl.OW, OC
    dev = wl.X.device
    g = torch.Generator(device="cpu").manual_seed(4242)
    Xb = torch.randn((rows, M), generator=g) * 1.3 + 0.4          # the convolution's output that was normalised
    mean, var = Xb.double().mean(0).float(), Xb.double().var(0, unbiased=False).float()
    A = torch.rand((M,), generator=g) + 0.5
    dYv = wl.dYh.reshape(rows, M)
    d = {k: v.to(dev) for k, v in dict(X=Xb, mean=mean, var=var, A=A).items()}
    dX = torch.empty((rows, M), device=dev)
    dA, dB = torch.empty(M, device=dev), torch.empty(M, device=dev)
    eps = 1e-5

    def step():
        wl.engine.batchNorm2D_deltaX_v2(dX.data_ptr(), wl.dY.data_ptr(), d["X"].data_ptr(), d["mean"].data_ptr(), d["var"].data_ptr(), eps,
                                        rows, M, rows * M, M, M, A=d["A"].data_ptr(), deltaA=dA.data_ptr(), deltaB=dB.data_ptr())

    def kernel():
        pkg.Cuda_function.batchNorm_affined2D_row_deltaX_v2(wl.stream, wl.dY.data_ptr(), d["X"].data_ptr(), d["mean"].data_ptr(), d["var"].data_ptr(),
                                                            eps, d["A"].data_ptr(), dB.data_ptr(), dA.data_ptr(), M, dX.data_ptr(), rows * M, M, M)

    wall_ms, ev_ms = time_loop(torch, step, steps, warmup)
    wl.engine.sync()
    _, k_ms = time_loop(torch, kernel, steps, max(1, warmup // 2))
    by = 4.0 * 3 * rows * M
    roof = {"bound": "hbm", "achieved": round(by / (k_ms * 1e-3) / 1e9, 2), "peak": PEAK_HBM_GBPS, "unit": "GB/s", "kernel_ms": round(k_ms, 5),
            "traffic": None, "operator_GBps_on_two_passes": round((by + 4.0 * 2 * rows * M) / (wall_ms * 1e-3) / 1e9, 2)}
    roof["frac"] = round(roof["achieved"] / roof["peak"], 4)
    row = {"layer": wl.layer, "op": "bn_bwd", "ms_per_step": round(wall_ms, 5), "event_ms_per_step": round(ev_ms, 5), "tflops": None, "gflop": None,
           "algorithmic_MB": round(by / 1e6, 2), "GridZ": None, "roofline": roof}
    if with_parity:
        dX.fill_(float("nan"))
        step()
        wl.engine.sync()
        torch.cuda.synchronize()
        xn = O.batchNorm_xnorm("from_x", Xb.numpy(), X_mean=mean.numpy(), X_var=var.numpy(), eps=eps)
        wA, wB = O.batchNorm_deltaAB(dYv.numpy(), xn)
        want = O.batchNorm_deltaX(dYv.numpy(), xn, var.numpy(), eps, wB, wA, A=A.numpy())
        got = dX.cpu().numpy()
        rms = float(np.sqrt(np.mean(want * want)))
        tol_abs = ABS_TOL * max(1.0, rms)
        worst = max(O.max_err_ratio(got, want, REL_TOL, tol_abs), O.max_err_ratio(dA.cpu().numpy(), wA, REL_TOL, ABS_TOL * max(1.0, float(np.sqrt(np.mean(wA * wA))))),
                    O.max_err_ratio(dB.cpu().numpy(), wB, REL_TOL, ABS_TOL * max(1.0, float(np.sqrt(np.mean(wB * wB))))))
        row["parity"] = {"vs": "fp64 closed form (oracle)", "subset": "deltaX, deltaA, deltaB: every element", "checked": int(want.size + 2 * M),
                         "tol_rel": REL_TOL, "tol_abs": float("%.3g" % tol_abs), "max_err_ratio": round(worst, 4),
                         "max_err_ratio_at_abs_1e-5": round(O.max_err_ratio(got, want, REL_TOL, ABS_TOL), 4),
                         "max_abs_err": float("%.3g" % float(np.max(np.abs(got.astype(np.float64) - want)))), "rms_expected": float("%.4g" % rms),
                         "samePercentRelative_1e-4": round(O.samePercentRelative(want.astype(np.float32), got, 1e-4), 6),
                         "samePercentRelative_1e-5": round(O.samePercentRelative(want.astype(np.float32), got, 1e-5), 6),
                         "ok": bool(worst <= 1.0 and np.isfinite(got).all())}
    return row


def layer_ops(layer):
    N, IH, IW, IC, OC, F, s, p, ICl, ops = LAYERS[layer]
    ops = list(ops)
    if "fwd" in ops and F == 3 and s == 1 and IC >= 16:
        ops.append("wino")
    if "dx" in ops and F == 3 and s == 1:
        ops.append("dx_wino")
    if "dw" in ops:
        ops.append("dw_least")
    if "dw" in ops and F == 3 and s == 1:
        ops.append("dw_wino")
    if layer == "c3a":
        ops += ["fwd_bias", "fwd_cached", "fwd_fused", "bn_bwd"]
    return ops


FINAL_LINE_LIMIT = 4096   # bytes; a harness that keeps only the tail of stdout must still see the whole result line


def compact_parity(par):
    """The few parity figures the result line keeps of a row's full parity record."""
    if not par:
        return None
    keys = ("ok", "max_err_ratio", "max_err_ratio_at_abs_1e-5", "max_abs_err", "tol_rel", "tol_abs", "checked",
            "samePercentRelative_1e-4", "samePercentRelative_1e-5", "bit_reproducible_run_to_run")
    return {k: par[k] for k in keys if k in par}


def layers_min(rows):
    """One short entry per measured row: "layer/op": [kernel fraction of its binding roofline, operator ms, parity ok]."""
    return {"%s/%s" % (r["layer"], r["op"]): [round(r["roofline"]["frac"], 3), round(r["ms_per_step"], 4),
                                              (1 if r["parity"]["ok"] else 0) if "parity" in r else None] for r in rows}


def result_line(out, rows):
    """Serialises the result object with its per-row summary; sheds the optional parts, least important first, should the
    line ever exceed FINAL_LINE_LIMIT."""
    out = dict(out)
    if rows:
        out["layers_min"] = layers_min(rows)
        out["layers_min_key"] = "layer/op: [kernel frac of its roofline, operator ms, parity ok]"
    line = json.dumps(out, separators=(",", ":"))
    for drop in ("layers_min_key", "winograd", "layers_min", "parity"):
        if len(line) <= FINAL_LINE_LIMIT:
            break
        out.pop(drop, None)
        line = json.dumps(out, separators=(",", ":"))
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--layer", default="c3a", choices=sorted(LAYERS) + sorted(OTHER_LAYERS),
                    help="a layer of BASELINE.json's configs (default c3a, the headline) or one of --sweep's, measured alone (profiles)")
    ap.add_argument("--op", default=None, choices=["fwd", "fwd_bias", "fwd_cached", "fwd_fused", "dx", "dw", "dw_least", "wino", "dx_wino", "dw_wino"],
                    help="wino = forward through Winograd F(2x2,3x3) (3x3 stride-1 layers), reported in direct-conv-equivalent FLOPs")
    ap.add_argument("--layers", action="store_true", help="accepted for compatibility: the layers array is part of the default line")
    ap.add_argument("--no-layers", action="store_true", help="leave out the array with every layer/op of BASELINE.json's configs")
    ap.add_argument("--no-parity", action="store_true", help="leave out the per-row comparison with the CPU oracle")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-workspace", action="store_true",
                    help="do not lend the forward / backward-data entries scratch (the host layer's conv_workspace option off): "
                         "the natives as an unmodified Java engine calls them")
    ap.add_argument("--no-tickets", action="store_true",
                    help="lend the scratch but no ticket words: the pieces of the items left over are added by a second kernel")
    ap.add_argument("--sweep", action="store_true",
                    help="instead of the default line: kernel / operator time and parity of OTHER_LAYERS (layers outside the five "
                         "configs), one JSON line per row and a summary line")
    ap.add_argument("--probe-copy", action="store_true",
                    help="only run a plain 256 MiB device-to-device copy a few times (calibrates FETCH_SIZE/WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is built and measured on ONE GPU; --gpus %d is not supported "
              "(forward/backward-data shard over N with no exchange, backward-filter needs one all-reduce of deltaW)." % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    global NO_WORKSPACE, NO_TICKETS
    NO_WORKSPACE = args.no_workspace
    NO_TICKETS = args.no_tickets
    import torch
    if args.probe_copy:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"probe": "copy", "bytes_read": src.numel() * 4, "bytes_written": src.numel() * 4}))
        return
    from __graft_entry__ import package
    pkg = package()
    pkg.lib()   # raises if the HIP library is not built; there is no fallback
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.sweep:
        LAYERS.update(OTHER_LAYERS)
        worst, bad = None, []
        for i, layer in enumerate(OTHER_LAYERS):
            wl = Workload(pkg, torch, layer, 5000 + i)
            for o in OTHER_LAYERS[layer][9]:
                r = measure(wl, o, args.steps, args.warmup, with_parity=not args.no_parity)
                rf = r["roofline"]
                row = {"layer": layer, "op": o, "shape": list(OTHER_LAYERS[layer][:9]), "kernel_ms": rf["kernel_ms"], "ms_per_step": r["ms_per_step"],
                       "mfma_frac": rf["mfma_frac"], "hbm_frac": rf["hbm_frac"]}
                if "parity" in r:
                    row["parity_ok"] = r["parity"]["ok"]
                    row["max_err_ratio"] = r["parity"]["max_err_ratio"]
                    if not r["parity"]["ok"]:
                        bad.append(layer + "/" + o)
                    if worst is None or r["parity"]["max_err_ratio"] > worst:
                        worst = r["parity"]["max_err_ratio"]
                print(json.dumps(row, separators=(",", ":")), flush=True)
            wl.close()
            del wl
            torch.cuda.empty_cache()
        print(json.dumps({"sweep": "layers outside the five configs", "layers": len(OTHER_LAYERS), "steps": args.steps,
                          "parity_failed": bad, "worst_max_err_ratio": worst}, separators=(",", ":")), flush=True)
        return
    config_layers = sorted(LAYERS)
    if args.layer in OTHER_LAYERS:   # a layer outside the configs, alone: its seed as in --sweep, no array of the configs' layers
        LAYERS[args.layer] = OTHER_LAYERS[args.layer]
        args.no_layers = True
    op = args.op or LAYERS[args.layer][9][0]

    def seed_of(layer):
        return 1000 + config_layers.index(layer) if layer in config_layers else 5000 + list(OTHER_LAYERS).index(layer)

    wl = Workload(pkg, torch, args.layer, seed_of(args.layer))
    head = measure(wl, op, args.steps, args.warmup, with_parity=not args.no_parity)
    props = torch.cuda.get_device_properties(0)
    cus, clk_khz = pkg.device_info()
    clk_ghz = clk_khz / 1e6
    N, IH, IW, IC, OC, F, s, p, ICl, _ = LAYERS[args.layer]
    out = {
        "metric": "conv fwd/bwd TFLOP/s (fp32) + % of MI355X fp32 MFMA peak, 1 GPU",
        "value": head["tflops"], "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s %s: N=%d %dx%dx%d->%d %dx%d s%d p%d NHWC; step = one operator call through the host layer (scratch + remode/summary + conv entry)"
                               % (args.layer, op, N, IH, IW, ICl, OC, F, F, s, p),
                   "layer": args.layer, "op": op, "gflop_per_step": head["gflop"],
                   "algorithmic_MB_per_step": head["algorithmic_MB"],
                   "frac_of_fp32_mfma_peak": round(head["tflops"] / PEAK_MFMA_F32_TFLOPS, 4),
                   "tolerance": "rel 1e-4, abs 1e-5*max(1, rms(expected)) vs the fp64 CPU oracle",
                   "clock_ramp_ms": CLOCK_RAMP_MS,   # untimed run-in of the same calls before the warmup steps of every measurement
                   "device": {"name": props.name, "cus": cus, "clock_ghz": round(clk_ghz, 3),
                              "fp32_mfma_peak_from_device_tflops": round(cus * 256 * clk_ghz / 1e3, 1)}},
        "roofline": head["roofline"],
    }
    if "parity" in head:
        out["parity"] = compact_parity(head["parity"])
    if op == "fwd" and F == 3 and s == 1 and IC >= 16:
        # the same layer through this build's second forward algorithm, in direct-convolution-equivalent FLOPs (2.25x the
        # multiplies executed; the executed-FLOP figure counts the 16 GEMMs only, not the transforms)
        wn = measure(wl, "wino", args.steps, args.warmup, with_parity=not args.no_parity)
        out["winograd"] = {"value": wn["tflops"], "unit": "TFLOP/s (direct-conv-equivalent)", "ms_per_step": wn["ms_per_step"],
                           "kernel_ms": wn["roofline"]["kernel_ms"], "kernel_tflops": wn["roofline"]["achieved"],
                           "direct_equivalent_over_fp32_mfma_peak": wn["roofline"]["frac"],
                           "executed_flop_frac_of_fp32_mfma_peak": round(wn["roofline"]["frac"] / 2.25, 4),
                           "parity": {k: v for k, v in (compact_parity(wn.get("parity")) or {}).items()
                                      if k in ("ok", "max_err_ratio", "max_abs_err", "samePercentRelative_1e-4")} or None}
    wl.close()
    del wl
    rows = []
    if not args.no_layers:
        for layer in config_layers:
            wl = Workload(pkg, torch, layer, seed_of(layer))
            for o in layer_ops(layer):
                if o == "bn_bwd":
                    row = measure_bn_backward(wl, args.steps, args.warmup, with_parity=not args.no_parity)
                else:
                    row = measure(wl, o, args.steps, args.warmup, with_parity=not args.no_parity)
                rows.append(row)
                print(json.dumps(row, separators=(",", ":")), flush=True)   # full row: a line of its own, before the result line
            wl.close()
            del wl
            torch.cuda.empty_cache()
        try:
            os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
            with open(os.path.join(ROOT, "gpurun_out", "bench_layers.json"), "w") as f:
                json.dump(rows, f, indent=1)
        except OSError as e:
            print("bench.py: could not write gpurun_out/bench_layers.json: %s" % e, file=sys.stderr)
        checked = [r for r in rows if "parity" in r]
        if checked:
            out["parity_summary"] = {"rows": len(checked), "rows_ok": sum(1 for r in checked if r["parity"]["ok"]),
                                     "worst_max_err_ratio": max(r["parity"]["max_err_ratio"] for r in checked),
                                     "worst_max_err_ratio_at_abs_1e-5": max(r["parity"]["max_err_ratio_at_abs_1e-5"] for r in checked),
                                     "least_samePercentRelative_1e-4": min(r["parity"]["samePercentRelative_1e-4"] for r in checked)}
    if args.no_cpu:
        out["cpu_baseline"] = None
    else:
        out["cpu_baseline"] = cpu_baseline(args.layer, op)
        if args.layer == "c3a" and op == "fwd":   # the default run: a CPU figure beside the backward rows and config 1 on one core
            out["cpu_baseline_dx"] = cpu_baseline("c5b", "dx", budget_s=5.0)
            out["cpu_baseline_dw"] = cpu_baseline("c5b", "dw", budget_s=5.0)
            out["cpu_baseline_c1_1core"] = cpu_baseline("c1", "fwd", budget_s=2.0, threads=1)
    print(result_line(out, rows), flush=True)


if __name__ == "__main__":
    main()
