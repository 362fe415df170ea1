#!/usr/bin/env python3
"""Benchmark of the conv3D hot path on one MI355X.

Default run: the headline workload of BASELINE.json's north_star — fp32 NHWC 3x3 stride-1 pad-1
forward, N=64, 56x56x64 -> 64 (config "c3a") — called the way the reference's Java engine calls it
(kernel_remode then the GemmR entry, both per step; CudaFloat32EngineBase.java:1363-1420), inputs
resident in HBM. One "step" = one forward pass over that batch. Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--layer c3a] [--op fwd|dx|dw] [--layers]

--layers adds a "layers" array with every layer of BASELINE.json's configs (fewer iterations each).
The cpu_baseline leg times the CPU oracle's float-accumulate direct convolution on a bounded batch
subset of the same workload on the host cores (baseline only, never a target).
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
    "c4a": (64, 224, 224, 4, 64, 7, 2, 3, 3, ("fwd",)),
    "c4b": (64, 56, 56, 64, 128, 3, 2, 1, 64, ("fwd",)),
    "c4c": (64, 56, 56, 64, 128, 1, 2, 0, 64, ("fwd",)),
    "c4d": (64, 14, 14, 256, 1024, 1, 1, 0, 256, ("fwd",)),
    "c5a": (32, 56, 56, 256, 64, 1, 1, 0, 256, ("dx", "dw")),
    "c5b": (32, 56, 56, 64, 64, 3, 1, 1, 64, ("dx", "dw")),
    "c5c": (32, 56, 56, 64, 256, 1, 1, 0, 64, ("dx", "dw")),
}
HBM_BOUND = {"c1", "c4c", "c5a", "c5c"}   # arithmetic intensity below the ridge


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


class Workload:
    """Device tensors of one layer plus closures that enqueue each operator the way the Java engine does."""

    def __init__(self, pkg, torch, layer, seed, fill_units=False, dw_winograd=False):
        self.pkg, self.torch, self.layer = pkg, torch, layer
        N, IH, IW, IC, OC, F, s, p, ICl, _ = LAYERS[layer]
        self.dims = (N, IH, IW, IC, OC, F, s, p)
        OH, OW = out_dim(IH, F, s, p), out_dim(IW, F, s, p)
        self.OH, self.OW = OH, OW
        dev = torch.device("cuda:0")
        g = torch.Generator(device="cpu").manual_seed(seed)
        X = torch.randn((N, IH, IW, IC), generator=g)
        W = torch.randn((OC, F, F, IC), generator=g) * float(np.sqrt(2.0 / (F * F * ICl)))
        if ICl < IC:
            X[..., ICl:] = 0
            W[..., ICl:] = 0
        dY = torch.randn((N, OH, OW, OC), generator=g)
        self.X, self.W, self.dY = X.to(dev), W.to(dev), dY.to(dev)
        self.Y = torch.empty((N, OH, OW, OC), device=dev)
        self.dX = torch.empty((N, IH, IW, IC), device=dev)
        self.dW = torch.empty((OC, F, F, IC), device=dev)
        self.CW = torch.empty(F * F * IC * OC, device=dev)
        self.Bias = torch.randn((OC,), generator=g).to(dev)
        self.stream = int(torch.cuda.current_stream().cuda_stream)
        self.streams = [self.stream]
        self.engine = pkg.engine.Engine(self.stream)
        if fill_units:
            # this build's option: raise the split-K factor until the launch fills the device (the reference's GridZ
            # is sized for at most 128 SMs)
            self.engine.config.deltaW_SK_fillUnits = pkg.device_info()[0]
        if dw_winograd:
            # this build's Winograd backward-filter, its split-K factor sized for the device's compute units
            self.engine.config.deltaW_winograd = pkg.device_info()[0]
        # split-K factor for the kernel-only timing: what the host layer would pass (CudaFloat32EngineBase.java:1707-1715)
        self.GridZ = max(1, pkg.engine.plan_deltaW(self.engine.config, IH, IW, OH, OW, F, F, N, IC, OC, s, s).GridZ)
        self.buf = torch.empty(max(1, self.GridZ - 1) * self.dW.numel(), device=dev)
        if F == 3 and s == 1:
            self.U = torch.empty(16 * IC * OC, device=dev)

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

    def wino(self):
        self.engine.config.conv3D_winograd = 1
        self.fwd()
        self.engine.config.conv3D_winograd = 0

    def fwd_bias(self):
        # conv3D_biased through the host layer: same plan as fwd, bias added in the kernel epilogue
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.engine.conv3D_biased(self.Y.data_ptr(), self.OH, self.OW, self.X.data_ptr(), IH, IW, self.W.data_ptr(), F, F,
                                  N, IC, OC, s, s, p, p, self.Bias.data_ptr(), N * self.OH * self.OW * OC, OC)

    def fwd_cached(self):
        # as fwd, with this build's option that keeps the re-laid-out filter between calls (inference, or training with
        # the weight update reported to the engine)
        self.engine.config.cache_filter_transforms = 1
        self.fwd()

    def fwd(self):
        # whole operator through the C++ host layer: entry selection, CW scratch, kernel_remode, conv entry
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.engine.conv3D(self.Y.data_ptr(), self.OH, self.OW, self.X.data_ptr(), IH, IW, self.W.data_ptr(), F, F,
                           N, IC, OC, s, s, p, p)

    def dx(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        D = self.pkg.Cuda_dconv3D_deltaX
        if F == 1:
            D.dconv3D_deltaX_W1(self.streams, 1, self.dY.data_ptr(), self.W.data_ptr(), self.dX.data_ptr(), IH, IW, N, IC, OC)
        else:
            D.dconv3D_deltaX_V2_s1(True, self.streams, 1, self.dY.data_ptr(), self.OH, self.OW, self.W.data_ptr(), F, F,
                                   self.dX.data_ptr(), IH, IW, N, IC, OC, p, p)

    def dw_gemm(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        D = self.pkg.Cuda_dconv3D_deltaW
        if F == 1:
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

    def dx_wino(self):
        self.engine.config.deltaX_winograd = 1
        self.dx_op()
        self.engine.config.deltaX_winograd = 0

    def dx_op(self):
        N, IH, IW, IC, OC, F, s, p = self.dims
        self.engine.dconv3D_deltaX(self.dX.data_ptr(), IH, IW, self.dY.data_ptr(), self.OH, self.OW, self.W.data_ptr(), F, F,
                                   N, IC, OC, s, s, p, p)


def time_loop(torch, fn, steps, warmup):
    """Wall-clock (sync'ed both sides) and HIP-event time of `steps` back-to-back calls, in ms per call."""
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


def cpu_baseline(layer, op, budget_s=12.0):
    """Times the oracle's float-accumulate direct convolution on a batch subset sized for ~budget_s."""
    from oracle import oracle as O
    N, IH, IW, IC, OC, F, s, p, ICl, _ = LAYERS[layer]
    OH, OW = out_dim(IH, F, s, p), out_dim(IW, F, s, p)
    r = np.random.Generator(np.random.PCG64(7))
    cores = O.num_threads()

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

    per_image = flops(layer) / N
    n0 = min(N, max(1, cores // 4))
    t_probe = run(n0)
    n = int(max(n0, min(N, n0 * budget_s / max(t_probe, 1e-6))))
    t1 = run(n) if n > n0 else t_probe
    n_used = n if n > n0 else n0
    reps = int(max(1, min(5000, budget_s / max(t1, 1e-6))))   # repeat the subset until ~budget_s of CPU work is timed
    t = sum(run(n_used) for _ in range(reps))
    return {
        "value": round(per_image * n_used * reps / t / 1e12, 6), "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": "%s %s on %d of %d images x %d repeats (%.1f s total, OpenMP over n,oh; float accumulate, direct loops)"
                  % (layer, op, n_used, N, reps, t),
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


def measure(pkg, torch, layer, op, steps, warmup):
    wl = Workload(pkg, torch, layer, seed=1000 + sorted(LAYERS).index(layer), fill_units=(op == "dw_fill"), dw_winograd=(op == "dw_wino"))
    step = {"fwd": wl.fwd, "fwd_cached": wl.fwd_cached, "fwd_bias": wl.fwd_bias, "dx": wl.dx_op, "dw": wl.dw, "dw_fill": wl.dw, "wino": wl.wino,
            "dx_wino": wl.dx_wino, "dw_wino": wl.dw}[op]
    kernel = {"fwd": wl.fwd_conv, "fwd_cached": wl.fwd_conv, "fwd_bias": wl.fwd_conv, "dx": wl.dx, "dw": wl.dw_gemm, "dw_fill": wl.dw_gemm,
              "wino": wl.wino_conv, "dx_wino": wl.dx_wino_conv, "dw_wino": wl.dw_wino_gemm}[op]
    if op in ("fwd", "fwd_bias", "fwd_cached"):
        wl.fwd_remode()
    if op == "wino":
        N_, IH_, IW_, IC_, OC_, F_, s_, p_ = wl.dims
        pkg.Cuda_conv3D.winograd_filter_transform(wl.stream, wl.W.data_ptr(), wl.U.data_ptr(), IC_, OC_)
    if op == "dx_wino":
        N_, IH_, IW_, IC_, OC_, F_, s_, p_ = wl.dims
        pkg.Cuda_dconv3D_deltaX.winograd_filter_transform_deltaX(wl.stream, wl.W.data_ptr(), wl.U.data_ptr(), IC_, OC_)
    def step_and_recycle():
        step()
    wall_ms, ev_ms = time_loop(torch, step_and_recycle, steps, warmup)
    wl.engine.sync()
    _, k_ms = time_loop(torch, kernel, steps, max(1, warmup // 2))   # dominant kernel alone, HIP events on its stream
    gridz = wl.GridZ
    wl.engine.close()
    fl, by = flops(layer), algorithmic_bytes(layer)
    hbm = layer in HBM_BOUND
    roof = {
        "bound": "hbm" if hbm else "mfma",
        "achieved": round(by / (k_ms * 1e-3) / 1e9, 2) if hbm else round(fl / (k_ms * 1e-3) / 1e12, 3),
        "peak": PEAK_HBM_GBPS if hbm else PEAK_MFMA_F32_TFLOPS,
        "unit": "GB/s" if hbm else "TFLOP/s",
        "kernel_ms": round(k_ms, 5),
        "traffic": load_traffic(layer, op),
    }
    roof["frac"] = round(roof["achieved"] / roof["peak"], 4)
    return {"layer": layer, "op": op, "ms_per_step": round(wall_ms, 5), "event_ms_per_step": round(ev_ms, 5),
            "tflops": round(fl / (wall_ms * 1e-3) / 1e12, 3), "gflop": round(fl / 1e9, 3),
            "algorithmic_MB": round(by / 1e6, 2), "GridZ": gridz if op in ("dw", "dw_fill") else None, "roofline": roof}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--layer", default="c3a", choices=sorted(LAYERS))
    ap.add_argument("--op", default=None, choices=["fwd", "fwd_bias", "fwd_cached", "dx", "dw", "dw_fill", "wino", "dx_wino", "dw_wino"],
                    help="wino = forward through Winograd F(2x2,3x3) (3x3 stride-1 layers), reported in direct-conv-equivalent FLOPs")
    ap.add_argument("--layers", action="store_true", help="also measure every layer/op of BASELINE.json's configs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--probe-copy", action="store_true",
                    help="only run a plain 256 MiB device-to-device copy a few times (calibrates FETCH_SIZE/WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is built and measured on ONE GPU; --gpus %d is not supported "
              "(forward/backward-data shard over N with no exchange, backward-filter needs one all-reduce of deltaW)." % args.gpus,
              file=sys.stderr)
        sys.exit(2)

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
    op = args.op or LAYERS[args.layer][9][0]

    head = measure(pkg, torch, args.layer, op, args.steps, args.warmup)
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
                   "device": {"name": props.name, "cus": cus, "clock_ghz": round(clk_ghz, 3),
                              "fp32_mfma_peak_from_device_tflops": round(cus * 256 * clk_ghz / 1e3, 1)}},
        "roofline": head["roofline"],
    }
    if op == "fwd" and F == 3 and s == 1 and IC >= 16:
        # the same layer through this build's second forward algorithm, in direct-convolution-equivalent FLOPs
        wn = measure(pkg, torch, args.layer, "wino", args.steps, args.warmup)
        out["winograd"] = {"value": wn["tflops"], "unit": "TFLOP/s (direct-conv-equivalent)", "ms_per_step": wn["ms_per_step"],
                           "kernel_ms": wn["roofline"]["kernel_ms"], "kernel_tflops": wn["roofline"]["achieved"],
                           "frac_of_fp32_mfma_peak": wn["roofline"]["frac"],
                           "note": "Winograd F(2x2,3x3): 2.25x fewer multiplies than the FLOP count credited"}
    if args.layers:
        out["layers"] = []
        for layer in sorted(LAYERS):
            ops = list(LAYERS[layer][9])
            if "fwd" in ops and LAYERS[layer][5] == 3 and LAYERS[layer][6] == 1 and LAYERS[layer][3] >= 16:
                ops.append("wino")
            if "dx" in ops and LAYERS[layer][5] == 3 and LAYERS[layer][6] == 1:
                ops.append("dx_wino")
            if "dw" in ops:
                ops.append("dw_fill")
            if "dw" in ops and LAYERS[layer][5] == 3 and LAYERS[layer][6] == 1:
                ops.append("dw_wino")
            if layer == "c3a":
                ops += ["fwd_bias", "fwd_cached"]
            for o in ops:
                out["layers"].append(measure(pkg, torch, layer, o, max(5, args.steps // 5), max(2, args.warmup // 3)))
                torch.cuda.empty_cache()
    out["cpu_baseline"] = None if args.no_cpu else cpu_baseline(args.layer, op)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
