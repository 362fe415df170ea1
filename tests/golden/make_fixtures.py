"""Writes tests/golden/conv_golden.npz: small seeded cases of the conv3D path with the expected results of the CPU oracle
at the time of writing (fp64 direct convolution, backward-data, backward-filter; the three filter re-layouts; the fp32
Kahan sum over split-K partials). The reference holds no golden vectors for this path (its tests draw unseeded random
numbers), so these freeze the pinned oracle: a later change to oracle/conv_oracle.c that alters any result, and a HIP
kernel that drifts from it, both show up against this file.

Run from the repository root:  python tests/golden/make_fixtures.py
Inputs come from numpy's PCG64 with the seeds below, uniform [-1, 1) rounded to float32; every array is stored in the
file, so the fixtures do not depend on numpy's generator staying the same."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as O   # noqa: E402

# name: N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw
CASES = {
    "s1_3x3": (4, 6, 6, 8, 8, 3, 3, 1, 1, 1, 1),
    "s2_3x3": (4, 7, 5, 4, 8, 3, 3, 2, 2, 1, 1),
    "s1_1x1": (4, 4, 5, 8, 12, 1, 1, 1, 1, 0, 0),
    "s2_5x4_ragged": (4, 8, 7, 4, 12, 5, 4, 2, 2, 2, 1),
    "stem_7x7_ic3": (4, 10, 10, 4, 8, 7, 7, 2, 2, 3, 3),
}
GRIDZ = 3


def make():
    out = {}
    for i, (name, (N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw)) in enumerate(sorted(CASES.items())):
        r = np.random.Generator(np.random.PCG64(20240 + i))
        OH, OW = O.out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
        X = r.uniform(-1, 1, (N, IH, IW, IC)).astype(np.float32)
        W = r.uniform(-1, 1, (OC, FH, FW, IC)).astype(np.float32)
        dY = r.uniform(-1, 1, (N, OH, OW, OC)).astype(np.float32)
        if name == "stem_7x7_ic3":   # three logical channels stored as four
            X[..., 3] = 0
            W[..., 3] = 0
        out[name + "/dims"] = np.array([N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw], dtype=np.int32)
        out[name + "/X"], out[name + "/W"], out[name + "/dY"] = X, W, dY
        out[name + "/Y"] = O.conv3D_f64(X, W, sh, sw, ph, pw)
        out[name + "/dX"] = O.deltaX_f64(dY, W, IH, IW, sh, sw, ph, pw)
        out[name + "/dW"] = O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw)
        out[name + "/CW"] = O.kernel_remode(W)
        out[name + "/ksCW1"] = O.ks_remode(W, sh, sw)
        out[name + "/ksCW2"] = O.ks_remodev2(W, sh, sw)
        parts = np.stack([O.deltaW_slice_f64(X, dY, FH, FW, sh, sw, ph, pw, GRIDZ, z).astype(np.float32) for z in range(GRIDZ)])
        out[name + "/dW_parts"] = parts
        out[name + "/dW_kahan"] = O.buf_summary(parts[1:].reshape(GRIDZ - 1, -1), parts[0]).reshape(OC, FH, FW, IC)
    return out


if __name__ == "__main__":
    path = os.path.join(HERE, "conv_golden.npz")
    np.savez_compressed(path, **make())
    print(path, os.path.getsize(path), "bytes")
