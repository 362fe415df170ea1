"""Shared helpers for the tests: loads the product package (its directory name is not a valid
Python identifier, so it is imported by path) and wraps device buffers for the C ABI."""
import importlib.util
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "dragon-alpha-v1.0_amd")


def load_package():
    name = "dragon_alpha_amd"
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(name, os.path.join(PKG_DIR, "__init__.py"),
                                                  submodule_search_locations=[PKG_DIR])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def uniform(shape, seed, lo=-1.0, hi=1.0):
    return rng(seed).uniform(lo, hi, size=shape).astype(np.float32)


def normal(shape, seed, std=1.0):
    return (rng(seed).standard_normal(size=shape) * std).astype(np.float32)


def he_normal(OC, FH, FW, IC, seed):
    return normal((OC, FH, FW, IC), seed, std=float(np.sqrt(2.0 / (FH * FW * IC))))


GUARD = 16384          # floats on either side of a guarded output (a multiple of 4: the tensor stays 16-byte aligned)
SENTINEL = 1.5e30


class Dev:
    """Device-side helpers built on torch (allocation, copies, the current stream handle)."""

    def __init__(self):
        import torch
        self.torch = torch
        assert torch.cuda.is_available(), "GPU tests need a GPU"
        self.dev = torch.device("cuda:0")
        self.stream = int(torch.cuda.current_stream().cuda_stream)
        self.streams = [self.stream]

    def put(self, a):
        return self.torch.from_numpy(np.ascontiguousarray(a)).to(self.dev)

    def empty(self, *shape, fill=None):
        t = self.torch.empty(shape, dtype=self.torch.float32, device=self.dev)
        if fill is not None:
            t.fill_(fill)
        return t

    def guarded(self, *shape):
        """An output tensor filled with NaN that sits between two guard bands of a sentinel value; `check_guards`
        tells whether a kernel wrote outside the tensor."""
        n = int(np.prod(shape))
        flat = self.torch.full((2 * GUARD + n,), SENTINEL, dtype=self.torch.float32, device=self.dev)
        inner = flat[GUARD:GUARD + n].view(*shape)
        inner.fill_(float("nan"))
        inner._guard_owner = flat
        return inner

    def check_guards(self, t):
        flat = t._guard_owner
        self.torch.cuda.synchronize()
        n = flat.numel() - 2 * GUARD
        lo, hi = flat[:GUARD].cpu().numpy(), flat[GUARD + n:].cpu().numpy()
        assert np.all(lo == np.float32(SENTINEL)), "write before the output tensor"
        assert np.all(hi == np.float32(SENTINEL)), "write past the output tensor"

    def get(self, t):
        self.torch.cuda.synchronize()
        if hasattr(t, "_guard_owner"):
            self.check_guards(t)
        return t.cpu().numpy()

    def sync(self):
        self.torch.cuda.synchronize()


def out_dim(IH, IW, FH, FW, sh, sw, ph, pw):
    return (IH + 2 * ph - FH) // sh + 1, (IW + 2 * pw - FW) // sw + 1
