"""MI355X (gfx950) replacement for Dragon-Alpha's cu32 conv3D hot path.

The product is the shared library libalpha_conv_hip.so (HIP kernels + C ABI + JNI symbols) built
from csrc/. This Python package is only a thin ctypes mirror of the reference's Java native classes
(same class names, method names and argument order), used by tests and the benchmark. It never
falls back to a CPU or PyTorch implementation: if the library is missing, loading raises.
"""
from .native import (Cuda_conv3D, Cuda_dconv3D_deltaX, Cuda_dconv3D_deltaW, Cuda_function, Cuda_reduce, Epilogue, AlphaConvError, lib,  # noqa: F401
                     lib_path, exported_symbols, device_info)
from . import engine  # noqa: F401,E402
from . import runtime  # noqa: F401,E402
from .runtime import Cuda, CudaDevice  # noqa: F401,E402
