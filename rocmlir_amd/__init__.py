"""rocmlir_amd: MI355X (gfx950) kernels for the Rock-dialect contraction ops
behind a Miir-shaped C ABI (include/rocmlir_amd.h).

The compute path is librocmlir_amd.so (hand-written HIP, built by
rocmlir_amd._build).  This package is the thin Python host side: a ctypes
binding plus helpers that take torch tensors as device memory.  There is no
CPU or eager fallback: if the library is missing, importing the binding
raises.
"""
from .api import (RockError, RockKernel, RockProgram, attention, conv2d, conv2d_bwd_data,  conv3d,  # noqa: F401
                  conv2d_bwd_weight, conv3d_bwd_data, conv3d_bwd_weight, gemm, library_path, load_library,
                  mfma_rate)

__all__ = ["RockError", "RockKernel", "RockProgram", "gemm", "conv2d", "conv3d", "conv2d_bwd_data", "conv2d_bwd_weight",
           "conv3d_bwd_data", "conv3d_bwd_weight", "attention", "library_path", "load_library", "mfma_rate"]
# rocmlir_amd.tuning (tuning table + in-process tuner) is imported on demand
