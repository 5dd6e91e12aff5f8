"""MI355X-native low-bit GEMM/GEMV path behind nnfusion's kernel-plugin surface.

Python here is plumbing only: it loads the two native libraries built from ``csrc/``
(``libnnf_hip_kernels.so``: the gfx950 kernels behind a C ABI; ``libnnf_host.so``: the C++ host
side -- registry, emitters, codegen, data generator) and hands them device pointers.
"""
from . import _lib  # noqa: F401
from .ops import (  # noqa: F401
    NnfError,
    w4a16_gemm,
    w4a16_gemm_fused,
    w8a8_gemm,
    w8a8_gemm_acc,
    fused_mlp_w4a16,
)

__all__ = ["NnfError", "w4a16_gemm", "w4a16_gemm_fused", "w8a8_gemm", "w8a8_gemm_acc", "fused_mlp_w4a16"]
