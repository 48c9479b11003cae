"""MI355X-native fast Hadamard transform library (gfx950 HIP kernels behind a C ABI).

Import by string, the package name starts with a digit::

    import importlib
    hada = importlib.import_module("6s894_project_2025_amd")
    y = hada.hadamard_transform(x)                 # scale = n ** -0.5
    hada.hadamard_transform(x, inplace=True)       # the reference's call shape
"""
from .ops import (fp8_gemm_rowscale, fused_ht_gemm, fused_ht_gemv, hadamard_transform,
                  rht_quant_fp8)

__all__ = ["hadamard_transform", "fused_ht_gemv", "fused_ht_gemm", "rht_quant_fp8",
           "fp8_gemm_rowscale"]
