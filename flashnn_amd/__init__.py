"""flashnn_amd: the FLASHNN quantized-GEMM operators on MI355X (gfx950).

Same public names as the reference's package for this path (flashnn/__init__.py:7-10):
DynamicQuantize, GemmA8W8, GemmWeightOnly, RMSNormDquant, set_use_triton,
set_autotune_triton_kernels - and for the layers one step before it: RMSNorm, LayerNorm,
LayernormDquant.
"""
from .kernel_backend import (get_use_triton, set_autotune_triton_kernels,  # noqa: F401
                             set_use_triton)
from .norm import LayerNorm, LayernormDquant, RMSNorm, RMSNormDquant  # noqa: F401
from .quant_gemm import DynamicQuantize, GemmA8W8, GemmWeightOnly  # noqa: F401

__all__ = ["DynamicQuantize", "GemmA8W8", "GemmWeightOnly", "RMSNormDquant", "RMSNorm", "LayerNorm",
           "LayernormDquant", "set_use_triton",
           "set_autotune_triton_kernels", "get_use_triton"]
