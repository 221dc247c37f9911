"""flashnn_amd: the FLASHNN quantized-GEMM operators on MI355X (gfx950).

Same public names as the reference's package for this path (flashnn/__init__.py:7-10):
DynamicQuantize, GemmA8W8, GemmWeightOnly, RMSNormDquant, set_use_triton,
set_autotune_triton_kernels - for the layers one step before it: RMSNorm, LayerNorm,
LayernormDquant - and for the mixture-of-experts forms of the int8 and int4 GEMMs:
fused_moe_a8w8_forward, fused_moe_a16w4_forward (flashnn/__init__.py:14-15).
"""
from .fused_moe import fused_moe_a8w8_forward, fused_moe_a16w4_forward  # noqa: F401
from .kernel_backend import (get_use_triton, set_autotune_triton_kernels,  # noqa: F401
                             set_use_triton)
from .norm import LayerNorm, LayernormDquant, RMSNorm, RMSNormDquant  # noqa: F401
from .quant_gemm import DynamicQuantize, GemmA8W8, GemmWeightOnly  # noqa: F401

__all__ = ["DynamicQuantize", "GemmA8W8", "GemmWeightOnly", "RMSNormDquant", "RMSNorm", "LayerNorm",
           "LayernormDquant", "fused_moe_a8w8_forward", "fused_moe_a16w4_forward", "set_use_triton",
           "set_autotune_triton_kernels", "get_use_triton"]
