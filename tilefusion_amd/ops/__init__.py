"""Core operations (counterpart of python/ops/__init__.py in the reference)."""

from .flash_attention import FlashAttention, flash_attention
from .flash_decode import flash_decode
from .fused_two_gemms import fused_two_gemms
from .gemm import gemm
from .scatter_nd import scatter_nd

__all__ = [
    "FlashAttention",
    "flash_attention",
    "flash_decode",
    "fused_two_gemms",
    "gemm",
    "scatter_nd",
]
