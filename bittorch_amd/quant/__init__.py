"""Quantizers and the packed-weight codec (same names as ``bittorch.quant``; its INT4 module, in which every
function raises ``NotImplementedError``, has no counterpart here)."""

from .base import QuantConfig, QuantType, Quantizer, ScaleType, compute_scale
from .ternary import (TernaryQuantConfig, TernaryQuantizer, dequantize_ternary,
                      ternary_quantize, ternary_quantize_ste)
from .ternary_packed import (get_memory_reduction, get_packed_size, pack_ternary,
                             pack_ternary_transposed, pack_ternary_with_scale,
                             unpack_ternary, unpack_ternary_transposed)

__all__ = [
    "QuantConfig", "QuantType", "Quantizer", "ScaleType", "compute_scale",
    "TernaryQuantConfig", "TernaryQuantizer", "ternary_quantize", "ternary_quantize_ste",
    "dequantize_ternary",
    "pack_ternary", "unpack_ternary", "pack_ternary_with_scale", "pack_ternary_transposed",
    "unpack_ternary_transposed", "get_packed_size", "get_memory_reduction",
]
