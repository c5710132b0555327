"""Quantizers and the packed-weight codec (same names as ``bittorch.quant``)."""

from .base import QuantConfig, QuantType, Quantizer, ScaleType, compute_scale
from .int4 import (Int4QuantConfig, Int4Quantizer, dequantize_int4, int4_quantize,
                   int4_quantize_ste)
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
    "Int4QuantConfig", "Int4Quantizer", "int4_quantize", "int4_quantize_ste", "dequantize_int4",
]
