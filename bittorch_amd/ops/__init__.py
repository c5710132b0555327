"""Functional operations (same names as ``bittorch.ops``)."""

from .ternary_linear import ternary_linear, ternary_linear_forward_cuda
from .ternary_linear_packed import has_packed_cuda_support, ternary_linear_packed_forward
from .ternary_linear_tensor_core import ternary_linear_tensor_core_forward
from .fused import act_quant_int8, rmsnorm, swiglu, ternary_linear_int8
from .grouped import ternary_linear_grouped, ternary_linear_int8_grouped

__all__ = [
    "ternary_linear",
    "ternary_linear_forward_cuda",
    "ternary_linear_packed_forward",
    "has_packed_cuda_support",
    "ternary_linear_tensor_core_forward",
    "swiglu",
    "rmsnorm",
    "ternary_linear_int8",
    "act_quant_int8",
    "ternary_linear_grouped",
    "ternary_linear_int8_grouped",
]
