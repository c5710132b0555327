"""Ternary layers (same names as ``bittorch.nn``)."""

from .ternary_linear import TernaryLinear
from .ternary_linear_cuda import TernaryLinearCUDA
from .ternary_linear_infer import TernaryLinearInference, create_ternary_linear_inference
from .ternary_mlp import TernarySwiGLU

__all__ = ["TernaryLinear", "TernaryLinearCUDA", "TernaryLinearInference",
           "create_ternary_linear_inference", "TernarySwiGLU"]
