"""``TernaryLinear``: ``nn.Linear`` look-alike whose weights are ternarised on the fly.

Keeps the constructor, attributes, backend dispatch and error texts of the
reference module (``bittorch/nn/ternary_linear.py:29-242``).  Full-precision
master weights are trained; each forward quantizes them to {-1,0,+1} with an
absmax scale and a straight-through gradient.
"""

from __future__ import annotations

import math
import warnings
from typing import Literal, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from ..quant.ternary import ternary_quantize, ternary_quantize_ste
from ._packed_cache import PackedWeightCache, cache_usable

BackendType = Literal["auto", "cuda", "python"]
_BACKENDS = ("auto", "cuda", "python")


def _cuda_kernel_available() -> bool:
    """True when the HIP library is built and loadable (reference ``:20-26``)."""
    try:
        from .. import _C
    except ImportError:
        return False
    return hasattr(_C, "ternary_linear_forward")


def _init_linear_params(weight: Tensor, bias: Optional[Tensor]) -> None:
    """The default ``nn.Linear`` initialisation (reference ``:136-142``)."""
    nn.init.kaiming_uniform_(weight, a=math.sqrt(5))
    if bias is not None:
        fan_in = weight.shape[1]
        bound = 1.0 / math.sqrt(fan_in) if fan_in > 0 else 0.0
        nn.init.uniform_(bias, -bound, bound)


class TernaryLinear(nn.Module):
    """``y = x @ (w_tern * scale).T + bias`` with ``w_tern = ternary_quantize(weight)``.

    ``backend``: ``"auto"`` runs the HIP kernels for GPU tensors and plain torch
    otherwise; ``"cuda"`` insists on the kernels (``RuntimeError`` on CPU tensors
    or when the library is not built); ``"python"`` always uses plain torch ops.
    ``quantize=False`` turns the layer into an ordinary ``nn.Linear``.
    ``use_cuda_kernel`` is the deprecated boolean spelling of ``backend``.
    """

    def __init__(self, in_features: int, out_features: int, bias: bool = True,
                 threshold_factor: float = 0.05, per_channel: bool = True, quantize: bool = True,
                 backend: BackendType = "auto", use_cuda_kernel: Optional[bool] = None) -> None:
        super().__init__()
        if use_cuda_kernel is not None:
            warnings.warn("use_cuda_kernel is deprecated, use backend='auto'|'cuda'|'python' instead",
                          DeprecationWarning, stacklevel=2)
            backend = "auto" if use_cuda_kernel else "python"
        elif backend not in _BACKENDS:
            raise ValueError(f"backend must be 'auto', 'cuda', or 'python', got {backend!r}")
        self.in_features = in_features
        self.out_features = out_features
        self.threshold_factor = threshold_factor
        self.per_channel = per_channel
        self.quantize = quantize
        self.backend = backend
        self.use_cuda_kernel = backend != "python"
        self.weight = nn.Parameter(torch.empty(out_features, in_features))
        if bias:
            self.bias = nn.Parameter(torch.empty(out_features))
        else:
            self.register_parameter("bias", None)
        self._packed = PackedWeightCache()
        self.reset_parameters()

    def reset_parameters(self) -> None:
        _init_linear_params(self.weight, self.bias)

    def _should_use_cuda_kernel(self, x: Tensor) -> bool:
        """Backend decision for this input (reference ``:144-166``)."""
        if self.backend == "python":
            return False
        on_gpu = x.is_cuda and self.weight.is_cuda
        built = _cuda_kernel_available()
        if self.backend == "cuda":
            if not on_gpu:
                raise RuntimeError("backend='cuda' requires input and weights on CUDA device")
            if not built:
                raise RuntimeError("backend='cuda' requires CUDA extension to be built. "
                                   "Rebuild with CUDA support or use backend='python'")
            return True
        if on_gpu and not built:
            # never fall back silently on a GPU: the kernels are the product
            raise RuntimeError("GPU tensors given but the HIP library is not built "
                               "(python -m bittorch_amd.build); pass backend='python' to "
                               "run the plain torch path on purpose")
        return on_gpu

    def forward(self, x: Tensor) -> Tensor:
        if not self.quantize:
            return F.linear(x, self.weight, self.bias)
        if self._should_use_cuda_kernel(x):
            from .ternary_linear_cuda import TernaryLinearCUDAFunction
            cached = None
            if cache_usable(x, self.weight):  # packed weights are kept until the masters change
                cached = self._packed.get(self.weight, self.threshold_factor, self.per_channel)
            return TernaryLinearCUDAFunction.apply(x, self.weight, self.bias, self.threshold_factor,
                                                   self.per_channel, cached)
        # plain torch path (reference :194-213): the scale is folded into the
        # weights, which are rounded to the activation dtype before the product
        w_q, scale = ternary_quantize_ste(self.weight, self.threshold_factor, self.per_channel)
        w_eff = (w_q * scale.reshape(-1, 1)).to(x.dtype)
        bias = None if self.bias is None else self.bias.to(x.dtype)
        return F.linear(x, w_eff, bias)

    def invalidate_packed_cache(self) -> None:
        """Forget the cached packed weights (needed only after an evaluation-time write through ``weight.data``,
        which the version counter the cache is keyed on does not see)."""
        self._packed.clear()

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.bias is not None}, threshold_factor={self.threshold_factor}, "
                f"per_channel={self.per_channel}, quantize={self.quantize}, "
                f"backend={self.backend!r}")

    def get_quantized_weight(self) -> Tuple[Tensor, Tensor]:
        """Current ``(w_tern, scale)`` without gradient tracking (reference ``:228-242``)."""
        with torch.no_grad():
            return ternary_quantize(self.weight, self.threshold_factor, self.per_channel)
