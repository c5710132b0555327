"""GPU-only ternary linear layer and its autograd function.

API mirror of ``bittorch/nn/ternary_linear_cuda.py:23-228``.  Forward: one fused
HIP kernel quantizes and packs the master weights, a second one multiplies the
activations with the packed weights (fp32 accumulation).  Backward is the
straight-through estimator with torch matmuls, as in the reference
(``:73-111``); the dense effective weights it needs are rebuilt from the packed
bytes instead of being kept alive from the forward.
"""

from __future__ import annotations

import os
from typing import Optional, Tuple

import torch
import torch.nn as nn
from torch import Tensor

from ..quant.ternary import ternary_quantize
from ._packed_cache import PackedWeightCache, cache_usable
from .ternary_linear import _init_linear_params


class TernaryLinearCUDAFunction(torch.autograd.Function):
    """``y = x @ (ternary(weight) * scale).T + bias`` with STE gradients."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.float16)
    def forward(ctx, x: Tensor, weight: Tensor, bias: Optional[Tensor], threshold_factor: float,
                per_channel: bool, cached=None) -> Tensor:
        """``cached``: optional ``(packed_T, scale, tiled copy or None)`` of exactly these weights (see
        ``_packed_cache.py``); the quantize+pack kernel is skipped when it is given."""
        from .. import _C

        if weight.dtype == torch.float64 or x.dtype == torch.float64:
            w_tern, scale = ternary_quantize(weight, threshold_factor, per_channel)
            out = _C.ternary_linear_forward(x.contiguous(), w_tern.to(torch.int8),
                                            scale.reshape(-1).to(x.dtype),
                                            None if bias is None else bias.to(x.dtype))
            packed = None
            ctx.w_eff = w_tern * scale.reshape(-1, 1)
        else:
            tiled = None
            if cached is not None:
                packed, scale, tiled = cached
            else:
                packed, scale, _ = _C.ternary_quantize_pack(weight, threshold_factor, per_channel)
            b = None if bias is None else bias.to(x.dtype).contiguous()
            if (tiled is not None and x.dtype in (torch.float16, torch.bfloat16, torch.float32)
                    and os.environ.get("BITTORCH_KERNEL") != "generic"):  # (the shape-generic kernel reads packed_T)
                out = _C.ternary_linear_tiled_forward(x.contiguous(), tiled, scale.reshape(-1).to(x.dtype), b,
                                                      weight.shape[1], weight.shape[0])
            else:
                out = _C.ternary_linear_packed_forward(x.contiguous(), packed, scale.reshape(-1).to(x.dtype), b,
                                                       weight.shape[1])
            ctx.w_eff = None
        ctx.save_for_backward(x, packed, scale)
        ctx.in_features = weight.shape[1]
        ctx.weight_dtype = weight.dtype
        ctx.has_bias = bias is not None
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output: Tensor):
        from .. import _C

        x, packed, scale = ctx.saved_tensors
        scale_col = scale.reshape(-1, 1)
        g2 = grad_output.reshape(-1, grad_output.shape[-1])
        x2 = x.reshape(-1, x.shape[-1])
        grad_x = grad_w = grad_b = None
        if ctx.needs_input_grad[0]:
            if packed is not None:
                w_eff = _C.unpack_dequant(packed, ctx.in_features, scale.reshape(-1),
                                          out_dtype=ctx.weight_dtype)
            else:
                w_eff = ctx.w_eff
            grad_x = (g2 @ w_eff.to(g2.dtype)).reshape(x.shape)
        if ctx.needs_input_grad[1]:
            # d(w_eff)/d(weight) = scale under the straight-through estimator
            grad_w = (g2.t() @ x2) * scale_col.to(g2.dtype)
        if ctx.has_bias and ctx.needs_input_grad[2]:
            grad_b = g2.sum(dim=0)
        return grad_x, grad_w, grad_b, None, None, None


class TernaryLinearCUDA(nn.Module):
    """Ternary linear layer that only accepts GPU tensors (reference ``:114-228``)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True,
                 threshold_factor: float = 0.05, per_channel: bool = True) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.threshold_factor = threshold_factor
        self.per_channel = per_channel
        self.weight = nn.Parameter(torch.empty(out_features, in_features))
        if bias:
            self.bias = nn.Parameter(torch.empty(out_features))
        else:
            self.register_parameter("bias", None)
        self._packed = PackedWeightCache()
        self.reset_parameters()

    def reset_parameters(self) -> None:
        _init_linear_params(self.weight, self.bias)

    def forward(self, x: Tensor) -> Tensor:
        if not x.is_cuda:
            raise RuntimeError("TernaryLinearCUDA requires CUDA tensors. Use TernaryLinear for CPU.")
        cached = None
        if cache_usable(x, self.weight):
            cached = self._packed.get(self.weight, self.threshold_factor, self.per_channel)
        return TernaryLinearCUDAFunction.apply(x, self.weight, self.bias, self.threshold_factor,
                                               self.per_channel, cached)

    def invalidate_packed_cache(self) -> None:
        """Forget the cached packed weights (needed only after an evaluation-time write through ``weight.data``,
        which the version counter the cache is keyed on does not see)."""
        self._packed.clear()

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.bias is not None}, threshold_factor={self.threshold_factor}, "
                f"per_channel={self.per_channel}")

    def get_quantized_weight(self) -> Tuple[Tensor, Tensor]:
        with torch.no_grad():
            return ternary_quantize(self.weight, self.threshold_factor, self.per_channel)
