"""Functional forward with dense (unpacked) ternary weights.

Host wrapper over ``_C.ternary_linear_forward``; mirrors the reference's
``bittorch/ops/ternary_linear.py:15-86``.
"""

from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from ..quant.ternary import ternary_quantize


def ternary_linear_forward_cuda(x: Tensor, w_tern: Tensor, scale: Tensor,
                                bias: Optional[Tensor] = None) -> Tensor:
    """``Y = X @ (W_tern * scale).T + bias`` on the GPU.

    ``x`` is ``(*, K)``, ``w_tern`` int8 ``(N, K)``, ``scale`` ``(N,)``; scale and
    bias are cast to ``x.dtype`` first, as the reference does (``:40-47``).
    """
    from .. import _C  # ImportError if the HIP library is not built

    scale = scale.to(dtype=x.dtype)
    if bias is not None:
        bias = bias.to(dtype=x.dtype)
    return _C.ternary_linear_forward(x.contiguous(), w_tern.contiguous(), scale.contiguous(),
                                     None if bias is None else bias.contiguous())


def ternary_linear(x: Tensor, weight: Tensor, bias: Optional[Tensor] = None,
                   threshold_factor: float = 0.05, per_channel: bool = True) -> Tensor:
    """Quantize ``weight`` on the fly, then run the GPU forward (reference ``:52-86``).

    The quantizer and the 2-bit packing run as one fused HIP kernel and the
    product reads the packed weights, so no dense int8 copy is materialised.
    """
    from .. import _C
    from .ternary_linear_packed import ternary_linear_packed_forward

    if not weight.is_cuda or weight.dtype == torch.float64:
        w_tern, scale = ternary_quantize(weight, threshold_factor, per_channel)
        return ternary_linear_forward_cuda(x, w_tern.to(torch.int8), scale.reshape(-1), bias)
    packed, scale, _ = _C.ternary_quantize_pack(weight, threshold_factor, per_channel)
    scale = scale.reshape(-1).to(x.dtype)
    if bias is not None:
        bias = bias.to(x.dtype)
    return ternary_linear_packed_forward(x, packed, scale, weight.shape[1], bias)
