"""Ternary {-1, 0, +1} quantizer with absmax scales.

Host-side (torch) statement of the reference quantizer,
``bittorch/quant/ternary.py:100-150``; the fused HIP quantize+pack kernel is
bit-exact with what these functions return.
"""

from __future__ import annotations

import dataclasses
from typing import Optional, Tuple

import torch
from torch import Tensor

from .base import QuantConfig, Quantizer, QuantType, ScaleType

_SCALE_FLOOR = 1e-8


@dataclasses.dataclass
class TernaryQuantConfig(QuantConfig):
    """threshold = threshold_factor * scale; scale per output row or per tensor
    (reference ``ternary.py:16-45``)."""

    threshold_factor: float = 0.05
    per_channel: bool = True

    def __post_init__(self) -> None:
        self.scale_type = ScaleType.PER_CHANNEL if self.per_channel else ScaleType.PER_TENSOR

    def validate(self) -> None:
        super().validate()
        if not 0.0 <= self.threshold_factor <= 1.0:
            raise ValueError(f"threshold_factor must be in [0, 1], got {self.threshold_factor}")


def ternary_quantize(weight: Tensor, threshold_factor: float = 0.05,
                     per_channel: bool = True) -> Tuple[Tensor, Tensor]:
    """``(w_tern, scale)`` with ``w_tern`` in {-1,0,+1} (dtype/shape of ``weight``).

    scale is the row absmax (shape ``(N,)``) or the tensor absmax (0-dim), floored
    at 1e-8; an entry survives iff ``|w| > threshold_factor * scale`` (strict).
    Reference: ``bittorch/quant/ternary.py:122-148``.
    """
    mag = weight.abs()
    if per_channel:
        scale = mag.max(dim=1, keepdim=True).values.clamp(min=_SCALE_FLOOR)
    else:
        scale = mag.max().reshape(1).clamp(min=_SCALE_FLOOR)
    if scale.dtype in (torch.float16, torch.bfloat16):
        # ``threshold_factor * scale`` on a 16-bit tensor is float(threshold_factor) * float(scale), rounded to fp32 and
        # then to the tensor's dtype -- two roundings, which is what torch's CPU kernels and the quantize+pack kernel
        # do.  torch's ROCm kernel fuses them into ONE rounding of the exact product, which lands on the other
        # neighbour where the fp32 product is a tie (a few elements per million at threshold_factor = 0.7): the two
        # steps are spelled out so that every device gives the same threshold.
        threshold = (scale.float() * threshold_factor).to(scale.dtype)
    else:
        threshold = threshold_factor * scale
    keep = mag > threshold
    w_tern = torch.where(keep, torch.sign(weight), torch.zeros_like(weight))
    return w_tern, (scale.squeeze(1) if per_channel else scale.squeeze(0))


def ternary_quantize_ste(weight: Tensor, threshold_factor: float = 0.05,
                         per_channel: bool = True) -> Tuple[Tensor, Tensor]:
    """Forward value = quantized weights, backward = identity onto ``weight``.

    The scale carries no gradient.  Reference: ``bittorch/quant/ternary.py:153-195``.
    """
    w_tern, scale = ternary_quantize(weight, threshold_factor, per_channel)
    passthrough = weight + (w_tern - weight).detach()
    return passthrough, scale.detach()


def dequantize_ternary(w_tern: Tensor, scale: Tensor) -> Tensor:
    """``w_tern * scale[:, None]`` (reference ``ternary.py:198-209``)."""
    return w_tern * scale.unsqueeze(1)


class TernaryQuantizer(Quantizer):
    """Object form of the three functions above (reference ``ternary.py:48-97``)."""

    def __init__(self, config: Optional[TernaryQuantConfig] = None):
        self._config = config if config is not None else TernaryQuantConfig()
        super().__init__(self._config)

    @property
    def quant_type(self) -> QuantType:
        return QuantType.TERNARY

    @property
    def bits_per_weight(self) -> float:
        return 1.58

    def quantize(self, weight: Tensor) -> Tuple[Tensor, Tensor]:
        return ternary_quantize(weight, self._config.threshold_factor, self._config.per_channel)

    def dequantize(self, w_tern: Tensor, scale: Tensor) -> Tensor:
        return dequantize_ternary(w_tern, scale)

    def quantize_ste(self, weight: Tensor) -> Tuple[Tensor, Tensor]:
        return ternary_quantize_ste(weight, self._config.threshold_factor,
                                    self._config.per_channel)
