"""Shared vocabulary of the quantizers: enums, the config base and the ABC.

API mirror of the reference's ``bittorch/quant/base.py:16-181`` (pure host
code; nothing here touches a device kernel).
"""

from __future__ import annotations

import abc
import dataclasses
import enum
from typing import Tuple

import torch
from torch import Tensor


class QuantType(enum.Enum):
    TERNARY = "ternary"
    INT4 = "int4"


class ScaleType(enum.Enum):
    PER_TENSOR = "per_tensor"
    PER_CHANNEL = "per_channel"
    PER_GROUP = "per_group"


@dataclasses.dataclass
class QuantConfig:
    """Options common to all schemes (reference ``base.py:31-54``)."""

    scale_type: ScaleType = ScaleType.PER_CHANNEL
    group_size: int = 128

    @property
    def per_channel(self) -> bool:
        return self.scale_type is ScaleType.PER_CHANNEL

    def validate(self) -> None:
        if self.scale_type is ScaleType.PER_GROUP and self.group_size < 1:
            raise ValueError(f"group_size must be >= 1, got {self.group_size}")


class Quantizer(abc.ABC):
    """quantize / dequantize / quantize_ste contract (reference ``base.py:57-136``)."""

    def __init__(self, config: QuantConfig):
        config.validate()
        self.config = config

    @abc.abstractmethod
    def quantize(self, weight: Tensor) -> Tuple[Tensor, Tensor]: ...

    @abc.abstractmethod
    def dequantize(self, w_quant: Tensor, scale: Tensor) -> Tensor: ...

    @abc.abstractmethod
    def quantize_ste(self, weight: Tensor) -> Tuple[Tensor, Tensor]: ...

    @property
    @abc.abstractmethod
    def quant_type(self) -> QuantType: ...

    @property
    @abc.abstractmethod
    def bits_per_weight(self) -> float: ...


def compute_scale(weight: Tensor, scale_type: ScaleType, group_size: int = 128,
                  eps: float = 1e-8) -> Tensor:
    """absmax scale per tensor / row / group of a row (reference ``base.py:139-181``)."""
    mag = weight.abs()
    if scale_type is ScaleType.PER_TENSOR:
        return mag.max().clamp(min=eps).reshape(1)
    if scale_type is ScaleType.PER_CHANNEL:
        return mag.amax(dim=1).clamp(min=eps)
    if scale_type is ScaleType.PER_GROUP:
        rows, cols = mag.shape
        tail = (-cols) % group_size
        if tail:
            mag = torch.nn.functional.pad(mag, (0, tail))
        return mag.reshape(rows, -1, group_size).amax(dim=2).clamp(min=eps)
    raise ValueError(f"Unknown scale_type: {scale_type}")
