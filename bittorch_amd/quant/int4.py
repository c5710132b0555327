"""INT4 placeholders.  The reference declares this API and implements none of it
(``bittorch/quant/int4.py:76-157`` all raise); the same holds here."""

from __future__ import annotations

import dataclasses
from typing import Optional, Tuple

from torch import Tensor

from .base import QuantConfig, Quantizer, QuantType, ScaleType

_MSG = "INT4 quantization is not implemented."


@dataclasses.dataclass
class Int4QuantConfig(QuantConfig):
    scale_type: ScaleType = ScaleType.PER_GROUP
    group_size: int = 128
    symmetric: bool = True

    def validate(self) -> None:
        super().validate()
        if self.group_size < 1:
            raise ValueError(f"group_size must be >= 1, got {self.group_size}")


class Int4Quantizer(Quantizer):
    def __init__(self, config: Optional[Int4QuantConfig] = None):
        self._config = config if config is not None else Int4QuantConfig()
        super().__init__(self._config)

    @property
    def quant_type(self) -> QuantType:
        return QuantType.INT4

    @property
    def bits_per_weight(self) -> float:
        return 4.0

    def quantize(self, weight: Tensor) -> Tuple[Tensor, Tensor]:
        raise NotImplementedError(_MSG)

    def dequantize(self, w_int4: Tensor, scale: Tensor) -> Tensor:
        raise NotImplementedError(_MSG)

    def quantize_ste(self, weight: Tensor) -> Tuple[Tensor, Tensor]:
        raise NotImplementedError(_MSG)


def int4_quantize(weight: Tensor, group_size: int = 128, symmetric: bool = True):
    raise NotImplementedError(_MSG)


def int4_quantize_ste(weight: Tensor, group_size: int = 128, symmetric: bool = True):
    raise NotImplementedError(_MSG)


def dequantize_int4(w_int4: Tensor, scale: Tensor) -> Tensor:
    raise NotImplementedError(_MSG)
