"""2-bit codec for ternary weights: four weights per byte.

Codes: 0 -> 0b00, +1 -> 0b01, -1 -> 0b10, 0b11 is reserved and decodes to 0.
Weight ``k = 4*kb + i`` of a row sits in bits ``2i, 2i+1`` of byte ``kb``.
Two layouts exist: row-major ``[N, ceil(K/4)]`` and the transposed
``[ceil(K/4), N]`` that the device kernels and ``TernaryLinearInference`` use.
Reference: ``bittorch/quant/ternary_packed.py:22-223``.
"""

from __future__ import annotations

from typing import Tuple

import torch
from torch import Tensor

_SHIFTS = (0, 2, 4, 6)


def _require_2d(t: Tensor) -> None:
    if t.dim() != 2:
        raise ValueError(f"Expected 2D tensor, got {t.dim()}D")


def pack_ternary(w_tern: Tensor) -> Tuple[Tensor, int]:
    """``(uint8 [N, ceil(K/4)], K)``; K is zero-padded to a multiple of four
    (reference ``ternary_packed.py:22-75``)."""
    _require_2d(w_tern)
    rows, cols = w_tern.shape
    tail = (-cols) % 4
    if tail:
        w_tern = torch.nn.functional.pad(w_tern, (0, tail), value=0)
    codes = (w_tern == 1).to(torch.uint8) + 2 * (w_tern == -1).to(torch.uint8)
    quads = codes.reshape(rows, -1, 4)
    packed = quads[..., 0].clone()
    for i in (1, 2, 3):
        packed |= quads[..., i] << _SHIFTS[i]
    return packed, cols


def unpack_ternary(packed: Tensor, in_features: int) -> Tensor:
    """int8 ``[N, in_features]`` from ``[N, ceil(K/4)]`` bytes
    (reference ``ternary_packed.py:78-120``)."""
    _require_2d(packed)
    rows = packed.shape[0]
    codes = torch.stack([(packed >> s) & 0x3 for s in _SHIFTS], dim=2).reshape(rows, -1)
    values = (codes == 1).to(torch.int8) - (codes == 2).to(torch.int8)
    return values[:, :in_features]


def pack_ternary_with_scale(w_tern: Tensor, scale: Tensor) -> Tuple[Tensor, Tensor, int]:
    """Packed bytes plus the scale cast to fp16 (reference ``ternary_packed.py:123-141``)."""
    packed, in_features = pack_ternary(w_tern)
    return packed, scale.to(torch.float16), in_features


def get_packed_size(out_features: int, in_features: int) -> int:
    """Bytes of packed weights, scales excluded (reference ``ternary_packed.py:144-155``)."""
    return out_features * ((in_features + 3) // 4)


def get_memory_reduction(out_features: int, in_features: int) -> float:
    """fp32 bytes / (packed bytes + fp16 scales) (reference ``ternary_packed.py:158-171``)."""
    dense = 4 * out_features * in_features
    return dense / (get_packed_size(out_features, in_features) + 2 * out_features)


def pack_ternary_transposed(w_tern: Tensor) -> Tuple[Tensor, int]:
    """``(uint8 [ceil(K/4), N] contiguous, K)``: byte ``[kb, n]`` holds
    ``W[n, 4kb:4kb+4]`` (reference ``ternary_packed.py:174-206``)."""
    packed, in_features = pack_ternary(w_tern)
    return packed.t().contiguous(), in_features


def unpack_ternary_transposed(packed_T: Tensor, in_features: int) -> Tensor:
    """Inverse of :func:`pack_ternary_transposed` (reference ``ternary_packed.py:209-223``)."""
    return unpack_ternary(packed_T.t().contiguous(), in_features)
