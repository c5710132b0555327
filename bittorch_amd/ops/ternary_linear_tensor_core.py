"""Matrix-core (int8 MFMA) forward over packed ternary weights.

Mirrors ``bittorch/ops/ternary_linear_tensor_core.py:17-41``: ``version=1`` is the
float-compute path, ``version=2`` quantizes each activation row to int8 and
accumulates in int32 on the matrix cores.
"""

from __future__ import annotations

from typing import Optional

from torch import Tensor


def ternary_linear_tensor_core_forward(x: Tensor, w_packed_T: Tensor, scale: Tensor, in_features: int,
                                       bias: Optional[Tensor] = None, version: int = 1) -> Tensor:
    from .. import _C

    return _C.ternary_linear_tensor_core_forward(x, w_packed_T, scale, bias, in_features, version)
