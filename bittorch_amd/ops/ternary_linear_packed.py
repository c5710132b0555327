"""Functional forward that reads 2-bit packed weights directly.

Mirrors ``bittorch/ops/ternary_linear_packed.py:21-90``.  The weights are in the
transposed layout ``[ceil(K/4), N]`` produced by ``pack_ternary_transposed``.
Decode-shape batches stream the packed bytes once from HBM through the matrix
cores; the kernel choice can be overridden with the environment variable
``BITTORCH_KERNEL`` (``auto`` | ``generic``), read on every call.
"""

from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor


def ternary_linear_packed_forward(x: Tensor, w_packed_T: Tensor, scale: Tensor, in_features: int,
                                  bias: Optional[Tensor] = None, residual: Optional[Tensor] = None) -> Tensor:
    """``Y = X @ (decode(W_packed_T) * scale).T + bias``; ``x`` is ``(*, K)``.

    ``residual`` (not in the reference) is added to the result inside the kernel."""
    from .. import _C

    return _C.ternary_linear_packed_forward(
        x.contiguous(), w_packed_T.contiguous(), scale.contiguous(),
        None if bias is None else bias.contiguous(), in_features, residual)


def has_packed_cuda_support() -> bool:
    """True when the packed kernel is built and a GPU is visible (reference ``:80-90``)."""
    try:
        from .. import _C  # noqa: F401
    except ImportError:
        return False
    return hasattr(_C, "ternary_linear_packed_forward") and torch.cuda.is_available()
