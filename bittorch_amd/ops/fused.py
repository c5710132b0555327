"""Fused glue between the ternary layers of a transformer block (HIP, no counterpart in
``bittorch.ops``; block structure of the reference's JS runtime,
``js/src/models/TernaryTransformer.ts:366-423`` and ``:489-521``).

* :func:`swiglu` -- ``silu(gate) * up`` in one pass, optionally leaving the result already
  quantized per row to int8 for the int8 matrix-core GEMM;
* :func:`rmsnorm` -- RMSNorm, optionally with the same quantization fused in;
* :func:`ternary_linear_int8` -- the int8 GEMM on pre-quantized activations, so that one
  quantization feeds several projections (q/k/v, gate/up), with an optional residual;
* ``operand_order=True`` on the quantizing side with ``q_operand_order=True`` on the GEMM side
  hands the int8 activations over in the order the matrix cores consume them.

The residual connection itself is an argument of the linear layers' forward
(``residual=``): the add happens in the GEMM epilogue.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor


def swiglu(gate: Tensor, up: Tensor, store: bool = True, quantize: bool = False, operand_order: bool = False,
           return_rowsum: bool = False):
    from .. import _C

    return _C.swiglu(gate, up, store, quantize, operand_order, return_rowsum)


def rmsnorm(x: Tensor, weight: Optional[Tensor] = None, eps: float = 1e-6, store: bool = True,
            quantize: bool = False, operand_order: bool = False, return_rowsum: bool = False):
    from .. import _C

    return _C.rmsnorm(x, weight, eps, store, quantize, operand_order, return_rowsum)


def act_quant_int8(x: Tensor, operand_order: bool = False, return_rowsum: bool = False):
    """Per-row int8 quantization of ``x`` ``(*, K)``: ``(q int8 (*, K), s_x fp32 (*))``; with ``return_rowsum`` also the
    rows' sums of ``q`` (int32 ``(*)``), which ``TernaryLinearInference.forward_int8`` hands to the prefill GEMM on a
    layer's field-layout copy (``prepare_prefill``)."""
    from .. import _C

    out = _C.act_quant_int8(x.reshape(-1, x.shape[-1]), operand_order, return_rowsum)
    lead = x.shape[:-1]
    if return_rowsum:
        return out[0].reshape(x.shape), out[1].reshape(lead), out[2].reshape(lead)
    return out[0].reshape(x.shape), out[1].reshape(lead)


def ternary_linear_int8(q: Tensor, s_x: Tensor, w_packed_T: Tensor, scale: Tensor, in_features: int,
                        bias: Optional[Tensor] = None, out_dtype: torch.dtype = torch.bfloat16,
                        residual: Optional[Tensor] = None, q_operand_order: bool = False) -> Tensor:
    """``q`` int8 ``(*, K)`` with per-row scales ``s_x`` ``(*)`` -> ``(*, N)`` in ``out_dtype``.

    ``q_operand_order``: ``q`` was produced with ``operand_order=True`` (every 16-byte group already
    in the order the matrix cores take it; K % 16 == 0), which spares the GEMM a permutation."""
    from .. import _C

    lead = q.shape[:-1]
    y = _C.ternary_gemm_int8(q.reshape(-1, q.shape[-1]), s_x.reshape(-1), w_packed_T, scale, bias, in_features,
                             out_dtype, False,
                             None if residual is None else residual.reshape(-1, residual.shape[-1]),
                             q_operand_order)
    return y.reshape(*lead, y.shape[-1])
