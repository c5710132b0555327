"""``TernarySwiGLU``: the block MLP ``down(silu(gate(h)) * up(h))`` over packed ternary weights
with the glue fused (no counterpart in ``bittorch.nn``; structure of the reference's JS runtime,
``js/src/models/TernaryTransformer.ts:366-423``, and of its pre-norm block, ``:489-521``).

``compute="float"`` keeps the reference's arithmetic (fp32-accumulate packed kernels) and only
fuses ``silu * up`` and the residual add.  ``compute="int8"`` is the BitNet-style path: the
RMSNorm (or the input) and the SwiGLU product leave their kernels already quantized per row to
int8, and the three projections run on the int8 matrix cores.
"""

from __future__ import annotations

from typing import Optional

import torch.nn as nn
from torch import Tensor

from .ternary_linear_infer import TernaryLinearInference


class TernarySwiGLU(nn.Module):
    def __init__(self, gate: TernaryLinearInference, up: TernaryLinearInference, down: TernaryLinearInference,
                 compute: str = "float"):
        super().__init__()
        if compute not in ("float", "int8"):
            raise ValueError(f"compute must be 'float' or 'int8', got {compute!r}")
        if not (gate.in_features == up.in_features and gate.out_features == up.out_features
                and down.in_features == gate.out_features):
            raise ValueError("gate/up/down shapes do not form an MLP")
        self.gate, self.up, self.down = gate, up, down
        self.compute = compute

    def forward(self, x: Tensor, norm_weight: Optional[Tensor] = None, eps: Optional[float] = None,
                residual: Optional[Tensor] = None) -> Tensor:
        """``down(silu(gate(h)) * up(h)) [+ residual]`` with ``h = rmsnorm(x, norm_weight, eps)`` when
        ``eps`` is given and ``h = x`` otherwise."""
        from ..ops import fused

        if not x.is_cuda:
            import torch.nn.functional as F
            h = x if eps is None else F.rms_norm(x, (x.shape[-1],), norm_weight, eps)
            return self.down(F.silu(self.gate(h)) * self.up(h), residual)
        if self.compute == "float":
            h = x if eps is None else fused.rmsnorm(x, norm_weight, eps)
            return self.down(fused.swiglu(self.gate(h), self.up(h)), residual)
        if eps is None:
            from .. import _C
            q, s = _C.act_quant_int8(x.reshape(-1, x.shape[-1]))
            q, s = q.reshape(x.shape), s.reshape(x.shape[:-1])
        else:
            q, s = fused.rmsnorm(x, norm_weight, eps, store=False, quantize=True)
        g = self.gate.forward_int8(q, s, x.dtype)
        u = self.up.forward_int8(q, s, x.dtype)
        q2, s2 = fused.swiglu(g, u, store=False, quantize=True)
        return self.down.forward_int8(q2, s2, x.dtype, residual)
