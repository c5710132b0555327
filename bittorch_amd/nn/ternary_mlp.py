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
    """``fuse_gate_up=True`` stores gate and up as one layer of ``2 * ffn`` columns (one GEMM launch;
    SwiGLU then reads the two halves of its output in place)."""

    def __init__(self, gate: TernaryLinearInference, up: TernaryLinearInference, down: TernaryLinearInference,
                 compute: str = "float", fuse_gate_up: bool = False):
        super().__init__()
        if compute not in ("float", "int8"):
            raise ValueError(f"compute must be 'float' or 'int8', got {compute!r}")
        if not (gate.in_features == up.in_features and gate.out_features == up.out_features
                and down.in_features == gate.out_features):
            raise ValueError("gate/up/down shapes do not form an MLP")
        self.ffn = gate.out_features
        self.down = down
        if fuse_gate_up:
            from ..utils.convert import fuse_ternary_linear_inference
            self.gate_up = fuse_ternary_linear_inference(gate, up)
            self.gate = self.up = None
        else:
            self.gate_up = None
            self.gate, self.up = gate, up
        self.compute = compute

    @property
    def compute(self) -> str:
        return self._compute

    @compute.setter
    def compute(self, mode: str) -> None:
        if mode not in ("float", "int8"):
            raise ValueError(f"compute must be 'float' or 'int8', got {mode!r}")
        self._compute = mode
        if self.gate_up is not None:
            # float: decode-shape calls let the SwiGLU product leave the gate|up GEMV's own output stage, which wants
            # the tiles of the two halves alternating; int8: the GEMMs read the copy in natural order
            self.gate_up.tile_order = "gate_up_pairs" if (mode == "float" and self.ffn % 16 == 0) else "natural"

    def _gate_up(self, h: Tensor, norm=None):
        if self.gate_up is None:
            return self.gate(h, None, norm), self.up(h, None, norm)
        gu = self.gate_up(h, None, norm)
        return gu[..., :self.ffn], gu[..., self.ffn:]

    def _gate_up_int8(self, q: Tensor, s: Tensor, dtype, oo: bool, rs: Optional[Tensor] = None):
        if self.gate_up is None:
            return (self.gate.forward_int8(q, s, dtype, None, oo, rs), self.up.forward_int8(q, s, dtype, None, oo, rs))
        gu = self.gate_up.forward_int8(q, s, dtype, None, oo, rs)
        return gu[..., :self.ffn], gu[..., self.ffn:]

    def _linears(self):
        return [m for m in (self.gate_up, self.gate, self.up, self.down) if m is not None]

    def prepare_prefill(self) -> "TernarySwiGLU":
        """``TernaryLinearInference.prepare_prefill()`` on every projection (a second, prefill-only copy of the weights
        each): the int8 compute mode then hands its quantizers' row sums to the GEMMs of prefill-sized batches."""
        for m in self._linears():
            m.prepare_prefill()
        return self

    def drop_prefill(self) -> "TernarySwiGLU":
        for m in self._linears():
            m.drop_prefill()
        return self

    def _wants_rowsum(self, rows: int) -> bool:
        from .ternary_linear_infer import PREFILL_ROWS
        return rows >= PREFILL_ROWS and any(m._prefill_copy() is not None for m in self._linears())

    def forward(self, x: Tensor, norm_weight: Optional[Tensor] = None, eps: Optional[float] = None,
                residual: Optional[Tensor] = None) -> Tensor:
        """``down(silu(gate(h)) * up(h)) [+ residual]`` with ``h = rmsnorm(x, norm_weight, eps)`` when
        ``eps`` is given and ``h = x`` otherwise."""
        from ..ops import fused

        if not x.is_cuda:
            import torch.nn.functional as F
            h = x if eps is None else F.rms_norm(x, (x.shape[-1],), norm_weight, eps)
            g, u = self._gate_up(h)
            return self.down(F.silu(g) * u, residual)
        if self.compute == "float":
            # norm and SwiGLU ride on the projections that consume them (for one decode token they run
            # inside the GEMV kernels; otherwise as one fused kernel each ahead of the GEMM)
            norm = None if eps is None else (norm_weight, eps)
            if self.gate_up is not None and self.gate_up.tile_order == "gate_up_pairs":
                return self.down(self.gate_up.forward_swiglu(x, norm), residual)
            g, u = self._gate_up(x, norm)
            return self.down(g, residual, None, u)
        # the int8 activations stay inside this call: hand them over in the matrix cores' own order
        oo1, oo2 = x.shape[-1] % 16 == 0, self.ffn % 16 == 0
        # row sums of the quantized activations ride along where a projection holds a prefill copy that wants them
        want = self._wants_rowsum(x.numel() // max(x.shape[-1], 1))
        if eps is None:
            q, s, *rs = fused.act_quant_int8(x, oo1, return_rowsum=want)
        else:
            q, s, *rs = fused.rmsnorm(x, norm_weight, eps, store=False, quantize=True, operand_order=oo1, return_rowsum=want)
        g, u = self._gate_up_int8(q, s, x.dtype, oo1, rs[0] if rs else None)
        q2, s2, *rs2 = fused.swiglu(g, u, store=False, quantize=True, operand_order=oo2, return_rowsum=want)
        return self.down.forward_int8(q2, s2, x.dtype, residual, oo2, rs2[0] if rs2 else None)
