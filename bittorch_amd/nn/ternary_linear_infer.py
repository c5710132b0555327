"""``TernaryLinearInference``: deployment layer that holds only packed weights.

API mirror of ``bittorch/nn/ternary_linear_infer.py:22-193``.  State: ``weight_packed`` uint8
``[ceil(K/4), N]`` (transposed layout), ``scale`` ``[N]``, optional ``bias``; nothing is trainable.  GPU inputs go
to the packed HIP kernels; CPU inputs unpack and use ``F.linear`` as the reference does.

On the GPU the layer keeps ONE copy of its weights: on its first GPU call it re-arranges ``weight_packed``
into the *decode-tiled* layout every matrix-core kernel of the library reads (same 2 bits per weight; 15-25 %
less time per decode GEMV because every load then covers whole cache lines, a few per cent on the prefill GEMMs)
and releases the row-major buffer.  ``state_dict()`` still holds ``weight_packed`` in the reference's layout
(rebuilt from the tiled copy with ``bt_untile_weights``, bit for bit), ``load_state_dict`` and ``.to()`` /
``.cpu()`` work as usual.  Reading the attribute ``layer.weight_packed`` brings the row-major buffer back as a
real buffer (so that in-place edits of it keep their meaning) and the layer then holds both copies until
``drop_row_major()``; so does a call that only the row-major kernels can serve once the buffer has been released
(the shape-generic kernel; int8 activations on a fused gate|up layer stored in pair order).  A fused gate|up layer
in pair order (``TernarySwiGLU``'s float default) serves decode and prefill, 16-bit and fp32, from its one tiled
copy.  ``packed_weights()`` returns the reference-layout bytes without changing what the layer holds.  ``decode_tiled=False`` or ``BITTORCH_DECODE_TILED=0`` keeps the layer on ``weight_packed``
alone.
"""

from __future__ import annotations

import os
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from ..quant.ternary import ternary_quantize
from ..quant.ternary_packed import pack_ternary_transposed, unpack_ternary_transposed


# batches up to this many rows stream the tiled weights (once per 16 rows) instead of running the tiled GEMM
DECODE_ROWS = 128
# From this many rows an int8 call with row sums takes the prefill GEMM on the field-layout copy (prepare_prefill):
# below it the routing between the streaming kernel and the tiled GEMM on the decode-tiled copy does as well or better.
PREFILL_ROWS = 384


class TernaryLinearInference(nn.Module):
    def __init__(self, in_features: int, out_features: int, weight_packed: Tensor, scale: Tensor,
                 bias: Optional[Tensor] = None, decode_tiled: Optional[bool] = None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.register_buffer("weight_packed", weight_packed)
        self.register_buffer("scale", scale)
        self.register_buffer("bias", bias)
        self.requires_grad_(False)
        if decode_tiled is None:
            decode_tiled = os.environ.get("BITTORCH_DECODE_TILED", "1") != "0"
        self.decode_tiled = bool(decode_tiled)
        # True: hold the reference-layout buffer beside the tiled copy (set once somebody needs it, see above)
        self.keep_row_major = False
        # "natural", or "gate_up_pairs" for a fused [gate | up] layer whose decode calls go through
        # forward_swiglu (set by TernarySwiGLU; such a copy serves only that output stage)
        self._tile_order = "natural"
        self._tiled: Optional[Tensor] = None
        self._tiled_key = None
        # prefill-only second copy (prepare_prefill) and the tiled copy it was made from
        self._fields: Optional[Tensor] = None
        self._fields_src: Optional[Tensor] = None

    # ---- which copies of the weights the layer holds ----------------------------------------
    def _has_row_major(self) -> bool:
        return "weight_packed" in self.__dict__["_buffers"]

    def __getattr__(self, name: str):
        if name == "weight_packed" and "_buffers" in self.__dict__ and not self._has_row_major() \
                and self.__dict__.get("_tiled") is not None:
            # somebody wants the buffer itself: bring it back for good (in-place edits must keep their meaning)
            self._restore_row_major(keep=True)
            return self._buffers["weight_packed"]
        return super().__getattr__(name)

    def _untiled(self) -> Tensor:
        from .. import _C
        return _C.untile_weights(self._tiled, self.out_features, self.in_features, self._tile_order == "gate_up_pairs")

    def _restore_row_major(self, keep: bool) -> Tensor:
        if not self._has_row_major():
            wp = self._untiled()
            self._buffers["weight_packed"] = wp
            self._tiled_key = (wp.data_ptr(), wp._version, wp.device, self._tile_order)
        if keep:
            self.keep_row_major = True
        return self._buffers["weight_packed"]

    def packed_weights(self) -> Tensor:
        """``W_T`` uint8 ``[ceil(K/4), N]`` in the reference's layout: the buffer if the layer holds it, otherwise a
        fresh tensor rebuilt from the tiled copy (what the layer holds does not change)."""
        return self._buffers["weight_packed"] if self._has_row_major() else self._untiled()

    def invalidate_packed_cache(self) -> "TernaryLinearInference":
        """Forget the decode-tiled copy when the layer also holds ``weight_packed``, so that the next call rebuilds it:
        for code that wrote ``weight_packed`` through ``.data`` (a write the tensor's version counter does not see)."""
        if self._has_row_major():
            self._tiled, self._tiled_key = None, None
        return self

    def drop_row_major(self) -> "TernaryLinearInference":
        """Back to one resident copy: build the tiled copy if need be and release the row-major buffer."""
        self.keep_row_major = False
        if self.decode_tiled and self._has_row_major() and self._buffers["weight_packed"].is_cuda:
            self.tiled_weights()
        return self

    @property
    def tile_order(self) -> str:
        return self._tile_order

    @tile_order.setter
    def tile_order(self, order: str) -> None:
        if order not in ("natural", "gate_up_pairs"):
            raise ValueError(f"tile_order must be 'natural' or 'gate_up_pairs', got {order!r}")
        if order != self._tile_order and self._tiled is not None:
            self._restore_row_major(keep=False)  # (in the old order) and re-tile on the next call
            self._tiled, self._tiled_key = None, None
        self._tile_order = order

    # ---- decode-tiled copy of the weights ---------------------------------------------------
    def tiled_weights(self) -> Tensor:
        """The decode-tiled copy of the weights (GPU only).  Built on first use from ``weight_packed``, which is
        then released unless ``keep_row_major``; rebuilt when a held ``weight_packed`` has moved or been written."""
        if not self._has_row_major():
            return self._tiled
        wp = self._buffers["weight_packed"]
        key = (wp.data_ptr(), wp._version, wp.device, self._tile_order)
        if self._tiled is None or self._tiled_key != key:
            from .. import _C
            self._tiled = _C.retile_weights(wp, self.in_features, self._tile_order == "gate_up_pairs")
            # built once on the current stream; later calls may come from any stream
            torch.cuda.current_stream(wp.device).synchronize()
            self._tiled_key = key
        if not self.keep_row_major and not torch.cuda.is_current_stream_capturing():
            del self._buffers["weight_packed"]  # one resident copy
        return self._tiled

    def resident_weight_bytes(self) -> int:
        """Bytes of packed weights the layer holds right now (tiled copy and / or row-major buffer, and the prefill
        copy if one was asked for)."""
        n = self._buffers["weight_packed"].numel() if self._has_row_major() else 0
        n += self._fields.numel() if self._prefill_copy() is not None else 0
        return n + (self._tiled.numel() if self._tiled is not None else 0)

    # state_dict / load_state_dict / .to() / pickling see the reference's layout whatever the layer holds
    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        if not self._has_row_major():
            moved = {prefix + name: destination.pop(prefix + name) for name in ("scale", "bias") if prefix + name in destination}
            destination[prefix + "weight_packed"] = self._untiled()
            destination.update(moved)  # the reference's key order: weight_packed, scale, bias

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        if not self._has_row_major():
            self._restore_row_major(keep=False)
        self._tiled, self._tiled_key = None, None
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def _apply(self, fn, *args, **kwargs):
        if not self._has_row_major():
            self._restore_row_major(keep=False)
        self._tiled, self._tiled_key = None, None
        return super()._apply(fn, *args, **kwargs)

    def __getstate__(self):
        # the tiled copy is derived data: rebuilt on demand, never pickled or deep-copied
        state = super().__getstate__() if hasattr(super(), "__getstate__") else self.__dict__.copy()
        state = dict(state)
        if not self._has_row_major():
            bufs = type(state["_buffers"])()
            bufs["weight_packed"] = self._untiled()
            bufs.update(state["_buffers"])
            state["_buffers"] = bufs
        state["_tiled"], state["_tiled_key"] = None, None
        state["_fields"], state["_fields_src"] = None, None
        return state

    def prepare_decode(self) -> "TernaryLinearInference":
        """Build the decode-tiled copy now (e.g. before capturing decode steps into a HIP graph: a
        capture never builds it, it falls back to ``weight_packed``)."""
        if self.decode_tiled and (not self._has_row_major() or self._buffers["weight_packed"].is_cuda):
            self.tiled_weights()
        return self

    def prepare_prefill(self) -> "TernaryLinearInference":
        """Opt in to a SECOND resident copy of the weights (0.25 bytes per weight more) in the field layout that only
        the prefill int8 GEMM reads: ``forward_int8(..., q_rowsum=...)`` with at least ``PREFILL_ROWS`` rows then
        decodes a weight operand with one AND.  The same bits as without it; 10-16 % faster GEMMs for prefill chunks
        of 512-1024 rows, nothing at 2048 rows and more.  Needs ``in_features % 128 == 0`` and the decode-tiled copy
        (GPU); ``drop_prefill()`` releases it."""
        self.prepare_decode()
        if self._tiled is not None and self.in_features % 128 == 0:
            from .. import _C
            self._fields = _C.retile_fields(self._tiled, self.in_features, self.out_features)
            self._fields_src = self._tiled
            torch.cuda.current_stream(self._tiled.device).synchronize()
        return self

    def drop_prefill(self) -> "TernaryLinearInference":
        self._fields, self._fields_src = None, None
        return self

    def _prefill_copy(self) -> Optional[Tensor]:
        """The field-layout copy if it still matches the tiled copy the layer holds (a layer whose weights were
        reloaded, moved or re-tiled simply stops using it until ``prepare_prefill`` is called again)."""
        if self._fields is not None and self._fields_src is self._tiled and self._tiled is not None:
            return self._fields
        return None

    def _tiled_for(self, x: Tensor, rows: int, order: str = "natural") -> Optional[Tensor]:
        """The tiled copy if this call can run on it, else None.  ``order`` is what the call wants: ``"natural"`` (a
        plain linear output; a copy in gate/up pair order serves it too, the kernels looking every column tile up
        where the pair order put it -- float activations only, see ``_natural_from_pairs``) or ``"gate_up_pairs"``
        (the SwiGLU output stage: pair-ordered copy, decode shapes)."""
        if not (self.decode_tiled and x.is_cuda):
            return None
        if order == "gate_up_pairs":
            if self._tile_order != order or rows > DECODE_ROWS:
                return None
        elif self._tile_order != "natural" and x.dtype == torch.int8:
            return None  # the int8 entry point reads natural-order copies only
        if os.environ.get("BITTORCH_KERNEL") == "generic":  # the shape-generic kernel reads weight_packed
            return None
        if x.dtype not in (torch.float16, torch.bfloat16, torch.float32, torch.int8):
            return None
        kb = (self.in_features + 3) // 4
        if ((self.out_features + 15) // 16) * ((kb + 15) // 16) * 256 >= 2 ** 32:  # beyond the kernels' 32-bit offsets
            return None
        if not self._has_row_major():
            return self._tiled
        wp = self._buffers["weight_packed"]
        fresh = self._tiled is not None and self._tiled_key == (wp.data_ptr(), wp._version, wp.device, self._tile_order)
        if not fresh and torch.cuda.is_current_stream_capturing():
            return None
        return self.tiled_weights()

    @property
    def _natural_from_pairs(self) -> bool:
        """True when a plain (natural column order) call reads a copy stored in gate/up pair order."""
        return self._tile_order == "gate_up_pairs"

    def _row_major_for_call(self) -> Tensor:
        """``weight_packed`` for a call that only the row-major kernels serve (the shape-generic kernel, int8
        activations on a pair-ordered copy, a first call inside a graph capture).  A layer that still holds the
        buffer just hands it over; one that had released it rebuilds it and holds both copies from then on
        (``drop_row_major()`` undoes that).  Inside a stream capture a released buffer cannot come back: the kernel
        that rebuilds it would be recorded instead of run, and ``weight_packed`` would hold nothing until the first
        replay."""
        if self._has_row_major():
            return self._buffers["weight_packed"]
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(
                "TernaryLinearInference: this call needs the row-major weight_packed, which the layer released after "
                "building its decode-tiled copy, and a stream capture cannot rebuild it; read layer.weight_packed "
                "(or make this call once) before capturing")
        return self._restore_row_major(keep=True)

    def forward(self, x: Tensor, residual: Optional[Tensor] = None, norm=None,
                swiglu_up: Optional[Tensor] = None) -> Tensor:
        """Additions to the reference's ``forward(x)``, all optional and GPU-fused: ``residual`` is added to
        the output inside the kernel; ``norm=(weight or None, eps)`` applies RMSNorm to ``x`` first;
        ``swiglu_up=u`` makes the input ``silu(x) * u`` (for a single decode token both run inside the
        GEMV kernel itself)."""
        if x.is_cuda:
            tiled = self._tiled_for(x, x.numel() // max(x.shape[-1], 1))
            if tiled is not None:
                from .. import _C
                return _C.ternary_linear_tiled_forward(x, tiled, self.scale, self.bias, self.in_features,
                                                       self.out_features, residual, norm, swiglu_up, False,
                                                       self._natural_from_pairs)
        if x.is_cuda and (norm is not None or swiglu_up is not None):
            from .. import _C
            return _C.ternary_linear_packed_forward_fused(x, self._row_major_for_call(), self.scale, self.bias,
                                                          self.in_features, residual, norm, swiglu_up)
        if norm is not None:
            x = F.rms_norm(x, (x.shape[-1],), norm[0], norm[1])
        if swiglu_up is not None:
            x = F.silu(x) * swiglu_up
        if x.is_cuda:
            from ..ops.ternary_linear_packed import ternary_linear_packed_forward
            return ternary_linear_packed_forward(x, self._row_major_for_call(), self.scale,
                                                 self.in_features, self.bias, residual)
        # CPU (reference :98-104): unpack, fold the scale in, dense product
        w = unpack_ternary_transposed(self.packed_weights(), self.in_features).to(x.dtype)
        w = w * self.scale.unsqueeze(1).to(x.dtype)
        y = F.linear(x, w, self.bias)
        return y if residual is None else y + residual

    def forward_swiglu(self, x: Tensor, norm=None) -> Tensor:
        """For a layer whose columns are ``[gate | up]``: ``swiglu(gate(h), up(h))`` ``(*, N/2)`` with ``h = x`` or
        ``rmsnorm(x, *norm)``.  Decode-shape calls on a layer with ``tile_order == "gate_up_pairs"`` form the product
        in the output stage of the GEMV kernel; everything else runs the projection and the SwiGLU kernel."""
        if x.is_cuda:
            tiled = self._tiled_for(x, x.numel() // max(x.shape[-1], 1), "gate_up_pairs")
            if tiled is not None and x.dtype in (torch.float16, torch.bfloat16):
                from .. import _C
                return _C.ternary_linear_tiled_forward(x, tiled, self.scale, self.bias, self.in_features,
                                                       self.out_features, None, norm, None, True)
        gu = self.forward(x, None, norm)
        half = self.out_features // 2
        if x.is_cuda:
            from ..ops import fused
            return fused.swiglu(gu[..., :half], gu[..., half:])
        return F.silu(gu[..., :half]) * gu[..., half:]

    def forward_int8(self, q: Tensor, s_x: Tensor, out_dtype: torch.dtype = torch.bfloat16,
                     residual: Optional[Tensor] = None, q_operand_order: bool = False,
                     q_rowsum: Optional[Tensor] = None) -> Tensor:
        """Forward from activations already quantized per row to int8 (``ops.rmsnorm`` /
        ``ops.swiglu`` / ``ops.act_quant_int8`` with ``quantize=True``): int8 matrix cores, int32
        accumulators (GPU only).  ``q_operand_order`` as in :func:`ops.ternary_linear_int8`.  ``q_rowsum`` (the rows'
        sums of ``q``, ``ops.act_quant_int8(..., return_rowsum=True)``) lets a prefill batch run on the layer's
        field-layout copy where ``prepare_prefill`` built one; the result does not depend on it."""
        rows = q.numel() // max(q.shape[-1], 1)
        fields = self._prefill_copy() if (q_rowsum is not None and rows >= PREFILL_ROWS and q.is_cuda) else None
        if fields is not None and os.environ.get("BITTORCH_KERNEL") != "generic":
            from .. import _C
            y = _C.ternary_gemm_int8_fields(q.reshape(-1, q.shape[-1]), s_x.reshape(-1), q_rowsum.reshape(-1), fields,
                                            self.scale, self.bias, self.in_features, self.out_features, out_dtype, False,
                                            None if residual is None else residual.reshape(-1, residual.shape[-1]),
                                            q_operand_order, self._natural_from_pairs)
            return y.reshape(*q.shape[:-1], self.out_features)
        tiled = self._tiled_for(q, rows)
        if tiled is not None:
            from .. import _C
            lead = q.shape[:-1]
            y = _C.ternary_gemm_int8_tiled(q.reshape(-1, q.shape[-1]), s_x.reshape(-1), tiled, self.scale, self.bias,
                                           self.in_features, self.out_features, out_dtype, False,
                                           None if residual is None else residual.reshape(-1, residual.shape[-1]),
                                           q_operand_order)
            return y.reshape(*lead, self.out_features)
        from ..ops.fused import ternary_linear_int8
        return ternary_linear_int8(q, s_x, self._row_major_for_call(), self.scale, self.in_features, self.bias,
                                   out_dtype, residual, q_operand_order)

    def extra_repr(self) -> str:
        dense = 4 * self.out_features * self.in_features
        ratio = dense / (self.packed_size_bytes + 2 * self.scale.numel())
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.bias is not None}, packed_bytes={self.packed_size_bytes}, "
                f"resident_weight_bytes={self.resident_weight_bytes()}, reduction={ratio:.1f}x")

    @classmethod
    def from_unpacked(cls, w_tern: Tensor, scale: Tensor,
                      bias: Optional[Tensor] = None) -> "TernaryLinearInference":
        """Pack already-quantized ``w_tern`` ``(N, K)`` (reference ``:119-148``)."""
        packed_t, in_features = pack_ternary_transposed(w_tern)
        return cls(in_features, w_tern.shape[0], packed_t, scale, bias)

    @property
    def packed_size_bytes(self) -> int:
        """Bytes of ``weight_packed`` (``ceil(K/4) * N``), whichever copy the layer holds."""
        return ((self.in_features + 3) // 4) * self.out_features

    @property
    def effective_bits_per_weight(self) -> float:
        bits = 8 * self.packed_size_bytes + 16 * self.scale.numel()
        return bits / (self.out_features * self.in_features)


def create_ternary_linear_inference(in_features: int, out_features: int, weight: Tensor,
                                    bias: Optional[Tensor] = None,
                                    threshold_factor: float = 0.05) -> TernaryLinearInference:
    """Quantize + pack full-precision ``weight`` into an inference layer (reference ``:163-193``).

    GPU weights go through the fused quantize+pack kernel, whose bytes and scales
    equal those of the torch path bit for bit.
    """
    if weight.is_cuda and weight.dtype in (torch.float32, torch.float16, torch.bfloat16):
        from .ternary_linear import _cuda_kernel_available
        if _cuda_kernel_available():
            from .. import _C
            packed, scale, _ = _C.ternary_quantize_pack(weight, threshold_factor, True)
            return TernaryLinearInference(in_features, out_features, packed, scale, bias)
    w_tern, scale = ternary_quantize(weight, threshold_factor=threshold_factor)
    return TernaryLinearInference.from_unpacked(w_tern, scale, bias)
