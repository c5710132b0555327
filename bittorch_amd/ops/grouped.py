"""``ternary_linear_grouped``: G decode GEMVs of same-shaped inference layers in ONE kernel launch.

No counterpart in ``bittorch.ops``: the reference's packed kernel serves one matrix per launch
(``csrc/kernels/ternary_gemm_production.cu:286-362``, called from ``bittorch/nn/ternary_linear_infer.py:78-104``).  A
4 MiB weight matrix streams in less time than a kernel takes to start and drain, so a decode step that has several
independent GEMVs of one shape -- q, k and v of a block kept as separate layers, the same projection of several
models or adapters, one row per user times per-user layers -- pays that start once for all of them here
(``bt_ternary_gemv_grouped``).  Every unit's output equals ``layer(x_row)`` bit for bit for fp16 rows; bf16 rows are
summed exactly (each row scaled by its own largest exponent) and agree with the single call's fp32 sums to their
rounding.  Whatever the grouped kernel does not take (CPU tensors, fp32 rows, K % 16 != 0, layers without a natural
tiled copy) runs as single calls, same results as ``layer(x)``.
"""

from __future__ import annotations

from collections import OrderedDict
from typing import List, Optional, Sequence, Union

import torch
from torch import Tensor

_MAX_K = 16384     # the grouped kernel keeps a row's digit planes in LDS
_PLANS: "OrderedDict[tuple, _Plan]" = OrderedDict()
_MAX_PLANS = 16


class _Plan:
    """Pointer tables of one set of layers (device arrays of G addresses), rebuilt when a layer's buffers move."""

    def __init__(self, layers):
        from .. import _C
        # (scales and biases go to the kernel in their own dtype, as the single call hands them over: same bits)
        self.tiled = [L.tiled_weights() for L in layers]       # keeps the copies alive
        self.scales = [L.scale.contiguous() for L in layers]
        self.biases = None if layers[0].bias is None else [L.bias.contiguous() for L in layers]
        self.key = self.fingerprint(layers)
        self.w_tab = _C.pointer_table(self.tiled)
        self.s_tab = _C.pointer_table(self.scales)
        self.b_tab = None if self.biases is None else _C.pointer_table(self.biases)
        self.io_tabs: "OrderedDict[tuple, tuple]" = OrderedDict()

    @staticmethod
    def fingerprint(layers):
        return tuple((L._tiled.data_ptr() if L._tiled is not None else 0, L.scale.data_ptr(), L.scale._version,
                      0 if L.bias is None else L.bias.data_ptr(), 0 if L.bias is None else L.bias._version)
                     for L in layers)

    def io_tab(self, x: Tensor, y: Tensor, shared_x: bool):
        """Tables of the G row addresses of x [G, K] (or of one shared row) and y [G, N]; cached by address, so a
        decode loop whose buffers repeat (and a captured graph, whose buffers are fixed) builds them once."""
        key = (x.data_ptr(), y.data_ptr(), shared_x)
        hit = self.io_tabs.get(key)
        if hit is not None:
            self.io_tabs.move_to_end(key)
            return hit
        g = y.shape[0]
        step = 0 if shared_x else x.stride(0) * x.element_size()
        xt = torch.tensor([x.data_ptr() + u * step for u in range(g)], dtype=torch.int64, device=x.device)
        yt = torch.tensor([y.data_ptr() + u * y.stride(0) * y.element_size() for u in range(g)], dtype=torch.int64,
                          device=x.device)
        self.io_tabs[key] = (xt, yt)
        if len(self.io_tabs) > 8:
            self.io_tabs.popitem(last=False)
        return xt, yt


def _plan_for(layers) -> _Plan:
    ident = tuple(id(L) for L in layers)
    plan = _PLANS.get(ident)
    if plan is not None and plan.key == _Plan.fingerprint(layers):
        _PLANS.move_to_end(ident)
        return plan
    plan = _Plan(layers)
    _PLANS[ident] = plan
    if len(_PLANS) > _MAX_PLANS:
        _PLANS.popitem(last=False)
    return plan


def _groupable(layers, x: Tensor) -> bool:
    L0 = layers[0]
    if not x.is_cuda or x.dtype not in (torch.float16, torch.bfloat16):
        return False
    if L0.in_features % 16 != 0 or L0.in_features > _MAX_K:
        return False
    kinds = (torch.float32, torch.float16, torch.bfloat16)
    for L in layers:
        if not (L.decode_tiled and L.tile_order == "natural" and L.scale.is_cuda):
            return False
        if L.scale.dtype != L0.scale.dtype or L.scale.dtype not in kinds:
            return False
        if L.bias is not None and (L.bias.dtype != L0.bias.dtype or L.bias.dtype not in kinds):
            return False
        if L._tiled is None and torch.cuda.is_current_stream_capturing():
            return False  # (a capture never builds the tiled copy)
    import os
    return os.environ.get("BITTORCH_KERNEL", "auto") != "generic"


def ternary_linear_grouped(layers: Sequence, xs: Union[Tensor, Sequence[Tensor]], out: Optional[Tensor] = None) -> Tensor:
    """``Y[u] = layers[u](xs[u])`` for ``G`` :class:`~bittorch_amd.nn.TernaryLinearInference` layers of one shape,
    one activation row each, in one launch.

    ``xs``: ``[G, K]`` (row ``u`` goes to layer ``u``), a single row ``[K]`` / ``[1, K]`` shared by every layer, or a
    sequence of ``G`` rows.  Returns ``[G, N]`` in the rows' dtype (written into ``out`` if given)."""
    layers = list(layers)
    if not layers:
        raise ValueError("ternary_linear_grouped: no layers")
    from ..nn.ternary_linear_infer import TernaryLinearInference
    for L in layers:
        if not isinstance(L, TernaryLinearInference):
            raise TypeError("ternary_linear_grouped takes TernaryLinearInference layers")
    g, k, n = len(layers), layers[0].in_features, layers[0].out_features
    for L in layers:
        if (L.in_features, L.out_features) != (k, n):
            raise ValueError("ternary_linear_grouped: every layer must have the same in_features and out_features")
        if (L.bias is None) != (layers[0].bias is None) or L.scale.numel() != layers[0].scale.numel():
            raise ValueError("ternary_linear_grouped: layers must agree on having a bias and on the scale's length")
    if not isinstance(xs, Tensor):
        xs = torch.stack([t.reshape(-1) for t in xs])
    shared = xs.numel() == k
    if shared:
        x = xs.reshape(1, k)
    else:
        if xs.dim() != 2 or xs.shape != (g, k):
            raise RuntimeError(f"input K doesn't match in_features: expected [{g}, {k}] or one row of {k}, got {tuple(xs.shape)}")
        x = xs
    if any(t is not None and t.is_cuda != x.is_cuda for L in layers for t in (L.scale,)):
        raise RuntimeError("All tensors must be CUDA")
    if out is not None and (out.shape != (g, n) or out.dtype != x.dtype or out.device != x.device or out.stride(1) != 1):
        raise ValueError("ternary_linear_grouped: out must be [G, N] in the rows' dtype on their device, rows contiguous")
    if not _groupable(layers, x):
        ys = [L(x if shared else x[u:u + 1]) for u, L in enumerate(layers)]
        y = torch.cat(ys, dim=0)
        return y if out is None else out.copy_(y)
    from .. import _C
    if x.stride(-1) != 1 or (x.data_ptr() % 16) or (not shared and (x.stride(0) * x.element_size()) % 16):
        x = x.contiguous()
    plan = _plan_for(layers)
    y = out if out is not None else torch.empty((g, n), dtype=x.dtype, device=x.device)
    xt, yt = plan.io_tab(x, y, shared)
    _C.ternary_gemv_grouped(xt, plan.w_tab, plan.s_tab, plan.b_tab, yt, k, n,
                            scale_len=layers[0].scale.numel(), scale_dtype=layers[0].scale.dtype,
                            bias_dtype=torch.float32 if layers[0].bias is None else layers[0].bias.dtype,
                            x_dtype=x.dtype)
    return y
