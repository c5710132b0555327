"""``ternary_linear_grouped`` / ``ternary_linear_int8_grouped``: G decode-shape products of same-shaped inference
layers in ONE kernel launch.

No counterpart in ``bittorch.ops``: the reference's packed kernel serves one matrix per launch
(``csrc/kernels/ternary_gemm_production.cu:286-362``, called from ``bittorch/nn/ternary_linear_infer.py:78-104``).  A
4 MiB weight matrix streams in less time than a kernel takes to start and drain, so a decode step that has several
independent GEMVs of one shape -- q, k and v of a block kept as separate layers, the same projection of several
models or adapters, one row per user times per-user layers -- pays that start once for all of them here
(``bt_ternary_gemv_grouped``).  Every unit's output equals ``layer(x_row)`` bit for bit for fp16 rows; bf16 rows are
summed exactly (each row scaled by its own largest exponent) and agree with the single call's fp32 sums to their
rounding.  Whatever the grouped kernel does not take (CPU tensors, fp32 rows, K % 16 != 0, layers without a natural
tiled copy) runs as single calls, same results as ``layer(x)``.

``ternary_linear_int8_grouped`` is the same for the int8 path with up to 16 rows per layer (a batched decode step;
``bt_ternary_gemm_i8_grouped``): per-row int8 activations, int32 accumulators on the matrix cores, every unit equal to
``layer.forward_int8`` on its rows bit for bit.
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
        self.i8_tabs: "OrderedDict[tuple, tuple]" = OrderedDict()

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


    def i8_tab(self, q: Tensor, s_x: Tensor, y: Tensor):
        """Tables of the G units' addresses inside q [G, M, K], s_x [G, M] and y [G, M, N]; cached by address."""
        key = (q.data_ptr(), s_x.data_ptr(), y.data_ptr())
        hit = self.i8_tabs.get(key)
        if hit is not None:
            self.i8_tabs.move_to_end(key)
            return hit
        g = q.shape[0]

        def tab(t):
            step = t.stride(0) * t.element_size()
            return torch.tensor([t.data_ptr() + u * step for u in range(g)], dtype=torch.int64, device=t.device)

        self.i8_tabs[key] = (tab(q), tab(s_x), tab(y))
        if len(self.i8_tabs) > 8:
            self.i8_tabs.popitem(last=False)
        return self.i8_tabs[key]


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


_MAX_K_I8 = 11264  # the grouped int8 kernel holds a wave's K slice of the 16 rows in registers
_MIN_G_I8 = 3  # below this the one-matrix kernel, one call per unit, is the faster route (persistent workgroups
               # that walk a single matrix leave most of the chip's request queues empty)


def ternary_linear_int8_grouped(layers: Sequence, xs: Optional[Tensor] = None, q: Optional[Tensor] = None,
                                s_x: Optional[Tensor] = None, out_dtype: Optional[torch.dtype] = None,
                                q_operand_order: bool = False, out: Optional[Tensor] = None) -> Tensor:
    """``Y[u] = layers[u].forward_int8(q[u], s_x[u])`` for ``G`` same-shaped layers with up to 16 activation rows each,
    in one launch.

    Either ``xs`` ``[G, M, K]`` float activations (quantized here per row, one launch for all units) or already
    quantized ``q`` ``[G, M, K]`` int8 with row scales ``s_x`` ``[G, M]`` (``q_operand_order`` as in
    :func:`ops.ternary_linear_int8`).  Returns ``[G, M, N]`` in ``out_dtype`` (default: ``xs.dtype``, or bf16)."""
    layers = list(layers)
    if not layers:
        raise ValueError("ternary_linear_int8_grouped: no layers")
    from ..nn.ternary_linear_infer import TernaryLinearInference
    from .. import _C
    for L in layers:
        if not isinstance(L, TernaryLinearInference):
            raise TypeError("ternary_linear_int8_grouped takes TernaryLinearInference layers")
    g, k, n = len(layers), layers[0].in_features, layers[0].out_features
    for L in layers:
        if (L.in_features, L.out_features) != (k, n):
            raise ValueError("ternary_linear_int8_grouped: every layer must have the same in_features and out_features")
        if (L.bias is None) != (layers[0].bias is None) or L.scale.numel() != layers[0].scale.numel():
            raise ValueError("ternary_linear_int8_grouped: layers must agree on having a bias and on the scale's length")
    if (xs is None) == (q is None) or (q is not None and s_x is None):
        raise ValueError("ternary_linear_int8_grouped: give xs, or q together with s_x")
    src = xs if xs is not None else q
    if src.dim() != 3 or src.shape[0] != g or src.shape[2] != k:
        raise RuntimeError(f"input K doesn't match in_features: expected [{g}, M, {k}], got {tuple(src.shape)}")
    m = src.shape[1]
    if not src.is_cuda:
        raise RuntimeError("All tensors must be CUDA")
    if out_dtype is None:
        out_dtype = xs.dtype if xs is not None and xs.dtype in (torch.float16, torch.bfloat16, torch.float32) else torch.bfloat16
    if xs is not None:
        q_operand_order = k % 16 == 0
        q2, s2 = _C.act_quant_int8(xs.reshape(g * m, k), q_operand_order)
        q, s_x = q2.view(g, m, k), s2.view(g, m)
    else:
        if q.dtype != torch.int8 or s_x.shape != (g, m) or s_x.dtype != torch.float32:
            raise RuntimeError("q must be int8 [G, M, K] and s_x fp32 [G, M]")
        q, s_x = q.contiguous(), s_x.contiguous()
    kinds = (torch.float32, torch.float16, torch.bfloat16)
    groupable = (g >= _MIN_G_I8 and m <= 16 and k % 16 == 0 and k <= _MAX_K_I8 and _groupable(layers, torch.empty(0, dtype=torch.float16, device=q.device))
                 and all(L.scale.dtype in kinds for L in layers))
    if out is not None and (out.shape != (g, m, n) or out.dtype != out_dtype or not out.is_contiguous()):
        raise ValueError("ternary_linear_int8_grouped: out must be a contiguous [G, M, N] tensor of out_dtype")
    if not groupable:
        y = torch.stack([L.forward_int8(q[u], s_x[u], out_dtype, None, q_operand_order) for u, L in enumerate(layers)])
        return y if out is None else out.copy_(y)
    plan = _plan_for(layers)
    y = out if out is not None else torch.empty((g, m, n), dtype=out_dtype, device=q.device)
    qt, st, yt = plan.i8_tab(q, s_x, y)
    _C.ternary_gemm_int8_grouped(qt, st, plan.w_tab, plan.s_tab, plan.b_tab, yt, m, k, n,
                                 scale_len=layers[0].scale.numel(), scale_dtype=layers[0].scale.dtype,
                                 bias_dtype=torch.float32 if layers[0].bias is None else layers[0].bias.dtype,
                                 out_dtype=out_dtype, q_operand_order=q_operand_order)
    return y
