"""``bittorch._C`` look-alike over the C-ABI HIP library.

Same four entry points, argument order and keyword names as the reference's
pybind11 module (``csrc/bindings/bittorch_bindings.cpp:34-88``) with the host
checks of ``csrc/core/dispatch.cpp:52-142``; additional entry points expose
the fused quantize+pack kernel and the int8 pipeline stages.  Tensors are
passed to the library as raw device pointers; outputs and scratch are
allocated here with torch so the library itself never allocates.

Importing this module raises ``ImportError`` when the library is not built.
"""

from __future__ import annotations

import os

from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _lib

_L = _lib.load()  # ImportError here == "extension not available"

_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
_INT8_OUT = 3


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _status(rc: int) -> None:
    if rc != 0:
        raise RuntimeError(_lib.last_error() or f"libbittorch_hip call failed ({rc})")


def _stream(t: Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: Optional[Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _dt(t: Tensor, what: str) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise RuntimeError(f"{what} must be float32, float16 or bfloat16, got {t.dtype}") from None


_ws_cache = {}


def _workspace(nbytes: int, device) -> Optional[Tensor]:
    """Scratch buffer for the current stream of ``device``, kept between calls (the library
    needs no initialisation of it).  One buffer per (device, stream): calls on one stream
    run in order."""
    if nbytes <= 0:
        return None
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    buf = _ws_cache.get(key)
    if buf is None or buf.numel() < nbytes:
        size = max(nbytes, 1 << 20)
        buf = torch.empty(size, dtype=torch.uint8, device=device)
        _ws_cache[key] = buf
    return buf


def _all_cuda(*ts: Optional[Tensor]) -> bool:
    return all(t is None or t.is_cuda for t in ts)


def _prep_vec(v: Tensor, x: Tensor) -> Tensor:
    """scale / bias operand: contiguous, in a dtype the kernels read (fp32 or 16-bit)."""
    if v.dtype not in _DT:
        v = v.to(x.dtype if x.dtype in _DT else torch.float32)
    return v.contiguous()


def dummy(input: Tensor) -> Tensor:
    """Copy of the input (reference ``dispatch.cpp:7-9``)."""
    return input.clone()


def _float64_packed(X, W_T, scale, bias, in_features):
    from .quant.ternary_packed import unpack_ternary_transposed
    w = unpack_ternary_transposed(W_T, in_features).to(X.dtype) * scale.to(X.dtype).unsqueeze(1)
    return torch.nn.functional.linear(X, w, None if bias is None else bias.to(X.dtype))


def pack_ternary_int8(W_tern: Tensor) -> Tensor:
    """Dense ternary ``[N, K]`` int8 on the GPU -> packed transposed ``[ceil(K/4), N]`` uint8
    (the bytes of ``quant.pack_ternary_transposed``)."""
    _check(W_tern.dim() == 2 and W_tern.dtype == torch.int8, "W_tern must be 2D int8")
    _check(W_tern.is_cuda, "All tensors must be CUDA")
    W_tern = W_tern.contiguous()
    N, K = W_tern.shape
    packed = torch.empty(((K + 3) // 4, N), dtype=torch.uint8, device=W_tern.device)
    with torch.cuda.device(W_tern.device):
        _status(_L.bt_pack_ternary_i8(W_tern.data_ptr(), N, K, packed.data_ptr(), _stream(W_tern)))
    return packed


def ternary_linear_forward(X: Tensor, W_tern: Tensor, scale: Tensor,
                           bias: Optional[Tensor] = None) -> Tensor:
    """``Y = X @ (W_tern * scale).T + bias`` with dense int8 ternary weights ``[N, K]``.

    Reference: ``bittorch_bindings.cpp:41-46``, ``dispatch.cpp:52-87``.
    """
    _check(X.dim() >= 1, "X must have at least 1 dimension")
    _check(X.numel() > 0, "X is empty")
    _check(W_tern.dim() == 2, "W_tern must be 2D [N, K]")
    _check(W_tern.dtype == torch.int8, "W_tern must be int8")
    _check(scale.dim() == 1, "scale must be 1D [N]")
    K = X.shape[-1]
    N, WK = W_tern.shape
    _check(K == WK, "input K doesn't match weight K")
    _check(scale.shape[0] in (N, 1), "scale size doesn't match N")
    if bias is not None:
        _check(bias.dim() == 1 and bias.shape[0] == N, "bias shape mismatch")
    _check(_all_cuda(X, W_tern, scale, bias), "All tensors must be CUDA")
    if X.dtype == torch.float64:
        w = W_tern.to(X.dtype) * scale.to(X.dtype).unsqueeze(1)
        return torch.nn.functional.linear(X, w, None if bias is None else bias.to(X.dtype))
    W_tern = W_tern.contiguous()
    if os.environ.get("BITTORCH_KERNEL", "auto") != "generic":
        # the weights are packed on the device (one read of N*K bytes) and the call joins the
        # packed matrix-core path; entries are taken as ternary (sign of anything non-zero)
        return ternary_linear_packed_forward(X, pack_ternary_int8(W_tern), scale, bias, K)
    x2 = X.contiguous().reshape(-1, K)
    scale = _prep_vec(scale, x2)
    bias = None if bias is None else _prep_vec(bias, x2)
    B = x2.shape[0]
    y = torch.empty((B, N), dtype=X.dtype, device=X.device)
    with torch.cuda.device(X.device):
        _status(_L.bt_ternary_linear_forward(
            x2.data_ptr(), _dt(x2, "X"), W_tern.data_ptr(), scale.data_ptr(), _dt(scale, "scale"),
            scale.numel(), _ptr(bias), 0 if bias is None else _dt(bias, "bias"), y.data_ptr(),
            B, N, K, _stream(X)))
    return y.reshape(*X.shape[:-1], N)


def _packed_checks(X, W_T, scale, bias, in_features, flatten: bool = True):
    _check(X.dim() >= 1, "X must have at least 1 dimension")
    _check(X.numel() > 0, "X is empty")
    _check(W_T.dim() == 2, "W_T must be 2D [K_bytes, N]")
    _check(W_T.dtype == torch.uint8, "W_T must be uint8")
    _check(scale.dim() == 1, "scale must be 1D [N]")
    K = X.shape[-1]
    K_bytes, N = W_T.shape
    _check(K == in_features, "input K doesn't match in_features")
    _check(K_bytes == (in_features + 3) // 4, "K_bytes doesn't match ceil(K/4)")
    _check(scale.shape[0] in (N, 1), "scale size doesn't match N")
    if bias is not None:
        _check(bias.dim() == 1 and bias.shape[0] == N, "bias shape mismatch")
    _check(_all_cuda(X, W_T, scale, bias), "All tensors must be CUDA")
    return K, N


def _residual_2d(residual: Tensor, like: Tensor, lead_shape, N: int) -> Tensor:
    _check(residual.shape == (*lead_shape, N), "residual shape doesn't match the output")
    _check(residual.dtype == like.dtype, "residual must have the output's dtype")
    _check(residual.device == like.device, "All tensors must be CUDA")
    r = residual.contiguous()
    if r.data_ptr() % 16:  # a view that starts inside a buffer: the epilogues read the residual in 16-byte pieces
        r = r.clone()
    return r.reshape(-1, N)


def ternary_linear_packed_forward(X: Tensor, W_T: Tensor, scale: Tensor,
                                  bias: Optional[Tensor] = None, in_features: int = -1,
                                  residual: Optional[Tensor] = None) -> Tensor:
    """Packed-weight forward, fp32 accumulation; ``W_T`` is ``[ceil(K/4), N]`` uint8.

    Reference: ``bittorch_bindings.cpp:48-63``, ``dispatch.cpp:105-142``.  ``scale``
    may be fp32 or the activation dtype and may have one entry (per-tensor scale).
    ``residual`` (additive, not in the reference): a tensor of the output's shape and dtype
    added in the kernel's epilogue with the two roundings of ``linear(x) + residual``.
    """
    if in_features < 0:
        in_features = X.shape[-1]
    K, N = _packed_checks(X, W_T, scale, bias, in_features)
    if X.dtype == torch.float64:
        y = _float64_packed(X, W_T, scale, bias, in_features)
        return y if residual is None else y + residual
    x2 = X.contiguous().reshape(-1, K)
    W_T = W_T.contiguous()
    scale = _prep_vec(scale, x2)
    bias = None if bias is None else _prep_vec(bias, x2)
    B = x2.shape[0]
    xdt = _dt(x2, "X")
    y = torch.empty((B, N), dtype=X.dtype, device=X.device)
    with torch.cuda.device(X.device):
        ws_bytes = _L.bt_packed_forward_workspace_bytes(B, N, K, xdt)
        ws = _workspace(ws_bytes, X.device)
        if residual is None:
            _status(_L.bt_ternary_linear_packed_forward(
                x2.data_ptr(), xdt, W_T.data_ptr(), scale.data_ptr(), _dt(scale, "scale"), scale.numel(),
                _ptr(bias), 0 if bias is None else _dt(bias, "bias"), y.data_ptr(), B, N, K,
                _ptr(ws), 0 if ws is None else ws.numel(), _stream(X)))
        else:
            res = _residual_2d(residual, X, X.shape[:-1], N)
            _status(_L.bt_ternary_linear_packed_forward_res(
                x2.data_ptr(), xdt, W_T.data_ptr(), scale.data_ptr(), _dt(scale, "scale"), scale.numel(),
                _ptr(bias), 0 if bias is None else _dt(bias, "bias"), res.data_ptr(), y.data_ptr(), B, N, K,
                _ptr(ws), 0 if ws is None else ws.numel(), _stream(X)))
    return y.reshape(*X.shape[:-1], N)


def ternary_linear_packed_forward_fused(X: Tensor, W_T: Tensor, scale: Tensor, bias: Optional[Tensor] = None,
                                        in_features: int = -1, residual: Optional[Tensor] = None,
                                        norm: Optional[Tuple[Optional[Tensor], float]] = None,
                                        swiglu_up: Optional[Tensor] = None) -> Tensor:
    """``linear(pro(X)) [+ residual]`` with ``pro`` = RMSNorm (``norm=(weight or None, eps)``) or
    SwiGLU (``X`` is the gate, ``swiglu_up`` the other factor): the values :func:`rmsnorm` /
    :func:`swiglu` would store, without the extra launch when ``X`` is one 16-bit row (a decode token)."""
    _check((norm is None) != (swiglu_up is None), "exactly one of norm and swiglu_up must be given")
    if in_features < 0:
        in_features = X.shape[-1]
    K, N = _packed_checks(X, W_T, scale, bias, in_features)
    _check(X.dtype in _DT, "X must be float32, float16 or bfloat16")
    x2 = _rows_2d(X, K)
    W_T = W_T.contiguous()
    scale = _prep_vec(scale, x2)
    bias = None if bias is None else _prep_vec(bias, x2)
    B = x2.shape[0]
    if norm is not None:
        w, eps = norm
        if w is not None:
            _check(w.dim() == 1 and w.shape[0] == K, "norm weight must be 1D [K]")
            w = w.to(X.dtype).contiguous()
        op, pb, ldb = 1, w, 0
    else:
        _check(swiglu_up.shape == X.shape and swiglu_up.dtype == X.dtype, "gate and up must match in shape and dtype")
        u2 = _rows_2d(swiglu_up, K)
        op, pb, ldb, eps = 2, u2, u2.stride(0), 0.0
    _check(_all_cuda(pb), "All tensors must be CUDA")
    xdt = _dt(x2, "X")
    y = torch.empty((B, N), dtype=X.dtype, device=X.device)
    res = None if residual is None else _residual_2d(residual, X, X.shape[:-1], N)
    with torch.cuda.device(X.device):
        ws = _workspace(_L.bt_packed_forward_fused_workspace_bytes(B, N, K, xdt), X.device)
        _status(_L.bt_ternary_linear_packed_forward_fused(
            x2.data_ptr(), x2.stride(0), xdt, op, _ptr(pb), ldb, float(eps), W_T.data_ptr(), scale.data_ptr(),
            _dt(scale, "scale"), scale.numel(), _ptr(bias), 0 if bias is None else _dt(bias, "bias"), _ptr(res),
            y.data_ptr(), B, N, K, _ptr(ws), 0 if ws is None else ws.numel(), _stream(X)))
    return y.reshape(*X.shape[:-1], N)


def retile_weights(W_T: Tensor, in_features: int, gate_up_pairs: bool = False) -> Tensor:
    """Decode-tiled copy of ``W_T [ceil(K/4), N]`` (flat uint8 tensor): per 16-column tile and 16-row step
    the 64 dwords a wave of the decode kernel loads, contiguous.  Built once; :func:`untile_weights` inverts it.
    ``gate_up_pairs`` (N % 32 == 0): the tiles of the two column halves alternate, for the SwiGLU output stage
    of :func:`ternary_linear_tiled_forward` (such a copy serves only that)."""
    _check(W_T.dim() == 2 and W_T.dtype == torch.uint8, "W_T must be 2D uint8 [K_bytes, N]")
    _check(not gate_up_pairs or W_T.shape[1] % 32 == 0, "gate/up pair order needs N % 32 == 0")
    _check(W_T.shape[0] == (in_features + 3) // 4, "K_bytes doesn't match ceil(K/4)")
    _check(_all_cuda(W_T), "All tensors must be CUDA")
    W_T = W_T.contiguous()
    N = W_T.shape[1]
    with torch.cuda.device(W_T.device):
        out = torch.empty((_L.bt_tiled_weights_bytes(N, in_features),), dtype=torch.uint8, device=W_T.device)
        _status(_L.bt_retile_weights(W_T.data_ptr(), N, in_features, 1 if gate_up_pairs else 0, out.data_ptr(),
                                     _stream(W_T)))
    return out


def _tiled_checks(W_tiled: Tensor, N: int, K: int):
    _check(W_tiled.dtype == torch.uint8 and W_tiled.dim() == 1 and W_tiled.is_contiguous(),
           "W_tiled must be the flat uint8 tensor retile_weights returned")
    _check(N > 0 and K > 0 and W_tiled.numel() == _L.bt_tiled_weights_bytes(N, K),
           "W_tiled size doesn't match out_features x in_features")


def untile_weights(W_tiled: Tensor, out_features: int, in_features: int, gate_up_pairs: bool = False) -> Tensor:
    """``W_T [ceil(K/4), N]`` back from its decode-tiled copy (exact inverse of :func:`retile_weights`)."""
    _tiled_checks(W_tiled, out_features, in_features)
    _check(_all_cuda(W_tiled), "All tensors must be CUDA")
    with torch.cuda.device(W_tiled.device):
        out = torch.empty(((in_features + 3) // 4, out_features), dtype=torch.uint8, device=W_tiled.device)
        _status(_L.bt_untile_weights(W_tiled.data_ptr(), out_features, in_features, 1 if gate_up_pairs else 0,
                                     out.data_ptr(), _stream(W_tiled)))
    return out


def ternary_linear_tiled_forward(X: Tensor, W_tiled: Tensor, scale: Tensor, bias: Optional[Tensor] = None,
                                 in_features: int = -1, out_features: int = -1, residual: Optional[Tensor] = None,
                                 norm: Optional[Tuple[Optional[Tensor], float]] = None,
                                 swiglu_up: Optional[Tensor] = None, swiglu_pairs: bool = False,
                                 natural_from_pairs: bool = False) -> Tensor:
    """:func:`ternary_linear_packed_forward` / ``_fused`` on the decode-tiled copy of the weights: the same results
    bit for bit wherever both layouts take the same kernel -- always up to 32 rows; the rule that hands larger
    batches to the tiled GEMM prices a tiled launch's remainder lower, so a batch near the crossover may stream on one
    layout and run the GEMM on the other, with fp32 sums that differ in their last bits.
    ``swiglu_pairs`` (copy built with ``gate_up_pairs=True``): the layer's columns are ``[gate | up]`` and the
    output is the MLP's hidden vector ``swiglu(gate(x), up(x))`` ``[*, N/2]``, formed in the kernel's output stage.
    ``natural_from_pairs``: the same pair-ordered copy read as an ordinary linear layer (output ``[*, N]`` in natural
    column order, bit-identical to a natural-order copy's)."""
    _check(not (swiglu_pairs and natural_from_pairs), "swiglu_pairs and natural_from_pairs exclude each other")
    _check(not natural_from_pairs or out_features % 32 == 0, "a pair-ordered copy has N % 32 == 0")
    _check(not swiglu_pairs or (residual is None and swiglu_up is None and out_features % 32 == 0),
           "swiglu_pairs needs N % 32 == 0 and takes neither a residual nor a SwiGLU prologue")
    _check(norm is None or swiglu_up is None, "at most one of norm and swiglu_up may be given")
    _check(X.dim() >= 1 and X.numel() > 0, "X is empty")
    K, N = X.shape[-1], out_features
    _check(K == in_features, "input K doesn't match in_features")
    _tiled_checks(W_tiled, N, K)
    _check(scale.dim() == 1 and scale.shape[0] in (N, 1), "scale size doesn't match N")
    _check(bias is None or (bias.dim() == 1 and bias.shape[0] == N), "bias shape mismatch")
    _check(_all_cuda(X, W_tiled, scale, bias), "All tensors must be CUDA")
    _check(X.dtype in _DT, "X must be float32, float16 or bfloat16")
    x2 = _rows_2d(X, K) if (norm is not None or swiglu_up is not None) else X.contiguous().reshape(-1, K)
    scale = _prep_vec(scale, x2)
    bias = None if bias is None else _prep_vec(bias, x2)
    B = x2.shape[0]
    op, pb, ldb, eps = 0, None, 0, 0.0
    if norm is not None:
        w, eps = norm
        if w is not None:
            _check(w.dim() == 1 and w.shape[0] == K, "norm weight must be 1D [K]")
            w = w.to(X.dtype).contiguous()
        op, pb = 1, w
    elif swiglu_up is not None:
        _check(swiglu_up.shape == X.shape and swiglu_up.dtype == X.dtype, "gate and up must match in shape and dtype")
        pb = _rows_2d(swiglu_up, K)
        op, ldb = 2, pb.stride(0)
    _check(_all_cuda(pb), "All tensors must be CUDA")
    xdt = _dt(x2, "X")
    Ny = N // 2 if swiglu_pairs else N
    y = torch.empty((B, Ny), dtype=X.dtype, device=X.device)
    res = None if residual is None else _residual_2d(residual, X, X.shape[:-1], N)
    with torch.cuda.device(X.device):
        ws = _workspace(_L.bt_packed_forward_fused_workspace_bytes(B, N, K, xdt), X.device)
        _status(_L.bt_ternary_linear_tiled_forward(
            x2.data_ptr(), x2.stride(0), xdt, op, _ptr(pb), ldb, float(eps), W_tiled.data_ptr(), scale.data_ptr(),
            _dt(scale, "scale"), scale.numel(), _ptr(bias), 0 if bias is None else _dt(bias, "bias"), _ptr(res),
            1 if swiglu_pairs else 2 if natural_from_pairs else 0, y.data_ptr(), B, N, K, _ptr(ws), 0 if ws is None else ws.numel(), _stream(X)))
    return y.reshape(*X.shape[:-1], Ny)


def pointer_table(tensors) -> Tensor:
    """Device array of the tensors' device addresses (int64), the form :func:`ternary_gemv_grouped` takes its
    operands in.  The caller keeps the tensors alive for as long as the table is used."""
    tensors = list(tensors)
    _check(len(tensors) > 0 and _all_cuda(*tensors), "All tensors must be CUDA")
    return torch.tensor([t.data_ptr() for t in tensors], dtype=torch.int64, device=tensors[0].device)


def ternary_gemv_grouped(x_tab: Tensor, w_tiled_tab: Tensor, scale_tab: Tensor, bias_tab: Optional[Tensor],
                         y_tab: Tensor, in_features: int, out_features: int, scale_len: int = -1,
                         scale_dtype: torch.dtype = torch.float32, bias_dtype: torch.dtype = torch.float16,
                         x_dtype: torch.dtype = torch.float16) -> None:
    """``G`` independent decode GEMVs in one launch: unit ``u`` multiplies the fp16 row at ``x_tab[u]`` with the
    decode-tiled weights at ``w_tiled_tab[u]`` into the fp16 row at ``y_tab[u]``, exactly as
    :func:`ternary_linear_tiled_forward` would on that row (same bits).  The tables are int64 device tensors of
    ``G`` device addresses (:func:`pointer_table`); nothing is allocated or returned.
    ``x_dtype=torch.bfloat16``: bf16 rows and outputs; each row is scaled by its own largest exponent and summed
    exactly on the int8 matrix cores."""
    G = x_tab.numel()
    tabs = (x_tab, w_tiled_tab, scale_tab, y_tab) + (() if bias_tab is None else (bias_tab,))
    for t in tabs:
        _check(t.dtype == torch.int64 and t.dim() == 1 and t.numel() == G and t.is_contiguous(),
               "pointer tables must be contiguous int64 tensors of one length")
    _check(_all_cuda(*tabs), "All tensors must be CUDA")
    _check(scale_dtype in _DT and bias_dtype in _DT, "scale / bias dtype must be float32, float16 or bfloat16")
    _check(x_dtype in (torch.float16, torch.bfloat16), "x_dtype must be float16 or bfloat16")
    with torch.cuda.device(x_tab.device):
        _status(_L.bt_ternary_gemv_grouped(
            x_tab.data_ptr(), _DT[x_dtype], w_tiled_tab.data_ptr(), scale_tab.data_ptr(), _DT[scale_dtype],
            out_features if scale_len < 0 else scale_len, _ptr(bias_tab), _DT[bias_dtype], y_tab.data_ptr(), G,
            out_features, in_features, _stream(x_tab)))


def ternary_gemm_int8_grouped(q_tab: Tensor, sx_tab: Tensor, w_tiled_tab: Tensor, scale_tab: Tensor,
                              bias_tab: Optional[Tensor], y_tab: Tensor, rows: int, in_features: int, out_features: int,
                              scale_len: int = -1, scale_dtype: torch.dtype = torch.float32,
                              bias_dtype: torch.dtype = torch.float32, out_dtype: torch.dtype = torch.bfloat16,
                              q_operand_order: bool = False, acc_tab: Optional[Tensor] = None) -> None:
    """``G`` independent int8 units of ``rows`` (at most 16) activation rows each in one launch: unit ``u`` multiplies
    the int8 rows at ``q_tab[u]`` (row scales at ``sx_tab[u]``) with the decode-tiled weights at ``w_tiled_tab[u]``
    into ``y_tab[u]`` ``[rows, N]``, exactly as :func:`ternary_gemm_int8_tiled` would (same accumulators, same bits).
    The tables are int64 device tensors of ``G`` device addresses (:func:`pointer_table`); ``acc_tab`` optionally
    receives the int32 accumulators; nothing is allocated or returned."""
    G = q_tab.numel()
    tabs = (q_tab, sx_tab, w_tiled_tab, scale_tab, y_tab) + tuple(t for t in (bias_tab, acc_tab) if t is not None)
    for t in tabs:
        _check(t.dtype == torch.int64 and t.dim() == 1 and t.numel() == G and t.is_contiguous(),
               "pointer tables must be contiguous int64 tensors of one length")
    _check(_all_cuda(*tabs), "All tensors must be CUDA")
    _check(scale_dtype in _DT and bias_dtype in _DT and out_dtype in _DT,
           "scale / bias / output dtype must be float32, float16 or bfloat16")
    with torch.cuda.device(q_tab.device):
        _status(_L.bt_ternary_gemm_i8_grouped(
            q_tab.data_ptr(), 1 if q_operand_order else 0, sx_tab.data_ptr(), w_tiled_tab.data_ptr(), scale_tab.data_ptr(),
            _DT[scale_dtype], out_features if scale_len < 0 else scale_len, _ptr(bias_tab), _DT[bias_dtype],
            y_tab.data_ptr(), _DT[out_dtype], _ptr(acc_tab), G, rows, out_features, in_features, _stream(q_tab)))


def retile_fields(W_tiled: Tensor, in_features: int, out_features: int) -> Tensor:
    """The prefill-only field layout of a decode-tiled copy (same size; natural or pair-ordered tiles are kept in
    their order): what :func:`ternary_gemm_int8_fields` reads."""
    _tiled_checks(W_tiled, out_features, in_features)
    _check(W_tiled.is_cuda, "All tensors must be CUDA")
    with torch.cuda.device(W_tiled.device):
        out = torch.empty_like(W_tiled)
        _status(_L.bt_retile_fields(W_tiled.data_ptr(), out_features, in_features, out.data_ptr(), _stream(W_tiled)))
    return out


def ternary_gemm_int8_fields(Q: Tensor, s_x: Tensor, q_rowsum: Tensor, W_fields: Tensor, scale: Tensor,
                             bias: Optional[Tensor] = None, in_features: int = -1, out_features: int = -1,
                             out_dtype: torch.dtype = torch.float32, return_acc: bool = False,
                             residual: Optional[Tensor] = None, q_operand_order: bool = False,
                             natural_from_pairs: bool = False):
    """:func:`ternary_gemm_int8_tiled` on the field layout (:func:`retile_fields`) with the rows' sums of ``Q``
    (``act_quant_int8(..., return_rowsum=True)``): the same results bit for bit through a cheaper weight decode.
    Always the tiled matrix-core GEMM (prefill batches); ``in_features`` a multiple of 128."""
    _check(Q.dim() == 2 and Q.dtype == torch.int8 and Q.numel() > 0, "Q must be 2D int8")
    K, N = Q.shape[-1], out_features
    _check(K == in_features, "input K doesn't match in_features")
    _tiled_checks(W_fields, N, K)
    _check(scale.dim() == 1 and scale.shape[0] in (N, 1), "scale size doesn't match N")
    _check(bias is None or (bias.dim() == 1 and bias.shape[0] == N), "bias shape mismatch")
    _check(s_x.dtype == torch.float32 and s_x.numel() == Q.shape[0], "s_x must be fp32 [B]")
    _check(q_rowsum.dtype == torch.int32 and q_rowsum.numel() == Q.shape[0], "q_rowsum must be int32 [B]")
    _check(_all_cuda(Q, s_x, q_rowsum, W_fields, scale, bias), "All tensors must be CUDA")
    _check(out_dtype in _DT, "out_dtype must be float32, float16 or bfloat16")
    q = Q.contiguous()
    s_x = s_x.contiguous()
    q_rowsum = q_rowsum.contiguous()
    scale = _prep_vec(scale, s_x)
    bias = None if bias is None else _prep_vec(bias, s_x)
    B = q.shape[0]
    y = torch.empty((B, N), dtype=out_dtype, device=q.device)
    acc = torch.empty((B, N), dtype=torch.int32, device=q.device) if return_acc else None
    res = None if residual is None else _residual_2d(residual, y, (B,), N)
    with torch.cuda.device(q.device):
        _status(_L.bt_ternary_gemm_i8_fields(
            q.data_ptr(), 1 if q_operand_order else 0, s_x.data_ptr(), q_rowsum.data_ptr(), W_fields.data_ptr(),
            1 if natural_from_pairs else 0, scale.data_ptr(), _dt(scale, "scale"), scale.numel(), _ptr(bias),
            0 if bias is None else _dt(bias, "bias"), _ptr(res), y.data_ptr(), _DT[out_dtype], _ptr(acc), B, N, K,
            _stream(q)))
    return (y, acc) if return_acc else y


def ternary_gemm_int8_tiled(Q: Tensor, s_x: Tensor, W_tiled: Tensor, scale: Tensor, bias: Optional[Tensor] = None,
                            in_features: int = -1, out_features: int = -1,
                            out_dtype: torch.dtype = torch.float32, return_acc: bool = False,
                            residual: Optional[Tensor] = None, q_operand_order: bool = False):
    """:func:`ternary_gemm_int8` on the decode-tiled copy of the weights (same results bit for bit)."""
    _check(Q.dim() == 2 and Q.dtype == torch.int8 and Q.numel() > 0, "Q must be 2D int8")
    K, N = Q.shape[-1], out_features
    _check(K == in_features, "input K doesn't match in_features")
    _tiled_checks(W_tiled, N, K)
    _check(scale.dim() == 1 and scale.shape[0] in (N, 1), "scale size doesn't match N")
    _check(bias is None or (bias.dim() == 1 and bias.shape[0] == N), "bias shape mismatch")
    _check(s_x.dtype == torch.float32 and s_x.numel() == Q.shape[0], "s_x must be fp32 [B]")
    _check(_all_cuda(Q, s_x, W_tiled, scale, bias), "All tensors must be CUDA")
    _check(out_dtype in _DT, "out_dtype must be float32, float16 or bfloat16")
    q = Q.contiguous()
    s_x = s_x.contiguous()
    scale = _prep_vec(scale, s_x)
    bias = None if bias is None else _prep_vec(bias, s_x)
    B = q.shape[0]
    y = torch.empty((B, N), dtype=out_dtype, device=q.device)
    acc = torch.empty((B, N), dtype=torch.int32, device=q.device) if return_acc else None
    res = None if residual is None else _residual_2d(residual, y, (B,), N)
    with torch.cuda.device(q.device):
        _status(_L.bt_ternary_gemm_i8_tiled(
            q.data_ptr(), 1 if q_operand_order else 0, s_x.data_ptr(), W_tiled.data_ptr(), scale.data_ptr(),
            _dt(scale, "scale"), scale.numel(), _ptr(bias), 0 if bias is None else _dt(bias, "bias"), _ptr(res),
            y.data_ptr(), _DT[out_dtype], _ptr(acc), B, N, K, _stream(q)))
    return (y, acc) if return_acc else y


def ternary_linear_tensor_core_forward(X: Tensor, W_T: Tensor, scale: Tensor,
                                       bias: Optional[Tensor] = None, in_features: int = -1,
                                       version: int = 1) -> Tensor:
    """Matrix-core forward; ``X`` must be 2-D as in the reference.

    version 1: float compute (the reference's validation kernel,
    ``ternary_gemm_tensor_core.cu:120-271``) -- served by the fp32-accumulate
    packed kernel.  version 2: per-row int8 activations, int8 MFMA, int32
    accumulators (``:349-657`` with the whole-row activation scale).
    """
    _check(X.dim() == 2, "X must be 2D")
    _check(version in (1, 2), "version must be 1 (V1 float) or 2 (V2 mma.sync)")
    if in_features < 0:
        in_features = X.shape[-1]
    K, N = _packed_checks(X, W_T, scale, bias, in_features)
    if version == 1:
        return ternary_linear_packed_forward(X, W_T, scale, bias, in_features)
    _check(X.dtype in _DT, "X must be float32, float16 or bfloat16 for version 2")
    x2 = X.contiguous()
    W_T = W_T.contiguous()
    scale = _prep_vec(scale, x2)
    bias = None if bias is None else _prep_vec(bias, x2)
    B = x2.shape[0]
    y = torch.empty((B, N), dtype=X.dtype, device=X.device)
    with torch.cuda.device(X.device):
        ws_bytes = _L.bt_tensor_core_workspace_bytes(B, N, K)
        ws = _workspace(ws_bytes, X.device)
        _status(_L.bt_ternary_linear_tensor_core_forward(
            x2.data_ptr(), _dt(x2, "X"), W_T.data_ptr(), scale.data_ptr(), _dt(scale, "scale"),
            scale.numel(), _ptr(bias), 0 if bias is None else _dt(bias, "bias"), y.data_ptr(),
            B, N, K, _ptr(ws), 0 if ws is None else ws.numel(), _stream(X)))
    return y


# ---- additive entry points (no counterpart in the reference module) ----------------------


def ternary_quantize_pack(weight: Tensor, threshold_factor: float = 0.05, per_channel: bool = True,
                          want_packed: bool = True, want_tern: bool = False
                          ) -> Tuple[Optional[Tensor], Tensor, Optional[Tensor]]:
    """Fused quantize + pack of master weights ``[N, K]`` on the GPU.

    Returns ``(packed_T uint8 [ceil(K/4), N] | None, scale, w_tern int8 [N, K] | None)``;
    ``scale`` has the weight dtype and shape ``(N,)`` (per channel) or ``()`` (per tensor),
    exactly what ``quant.ternary_quantize`` returns.
    """
    _check(weight.dim() == 2, "weight must be 2D [N, K]")
    _check(weight.is_cuda, "All tensors must be CUDA")
    w = weight.detach().contiguous()
    N, K = w.shape
    _check(N > 0 and K > 0, "weight is empty")
    wdt = _dt(w, "weight")
    dev = w.device
    packed = torch.empty(((K + 3) // 4, N), dtype=torch.uint8, device=dev) if want_packed else None
    tern = torch.empty((N, K), dtype=torch.int8, device=dev) if want_tern else None
    scale = torch.empty((N if per_channel else 1,), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _status(_L.bt_quantize_pack(w.data_ptr(), wdt, N, K, float(threshold_factor),
                                    int(bool(per_channel)), _ptr(packed), scale.data_ptr(),
                                    _ptr(tern), _stream(w)))
    scale = scale.to(weight.dtype)
    if not per_channel:
        scale = scale.squeeze(0)
    return packed, scale, tern


def act_quant_int8(X: Tensor, operand_order: bool = False, return_rowsum: bool = False):
    """Per-row int8 activation quantization: ``(Q int8 [B,K], s_x fp32 [B])``.

    ``operand_order=True`` (K % 16 == 0) writes every 16-byte group of ``Q`` in the order the
    int8 GEMMs feed the matrix cores; such a ``Q`` must go to :func:`ternary_gemm_int8` with
    ``q_operand_order=True``.  ``return_rowsum=True`` adds the rows' sums of ``Q`` (int32 ``[B]``), which
    :func:`ternary_gemm_int8_fields` needs."""
    _check(X.dim() == 2 and X.numel() > 0, "X must be 2D and non-empty")
    _check(X.is_cuda, "All tensors must be CUDA")
    x = X.contiguous()
    B, K = x.shape
    q = torch.empty((B, K), dtype=torch.int8, device=x.device)
    s = torch.empty((B,), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        if return_rowsum:
            rs = torch.empty((B,), dtype=torch.int32, device=x.device)
            _status(_L.bt_act_quant_i8_rowsum(x.data_ptr(), _dt(x, "X"), B, K, q.data_ptr(), s.data_ptr(), rs.data_ptr(),
                                              1 if operand_order else 0, _stream(x)))
            return q, s, rs
        _status(_L.bt_act_quant_i8_layout(x.data_ptr(), _dt(x, "X"), B, K, q.data_ptr(), s.data_ptr(),
                                          1 if operand_order else 0, _stream(x)))
    return q, s


def ternary_gemm_int8(Q: Tensor, s_x: Tensor, W_T: Tensor, scale: Tensor,
                      bias: Optional[Tensor] = None, in_features: int = -1,
                      out_dtype: torch.dtype = torch.float32, return_acc: bool = False,
                      residual: Optional[Tensor] = None, q_operand_order: bool = False):
    """int8 activations x packed ternary weights; optionally also the int32 accumulators.
    ``residual`` ``[B, N]`` in ``out_dtype`` is added in the epilogue (``linear + residual``);
    ``q_operand_order`` says that ``Q`` was written with ``operand_order=True``."""
    _check(Q.dim() == 2 and Q.dtype == torch.int8, "Q must be 2D int8")
    if in_features < 0:
        in_features = Q.shape[-1]
    K, N = _packed_checks(Q, W_T, scale, bias, in_features)
    _check(s_x.dtype == torch.float32 and s_x.numel() == Q.shape[0], "s_x must be fp32 [B]")
    _check(_all_cuda(s_x), "All tensors must be CUDA")
    _check(out_dtype in _DT, "out_dtype must be float32, float16 or bfloat16")
    q = Q.contiguous()
    W_T = W_T.contiguous()
    s_x = s_x.contiguous()
    scale = _prep_vec(scale, s_x)
    bias = None if bias is None else _prep_vec(bias, s_x)
    B = q.shape[0]
    y = torch.empty((B, N), dtype=out_dtype, device=q.device)
    acc = torch.empty((B, N), dtype=torch.int32, device=q.device) if return_acc else None
    with torch.cuda.device(q.device):
        ws_bytes = _L.bt_gemm_i8_workspace_bytes(B, N, K)
        ws = _workspace(ws_bytes, q.device)
        if residual is None and not q_operand_order:
            _status(_L.bt_ternary_gemm_i8(
                q.data_ptr(), s_x.data_ptr(), W_T.data_ptr(), scale.data_ptr(), _dt(scale, "scale"),
                scale.numel(), _ptr(bias), 0 if bias is None else _dt(bias, "bias"), y.data_ptr(),
                _DT[out_dtype], _ptr(acc), B, N, K, _ptr(ws), 0 if ws is None else ws.numel(), _stream(q)))
        else:
            res = None if residual is None else _residual_2d(residual, y, (B,), N)
            _status(_L.bt_ternary_gemm_i8_res(
                q.data_ptr(), 1 if q_operand_order else 0, s_x.data_ptr(), W_T.data_ptr(), scale.data_ptr(),
                _dt(scale, "scale"), scale.numel(), _ptr(bias), 0 if bias is None else _dt(bias, "bias"), _ptr(res),
                y.data_ptr(), _DT[out_dtype], _ptr(acc), B, N, K, _stream(q)))
    return (y, acc) if return_acc else y


def _row_op_outputs(x2: Tensor, store: bool, quantize: bool):
    _check(store or quantize, "nothing to compute: store and quantize are both False")
    B, K = x2.shape
    h = torch.empty((B, K), dtype=x2.dtype, device=x2.device) if store else None
    q = torch.empty((B, K), dtype=torch.int8, device=x2.device) if quantize else None
    s = torch.empty((B,), dtype=torch.float32, device=x2.device) if quantize else None
    return h, q, s


def _row_op_result(h, q, s, lead_shape, K):
    if h is not None:
        h = h.reshape(*lead_shape, K)
    if q is None:
        return h
    return (q, s) if h is None else (h, q, s)


def _rows_2d(t: Tensor, K: int) -> Tensor:
    """A 2-D view with unit inner stride (row stride kept: slices of a wider matrix stay in place)."""
    if t.stride(-1) == 1 and t.dim() >= 2 and t.stride(-2) >= K:
        lead_ok = all(t.stride(i) == t.stride(i + 1) * t.shape[i + 1] for i in range(t.dim() - 2))
        if lead_ok:  # the leading dimensions collapse into one row index with a single stride
            rows = t.numel() // K
            return t if t.dim() == 2 else t.as_strided((rows, K), (t.stride(-2), 1), t.storage_offset())
    return t.contiguous().reshape(-1, K)


def swiglu(gate: Tensor, up: Tensor, store: bool = True, quantize: bool = False, operand_order: bool = False,
           return_rowsum: bool = False):
    """``silu(gate) * up`` in one pass, rounded as the two separate torch ops round it.

    Returns the product (``store``), or with ``quantize`` its per-row int8 form ``(Q, s_x)`` for
    :func:`ternary_gemm_int8` -- ``(h, Q, s_x)`` when both are asked for.  ``gate`` and ``up`` may
    be column slices of one wider matrix (the output of a fused gate/up projection).  ``return_rowsum`` (with
    ``quantize``) appends the rows' sums of ``Q`` (int32), which :func:`ternary_gemm_int8_fields` needs."""
    _check(gate.shape == up.shape and gate.dtype == up.dtype, "gate and up must match in shape and dtype")
    _check(gate.dim() >= 1 and gate.numel() > 0, "gate is empty")
    _check(gate.dtype in _DT, "gate must be float32, float16 or bfloat16")
    _check(_all_cuda(gate, up), "All tensors must be CUDA")
    K = gate.shape[-1]
    g2, u2 = _rows_2d(gate, K), _rows_2d(up, K)
    h, q, s = _row_op_outputs(g2, store, quantize)
    rs = None
    with torch.cuda.device(gate.device):
        if return_rowsum:
            _check(q is not None, "return_rowsum needs quantize=True")
            rs = torch.empty((g2.shape[0],), dtype=torch.int32, device=gate.device)
            _status(_L.bt_swiglu_rowsum(g2.data_ptr(), g2.stride(0), u2.data_ptr(), u2.stride(0), _dt(g2, "gate"),
                                        g2.shape[0], K, _ptr(h), _ptr(q), _ptr(s), rs.data_ptr(),
                                        1 if operand_order else 0, _stream(gate)))
        else:
            _status(_L.bt_swiglu(g2.data_ptr(), g2.stride(0), u2.data_ptr(), u2.stride(0), _dt(g2, "gate"),
                                 g2.shape[0], K, _ptr(h), _ptr(q), _ptr(s), 1 if operand_order else 0, _stream(gate)))
    if q is not None and gate.dim() != 2:
        q = q.reshape(*gate.shape[:-1], K)
        s = s.reshape(gate.shape[:-1])
    out = _row_op_result(h, q, s, gate.shape[:-1], K)
    return out if rs is None else (*out, rs.reshape(gate.shape[:-1]))


def rmsnorm(x: Tensor, weight: Optional[Tensor] = None, eps: float = 1e-6, store: bool = True,
            quantize: bool = False, operand_order: bool = False, return_rowsum: bool = False):
    """RMSNorm over the last dimension, ``(x * rsqrt(mean(x^2) + eps)) * weight``; with
    ``quantize`` also (or only, ``store=False``) the per-row int8 form of the result, and with ``return_rowsum``
    the rows' sums of that form appended (int32)."""
    _check(x.dim() >= 1 and x.numel() > 0, "x is empty")
    _check(x.dtype in _DT, "x must be float32, float16 or bfloat16")
    K = x.shape[-1]
    if weight is not None:
        _check(weight.dim() == 1 and weight.shape[0] == K, "weight must be 1D [K]")
        weight = weight.to(x.dtype).contiguous()
    _check(_all_cuda(x, weight), "All tensors must be CUDA")
    x2 = _rows_2d(x, K)
    h, q, s = _row_op_outputs(x2, store, quantize)
    rs = None
    with torch.cuda.device(x.device):
        if return_rowsum:
            _check(q is not None, "return_rowsum needs quantize=True")
            rs = torch.empty((x2.shape[0],), dtype=torch.int32, device=x.device)
            _status(_L.bt_rmsnorm_rowsum(x2.data_ptr(), x2.stride(0), _ptr(weight), float(eps), _dt(x2, "x"),
                                         x2.shape[0], K, _ptr(h), _ptr(q), _ptr(s), rs.data_ptr(),
                                         1 if operand_order else 0, _stream(x)))
        else:
            _status(_L.bt_rmsnorm(x2.data_ptr(), x2.stride(0), _ptr(weight), float(eps), _dt(x2, "x"),
                                  x2.shape[0], K, _ptr(h), _ptr(q), _ptr(s), 1 if operand_order else 0, _stream(x)))
    if q is not None and x.dim() != 2:
        q = q.reshape(*x.shape[:-1], K)
        s = s.reshape(x.shape[:-1])
    out = _row_op_result(h, q, s, x.shape[:-1], K)
    return out if rs is None else (*out, rs.reshape(x.shape[:-1]))


def unpack_dequant(W_T: Tensor, in_features: int, scale: Optional[Tensor] = None,
                   out_dtype: torch.dtype = torch.float32) -> Tensor:
    """Dense ``[N, K]`` weights from packed ``W_T``: ``decode * scale[:, None]``
    (``out_dtype`` float) or the plain ternary values (``out_dtype=torch.int8``)."""
    _check(W_T.dim() == 2 and W_T.dtype == torch.uint8, "W_T must be 2D uint8")
    _check(W_T.shape[0] == (in_features + 3) // 4, "K_bytes doesn't match ceil(K/4)")
    _check(_all_cuda(W_T, scale), "All tensors must be CUDA")
    W_T = W_T.contiguous()
    N = W_T.shape[1]
    if out_dtype == torch.int8:
        odt, scale_f = _INT8_OUT, None
    else:
        _check(out_dtype in _DT, "out_dtype must be float32, float16, bfloat16 or int8")
        odt = _DT[out_dtype]
        scale_f = None if scale is None else scale.reshape(-1).to(torch.float32).contiguous()
        if scale_f is not None:
            _check(scale_f.numel() in (N, 1), "scale size doesn't match N")
    out = torch.empty((N, in_features), dtype=out_dtype, device=W_T.device)
    with torch.cuda.device(W_T.device):
        _status(_L.bt_unpack_dequant(W_T.data_ptr(), _ptr(scale_f),
                                     0 if scale_f is None else scale_f.numel(), out.data_ptr(), odt,
                                     N, in_features, _stream(W_T)))
    return out
