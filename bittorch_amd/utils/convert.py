"""Model conversion, accounting and checkpoints for packed ternary layers.

API mirror of ``bittorch/utils/convert.py:19-246`` (same names, arguments and result
dictionaries).  Two things differ on purpose:
  * layers whose weights live on the GPU are converted by the fused quantize+pack kernel
    (one read of the master weights) instead of the quantize -> pack -> transpose chain of
    torch ops; the bytes and scales are the same bit for bit;
  * ``load_ternary_checkpoint`` reads with ``weights_only=True`` (a checkpoint is tensors plus
    a plain metadata dictionary; nothing in it needs unpickling of code).
"""

from __future__ import annotations

import copy
from typing import Any, Dict, Optional

import torch
import torch.nn as nn

from ..nn.ternary_linear import TernaryLinear
from ..nn.ternary_linear_infer import TernaryLinearInference, create_ternary_linear_inference
from ..quant.ternary import ternary_quantize


def fp_linear_to_ternary_infer(linear: nn.Linear, threshold_factor: float = 0.05) -> TernaryLinearInference:
    """``nn.Linear`` -> ``TernaryLinearInference`` (reference ``:19-49``): per-channel absmax
    quantization of the weights, packed transposed storage, bias kept as it is."""
    bias = linear.bias.data if linear.bias is not None else None
    return create_ternary_linear_inference(linear.in_features, linear.out_features, linear.weight.data, bias,
                                           threshold_factor)


def ternary_linear_to_infer(ternary_linear: TernaryLinear) -> TernaryLinearInference:
    """Trained ``TernaryLinear`` -> ``TernaryLinearInference`` with the weights the training
    module's forward uses (reference ``:52-73``: its threshold factor and scale granularity)."""
    bias = ternary_linear.bias.data if ternary_linear.bias is not None else None
    weight = ternary_linear.weight.data
    if weight.is_cuda and weight.dtype in (torch.float32, torch.float16, torch.bfloat16):
        from ..nn.ternary_linear import _cuda_kernel_available
        if _cuda_kernel_available():
            from .. import _C
            packed, scale, _ = _C.ternary_quantize_pack(weight, ternary_linear.threshold_factor,
                                                        ternary_linear.per_channel)
            scale = scale.reshape(-1).expand(ternary_linear.out_features).contiguous()
            return TernaryLinearInference(ternary_linear.in_features, ternary_linear.out_features, packed, scale,
                                          bias)
    w_tern, scale = ternary_linear.get_quantized_weight()
    scale = scale.reshape(-1).expand(ternary_linear.out_features).contiguous()
    return TernaryLinearInference.from_unpacked(w_tern, scale, bias)


def convert_linear_layers(module: nn.Module, threshold_factor: float = 0.05, skip_names: Optional[list] = None,
                          inplace: bool = False) -> nn.Module:
    """Replace every ``nn.Linear`` / ``TernaryLinear`` in the tree by a ``TernaryLinearInference``
    (reference ``:76-133``).  A child is skipped when any entry of ``skip_names`` is a substring of
    its dotted name; skipped and other modules are searched further down."""
    skip_names = skip_names or []
    if not inplace:
        module = copy.deepcopy(module)

    def skipped(name: str) -> bool:
        return any(pattern in name for pattern in skip_names)

    def walk(parent: nn.Module, prefix: str) -> None:
        for name, child in list(parent.named_children()):
            full = f"{prefix}.{name}" if prefix else name
            if isinstance(child, nn.Linear) and not skipped(full):
                setattr(parent, name, fp_linear_to_ternary_infer(child, threshold_factor))
            elif isinstance(child, TernaryLinear) and not skipped(full):
                setattr(parent, name, ternary_linear_to_infer(child))
            else:
                walk(child, full)

    walk(module, "")
    return module


def fuse_ternary_linear_inference(*layers: TernaryLinearInference) -> TernaryLinearInference:
    """One inference layer computing ``concat([l(x) for l in layers], dim=-1)``.

    Packed weights are laid out ``[ceil(K/4), N]``, so layers that share their input (q/k/v, or
    gate/up: the reference's JS runtime stores ``kv_proj`` fused the same way,
    ``js/src/models/TernaryTransformer.ts:141-188``) concatenate along the column axis; every
    output column keeps its own weights, scale and bias, so each slice of the result equals the
    separate layer's output bit for bit, while one launch covers all the columns (fewer, fuller
    waves of tiles on the 256 compute units)."""
    if not layers:
        raise ValueError("no layers to fuse")
    k = layers[0].in_features
    if any(l.in_features != k for l in layers):
        raise ValueError("layers must share in_features")
    if any((l.bias is None) != (layers[0].bias is None) for l in layers):
        raise ValueError("either all layers have a bias or none")
    packed = torch.cat([l.packed_weights() for l in layers], dim=1).contiguous()
    scale = torch.cat([l.scale.reshape(-1).expand(l.out_features) if l.scale.numel() == 1 else l.scale
                       for l in layers]).contiguous()
    bias = None if layers[0].bias is None else torch.cat([l.bias for l in layers]).contiguous()
    return TernaryLinearInference(k, sum(l.out_features for l in layers), packed, scale, bias)


def prepare_decode(module: nn.Module) -> nn.Module:
    """Build the decode-tiled weight copy of every ``TernaryLinearInference`` inside ``module`` now
    (they are otherwise built on each layer's first decode-shape call, and never during a HIP graph
    capture, which falls back to ``weight_packed``); the row-major buffer of a layer is released as its copy is built."""
    for m in module.modules():
        if isinstance(m, TernaryLinearInference):
            m.prepare_decode()
    return module


def count_ternary_params(module: nn.Module) -> Dict[str, int]:
    """Weights by storage type (reference ``:136-166``): ``fp32``, ``fp16``, ``packed_ternary``, ``total``
    (biases and scales are not counted; any non-fp16 dense weight counts as fp32, as in the reference)."""
    counts = {"fp32": 0, "fp16": 0, "packed_ternary": 0, "total": 0}
    for child in module.modules():
        if isinstance(child, TernaryLinearInference):
            n = child.out_features * child.in_features
            counts["packed_ternary"] += n
        elif isinstance(child, (nn.Linear, TernaryLinear)):
            n = child.weight.numel()
            counts["fp16" if child.weight.dtype == torch.float16 else "fp32"] += n
        else:
            continue
        counts["total"] += n
    return counts


def get_model_memory_bytes(module: nn.Module) -> Dict[str, int]:
    """Bytes by storage type (reference ``:169-207``): ``fp32``, ``fp16``, ``packed_ternary``,
    ``scales``, ``total`` (the total also includes the biases)."""
    out = {"fp32": 0, "fp16": 0, "packed_ternary": 0, "scales": 0, "total": 0}
    for child in module.modules():
        if isinstance(child, TernaryLinearInference):
            packed = child.resident_weight_bytes()  # what the layer holds: one copy unless it keeps the row-major buffer too
            scales = child.scale.numel() * child.scale.element_size()
            out["packed_ternary"] += packed
            out["scales"] += scales
            out["total"] += packed + scales
        elif isinstance(child, (nn.Linear, TernaryLinear)):
            nbytes = child.weight.numel() * child.weight.element_size()
            out["fp16" if child.weight.dtype == torch.float16 else "fp32"] += nbytes
            out["total"] += nbytes
        else:
            continue
        if child.bias is not None:
            out["total"] += child.bias.numel() * child.bias.element_size()
    return out


def save_ternary_checkpoint(module: nn.Module, path: str, metadata: Optional[Dict[str, Any]] = None) -> None:
    """``{"state_dict": ..., "metadata": ...}`` written with ``torch.save`` (reference ``:210-228``).
    State-dict keys of a packed layer: ``weight_packed`` uint8 ``[ceil(K/4), N]``, ``scale``, ``bias``."""
    torch.save({"state_dict": module.state_dict(), "metadata": metadata or {}}, path)


def load_ternary_checkpoint(path: str, module: nn.Module) -> Dict[str, Any]:
    """Load such a checkpoint into a module of matching architecture and return its metadata
    (reference ``:231-246``)."""
    checkpoint = torch.load(path, map_location="cpu", weights_only=True)
    module.load_state_dict(checkpoint["state_dict"])
    return checkpoint.get("metadata", {})


def save_ternary_safetensors(module: nn.Module, path: str, metadata: Optional[Dict[str, str]] = None) -> None:
    """The same state dict as a safetensors file: ``<layer>.weight_packed`` U8
    ``[ceil(K/4), N]`` and ``<layer>.scale`` F32 ``[N]`` are the tensors the reference's browser
    runtime reads (``js/src/loaders/SafeTensorsLoader.ts:223-234``).  Metadata values must be strings."""
    from safetensors.torch import save_file

    tensors = {}
    for k, v in module.state_dict().items():
        t = v.detach().cpu().contiguous()
        if k.endswith(".scale") or k == "scale":
            t = t.float()
        tensors[k] = t
    save_file(tensors, path, metadata=metadata or {})


def load_ternary_safetensors(path: str, module: nn.Module) -> Dict[str, str]:
    """Load a safetensors state dict (scales are cast to the dtype the module holds)."""
    from safetensors import safe_open

    state = {}
    with safe_open(path, framework="pt", device="cpu") as fh:
        meta = fh.metadata() or {}
        for k in fh.keys():
            state[k] = fh.get_tensor(k)
    own = module.state_dict()
    for k, v in state.items():
        if k in own and own[k].dtype != v.dtype and v.is_floating_point():
            state[k] = v.to(own[k].dtype)
    module.load_state_dict(state)
    return dict(meta)


# ---- interchange with the reference's browser runtime ----------------------------------------
# Tensor names and shapes of js/src/models/TernaryTransformer.ts:141-188: per block i
#   blocks.{i}.norm1.weight, blocks.{i}.norm2.weight                        F32 [dim]
#   blocks.{i}.attn.{q_proj, kv_proj, proj}.{weight_packed, scale}          U8 [inBytes, outFeatures], F32 [outFeatures]
#   blocks.{i}.mlp.{w_gate, w_up, w_down}.{weight_packed, scale}
# with k and v fused along the output columns as kv_proj (its output is [k | v], :575-590), no biases, and
# tok.weight / head.weight / norm.weight for the embedding, the output head and the final norm (:124-135).
# The packed bytes are this library's ``weight_packed`` as they are (same codes, same [ceil(K/4), N] layout,
# js/src/loaders/SafeTensorsLoader.ts:223-234).
_JS_LAYERS = ("attn.q_proj", "attn.kv_proj", "attn.proj", "mlp.w_gate", "mlp.w_up", "mlp.w_down")
_JS_DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "gate", "up": "up", "down": "down",
                     "norm1": "n1", "norm2": "n2"}


def _as_infer(layer: nn.Module) -> TernaryLinearInference:
    if isinstance(layer, TernaryLinearInference):
        return layer
    if isinstance(layer, TernaryLinear):
        return ternary_linear_to_infer(layer)
    if isinstance(layer, nn.Linear):
        return fp_linear_to_ternary_infer(layer)
    raise TypeError(f"cannot export a {type(layer).__name__} as a ternary layer")


def export_js_safetensors(blocks, path: str, tok_embedding: Optional[torch.Tensor] = None,
                          head: Optional[torch.Tensor] = None, final_norm: Optional[torch.Tensor] = None,
                          metadata: Optional[Dict[str, str]] = None, names: Optional[Dict[str, str]] = None) -> None:
    """Write a stack of transformer blocks as the ``model.safetensors`` the reference's browser runtime loads.

    ``blocks``: a sequence of modules whose attributes ``names[...]`` (default ``q k v o gate up down n1 n2``) are
    the block's seven ternary layers (``TernaryLinearInference``, or ``TernaryLinear`` / ``nn.Linear``, which are
    quantized and packed on the way) and its two RMSNorm modules (or weight tensors).  A block that already holds
    ``qkv`` fused keeps its ``q``, ``k``, ``v`` attributes, which are what is read.  Layers must have no bias and an
    input width that is a multiple of 4 (the runtime derives it from the packed rows)."""
    from safetensors.torch import save_file

    names = {**_JS_DEFAULT_NAMES, **(names or {})}
    tensors: Dict[str, torch.Tensor] = {}

    def put_layer(key: str, layer: TernaryLinearInference) -> None:
        if layer.bias is not None:
            raise ValueError(f"{key}: the browser runtime's ternary layers have no bias")
        if layer.in_features % 4 != 0:
            raise ValueError(f"{key}: in_features must be a multiple of 4 (got {layer.in_features})")
        tensors[key + ".weight_packed"] = layer.packed_weights().detach().cpu().contiguous()
        scale = layer.scale.detach().reshape(-1)
        if scale.numel() == 1:
            scale = scale.expand(layer.out_features)
        tensors[key + ".scale"] = scale.float().cpu().contiguous()

    def norm_weight(obj) -> torch.Tensor:
        w = obj.weight if isinstance(obj, nn.Module) else obj
        return w.detach().float().cpu().contiguous()

    for i, blk in enumerate(blocks):
        get = (lambda n: blk[names[n]]) if isinstance(blk, dict) else (lambda n: getattr(blk, names[n]))
        prefix = f"blocks.{i}"
        tensors[f"{prefix}.norm1.weight"] = norm_weight(get("norm1"))
        tensors[f"{prefix}.norm2.weight"] = norm_weight(get("norm2"))
        q, k, v, o = (_as_infer(get(n)) for n in ("q", "k", "v", "o"))
        put_layer(f"{prefix}.attn.q_proj", q)
        put_layer(f"{prefix}.attn.kv_proj", fuse_ternary_linear_inference(k, v))
        put_layer(f"{prefix}.attn.proj", o)
        for js, own in (("w_gate", "gate"), ("w_up", "up"), ("w_down", "down")):
            put_layer(f"{prefix}.mlp.{js}", _as_infer(get(own)))
    for key, t in (("tok.weight", tok_embedding), ("head.weight", head), ("norm.weight", final_norm)):
        if t is not None:
            tensors[key] = norm_weight(t)
    save_file(tensors, path, metadata=metadata or {})


def load_js_safetensors(path: str, device=None):
    """Read such a file back: ``(blocks, extras, metadata)`` with ``blocks[i]`` a dict of the six
    ``TernaryLinearInference`` layers under the runtime's names (``attn.q_proj``, ``attn.kv_proj``, ``attn.proj``,
    ``mlp.w_gate``, ``mlp.w_up``, ``mlp.w_down``) plus ``norm1`` / ``norm2`` weight tensors, and ``extras`` the
    ``tok.weight`` / ``head.weight`` / ``norm.weight`` tensors that are present."""
    from safetensors import safe_open

    raw: Dict[str, torch.Tensor] = {}
    with safe_open(path, framework="pt", device="cpu") as fh:
        meta = dict(fh.metadata() or {})
        for key in fh.keys():
            raw[key] = fh.get_tensor(key)
    n_blocks = 1 + max((int(k.split(".")[1]) for k in raw if k.startswith("blocks.")), default=-1)
    blocks = []
    for i in range(n_blocks):
        prefix = f"blocks.{i}"
        blk = {"norm1": raw[f"{prefix}.norm1.weight"], "norm2": raw[f"{prefix}.norm2.weight"]}
        for name in _JS_LAYERS:
            packed, scale = raw[f"{prefix}.{name}.weight_packed"], raw[f"{prefix}.{name}.scale"]
            if packed.dtype != torch.uint8 or packed.dim() != 2 or scale.dim() != 1 or packed.shape[1] != scale.shape[0]:
                raise ValueError(f"{prefix}.{name}: expected U8 [inBytes, outFeatures] and F32 [outFeatures]")
            blk[name] = TernaryLinearInference(packed.shape[0] * 4, packed.shape[1], packed, scale.float())
        if device is not None:
            blk = {k: v.to(device) for k, v in blk.items()}
        blocks.append(blk)
    extras = {k: (v if device is None else v.to(device)) for k, v in raw.items() if not k.startswith("blocks.")}
    return blocks, extras, meta
