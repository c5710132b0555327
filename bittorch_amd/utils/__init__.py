"""Model conversion, accounting and checkpoint helpers (reference ``bittorch/utils/__init__.py``)."""

from .convert import (
    convert_linear_layers,
    count_ternary_params,
    export_js_safetensors,
    fp_linear_to_ternary_infer,
    fuse_ternary_linear_inference,
    get_model_memory_bytes,
    load_js_safetensors,
    load_ternary_checkpoint,
    load_ternary_safetensors,
    prepare_decode,
    save_ternary_checkpoint,
    save_ternary_safetensors,
    ternary_linear_to_infer,
)

__all__ = [
    "fp_linear_to_ternary_infer",
    "ternary_linear_to_infer",
    "convert_linear_layers",
    "fuse_ternary_linear_inference",
    "prepare_decode",
    "count_ternary_params",
    "get_model_memory_bytes",
    "save_ternary_checkpoint",
    "load_ternary_checkpoint",
    "save_ternary_safetensors",
    "load_ternary_safetensors",
    "export_js_safetensors",
    "load_js_safetensors",
]
