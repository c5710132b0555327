"""ctypes binding of ``_hip/libbittorch_hip.so`` (declared in ``include/bittorch_hip.h``).

Importing this module never fails; :func:`load` raises ``ImportError`` when the
shared library has not been built, which is what makes ``bittorch_amd._C``
unimportable (and ``has_cuda_ext()`` false) on such a machine.
"""

from __future__ import annotations

import ctypes
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
# BITTORCH_HIP_LIBRARY points at another build of the library (A/B comparisons)
LIB_PATH = os.environ.get("BITTORCH_HIP_LIBRARY") or os.path.join(_HERE, "_hip", "libbittorch_hip.so")

ABI_VERSION = 2

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_sz = ctypes.c_size_t

# name -> (restype, argtypes); one entry per symbol the header declares
SIGNATURES = {
    "bt_abi_version": (_int, []),
    "bt_last_error": (ctypes.c_char_p, []),
    "bt_set_option": (_int, [ctypes.c_char_p, ctypes.c_char_p]),
    "bt_quantize_pack": (_int, [_vp, _int, _i64, _i64, ctypes.c_double, _int, _vp, _vp, _vp, _vp]),
    "bt_ternary_linear_forward": (_int, [_vp, _int, _vp, _vp, _int, _i64, _vp, _int, _vp, _i64, _i64,
                                         _i64, _vp]),
    "bt_packed_forward_workspace_bytes": (_sz, [_i64, _i64, _i64, _int]),
    "bt_ternary_linear_packed_forward": (_int, [_vp, _int, _vp, _vp, _int, _i64, _vp, _int, _vp, _i64,
                                                _i64, _i64, _vp, _sz, _vp]),
    "bt_act_quant_i8": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _vp]),
    "bt_gemm_i8_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "bt_ternary_gemm_i8": (_int, [_vp, _vp, _vp, _vp, _int, _i64, _vp, _int, _vp, _int, _vp, _i64,
                                  _i64, _i64, _vp, _sz, _vp]),
    "bt_tensor_core_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "bt_ternary_linear_tensor_core_forward": (_int, [_vp, _int, _vp, _vp, _int, _i64, _vp, _int, _vp,
                                                     _i64, _i64, _i64, _vp, _sz, _vp]),
    "bt_ternary_linear_tensor_core_forward_static": (_int, [_vp, _int, _vp, _vp, _int, _i64, _vp, _int, _vp,
                                                            _i64, _i64, _i64, _vp]),
    "bt_ternary_gemv_grouped": (_int, [_vp, _int, _vp, _vp, _int, _i64, _vp, _int, _vp, _i64, _i64, _i64, _vp]),
    "bt_ternary_gemm_i8_grouped": (_int, [_vp, _int, _vp, _vp, _vp, _int, _i64, _vp, _int, _vp, _int, _vp, _i64, _i64,
                                          _i64, _i64, _vp]),
    "bt_unpack_dequant": (_int, [_vp, _vp, _i64, _vp, _int, _i64, _i64, _vp]),
    "bt_pack_ternary_i8": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "bt_ternary_linear_packed_forward_res": (_int, [_vp, _int, _vp, _vp, _int, _i64, _vp, _int, _vp, _vp,
                                                    _i64, _i64, _i64, _vp, _sz, _vp]),
    "bt_ternary_gemm_i8_res": (_int, [_vp, _int, _vp, _vp, _vp, _int, _i64, _vp, _int, _vp, _vp, _int, _vp,
                                      _i64, _i64, _i64, _vp]),
    "bt_swiglu": (_int, [_vp, _i64, _vp, _i64, _int, _i64, _i64, _vp, _vp, _vp, _int, _vp]),
    "bt_rmsnorm": (_int, [_vp, _i64, _vp, ctypes.c_float, _int, _i64, _i64, _vp, _vp, _vp, _int, _vp]),
    "bt_act_quant_i8_layout": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _int, _vp]),
    "bt_packed_forward_fused_workspace_bytes": (_sz, [_i64, _i64, _i64, _int]),
    "bt_ternary_linear_packed_forward_fused": (_int, [_vp, _i64, _int, _int, _vp, _i64, ctypes.c_float, _vp, _vp, _int,
                                                      _i64, _vp, _int, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp]),
    "bt_tiled_weights_bytes": (_sz, [_i64, _i64]),
    "bt_retile_weights": (_int, [_vp, _i64, _i64, _int, _vp, _vp]),
    "bt_untile_weights": (_int, [_vp, _i64, _i64, _int, _vp, _vp]),
    "bt_ternary_linear_tiled_forward": (_int, [_vp, _i64, _int, _int, _vp, _i64, ctypes.c_float, _vp, _vp, _int,
                                               _i64, _vp, _int, _vp, _int, _vp, _i64, _i64, _i64, _vp, _sz, _vp]),
    "bt_ternary_gemm_i8_tiled": (_int, [_vp, _int, _vp, _vp, _vp, _int, _i64, _vp, _int, _vp, _vp, _int, _vp,
                                        _i64, _i64, _i64, _vp]),
    "bt_act_quant_i8_rowsum": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _vp, _int, _vp]),
    "bt_swiglu_rowsum": (_int, [_vp, _i64, _vp, _i64, _int, _i64, _i64, _vp, _vp, _vp, _vp, _int, _vp]),
    "bt_rmsnorm_rowsum": (_int, [_vp, _i64, _vp, ctypes.c_float, _int, _i64, _i64, _vp, _vp, _vp, _vp, _int, _vp]),
    "bt_retile_fields": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "bt_ternary_gemm_i8_fields": (_int, [_vp, _int, _vp, _vp, _vp, _int, _vp, _int, _i64, _vp, _int, _vp, _vp, _int, _vp,
                                         _i64, _i64, _i64, _vp]),
}

_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """The loaded library with prototypes set; ``ImportError`` if it is absent or stale."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m bittorch_amd.build` "
            "(needs hipcc; cross-compiles for gfx950 without a GPU)")
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as exc:  # e.g. libamdhip64 not found
        raise ImportError(f"cannot load {LIB_PATH}: {exc}") from exc
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise ImportError(f"{LIB_PATH} does not export {name}; rebuild it") from exc
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.bt_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has ABI {lib.bt_abi_version()}, expected {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


def last_error() -> str:
    return load().bt_last_error().decode("utf-8", "replace")


def set_option(name: Optional[str], value: Optional[str] = None) -> None:
    """Overrides one of the library's run-time options (``bt_set_option``): ``STREAM_MAX_ROWS``, ``GROUP_WALK`` ...;
    ``value=None`` un-sets it, ``name=None`` un-sets all of them.  The environment variable ``BITTORCH_<NAME>`` gives
    an option its initial value, read once per process."""
    rc = load().bt_set_option(None if name is None else name.encode(), None if value is None else str(value).encode())
    if rc != 0:
        raise ValueError(last_error())
