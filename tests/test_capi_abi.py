"""The C-ABI library loads without a GPU and exports every symbol the header declares;
argument validation fails cleanly (status + message) before any kernel launch."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "bittorch_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bt_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    syms = _declared_symbols()
    for name in ("bt_quantize_pack", "bt_ternary_linear_forward", "bt_ternary_linear_packed_forward",
                 "bt_act_quant_i8", "bt_ternary_gemm_i8", "bt_ternary_linear_tensor_core_forward",
                 "bt_unpack_dequant", "bt_pack_ternary_i8", "bt_ternary_gemv_grouped", "bt_ternary_linear_tensor_core_forward_static", "bt_last_error", "bt_abi_version",
                 "bt_ternary_linear_packed_forward_res", "bt_ternary_gemm_i8_res", "bt_tiled_weights_bytes",
                 "bt_retile_weights", "bt_untile_weights", "bt_ternary_linear_tiled_forward", "bt_ternary_gemm_i8_tiled", "bt_swiglu", "bt_rmsnorm",
                 "bt_act_quant_i8_layout", "bt_ternary_linear_packed_forward_fused",
                 "bt_packed_forward_fused_workspace_bytes", "bt_act_quant_i8_rowsum", "bt_retile_fields",
                 "bt_ternary_gemm_i8_fields", "bt_ternary_gemm_i8_grouped", "bt_set_option", "bt_swiglu_rowsum",
                 "bt_rmsnorm_rowsum"):
        assert name in syms


def test_library_exports_every_declared_symbol():
    from bittorch_amd import _lib
    lib = _lib.load()
    for name in _declared_symbols():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert set(_lib.SIGNATURES) == set(_declared_symbols())
    assert lib.bt_abi_version() == _lib.ABI_VERSION


def test_validation_errors_do_not_need_a_gpu():
    from bittorch_amd import _lib
    lib = _lib.load()
    # null pointers / empty shapes: rejected before any HIP call
    assert lib.bt_quantize_pack(None, 0, 4, 4, 0.05, 1, None, None, None, None) == -1
    assert "bt_quantize_pack" in _lib.last_error()
    assert lib.bt_act_quant_i8(None, 0, 1, 1, None, None, None) == -1
    assert lib.bt_ternary_linear_packed_forward(None, 1, None, None, 0, 1, None, 0, None, 1, 1, 1,
                                                None, 0, None) == -1
    assert "null" in _lib.last_error()
    buf = ctypes.create_string_buffer(64)
    addr = ctypes.addressof(buf)
    # unsupported dtype tag
    assert lib.bt_quantize_pack(addr, 9, 1, 4, 0.05, 1, addr, addr, None, None) == -1
    assert "dtype" in _lib.last_error()
    # scale length that matches neither N nor 1
    assert lib.bt_ternary_linear_forward(addr, 0, addr, addr, 0, 3, None, 0, addr, 1, 8, 4, None) == -1
    assert "scale" in _lib.last_error()
    # K beyond the int32 accumulator bound of the int8 path
    assert lib.bt_ternary_gemm_i8(addr, addr, addr, addr, 0, 1, None, 0, addr, 0, None, 1, 16, 200000,
                                  None, 0, None) == -1
    assert "overflow" in _lib.last_error()
    # workspace sizes are plain arithmetic
    assert lib.bt_tensor_core_workspace_bytes(16, 4096, 4096) >= 16 * 4096 + 16 * 4
    assert lib.bt_tensor_core_workspace_bytes(0, 1, 1) == 0


def test_extension_probes_are_truthful():
    import bittorch_amd as bt
    from bittorch_amd.nn.ternary_linear import _cuda_kernel_available
    import torch
    assert bt.has_cuda_ext() is True
    assert _cuda_kernel_available() is True
    assert bt.ops.has_packed_cuda_support() == torch.cuda.is_available()
    from bittorch_amd import _C
    for name in ("dummy", "ternary_linear_forward", "ternary_linear_packed_forward",
                 "ternary_linear_tensor_core_forward", "ternary_quantize_pack"):
        assert hasattr(_C, name)
    x = torch.arange(6.0).reshape(2, 3)
    y = _C.dummy(x)
    assert torch.equal(x, y) and y.data_ptr() != x.data_ptr()


def test_gpu_entry_points_reject_cpu_tensors():
    import torch
    from bittorch_amd import _C
    x = torch.randn(2, 8)
    with pytest.raises(RuntimeError, match="CUDA"):
        _C.ternary_linear_forward(x, torch.zeros(4, 8, dtype=torch.int8), torch.ones(4))
    with pytest.raises(RuntimeError, match="CUDA"):
        _C.ternary_linear_packed_forward(x, torch.zeros(2, 4, dtype=torch.uint8), torch.ones(4), None, 8)
    with pytest.raises(RuntimeError, match="W_T must be uint8"):
        _C.ternary_linear_packed_forward(x, torch.zeros(2, 4, dtype=torch.int8), torch.ones(4), None, 8)
    with pytest.raises(RuntimeError, match=r"K_bytes doesn't match ceil\(K/4\)"):
        _C.ternary_linear_packed_forward(x, torch.zeros(3, 4, dtype=torch.uint8), torch.ones(4), None, 8)
    with pytest.raises(RuntimeError, match="input K doesn't match in_features"):
        _C.ternary_linear_packed_forward(x, torch.zeros(2, 4, dtype=torch.uint8), torch.ones(4), None, 7)
    with pytest.raises(RuntimeError, match="scale size doesn't match N"):
        _C.ternary_linear_packed_forward(x, torch.zeros(2, 4, dtype=torch.uint8), torch.ones(3), None, 8)
    with pytest.raises(RuntimeError, match="W_tern must be int8"):
        _C.ternary_linear_forward(x, torch.zeros(4, 8), torch.ones(4))
    with pytest.raises(RuntimeError, match="version must be"):
        _C.ternary_linear_tensor_core_forward(x, torch.zeros(2, 4, dtype=torch.uint8), torch.ones(4), None, 8, 3)


def test_tiled_copy_size_and_argument_checks_without_a_gpu():
    """Host-side arithmetic and validation of the tiled-weight entry points (no kernel is launched)."""
    from bittorch_amd import _lib
    import numpy as np
    from oracle import oracle as o
    lib = _lib.load()
    for (n, k) in [(4096, 4096), (37, 100), (1, 1), (250, 1030), (11008, 512)]:
        kb = (k + 3) // 4
        expect = ((n + 15) // 16) * ((kb + 15) // 16) * 256
        assert lib.bt_tiled_weights_bytes(n, k) == expect
        # the oracle's restatement of the layout has exactly that many bytes
        assert o.retile_weights(np.zeros((kb, n), dtype=np.uint8), k).size == expect
    assert lib.bt_tiled_weights_bytes(0, 4) == 0
    buf = ctypes.create_string_buffer(1024)
    addr = (ctypes.addressof(buf) + 255) & ~255
    assert lib.bt_retile_weights(None, 16, 64, 0, addr, None) == -1
    assert "bt_retile_weights" in _lib.last_error()
    assert lib.bt_retile_weights(addr, 16, 64, 0, addr + 4, None) == -1      # tiled copy not 256-byte aligned
    assert "aligned" in _lib.last_error()
    assert lib.bt_retile_weights(addr, 48, 64, 1, addr, None) == -1          # pair order needs N % 32 == 0
    assert "N % 32" in _lib.last_error()
    assert lib.bt_retile_weights(addr, 16, 64, 7, addr, None) == -1          # unknown tile order
    # the prefill-only field layout: null row sums, K outside whole 128-wide stages, a misaligned copy
    assert lib.bt_act_quant_i8_rowsum(addr, 0, 1, 16, addr, addr, None, 0, None) == -1
    assert "bt_act_quant_i8_rowsum" in _lib.last_error()
    assert lib.bt_retile_fields(addr, 16, 64, addr + 4, None) == -1
    assert "aligned" in _lib.last_error()
    assert lib.bt_ternary_gemm_i8_fields(addr, 0, addr, None, addr, 0, addr, 0, 1, None, 0, None, addr, 0, None, 4, 16, 128,
                                         None) == -1
    assert "q_rowsum" in _lib.last_error()
    assert lib.bt_ternary_gemm_i8_fields(addr, 0, addr, addr, addr, 0, addr, 0, 1, None, 0, None, addr, 0, None, 4, 16, 192,
                                         None) == -1
    assert "multiple of 128" in _lib.last_error()
    # the fused quantizers' row-sum variants need both the codes and the sums
    assert lib.bt_swiglu_rowsum(addr, 16, addr, 16, 1, 1, 16, None, addr, addr, None, 0, None) == -1
    assert "bt_swiglu_rowsum" in _lib.last_error() and "q_rowsum" in _lib.last_error()
    assert lib.bt_rmsnorm_rowsum(addr, 16, None, 1e-5, 1, 1, 16, None, None, addr, addr, 0, None) == -1
    assert "bt_rmsnorm_rowsum" in _lib.last_error()


def test_set_option_validates_names_and_lengths():
    """bt_set_option is host-only: known names (with or without the BITTORCH_ prefix) are accepted, set and un-set;
    an unknown name or an over-long value is an error with a message."""
    from bittorch_amd import _lib
    lib = _lib.load()
    try:
        assert lib.bt_set_option(b"STREAM_MAX_ROWS", b"32") == 0
        assert lib.bt_set_option(b"BITTORCH_GROUP_WALK", b"chunk") == 0
        assert lib.bt_set_option(b"GROUP_WALK", None) == 0
        assert lib.bt_set_option(b"NO_SUCH_OPTION", b"1") == -1
        assert "unknown option" in _lib.last_error()
        assert lib.bt_set_option(b"STREAM_CFG", b"x" * 100) == -1
        assert "longer" in _lib.last_error()
        with pytest.raises(ValueError):
            _lib.set_option("KERNEL", "generic")  # read from the environment on every call, not an option
    finally:
        assert lib.bt_set_option(None, None) == 0
