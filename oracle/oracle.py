"""numpy/ctypes front end of the C oracle in ``bt_oracle.c``.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the
benchmark's ``cpu_baseline`` leg, never by the shipped package.  Each wrapper
keeps the name of the reference function it restates; the reference lines are
cited in the C source.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libbt_oracle.so")

F32, F16, BF16 = 0, 1, 2

_i64 = ctypes.c_int64
_vp = ctypes.c_void_p


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a few hundred ms)."""
    src = os.path.join(_HERE, "bt_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE, "-B", "libbt_oracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.bto_round_to_dtype.restype = ctypes.c_float
        _lib.bto_round_to_dtype.argtypes = [ctypes.c_float, ctypes.c_int]
        _lib.bto_quantize.argtypes = [_vp, _i64, _i64, ctypes.c_double, ctypes.c_int,
                                      ctypes.c_int, _vp, _vp]
        for name in ("bto_pack", "bto_pack_transposed", "bto_unpack", "bto_unpack_transposed"):
            getattr(_lib, name).argtypes = [_vp, _i64, _i64, _vp]
        _lib.bto_linear_packed.argtypes = [_vp, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64]
        _lib.bto_linear_packed_f64.argtypes = [_vp, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64]
        _lib.bto_linear_packed_fused_epilogue.argtypes = [_vp, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64]
        _lib.bto_linear_packed_rowscaled_bf16.argtypes = [_vp, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64]
        _lib.bto_linear_packed_rowscaled_bf16.restype = ctypes.c_int
        _lib.bto_linear_unpacked.argtypes = [_vp, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64]
        _lib.bto_linear_packed_exact_f16.restype = ctypes.c_int
        _lib.bto_linear_packed_exact_f16.argtypes = [_vp, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64]
        _lib.bto_act_quant_i8.argtypes = [_vp, _i64, _i64, _vp, _vp]
        _lib.bto_gemm_i8.argtypes = [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64]
        _lib.bto_exp_fixed.restype = ctypes.c_float
        _lib.bto_exp_fixed.argtypes = [ctypes.c_float]
        _lib.bto_swiglu.argtypes = [_vp, _vp, ctypes.c_int, _i64, _i64, _vp, _vp, _vp]
        _lib.bto_rmsnorm.argtypes = [_vp, _vp, ctypes.c_float, ctypes.c_int, _i64, _i64, _vp, _vp, _vp]
    return _lib


def num_threads() -> int:
    """OpenMP threads the oracle's loops run on."""
    fn = lib().bto_num_threads
    fn.restype = ctypes.c_int
    return int(fn())


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(_vp)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def round_to_dtype(v: float, dtype: int) -> float:
    return float(lib().bto_round_to_dtype(float(v), dtype))


def ternary_quantize(weight, threshold_factor: float = 0.05, per_channel: bool = True,
                     dtype: int = F32) -> Tuple[np.ndarray, np.ndarray]:
    """(w_tern int8 [N,K], scale f32 [N] or [1]); ``weight`` already widened to f32."""
    w = _f32(weight)
    n, k = w.shape
    w_tern = np.empty((n, k), dtype=np.int8)
    scale = np.empty((n if per_channel else 1,), dtype=np.float32)
    lib().bto_quantize(_p(w), n, k, float(threshold_factor), int(per_channel), dtype,
                       _p(w_tern), _p(scale))
    return w_tern, scale


def _i8(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a).astype(np.int8))


def pack_ternary(w_tern) -> Tuple[np.ndarray, int]:
    w = _i8(w_tern)
    n, k = w.shape
    out = np.empty((n, (k + 3) // 4), dtype=np.uint8)
    lib().bto_pack(_p(w), n, k, _p(out))
    return out, k


def pack_ternary_transposed(w_tern) -> Tuple[np.ndarray, int]:
    w = _i8(w_tern)
    n, k = w.shape
    out = np.empty(((k + 3) // 4, n), dtype=np.uint8)
    lib().bto_pack_transposed(_p(w), n, k, _p(out))
    return out, k


def unpack_ternary(packed, in_features: int) -> np.ndarray:
    p = np.ascontiguousarray(np.asarray(packed, dtype=np.uint8))
    n = p.shape[0]
    assert p.shape[1] == (in_features + 3) // 4
    out = np.empty((n, in_features), dtype=np.int8)
    lib().bto_unpack(_p(p), n, in_features, _p(out))
    return out


def unpack_ternary_transposed(packed_t, in_features: int) -> np.ndarray:
    p = np.ascontiguousarray(np.asarray(packed_t, dtype=np.uint8))
    n = p.shape[1]
    assert p.shape[0] == (in_features + 3) // 4
    out = np.empty((n, in_features), dtype=np.int8)
    lib().bto_unpack_transposed(_p(p), n, in_features, _p(out))
    return out


def retile_weights(packed_t, in_features: int, gate_up_pairs: bool = False) -> np.ndarray:
    """Decode-tiled copy of ``W_T [Kb, N]`` (a layout of this library, no counterpart in the reference):
    zero-pad to whole 16-row steps and 16-column tiles, then order the bytes as
    ``[tile t][step s][row group g][column j][row r]`` with ``kb = 16 s + 4 g + r``, ``n = 16 t + j``.
    ``gate_up_pairs`` (N % 32 == 0): the tiles of the first and of the second column half alternate."""
    w = np.ascontiguousarray(packed_t, dtype=np.uint8)
    kb, n = w.shape
    assert kb == (in_features + 3) // 4
    steps, tiles = (kb + 15) // 16, (n + 15) // 16
    padded = np.zeros((steps * 16, tiles * 16), dtype=np.uint8)
    padded[:kb, :n] = w
    tiled = np.ascontiguousarray(padded.reshape(steps, 4, 4, tiles, 16).transpose(3, 0, 1, 4, 2))
    if gate_up_pairs:
        assert n % 32 == 0
        tiled = np.ascontiguousarray(tiled.reshape(2, tiles // 2, steps, 4, 16, 4).transpose(1, 0, 2, 3, 4, 5))
    return tiled.reshape(-1)


def retile_fields(tiled, out_features: int, in_features: int) -> np.ndarray:
    """Field layout of a decode-tiled copy (a layout of this library for its prefill GEMM, no counterpart in the
    reference).  Every aligned 16 bytes of the tiled copy are four dwords, one per column ``t`` of a column quad, with
    the 2-bit code of ``k = 4 b + c`` at bits ``8 b + 2 c``.  The field layout keeps the group's place and stores, at
    bits ``8 b + 2 t`` of dword ``c``, column ``t`` at ``k = 4 b + c``: as ``w + 1`` for ``t < 3`` (codes 0 / +1 / -1
    become 1 / 2 / 0) and as ``w`` in two's complement for ``t = 3`` (0 / 1 / 3)."""
    t8 = np.ascontiguousarray(tiled, dtype=np.uint8)
    assert t8.size % 16 == 0 and t8.size == ((out_features + 15) // 16) * (((in_features + 3) // 4 + 15) // 16) * 256
    grp = t8.reshape(-1, 4, 4)                                     # [group][column t][byte b]
    codes = np.stack([(grp >> (2 * c)) & 3 for c in range(4)], axis=-1)  # [group][t][b][c]
    remap_lo = np.array([1, 2, 0, 0], dtype=np.uint8)              # w + 1 (code 3 never occurs)
    remap_hi = np.array([0, 1, 3, 0], dtype=np.uint8)              # two's complement
    out = np.zeros((grp.shape[0], 4, 4), dtype=np.uint8)           # [group][dword c][byte b]
    for t in range(4):
        f = (remap_lo if t < 3 else remap_hi)[codes[:, t]]         # [group][b][c]
        out |= (f.transpose(0, 2, 1) << (2 * t)).astype(np.uint8)
    return out.reshape(-1)


def _lin_args(x, w, scale, bias):
    x = _f32(x)
    scale = _f32(scale).reshape(-1)
    bias = None if bias is None else _f32(bias).reshape(-1)
    return x, scale, bias


def linear_packed(x, w_packed_t, scale, in_features: int, bias=None, f64: bool = False,
                  fused_epilogue: bool = False) -> np.ndarray:
    """fp32-accumulate packed linear (or the float64 truth with ``f64=True``); ``fused_epilogue`` rounds
    ``acc * scale + bias`` once (a contracting compiler's reading of the reference's source line)."""
    x, scale, bias = _lin_args(x, w_packed_t, scale, bias)
    w = np.ascontiguousarray(np.asarray(w_packed_t, dtype=np.uint8))
    b, k = x.shape
    assert k == in_features and w.shape[0] == (k + 3) // 4
    n = w.shape[1]
    assert scale.size in (1, n)
    y = np.empty((b, n), dtype=np.float64 if f64 else np.float32)
    fn = lib().bto_linear_packed_f64 if f64 else (lib().bto_linear_packed_fused_epilogue if fused_epilogue else lib().bto_linear_packed)
    fn(_p(x), _p(w), _p(scale), scale.size, _p(bias), _p(y), b, n, k)
    return y


def linear_packed_exact_f16(x, w_packed_t, scale, in_features: int, bias=None) -> np.ndarray:
    """Packed linear for fp16 activations (given widened to float) with the dot product summed exactly and
    rounded to fp32 once; fp32 result before the cast to the output dtype."""
    x, scale, bias = _lin_args(x, w_packed_t, scale, bias)
    w = np.ascontiguousarray(np.asarray(w_packed_t, dtype=np.uint8))
    b, k = x.shape
    assert k == in_features and w.shape[0] == (k + 3) // 4
    n = w.shape[1]
    assert scale.size in (1, n)
    y = np.empty((b, n), dtype=np.float32)
    rc = lib().bto_linear_packed_exact_f16(_p(x), _p(w), _p(scale), scale.size, _p(bias), _p(y), b, n, k)
    if rc != 0:
        raise ValueError("activations are not fp16 values" if rc == -1 else "out of memory")
    return y


def linear_packed_rowscaled_bf16(x, w_packed_t, scale, in_features: int, bias=None) -> np.ndarray:
    """Packed linear for bf16 activations (given widened to float): each row as integers scaled by its largest exponent,
    the dot product summed exactly and rounded to fp32 once; fp32 result before the cast to the output dtype."""
    x, scale, bias = _lin_args(x, w_packed_t, scale, bias)
    w = np.ascontiguousarray(np.asarray(w_packed_t, dtype=np.uint8))
    b, k = x.shape
    assert k == in_features and w.shape[0] == (k + 3) // 4
    n = w.shape[1]
    assert scale.size in (1, n)
    y = np.empty((b, n), dtype=np.float32)
    rc = lib().bto_linear_packed_rowscaled_bf16(_p(x), _p(w), _p(scale), scale.size, _p(bias), _p(y), b, n, k)
    if rc != 0:
        raise ValueError("linear_packed_rowscaled_bf16: the activations must be bf16 values" if rc == -1 else "out of memory")
    return y


def linear_unpacked(x, w_tern, scale, bias=None) -> np.ndarray:
    x, scale, bias = _lin_args(x, w_tern, scale, bias)
    w = _i8(w_tern)
    b, k = x.shape
    n = w.shape[0]
    assert w.shape[1] == k and scale.size in (1, n)
    y = np.empty((b, n), dtype=np.float32)
    lib().bto_linear_unpacked(_p(x), _p(w), _p(scale), scale.size, _p(bias), _p(y), b, n, k)
    return y


def act_quant_i8(x) -> Tuple[np.ndarray, np.ndarray]:
    x = _f32(x)
    b, k = x.shape
    q = np.empty((b, k), dtype=np.int8)
    s = np.empty((b,), dtype=np.float32)
    lib().bto_act_quant_i8(_p(x), b, k, _p(q), _p(s))
    return q, s


def gemm_i8(q, s_x, w_packed_t, scale, in_features: int, bias=None) -> Tuple[np.ndarray, np.ndarray]:
    """(acc int32 [B,N], y f32 [B,N]) from pre-quantized activations."""
    q = _i8(q)
    s_x = _f32(s_x).reshape(-1)
    scale = _f32(scale).reshape(-1)
    bias = None if bias is None else _f32(bias).reshape(-1)
    w = np.ascontiguousarray(np.asarray(w_packed_t, dtype=np.uint8))
    b, k = q.shape
    assert k == in_features and w.shape[0] == (k + 3) // 4
    n = w.shape[1]
    acc = np.empty((b, n), dtype=np.int32)
    y = np.empty((b, n), dtype=np.float32)
    lib().bto_gemm_i8(_p(q), _p(s_x), _p(w), _p(scale), scale.size, _p(bias), _p(acc), _p(y),
                      b, n, k)
    return acc, y


def linear_i8(x, w_packed_t, scale, in_features: int, bias=None):
    """Whole int8 path from float activations: (q, s_x, acc, y)."""
    q, s = act_quant_i8(x)
    acc, y = gemm_i8(q, s, w_packed_t, scale, in_features, bias)
    return q, s, acc, y


def exp_fixed(a: float) -> float:
    """The fixed-sequence fp32 exp the fused SwiGLU uses."""
    return float(lib().bto_exp_fixed(float(a)))


def swiglu(gate, up, dtype: int = 0):
    """(h f32 [B,K] on the dtype's grid, q int8 [B,K], s_x f32 [B]) of silu(gate)*up."""
    gate, up = _f32(gate), _f32(up)
    b, k = gate.shape
    h = np.empty((b, k), dtype=np.float32)
    q = np.empty((b, k), dtype=np.int8)
    s = np.empty((b,), dtype=np.float32)
    lib().bto_swiglu(_p(gate), _p(up), dtype, b, k, _p(h), _p(q), _p(s))
    return h, q, s


def rmsnorm(x, weight=None, eps: float = 1e-6, dtype: int = 0):
    """(y f32 [B,K] on the dtype's grid, q int8 [B,K], s_x f32 [B]) of RMSNorm(x) * weight."""
    x = _f32(x)
    weight = None if weight is None else _f32(weight).reshape(-1)
    b, k = x.shape
    y = np.empty((b, k), dtype=np.float32)
    q = np.empty((b, k), dtype=np.int8)
    s = np.empty((b,), dtype=np.float32)
    lib().bto_rmsnorm(_p(x), _p(weight), eps, dtype, b, k, _p(y), _p(q), _p(s))
    return y, q, s
