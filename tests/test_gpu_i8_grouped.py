"""GPU parity of the grouped int8 launch (`bt_ternary_gemm_i8_grouped`): G units of up to 16 int8-quantized rows.

Every unit must equal `bt_ternary_gemm_i8_tiled` on the same operands bit for bit, int32 accumulators included (the
sums are integers, so no split of K may show); one case is held to the CPU oracle directly.  Shapes cover both wave
counts of the kernel (K up to 4096: 8 waves; up to 11264: 16), every steps-per-wave instantiation that the K values
below select, ragged N and K, fewer than 16 rows, both activation layouts, per-tensor scales, shared operands and
BASELINE config 3's two shapes at full size.
"""
import numpy as np
import pytest
import torch

from conftest import announce
from _util import f32np, random_ternary, seeded_acts

pytestmark = pytest.mark.gpu


def _unit(oracle, n, k, m, seed, per_tensor=False, bias=True, operand_order=False):
    from bittorch_amd import _C
    w = random_ternary(n, k, seed=seed)
    packed, _ = oracle.pack_ternary_transposed(w.numpy())
    packed = torch.from_numpy(packed).cuda()
    g = torch.Generator().manual_seed(seed)
    scale = (torch.rand(1 if per_tensor else n, generator=g) * 0.05 + 0.01).cuda()
    b = (torch.randn(n, generator=g) * 0.01).cuda() if bias else None
    x = seeded_acts(m, k, seed=seed + 1, dtype=torch.bfloat16, outliers=True).cuda()
    q, s = _C.act_quant_int8(x, operand_order)
    return dict(packed=packed, tiled=_C.retile_weights(packed, k), scale=scale, bias=b, x=x, q=q, s=s)


def _run_grouped(units, m, n, k, out_dtype, operand_order, want_acc=True):
    from bittorch_amd import _C
    ys = [torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda") for _ in units]
    accs = [torch.full((m, n), -7, dtype=torch.int32, device="cuda") for _ in units] if want_acc else None
    bias_tab = None if units[0]["bias"] is None else _C.pointer_table([u["bias"] for u in units])
    _C.ternary_gemm_int8_grouped(
        _C.pointer_table([u["q"] for u in units]), _C.pointer_table([u["s"] for u in units]),
        _C.pointer_table([u["tiled"] for u in units]), _C.pointer_table([u["scale"] for u in units]), bias_tab,
        _C.pointer_table(ys), m, k, n, scale_len=units[0]["scale"].numel(), out_dtype=out_dtype,
        q_operand_order=operand_order, acc_tab=None if accs is None else _C.pointer_table(accs))
    torch.cuda.synchronize()
    return ys, accs


# (N, K, M, G): 8-wave kernel with 1..8 steps per wave, 16-wave kernel with 5..11; ragged N (odd tile count -> one tile
# in flight), ragged K (K % 64 != 0), M < 16
CASES = [(64, 64, 16, 3), (96, 528, 16, 5), (112, 1040, 7, 4), (256, 2048, 16, 9), (250, 2560, 1, 6), (640, 4096, 16, 40),
         (1000, 4112, 16, 3), (64, 6912, 5, 7), (128, 8192, 16, 4), (96, 11008, 16, 6), (32, 11264, 2, 2)]


@pytest.mark.parametrize("n,k,m,g", CASES)
def test_grouped_int8_units_equal_single_calls(oracle, n, k, m, g):
    from bittorch_amd import _C
    for operand_order, per_tensor, bias, out_dtype in ((False, False, True, torch.bfloat16), (True, True, False, torch.float32),
                                                      (True, False, True, torch.float16)):
        announce("grouped int8", n, k, m, g, operand_order, per_tensor, bias, out_dtype)
        units = [_unit(oracle, n, k, m, seed=10 * u + n, per_tensor=per_tensor, bias=bias, operand_order=operand_order)
                 for u in range(g)]
        ys, accs = _run_grouped(units, m, n, k, out_dtype, operand_order)
        for u, un in enumerate(units):
            y1, a1 = _C.ternary_gemm_int8_tiled(un["q"], un["s"], un["tiled"], un["scale"], un["bias"], k, n, out_dtype, True,
                                                None, operand_order)
            assert torch.equal(accs[u], a1), (u, "accumulators")
            assert torch.equal(ys[u], y1), (u, "outputs")


_rng = np.random.default_rng(20250311)


def _random_case(i):
    k = 16 * int(_rng.integers(1, 705))                       # 16 .. 11264, any multiple of 16
    if i % 3 == 0:
        k = 16 * int(_rng.integers(1, 257))                   # ... a third of them inside the 8-wave kernel's range
    n = int(_rng.choice([16, 20, 33, 48, 100, 250, 260, 512]))
    return n, k, int(_rng.integers(1, 17)), int(_rng.integers(1, 10)), bool(i % 2), i


@pytest.mark.parametrize("n,k,m,g,operand_order,seed", [_random_case(i) for i in range(18)])
def test_grouped_int8_random_shapes_against_the_oracle(oracle, n, k, m, g, operand_order, seed):
    """Seeded random unit counts, rows, ragged column counts and any K % 16 == 0 up to the kernel's limit, held to the
    CPU oracle directly: int32 accumulators and fp32 outputs bit for bit."""
    announce("grouped int8 random", n, k, m, g, operand_order)
    units = [_unit(oracle, n, k, m, seed=97 * seed + u, bias=bool(seed % 3), operand_order=operand_order) for u in range(g)]
    ys, accs = _run_grouped(units, m, n, k, torch.float32, operand_order)
    for u, un in enumerate(units):
        _, _, oacc, oy = oracle.linear_i8(f32np(un["x"].cpu()), un["packed"].cpu().numpy(), f32np(un["scale"].cpu()), k,
                                          None if un["bias"] is None else f32np(un["bias"].cpu()))
        np.testing.assert_array_equal(accs[u].cpu().numpy(), oacc)
        np.testing.assert_array_equal(ys[u].cpu().numpy(), oy)


def test_grouped_int8_against_oracle_and_shared_operands(oracle):
    """One case straight against the CPU oracle (quantized activations, accumulators, outputs), and units that
    share one weight matrix or one activation block."""
    from bittorch_amd import _C
    n, k, m = 96, 528, 11
    units = [_unit(oracle, n, k, m, seed=5 + u) for u in range(3)]
    units.append(dict(units[0], q=units[1]["q"], s=units[1]["s"], x=units[1]["x"]))   # unit 0's weights, unit 1's rows
    units.append(dict(units[2], tiled=units[0]["tiled"], packed=units[0]["packed"], scale=units[0]["scale"], bias=units[0]["bias"]))
    ys, accs = _run_grouped(units, m, n, k, torch.bfloat16, False)
    for u, un in enumerate(units):
        announce("grouped int8 vs oracle", u)
        oq, os_, oacc, oy = oracle.linear_i8(f32np(un["x"].cpu()), un["packed"].cpu().numpy(), f32np(un["scale"].cpu()), k,
                                             f32np(un["bias"].cpu()))
        np.testing.assert_array_equal(un["q"].cpu().numpy(), oq)
        np.testing.assert_array_equal(accs[u].cpu().numpy(), oacc)
        assert torch.equal(ys[u].cpu(), torch.from_numpy(oy).bfloat16())


@pytest.mark.parametrize("n,k", [(11008, 4096), (4096, 11008)])
def test_grouped_int8_config3_shapes_full_size(oracle, n, k):
    """BASELINE config 3: x bf16 [16, K] per-row int8, W [N, K]; four units per launch, each against the single call,
    and the launch replayed from a HIP graph with new activations in between."""
    from bittorch_amd import _C
    m, g = 16, 4
    announce("grouped int8 config 3", n, k)
    units = [_unit(oracle, n, k, m, seed=3 + u, operand_order=True) for u in range(g)]
    ys, accs = _run_grouped(units, m, n, k, torch.bfloat16, True)
    singles = []
    for u, un in enumerate(units):
        y1, a1 = _C.ternary_gemm_int8_tiled(un["q"], un["s"], un["tiled"], un["scale"], un["bias"], k, n, torch.bfloat16, True,
                                            None, True)
        assert torch.equal(accs[u], a1) and torch.equal(ys[u], y1)
        singles.append(y1)
    # graph replay: tables and buffers fixed, the activations refreshed by eager work between the replays
    ys2 = [torch.empty_like(y) for y in ys]
    tabs = (_C.pointer_table([u["q"] for u in units]), _C.pointer_table([u["s"] for u in units]),
            _C.pointer_table([u["tiled"] for u in units]), _C.pointer_table([u["scale"] for u in units]),
            _C.pointer_table([u["bias"] for u in units]), _C.pointer_table(ys2))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _C.ternary_gemm_int8_grouped(*tabs, m, k, n, out_dtype=torch.bfloat16, q_operand_order=True)
    for rep in range(2):
        for un in units:
            x = seeded_acts(m, k, seed=50 + rep, dtype=torch.bfloat16, outliers=True).cuda()
            q, s = _C.act_quant_int8(x, True)
            un["q"].copy_(q)
            un["s"].copy_(s)
        graph.replay()
        torch.cuda.synchronize()
        for u, un in enumerate(units):
            want = _C.ternary_gemm_int8_tiled(un["q"], un["s"], un["tiled"], un["scale"], un["bias"], k, n, torch.bfloat16,
                                              False, None, True)
            assert torch.equal(ys2[u], want)


def test_grouped_int8_argument_errors():
    from bittorch_amd import _C
    t = _C.pointer_table([torch.zeros(256, dtype=torch.uint8, device="cuda")])
    with pytest.raises(RuntimeError, match="at most 16"):
        _C.ternary_gemm_int8_grouped(t, t, t, t, None, t, 17, 64, 64)
    with pytest.raises(RuntimeError, match="multiple of 16"):
        _C.ternary_gemm_int8_grouped(t, t, t, t, None, t, 16, 72, 64)
    with pytest.raises(RuntimeError, match="at most 11264"):
        _C.ternary_gemm_int8_grouped(t, t, t, t, None, t, 16, 16384, 64)
    with pytest.raises(RuntimeError, match="scale size"):
        _C.ternary_gemm_int8_grouped(t, t, t, t, None, t, 16, 64, 64, scale_len=3)


def test_ops_ternary_linear_int8_grouped_equals_forward_int8(oracle):
    """The caller in the kept API: float activations [G, M, K] (quantized in one launch) or pre-quantized q / s_x
    through `ops.ternary_linear_int8_grouped`, unit by unit the bits of `layer.forward_int8` on the same rows; more
    than 16 rows per unit, or fewer than three units, fall back to single calls with the same result."""
    import bittorch_amd as bt
    from bittorch_amd import _C
    from bittorch_amd.nn import TernaryLinearInference
    n, k, g = 320, 1024, 5
    layers = []
    for u in range(g):
        w = random_ternary(n, k, seed=60 + u)
        packed, _ = oracle.pack_ternary_transposed(w.numpy())
        gen = torch.Generator().manual_seed(u)
        layers.append(TernaryLinearInference(k, n, torch.from_numpy(packed), torch.rand(n, generator=gen) * 0.05 + 0.01,
                                             torch.randn(n, generator=gen) * 0.01).cuda())
    for m in (16, 3, 20):
        announce("ops.ternary_linear_int8_grouped", m)
        xs = seeded_acts(g * m, k, seed=m, dtype=torch.bfloat16, outliers=True).view(g, m, k).cuda()
        got = bt.ops.ternary_linear_int8_grouped(layers, xs)
        assert got.shape == (g, m, n) and got.dtype == torch.bfloat16
        for u, L in enumerate(layers):
            q, s = bt.ops.act_quant_int8(xs[u], True)
            assert torch.equal(got[u], L.forward_int8(q, s, torch.bfloat16, None, True))
        # pre-quantized, row-major bytes, fp32 outputs, into a caller's buffer, twice (cached tables)
        q_all, s_all = bt.ops.act_quant_int8(xs, False)
        out = torch.empty(g, m, n, device="cuda")
        for _ in range(2):
            assert bt.ops.ternary_linear_int8_grouped(layers, q=q_all, s_x=s_all, out_dtype=torch.float32, out=out) is out
        for u, L in enumerate(layers):
            assert torch.equal(out[u], L.forward_int8(q_all[u], s_all[u], torch.float32))
    # two units are below the grouped kernel's break-even and go through single calls: the same bits
    got2 = bt.ops.ternary_linear_int8_grouped(layers[:2], xs[:2])
    for u in range(2):
        q, s = bt.ops.act_quant_int8(xs[u], True)
        assert torch.equal(got2[u], layers[u].forward_int8(q, s, torch.bfloat16, None, True))
    with pytest.raises(ValueError, match="give xs, or q together with s_x"):
        bt.ops.ternary_linear_int8_grouped(layers)
    with pytest.raises(RuntimeError, match="doesn't match in_features"):
        bt.ops.ternary_linear_int8_grouped(layers, torch.zeros(g, 4, k - 16, device="cuda"))
