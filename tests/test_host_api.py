"""Host-side mirror of the reference API on CPU tensors: quantizers, codec, modules,
backend dispatch and error behaviour (restating what the reference's CPU tests pin:
tests/test_ternary_quant.py, tests/test_packed_ternary.py, tests/test_ternary_linear.py)."""
import warnings

import pytest
import torch
import torch.nn as nn

import bittorch_amd as bt
from bittorch_amd.nn import (TernaryLinear, TernaryLinearCUDA, TernaryLinearInference,
                             create_ternary_linear_inference)
from bittorch_amd.quant import (TernaryQuantConfig, TernaryQuantizer, dequantize_ternary,
                                get_memory_reduction, pack_ternary, pack_ternary_transposed,
                                pack_ternary_with_scale, ternary_quantize, ternary_quantize_ste,
                                unpack_ternary, unpack_ternary_transposed)


def test_package_surface():
    assert bt.__version__ == "0.2.0"
    for name in ("TernaryLinear", "TernaryLinearCUDA", "TernaryLinearInference",
                 "create_ternary_linear_inference"):
        assert hasattr(bt.nn, name)
    for name in ("ternary_linear", "ternary_linear_forward_cuda", "ternary_linear_packed_forward",
                 "has_packed_cuda_support"):
        assert hasattr(bt.ops, name)
    for name in bt.quant.__all__:
        assert hasattr(bt.quant, name)


# ---- quantizer ---------------------------------------------------------------------------
def test_quantize_shapes_values_and_scale_kinds():
    torch.manual_seed(0)
    w = torch.randn(32, 64)
    t, s = ternary_quantize(w)
    assert t.shape == w.shape and s.shape == (32,) and t.dtype == w.dtype
    assert set(t.unique().tolist()) <= {-1.0, 0.0, 1.0}
    assert torch.equal(s, w.abs().amax(dim=1))
    t2, s2 = ternary_quantize(w, per_channel=False)
    assert s2.dim() == 0 and s2 == w.abs().max()
    lo = (ternary_quantize(w, 0.01)[0] == 0).sum()
    hi = (ternary_quantize(w, 0.5)[0] == 0).sum()
    assert hi > lo
    assert torch.equal(ternary_quantize(w)[0], ternary_quantize(w)[0])


def test_ste_passes_gradient_and_detaches_scale():
    w = torch.randn(8, 16, requires_grad=True)
    q, s = ternary_quantize_ste(w)
    assert torch.allclose(q.detach(), ternary_quantize(w.detach())[0], atol=1e-6)
    assert not s.requires_grad
    q.sum().backward()
    assert torch.equal(w.grad, torch.ones_like(w))


def test_dequantize_and_quantizer_object():
    t = torch.tensor([[1.0, -1.0, 0.0, 1.0], [0.0, 1.0, 1.0, -1.0]])
    s = torch.tensor([2.0, 0.5])
    assert torch.equal(dequantize_ternary(t, s), torch.tensor([[2.0, -2.0, 0.0, 2.0], [0.0, 0.5, 0.5, -0.5]]))
    cfg = TernaryQuantConfig()
    assert cfg.threshold_factor == 0.05 and cfg.per_channel is True
    assert TernaryQuantConfig(threshold_factor=0.1, per_channel=False).scale_type is bt.quant.ScaleType.PER_TENSOR
    with pytest.raises(ValueError, match="threshold_factor must be in"):
        TernaryQuantizer(TernaryQuantConfig(threshold_factor=1.5))
    qz = TernaryQuantizer()
    w = torch.randn(4, 8)
    t, sc = qz.quantize(w)
    assert torch.equal(qz.dequantize(t, sc), t * sc.unsqueeze(1))
    assert qz.bits_per_weight == 1.58 and qz.quant_type is bt.quant.QuantType.TERNARY


def test_compute_scale_variants():
    from bittorch_amd.quant import ScaleType, compute_scale
    w = torch.tensor([[1.0, -4.0, 2.0, 0.5], [0.0, 0.0, 0.0, 0.0]])
    assert compute_scale(w, ScaleType.PER_TENSOR).tolist() == [4.0]
    assert compute_scale(w, ScaleType.PER_CHANNEL).tolist() == [4.0, pytest.approx(1e-8)]
    assert compute_scale(w, ScaleType.PER_GROUP, group_size=2).tolist() == [[4.0, 2.0], [pytest.approx(1e-8)] * 2]


# ---- codec ---------------------------------------------------------------------------------
def test_codec_roundtrip_and_layouts():
    w = torch.tensor([[1.0, -1.0, 0.0, 1.0, -1.0, 0.0]])
    packed, k = pack_ternary(w)
    assert packed.shape == (1, 2) and packed.dtype == torch.uint8 and k == 6
    assert torch.equal(unpack_ternary(packed, k).float(), w)
    for shape in [(1, 4), (4, 4), (7, 13), (32, 64), (128, 256)]:
        t = torch.randint(-1, 2, shape).float()
        p, kk = pack_ternary(t)
        assert torch.equal(unpack_ternary(p, kk).float(), t)
        pt, _ = pack_ternary_transposed(t)
        assert pt.shape == ((shape[1] + 3) // 4, shape[0]) and pt.is_contiguous()
        assert torch.equal(pt, p.t())
        assert torch.equal(unpack_ternary_transposed(pt, kk).float(), t)
        assert unpack_ternary(p, kk).dtype == torch.int8
    with pytest.raises(ValueError, match="Expected 2D"):
        pack_ternary(torch.zeros(4))
    p, s16, k = pack_ternary_with_scale(torch.ones(2, 4), torch.tensor([1.0, 2.0]))
    assert s16.dtype == torch.float16 and k == 4
    assert 15.5 < get_memory_reduction(4096, 4096) < 16.5


# ---- TernaryLinear --------------------------------------------------------------------------
def test_ternary_linear_shapes_grads_and_debug_mode():
    torch.manual_seed(0)
    layer = TernaryLinear(64, 32)
    assert layer.weight.shape == (32, 64) and layer.bias.shape == (32,)
    assert layer(torch.randn(8, 64)).shape == (8, 32)
    assert layer(torch.randn(4, 16, 64)).shape == (4, 16, 32)
    assert TernaryLinear(64, 32, bias=False).bias is None
    x = torch.randn(8, 64, requires_grad=True)
    layer(x).sum().backward()
    assert layer.weight.grad is not None and layer.bias.grad is not None and x.grad is not None
    ref = nn.Linear(64, 32)
    dbg = TernaryLinear(64, 32, quantize=False)
    dbg.load_state_dict(ref.state_dict())
    xin = torch.randn(5, 64)
    assert torch.allclose(dbg(xin), ref(xin), atol=1e-6)
    w_t, sc = layer.get_quantized_weight()
    assert set(w_t.unique().tolist()) <= {-1.0, 0.0, 1.0} and sc.shape == (32,)
    assert torch.allclose(layer(xin), xin @ (w_t * sc.unsqueeze(1)).t() + layer.bias, atol=1e-5)
    assert "backend='auto'" in repr(layer) and "threshold_factor=0.05" in repr(layer)


def test_backend_validation_and_errors():
    assert TernaryLinear(8, 4).backend == "auto"
    for b in ("auto", "cuda", "python"):
        assert TernaryLinear(8, 4, backend=b).backend == b
    with pytest.raises(ValueError, match="backend must be"):
        TernaryLinear(8, 4, backend="invalid")
    with pytest.raises(RuntimeError, match="requires input and weights on CUDA"):
        TernaryLinear(8, 4, backend="cuda")(torch.randn(2, 8))
    with pytest.raises(RuntimeError, match="requires CUDA"):
        TernaryLinearCUDA(8, 4)(torch.randn(2, 8))
    with warnings.catch_warnings(record=True) as rec:
        warnings.simplefilter("always")
        assert TernaryLinear(8, 4, use_cuda_kernel=True).backend == "auto"
        assert TernaryLinear(8, 4, use_cuda_kernel=False).backend == "python"
    assert sum(issubclass(r.category, DeprecationWarning) for r in rec) == 2
    # CPU tensors with backend auto use the plain torch path and equal backend="python"
    a = TernaryLinear(16, 8, backend="auto")
    p = TernaryLinear(16, 8, backend="python")
    p.load_state_dict(a.state_dict())
    x = torch.randn(3, 16)
    assert torch.equal(a(x), p(x))


def test_per_tensor_scale_forward_works():
    layer = TernaryLinear(16, 8, per_channel=False)
    w_t, s = layer.get_quantized_weight()
    x = torch.randn(2, 16)
    assert torch.allclose(layer(x), x @ (w_t * s).t() + layer.bias, atol=1e-6)


# ---- TernaryLinearInference -------------------------------------------------------------------
def test_inference_module_matches_dense_formula():
    torch.manual_seed(1)
    w = torch.randn(32, 64)
    bias = torch.randn(32)
    w_t, s = ternary_quantize(w)
    mod = TernaryLinearInference.from_unpacked(w_t, s, bias)
    assert mod.weight_packed.shape == (16, 32) and mod.weight_packed.dtype == torch.uint8
    x = torch.randn(8, 64)
    assert torch.allclose(mod(x), x @ (w_t * s.unsqueeze(1)).t() + bias, rtol=1e-4, atol=1e-4)
    assert len(list(mod.parameters())) == 0 and {n for n, _ in mod.named_buffers()} == {"weight_packed", "scale", "bias"}
    assert mod.packed_size_bytes == 32 * 16
    assert mod.effective_bits_per_weight == (32 * 16 * 8 + 32 * 16) / (32 * 64)
    assert "reduction=" in repr(mod)
    mod2 = create_ternary_linear_inference(64, 32, w, bias)
    assert torch.equal(mod2.weight_packed, mod.weight_packed) and torch.equal(mod2.scale, mod.scale)
    sd = mod.state_dict()
    assert set(sd) == {"weight_packed", "scale", "bias"}
    # ragged K
    w = torch.randn(5, 13)
    m3 = create_ternary_linear_inference(13, 5, w)
    w_t, s = ternary_quantize(w)
    x = torch.randn(2, 13)
    assert torch.allclose(m3(x), x @ (w_t * s.unsqueeze(1)).t(), rtol=1e-4, atol=1e-5)


def test_config1_plumbing_cpu(oracle):
    """Benchmark config 1 on the plain torch backend: TernaryLinear(512->256), batch 32, fp32,
    N(0,0.02) masters, seed 0 -- quantize / pack / forward agree with the oracle."""
    g = torch.Generator().manual_seed(0)
    layer = TernaryLinear(512, 256, bias=True, threshold_factor=0.05, backend="python")
    with torch.no_grad():
        layer.weight.copy_(torch.randn(256, 512, generator=g) * 0.02)
        layer.bias.copy_(torch.randn(256, generator=g) * 0.01)
    x = torch.randn(32, 512, generator=g)
    y = layer(x)
    w_t, s = layer.get_quantized_weight()
    o_t, o_s = oracle.ternary_quantize(layer.weight.detach().numpy(), 0.05, True)
    assert (w_t.numpy() == o_t).all() and (s.numpy() == o_s).all()
    inf = create_ternary_linear_inference(512, 256, layer.weight.detach(), layer.bias.detach())
    assert (inf.weight_packed.numpy() == oracle.pack_ternary_transposed(o_t)[0]).all()
    truth = oracle.linear_packed(x.numpy(), inf.weight_packed.numpy(), o_s, 512, layer.bias.detach().numpy(), f64=True)
    assert abs(y.detach().numpy() - truth).max() / abs(truth).max() < 1e-5
    assert abs(inf(x).numpy() - truth).max() / abs(truth).max() < 1e-5


def test_xor_training_converges_on_cpu():
    """End-to-end training smoke (reference tests/test_xor_mlp.py:41-67)."""
    torch.manual_seed(42)
    model = nn.Sequential(TernaryLinear(2, 16), nn.ReLU(), TernaryLinear(16, 1))
    xs = torch.tensor([[0.0, 0.0], [0.0, 1.0], [1.0, 0.0], [1.0, 1.0]])
    ys = torch.tensor([[0.0], [1.0], [1.0], [0.0]])
    opt = torch.optim.Adam(model.parameters(), lr=0.01)
    first = None
    for _ in range(2000):
        opt.zero_grad()
        loss = nn.functional.binary_cross_entropy_with_logits(model(xs), ys)
        first = first if first is not None else loss.item()
        loss.backward()
        opt.step()
    acc = ((model(xs) > 0).float() == ys).float().mean().item()
    assert loss.item() < first and acc == 1.0
