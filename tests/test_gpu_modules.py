"""GPU parity at the module boundary: TernaryLinear / TernaryLinearCUDA /
TernaryLinearInference on the HIP kernels vs the plain torch backend and the oracle
(what the reference pins in tests/test_ternary_cuda.py, tests/test_gradient_consistency.py,
tests/test_amp.py, tests/test_packed_kernel.py:285-347, tests/test_robustness.py)."""
import numpy as np
import pytest
import torch
import torch.nn as nn

from conftest import announce
from _util import f32np, rel_err

pytestmark = pytest.mark.gpu


def _pair(in_f, out_f, **kw):
    from bittorch_amd.nn import TernaryLinear
    torch.manual_seed(0)
    hip = TernaryLinear(in_f, out_f, backend="cuda", **kw).cuda()
    ref = TernaryLinear(in_f, out_f, backend="python", **kw).cuda()
    ref.load_state_dict(hip.state_dict())
    return hip, ref


@pytest.mark.parametrize("shape", [(1, 1, 1), (4, 16, 8), (7, 33, 17), (32, 512, 256), (17, 123, 67),
                                   (2, 5, 64, 32), (8, 1024, 1024)])
def test_module_forward_matches_python_backend(shape):
    *lead, in_f, out_f = shape
    announce("module forward", shape)
    hip, ref = _pair(in_f, out_f)
    x = torch.randn(*lead, in_f, device="cuda")
    y, y_ref = hip(x), ref(x)
    assert y.shape == y_ref.shape == (*lead, out_f)
    assert torch.allclose(y, y_ref, rtol=1e-4, atol=1e-4)


def test_config1_plumbing_gpu(oracle, monkeypatch):
    """Config 1 on the GPU: TernaryLinear(512->256, bias), batch 32, fp32, seed 0."""
    from bittorch_amd.nn import TernaryLinear, create_ternary_linear_inference
    announce("config1 gpu")
    g = torch.Generator().manual_seed(0)
    layer = TernaryLinear(512, 256, bias=True, threshold_factor=0.05)
    with torch.no_grad():
        layer.weight.copy_(torch.randn(256, 512, generator=g) * 0.02)
        layer.bias.copy_(torch.randn(256, generator=g) * 0.01)
    x = torch.randn(32, 512, generator=g)
    o_t, o_s = oracle.ternary_quantize(layer.weight.detach().numpy(), 0.05, True)
    o_p, _ = oracle.pack_ternary_transposed(o_t)
    ref = oracle.linear_packed(x.numpy(), o_p, o_s, 512, layer.bias.detach().numpy())
    truth = oracle.linear_packed(x.numpy(), o_p, o_s, 512, layer.bias.detach().numpy(), f64=True)
    layer = layer.cuda()
    inf = create_ternary_linear_inference(512, 256, layer.weight.detach(), layer.bias.detach())
    np.testing.assert_array_equal(inf.weight_packed.cpu().numpy(), o_p)
    np.testing.assert_array_equal(inf.scale.cpu().numpy(), o_s)
    # default route for fp32 with K % 64 == 0: three exact bf16 planes on the matrix cores
    assert rel_err(f32np(layer(x.cuda())), truth) < 1e-5
    assert rel_err(f32np(inf(x.cuda())), truth) < 1e-5
    # the generic kernel sums in the oracle's k order: bit for bit
    monkeypatch.setenv("BITTORCH_KERNEL", "generic")
    np.testing.assert_array_equal(f32np(layer(x.cuda())), ref)
    np.testing.assert_array_equal(f32np(inf(x.cuda())), ref)


def test_gradients_match_python_backend():
    announce("gradients")
    for (b, in_f, out_f, bias) in [(8, 64, 32, True), (5, 33, 17, False), (16, 256, 128, True)]:
        hip, ref = _pair(in_f, out_f, bias=bias)
        x1 = torch.randn(b, in_f, device="cuda", requires_grad=True)
        x2 = x1.detach().clone().requires_grad_(True)
        g = torch.randn(b, out_f, device="cuda")
        (hip(x1) * g).sum().backward()
        (ref(x2) * g).sum().backward()
        assert torch.allclose(hip.weight.grad, ref.weight.grad, rtol=1e-4, atol=1e-4)
        assert torch.allclose(x1.grad, x2.grad, rtol=1e-4, atol=1e-4)
        if bias:
            assert torch.allclose(hip.bias.grad, ref.bias.grad, rtol=1e-4, atol=1e-4)
        cos = nn.functional.cosine_similarity(hip.weight.grad.flatten(), ref.weight.grad.flatten(), dim=0)
        assert cos > 0.99


def test_amp_autocast_forward_backward():
    from bittorch_amd.nn import TernaryLinearCUDA
    announce("amp")
    torch.manual_seed(0)
    layer = TernaryLinearCUDA(256, 128).cuda()
    x = torch.randn(16, 256, device="cuda", requires_grad=True)
    y32 = layer(x)
    with torch.autocast("cuda", dtype=torch.float16):
        y16 = layer(x)
    assert y16.dtype == torch.float16 and torch.isfinite(y16).all()
    assert torch.allclose(y16.float(), y32, rtol=1e-2, atol=1e-2)
    scaler_loss = y16.float().pow(2).mean()
    scaler_loss.backward()
    assert torch.isfinite(layer.weight.grad).all() and torch.isfinite(x.grad).all()
    assert layer.weight.grad.dtype == torch.float32


def test_amp_training_loop_with_grad_scaler():
    """What the reference's AMP tests pin beyond one forward (tests/test_amp.py:209-333): a GradScaler training loop on
    XOR lowers the loss on either backend, with no NaN or Inf in loss or gradients on the way."""
    from bittorch_amd.nn import TernaryLinear
    announce("amp training")
    xor_x = torch.tensor([[0., 0.], [0., 1.], [1., 0.], [1., 1.]], device="cuda")
    xor_y = torch.tensor([[0.], [1.], [1.], [0.]], device="cuda")
    for backend in ("cuda", "python"):
        torch.manual_seed(42)
        model = nn.Sequential(TernaryLinear(2, 16, backend=backend), nn.ReLU(), TernaryLinear(16, 1, backend=backend)).cuda()
        opt = torch.optim.Adam(model.parameters(), lr=0.01)
        scaler = torch.amp.GradScaler("cuda")
        losses = []
        for _ in range(100):
            opt.zero_grad()
            with torch.autocast("cuda", dtype=torch.float16):
                loss = nn.functional.binary_cross_entropy_with_logits(model(xor_x), xor_y)
            assert torch.isfinite(loss)
            scaler.scale(loss).backward()
            scaler.step(opt)
            scaler.update()
            losses.append(loss.item())
        assert losses[-1] < losses[0], (backend, losses[0], losses[-1])
        for prm in model.parameters():
            assert prm.grad is not None and prm.grad.shape == prm.shape


def test_autocast_contexts_mixed_nested_eval_and_batch_sizes():
    """tests/test_amp.py:335-405: one sample and a large batch under autocast, regular forwards before and after an
    autocast one agree, a disabled inner context gives fp32, eval mode under no_grad is finite."""
    from bittorch_amd.nn import TernaryLinear
    announce("autocast contexts")
    torch.manual_seed(3)
    layer = TernaryLinear(64, 32).cuda()
    for b in (1, 256):
        with torch.autocast("cuda", dtype=torch.float16):
            y = layer(torch.randn(b, 64, device="cuda"))
        assert y.shape == (b, 32) and torch.isfinite(y).all()
    x = torch.randn(8, 64, device="cuda")
    y1 = layer(x)
    with torch.autocast("cuda", dtype=torch.float16):
        ya = layer(x)
        with torch.autocast("cuda", enabled=False):
            yb = layer(x)
        yc = layer(x)
    y3 = layer(x)
    assert y1.dtype == y3.dtype == yb.dtype == torch.float32
    assert torch.equal(y1, y3) and torch.equal(yb, y1)
    assert torch.isfinite(ya).all() and torch.equal(ya, yc)
    assert torch.allclose(ya.float(), y1, rtol=1e-2, atol=1e-2)
    layer.eval()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        ye = layer(x)
    assert torch.isfinite(ye).all()


def test_gradient_consistency_over_seeds_shapes_and_double_precision():
    """tests/test_gradient_consistency.py:153-250: the kernels' gradients follow the torch backend's over several seeds
    and shapes, and the autograd function takes float64 operands (the reference runs gradcheck on it in double
    precision and accepts either outcome: the straight-through estimator is not the derivative of the forward)."""
    from bittorch_amd.nn.ternary_linear_cuda import TernaryLinearCUDAFunction
    announce("gradient consistency")
    for seed in (0, 1, 7, 42, 123):
        torch.manual_seed(seed)
        hip, ref = _pair(32, 16)
        x1 = torch.randn(4, 32, device="cuda", requires_grad=True)
        x2 = x1.detach().clone().requires_grad_(True)
        hip(x1).sum().backward()
        ref(x2).sum().backward()
        assert torch.allclose(hip.weight.grad, ref.weight.grad, rtol=1e-4, atol=1e-5)
        assert torch.allclose(x1.grad, x2.grad, rtol=1e-4, atol=1e-5)
    for (b, in_f, out_f) in [(1, 8, 4), (3, 100, 50), (64, 16, 128), (2, 7, 3)]:
        hip, ref = _pair(in_f, out_f)
        x1 = torch.randn(b, in_f, device="cuda", requires_grad=True)
        x2 = x1.detach().clone().requires_grad_(True)
        hip(x1).pow(2).sum().backward()
        ref(x2).pow(2).sum().backward()
        assert torch.allclose(hip.weight.grad, ref.weight.grad, rtol=1e-3, atol=1e-4)
        assert torch.allclose(hip.bias.grad, ref.bias.grad, rtol=1e-3, atol=1e-4)
        assert torch.allclose(x1.grad, x2.grad, rtol=1e-3, atol=1e-4)
    torch.manual_seed(42)
    x = torch.randn(2, 4, device="cuda", dtype=torch.float64, requires_grad=True)
    w = torch.randn(3, 4, device="cuda", dtype=torch.float64, requires_grad=True)
    bias = torch.randn(3, device="cuda", dtype=torch.float64, requires_grad=True)
    y = TernaryLinearCUDAFunction.apply(x, w, bias, 0.05, True)
    assert y.dtype == torch.float64 and y.shape == (2, 3)
    from bittorch_amd.quant import ternary_quantize
    w_t, s = ternary_quantize(w.detach(), 0.05, True)
    assert torch.allclose(y, x.detach() @ (w_t * s.unsqueeze(1)).t() + bias.detach(), rtol=1e-6, atol=1e-6)
    y.sum().backward()
    assert x.grad.dtype == w.grad.dtype == bias.grad.dtype == torch.float64
    assert torch.equal(bias.grad, torch.full_like(bias, 2.0))
    outcome = torch.autograd.gradcheck(lambda a, b_, c: TernaryLinearCUDAFunction.apply(a, b_, c, 0.05, True),
                                       (x, w, bias), eps=1e-4, atol=1e-3, rtol=1e-2, raise_exception=False)
    assert outcome in (True, False)


def test_half_and_bf16_modules():
    from bittorch_amd.nn import TernaryLinear
    announce("16-bit modules")
    for dtype in (torch.float16, torch.bfloat16):
        torch.manual_seed(1)
        hip = TernaryLinear(512, 256).cuda().to(dtype)
        x = torch.randn(4, 512, device="cuda", dtype=dtype)
        y = hip(x)
        assert y.dtype == dtype
        w_t, s = hip.get_quantized_weight()
        ref = x.float() @ (w_t.float() * s.float().unsqueeze(1)).t() + hip.bias.float()
        assert rel_err(f32np(y), f32np(ref)) < 1e-2


def test_inference_module_gpu_matches_cpu_route():
    from bittorch_amd.nn import TernaryLinearInference, create_ternary_linear_inference
    from bittorch_amd.quant import ternary_quantize
    announce("inference module")
    for (b, in_f, out_f) in [(1, 768, 768), (32, 1024, 4096), (3, 13, 5), (16, 4096, 4096), (8, 4096, 11008)]:
        torch.manual_seed(in_f)
        w = torch.randn(out_f, in_f) * 0.02
        bias = torch.randn(out_f) * 0.01
        w_t, s = ternary_quantize(w)
        cpu_mod = TernaryLinearInference.from_unpacked(w_t, s, bias)
        gpu_mod = create_ternary_linear_inference(in_f, out_f, w.cuda(), bias.cuda())
        assert torch.equal(gpu_mod.weight_packed.cpu(), cpu_mod.weight_packed)
        assert torch.equal(gpu_mod.scale.cpu(), cpu_mod.scale)
        x = torch.randn(b, in_f)
        for dtype, tol in ((torch.float32, 1e-3), (torch.float16, 1e-2), (torch.bfloat16, 1e-2)):
            y = gpu_mod.to(dtype)(x.cuda().to(dtype)) if dtype != torch.float32 else gpu_mod(x.cuda())
            truth = x.to(dtype).double() @ (w_t.double() * s.to(dtype).double().unsqueeze(1)).t() + bias.to(dtype).double()
            assert rel_err(f32np(y), truth.numpy()) < tol, (b, in_f, out_f, dtype)
        gpu_mod.float()
    # moving a CPU-built module to the GPU keeps the buffers and works
    moved = cpu_mod.cuda()
    assert moved.weight_packed.is_cuda and moved(x.cuda()).shape == (b, out_f)


def test_functional_ops():
    import bittorch_amd as bt
    from bittorch_amd.quant import pack_ternary_transposed, ternary_quantize
    announce("functional ops")
    torch.manual_seed(3)
    w = torch.randn(64, 128, device="cuda")
    bias = torch.randn(64, device="cuda")
    x = torch.randn(4, 7, 128, device="cuda")
    w_t, s = ternary_quantize(w)
    ref = x @ (w_t * s.unsqueeze(1)).t() + bias
    y1 = bt.ops.ternary_linear(x, w, bias)
    y2 = bt.ops.ternary_linear_forward_cuda(x, w_t.to(torch.int8), s, bias)
    y3 = bt.ops.ternary_linear_packed_forward(x, pack_ternary_transposed(w_t)[0], s, 128, bias)
    for y in (y1, y2, y3):
        assert y.shape == (4, 7, 64) and torch.allclose(y, ref, rtol=1e-4, atol=1e-4)
    x2 = x.reshape(-1, 128)
    y4 = bt.ops.ternary_linear_tensor_core_forward(x2, pack_ternary_transposed(w_t)[0], s, 128, bias, version=1)
    assert torch.allclose(y4, ref.reshape(-1, 64), rtol=1e-4, atol=1e-4)
    y5 = bt.ops.ternary_linear_tensor_core_forward(x2, pack_ternary_transposed(w_t)[0], s, 128, bias, version=2)
    assert rel_err(f32np(y5), f32np(ref.reshape(-1, 64))) < 2e-2
    # float64 inputs are served too (reference dispatches double)
    y6 = bt.ops.ternary_linear_packed_forward(x.double(), pack_ternary_transposed(w_t)[0], s.double(), 128, bias.double())
    assert y6.dtype == torch.float64 and torch.allclose(y6, ref.double(), rtol=1e-4, atol=1e-4)
    assert bt.ops.has_packed_cuda_support()


def test_determinism_and_batched_equals_looped():
    hip, _ = _pair(256, 128)
    announce("determinism")
    x = torch.randn(16, 256, device="cuda")
    y1, y2 = hip(x), hip(x)
    assert torch.equal(y1, y2)
    rows = torch.cat([hip(x[i:i + 1]) for i in range(16)])
    assert torch.allclose(rows, y1, atol=1e-6)
    assert torch.equal(hip(torch.zeros(3, 256, device="cuda")), hip.bias.detach().expand(3, 128))


def test_xor_training_on_gpu():
    from bittorch_amd.nn import TernaryLinearCUDA
    announce("xor gpu")
    torch.manual_seed(42)
    model = nn.Sequential(TernaryLinearCUDA(2, 16), nn.ReLU(), TernaryLinearCUDA(16, 1)).cuda()
    xs = torch.tensor([[0.0, 0.0], [0.0, 1.0], [1.0, 0.0], [1.0, 1.0]], device="cuda")
    ys = torch.tensor([[0.0], [1.0], [1.0], [0.0]], device="cuda")
    opt = torch.optim.Adam(model.parameters(), lr=0.01)
    for _ in range(1500):
        opt.zero_grad()
        loss = nn.functional.binary_cross_entropy_with_logits(model(xs), ys)
        loss.backward()
        opt.step()
    assert ((model(xs) > 0).float() == ys).all()


def test_packed_weight_cache_follows_the_weights(monkeypatch):
    """A training forward quantizes every time (as the reference does, bittorch/nn/ternary_linear.py:196-200), so
    writes through `.data` cannot go stale there; forwards without gradients keep the packed weights until a tracked
    change (in-place update, optimizer step, load_state_dict, dtype move) or `invalidate_packed_cache()`."""
    from bittorch_amd import _C
    from bittorch_amd.nn import TernaryLinear, TernaryLinearCUDA
    announce("packed weight cache")
    calls = {"n": 0}
    real = _C.ternary_quantize_pack

    def counting(*a, **k):
        calls["n"] += 1
        return real(*a, **k)

    def fresh_output(layer, x):
        packed, scale, _ = real(layer.weight.detach(), layer.threshold_factor, layer.per_channel)
        return _C.ternary_linear_packed_forward(x, packed, scale.reshape(-1).to(x.dtype), layer.bias.detach().to(x.dtype), 64)

    monkeypatch.setattr(_C, "ternary_quantize_pack", counting)
    for cls in (TernaryLinear, TernaryLinearCUDA):
        torch.manual_seed(1)
        layer = cls(64, 32).cuda()
        x = torch.randn(8, 64, device="cuda")
        calls["n"] = 0
        # gradient mode on, trainable weights: no caching, and a write through .data is seen at once
        y0 = layer(x)
        y1 = layer(x)
        assert calls["n"] == 2 and torch.equal(y0, y1)
        layer.weight.data.mul_(-1.0)
        y2 = layer(x)
        assert calls["n"] == 3 and torch.equal(y2, fresh_output(layer, x)) and not torch.equal(y2, y0)
        layer.weight.data.normal_(std=0.02)
        opt = torch.optim.SGD(layer.parameters(), lr=0.5)
        layer(x).pow(2).sum().backward()
        assert layer.weight.grad is not None and layer.weight.grad.abs().sum() > 0
        opt.step()
        assert torch.equal(layer(x), fresh_output(layer, x))
        # no gradients: quantized once, reused
        calls["n"] = 0
        with torch.no_grad():
            e0 = layer(x)
            e1 = layer(x)
            assert calls["n"] == 1 and torch.equal(e0, e1) and torch.equal(e0, fresh_output(layer, x))
            # tracked in-place writes are followed
            layer.weight.mul_(0.5)
            layer.weight[0, :8] = 1.0
            assert torch.equal(layer(x), fresh_output(layer, x)) and calls["n"] == 2
            # a write through .data is the one thing the version counter does not see: invalidate by hand
            layer.weight.data.mul_(-1.0)
            layer.invalidate_packed_cache()
            assert torch.equal(layer(x), fresh_output(layer, x)) and calls["n"] == 3
        # frozen weights cache with gradient mode on as well (inputs may still need gradients)
        layer.requires_grad_(False)
        xg = x.clone().requires_grad_(True)
        calls["n"] = 0
        layer(xg).sum().backward()
        layer(xg)
        assert calls["n"] == 0 and xg.grad is not None
        # load_state_dict copies in place
        other = cls(64, 32).cuda()
        layer.load_state_dict(other.state_dict())
        with torch.no_grad():
            assert torch.equal(layer(x), other(x))
        # dtype change replaces the storage
        layer.half()
        with torch.no_grad():
            yh = layer(x.half())
            assert yh.dtype == torch.float16 and torch.equal(yh, fresh_output(layer, x.half()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_cached_forwards_read_a_decode_tiled_copy_with_the_same_bits(dtype, monkeypatch):
    """A forward that may use the packed-weight cache runs on the decode-tiled copy the cache builds next to the packed
    bytes.  Up to 32 rows both layouts take the same kernel and the output equals the training forward's (which
    quantizes again and reads the row-major bytes) bit for bit; a larger batch may be routed to the streaming kernel
    on one layout and to the tiled GEMM on the other, whose fp32 sums differ in their last bits (held here to 4e-6 of the
    largest output in fp32 and to one unit in the last place of the largest output in 16 bits).
    BITTORCH_KERNEL=generic keeps the row-major bytes."""
    from bittorch_amd import _C
    from bittorch_amd.nn import TernaryLinear
    announce("tiled copy in the packed-weight cache", dtype)
    seen = {"tiled": 0}
    real = _C.ternary_linear_tiled_forward

    def counting(*a, **k):
        seen["tiled"] += 1
        return real(*a, **k)

    monkeypatch.setattr(_C, "ternary_linear_tiled_forward", counting)
    for (n, k) in [(32, 64), (250, 1032), (2560, 2560), (37, 100)]:
        torch.manual_seed(n + k)
        layer = TernaryLinear(k, n, backend="cuda").cuda().to(dtype)
        for rows in (1, 8, 200, 600):
            x = torch.randn(rows, k, device="cuda").to(dtype)
            before = seen["tiled"]
            y_train = layer(x)                      # gradient mode on, trainable weights: no cache
            assert seen["tiled"] == before
            with torch.no_grad():
                y_eval = layer(x)
            assert seen["tiled"] == before + 1
            if rows <= 32:
                assert torch.equal(y_train.detach(), y_eval)
            else:
                ulp = {torch.float32: 4e-6, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
                diff = (y_train.detach().float() - y_eval.float()).abs()
                assert float(diff.max()) <= ulp * float(y_eval.float().abs().max())
        packed, scale, tiled = layer._packed.value
        assert tiled is not None and torch.equal(_C.untile_weights(tiled, n, k), packed)
        monkeypatch.setenv("BITTORCH_KERNEL", "generic")
        before = seen["tiled"]
        with torch.no_grad():
            y_gen = layer(x)
        assert seen["tiled"] == before
        monkeypatch.delenv("BITTORCH_KERNEL")
        tol = {torch.float32: 1e-4, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dtype]
        assert torch.allclose(y_gen.float(), y_eval.float(), rtol=tol, atol=tol * float(y_eval.float().abs().max()))
