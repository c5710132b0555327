"""GPU robustness of the module path on the HIP kernels: the edge cases the reference pins in
tests/test_robustness.py:160-260, :284-400 and tests/test_kernel_regression.py:37-190 (zero,
tiny and huge inputs, constant weights, masked outputs in backward, batched == looped,
big shapes, multi-step training, kernel selection by BITTORCH_KERNEL)."""
import os

import pytest
import torch

from conftest import announce
from _util import random_ternary, seeded_acts

pytestmark = pytest.mark.gpu


def _layer(i, o, **kw):
    from bittorch_amd.nn import TernaryLinear
    torch.manual_seed(0)
    return TernaryLinear(i, o, backend="cuda", **kw).cuda()


def test_zero_tiny_and_huge_inputs():
    announce("robustness inputs")
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        layer = _layer(32, 16).to(dtype)
        y = layer(torch.zeros(4, 32, device="cuda", dtype=dtype))
        assert torch.equal(y, layer.bias.detach().unsqueeze(0).expand(4, -1))
        for mag in (1e-7, 1e3):
            y = layer((torch.randn(4, 32, device="cuda") * mag).to(dtype))
            assert torch.isfinite(y).all()
    layer = _layer(32, 16)
    y = layer(torch.randn(4, 32, device="cuda") * 1e4)
    assert torch.isfinite(y).all()


def test_constant_and_signed_weights():
    announce("robustness weights")
    layer = _layer(32, 16, threshold_factor=0.05)
    with torch.no_grad():
        layer.weight.fill_(0.05)            # every weight equals its row maximum -> all +1
    x = torch.randn(4, 32, device="cuda")
    y = layer(x)
    ref = x.sum(dim=1, keepdim=True) * 0.05 + layer.bias
    assert torch.allclose(y, ref, atol=1e-5)
    with torch.no_grad():
        layer.weight[:8] = layer.weight[:8].abs() * 2 + 0.1
        layer.weight[8:] = -(layer.weight[8:].abs() * 2 + 0.1)
    w_tern, _ = layer.get_quantized_weight()
    assert (w_tern[:8] == 1).all() and (w_tern[8:] == -1).all()
    assert torch.isfinite(layer(x)).all()
    with torch.no_grad():
        layer.weight.zero_()                 # all-zero rows: scale floor, codes 0, output = bias
    assert torch.equal(layer(x), layer.bias.detach().unsqueeze(0).expand(4, -1))


def test_backward_through_masked_outputs_and_noncontiguous_inputs():
    announce("robustness backward")
    layer = _layer(32, 16)
    x = torch.randn(4, 32, device="cuda", requires_grad=True)
    mask = torch.tensor([1, 0] * 8, device="cuda").float()
    (layer(x) * mask).sum().backward()
    assert torch.isfinite(x.grad).all() and torch.isfinite(layer.weight.grad).all()
    assert layer.bias.grad.tolist() == [4.0, 0.0] * 8
    # non-contiguous and 3-D inputs take the same path as their contiguous copies
    big = torch.randn(6, 5, 64, device="cuda")
    xs = big[:, :, ::2]
    assert not xs.is_contiguous()
    with torch.no_grad():
        assert torch.equal(layer(xs), layer(xs.contiguous()))
        assert layer(xs).shape == (6, 5, 16)


def test_batched_equals_looped_all_kernels():
    """Rows are independent in every kernel: one row at a time (streaming kernel) and 48 rows at
    once (tiled kernel) give the same rows up to the fp32 summation order."""
    announce("robustness batched vs looped")
    for dtype, tol in ((torch.float32, 1e-5), (torch.float16, 2e-3), (torch.bfloat16, 2e-2)):
        layer = _layer(256, 128).to(dtype)
        x = torch.randn(48, 256, device="cuda").to(dtype)
        with torch.no_grad():
            yb = layer(x)
            yl = torch.cat([layer(x[i:i + 1]) for i in range(48)])
        # different kernels sum in a different order; 16-bit outputs are rounded
        assert (yb.float() - yl.float()).abs().max() <= tol * yl.float().abs().max()


@pytest.mark.parametrize("shape", [(8, 4096, 4096), (512, 1024, 4096), (64, 11008, 4096)])
def test_big_shape_forward_backward(shape):
    b, i, o = shape
    announce("robustness big", shape)
    layer = _layer(i, o)
    x = torch.randn(b, i, device="cuda", requires_grad=True)
    y = layer(x)
    assert y.shape == (b, o) and torch.isfinite(y).all()
    y.float().pow(2).mean().backward()
    assert torch.isfinite(x.grad).all() and torch.isfinite(layer.weight.grad).all()
    # forward equals the plain torch backend of the same layer
    layer.backend = "python"
    with torch.no_grad():
        ref = layer(x.detach())
    assert (y.detach() - ref).abs().max() <= 1e-3 * ref.abs().max()


def test_multi_step_training_is_stable():
    announce("robustness training")
    torch.manual_seed(0)
    from bittorch_amd.nn import TernaryLinear
    model = torch.nn.Sequential(TernaryLinear(64, 128), torch.nn.ReLU(), TernaryLinear(128, 10)).cuda()
    opt = torch.optim.Adam(model.parameters(), lr=1e-2)
    x = torch.randn(256, 64, device="cuda")
    target = (x[:, :10] > 0).float()
    first = None
    for step in range(60):
        loss = torch.nn.functional.binary_cross_entropy_with_logits(model(x), target)
        opt.zero_grad()
        loss.backward()
        opt.step()
        assert torch.isfinite(loss)
        first = first if first is not None else float(loss.detach())
    assert float(loss.detach()) < 0.7 * first


def test_kernel_selection_env_matches_default():
    """BITTORCH_KERNEL is read on every call (tests/test_kernel_regression.py:17-34 flips it at run
    time): the generic kernel and the default dispatch agree."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("robustness kernel env")
    g = torch.Generator().manual_seed(4)
    old = os.environ.get("BITTORCH_KERNEL")
    try:
        for (b, n, k) in ((1, 64, 64), (7, 100, 36), (32, 512, 256), (128, 256, 1024)):
            w = torch.randint(-1, 2, (n, k), generator=g).float()
            packed = pack_ternary_transposed(w)[0].cuda()
            scale = (torch.rand(n, generator=g) + 0.5).half().cuda()
            x = torch.randn(b, k, generator=g).half().cuda()
            os.environ["BITTORCH_KERNEL"] = "generic"
            y_gen = _C.ternary_linear_packed_forward(x, packed, scale, None, k)
            os.environ["BITTORCH_KERNEL"] = "auto"
            y_def = _C.ternary_linear_packed_forward(x, packed, scale, None, k)
            assert (y_gen.float() - y_def.float()).abs().max() <= 1e-2 * y_gen.float().abs().max()
    finally:
        if old is None:
            os.environ.pop("BITTORCH_KERNEL", None)
        else:
            os.environ["BITTORCH_KERNEL"] = old


@pytest.mark.parametrize("n,k", [(128256, 4096), (50257, 768), (8192, 28672)])
def test_vocabulary_wide_and_very_deep_layers(n, k):
    """Output widths of a vocabulary projection (one of them odd: byte-granular loads) and a K beyond
    any FFN: both paths against a dense fp32 product of the dequantized weights."""
    from bittorch_amd import _C
    announce("wide / deep layer", n, k)
    dev = torch.device("cuda")
    w = torch.randn(n, k, device=dev, generator=torch.Generator(device="cuda").manual_seed(n)) * 0.02
    packed, scale, _ = _C.ternary_quantize_pack(w, 0.05, True)
    wd = _C.unpack_dequant(packed, k, scale, torch.float32)
    del w
    for m in (1, 7, 64):
        x = torch.randn(m, k, device=dev).bfloat16()
        ref = x.float() @ wd.t()
        y = _C.ternary_linear_packed_forward(x, packed, scale, None, k)
        assert ((y.float() - ref).abs().max() / ref.abs().max()).item() < 1e-2
        y8 = _C.ternary_linear_tensor_core_forward(x, packed, scale, None, k, 2)
        assert ((y8.float() - ref).abs().max() / ref.abs().max()).item() < 5e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_operands_that_start_inside_a_buffer(dtype):
    """Activations, scale, bias and residual handed over as views that start 1, 3 or 4 elements into a buffer (not
    16-byte aligned), rows that are a column slice of a wider matrix, a 3-D batch: the same results as the aligned
    call -- bit for bit on the integer paths, to the output rounding where another kernel takes the call."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed

    def off_view(t, off):
        buf = torch.empty(t.numel() + off, dtype=t.dtype, device=t.device)
        buf[off:] = t.reshape(-1)
        return buf[off:].view(t.shape)

    announce("offset operands", dtype)
    tol = {torch.float32: 3e-5, torch.bfloat16: 1.6e-2, torch.float16: 2e-3}[dtype]
    for (m, n, k) in [(1, 256, 512), (7, 100, 72), (40, 520, 1040), (130, 64, 333)]:
        w = random_ternary(n, k, seed=m + n)
        packed = pack_ternary_transposed(w)[0].cuda()
        x = seeded_acts(m, k, seed=3, dtype=dtype).cuda()
        scale = (torch.rand(n, generator=torch.Generator().manual_seed(1)) * 0.05 + 0.01).cuda()
        bias = seeded_acts(1, n, seed=4, dtype=dtype).reshape(-1).cuda()
        res = seeded_acts(m, n, seed=5, dtype=dtype).cuda()
        y0 = _C.ternary_linear_packed_forward(x, packed, scale, bias, k, res)
        for off in (1, 3, 4):
            y1 = _C.ternary_linear_packed_forward(off_view(x, off), packed, off_view(scale, off), off_view(bias, off), k,
                                                  off_view(res, off))
            assert float((y1.double() - y0.double()).abs().max()) <= tol * float(y0.double().abs().max())
            q0, s0 = _C.act_quant_int8(x)
            q1, s1 = _C.act_quant_int8(off_view(x, off))
            assert torch.equal(q0, q1) and torch.equal(s0, s1)
            u = seeded_acts(m, k, seed=6, dtype=dtype).cuda()
            a0 = _C.swiglu(x, u, store=True, quantize=True)
            a1 = _C.swiglu(off_view(x, off), off_view(u, off), store=True, quantize=True)
            assert all(torch.equal(p, q) for p, q in zip(a0, a1))
            if k % 16 == 0:
                y8 = _C.ternary_gemm_int8(q0, s0, packed, scale, bias.float(), k, dtype, True, res)
                y9 = _C.ternary_gemm_int8(q0, off_view(s0, off), packed, off_view(scale, off), off_view(bias.float(), off), k,
                                          dtype, True, off_view(res, off))
                assert torch.equal(y8[0], y9[0]) and torch.equal(y8[1], y9[1])
        wide = seeded_acts(m, k + 24, seed=7, dtype=dtype).cuda()
        xs = wide[:, 8:8 + k]
        y2 = _C.ternary_linear_packed_forward(xs, packed, scale, bias, k)
        y3 = _C.ternary_linear_packed_forward(xs.contiguous(), packed, scale, bias, k)
        assert float((y2.double() - y3.double()).abs().max()) <= tol * float(y3.double().abs().max())
        qa, sa = _C.act_quant_int8(xs)
        qb, sb = _C.act_quant_int8(xs.contiguous())
        assert torch.equal(qa, qb) and torch.equal(sa, sb)
