"""Seeded random shapes through the main entry points: every weight layout and activation order of the int8 family
must give the same accumulators and outputs, the accumulators must equal an exact integer product formed by torch,
the float family must sit within its output rounding of a float64 product (a single fp16 row: equal the correctly
rounded exact sum), and the row kernels' fast paths must equal the shape-generic kernel bit for bit.  The shapes are
drawn around the places where a launch changes its kernel, tile or remainder (16, 32, 96, 128, 384 ... rows; K in and
out of whole stages; N in and out of whole tiles)."""
import numpy as np
import pytest
import torch

from conftest import announce
from _util import set_option

pytestmark = pytest.mark.gpu

SPECIAL_M = [1, 2, 3, 15, 16, 17, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 255, 256, 257, 383, 384, 385, 511, 512,
             513, 1023, 1024, 1025]


def _rand_wt(n, k, dev):
    c = torch.randint(0, 3, (4, (k + 3) // 4, n), device=dev, dtype=torch.uint8)
    if k % 4:
        c[k % 4:, -1, :] = 0
    return (c[0] | (c[1] << 2) | (c[2] << 4) | (c[3] << 6)).contiguous()


def _pick_m(rng):
    return int(rng.choice(SPECIAL_M)) if rng.random() < 0.5 else int(rng.integers(1, 2200))


def _same(a, b):
    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("seed", [1, 2])
def test_int8_family_on_random_shapes(seed):
    from bittorch_amd import _C
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(seed)
    torch.manual_seed(seed)
    for it in range(20):
        m, n, k = _pick_m(rng), 4 * int(rng.integers(1, 1200)), 16 * int(rng.integers(1, 300))
        if rng.random() < 0.4:
            k = 128 * int(rng.integers(1, 40))
        if rng.random() < 0.3:
            n = 32 * int(rng.integers(1, 150))
        dt = [torch.float32, torch.bfloat16, torch.float16][int(rng.integers(0, 3))]
        announce("random int8", seed, it, m, n, k, dt)
        wt = _rand_wt(n, k, dev)
        w_dense = _C.unpack_dequant(wt, k, None, torch.int8).float()
        x = (torch.randn(m, k, device=dev) * (1 + 10 * torch.rand(m, 1, device=dev))).bfloat16()
        if m > 2:
            x[1] = 0
        scale = (torch.rand(n, device=dev) + 0.5) if rng.random() < 0.7 else (torch.rand(1, device=dev) + 0.5)
        bias = torch.randn(n, device=dev) if rng.random() < 0.5 else None
        res = torch.randn(m, n, device=dev).to(dt) if rng.random() < 0.4 else None
        q0, s0 = _C.act_quant_int8(x, False)
        q1, s1, rs = _C.act_quant_int8(x, True, return_rowsum=True)
        assert torch.equal(s0, s1) and torch.equal(rs, q0.int().sum(1).int())
        y_ref, a_ref = _C.ternary_gemm_int8(q0, s0, wt, scale, bias, k, dt, True, res, False)
        # |sum q w| <= 127 k < 2^24: the fp32 product is exact whatever order torch adds in
        assert torch.equal(a_ref, ((q0.float() @ w_dense.t()).to(torch.int64) * 127).to(torch.int32))
        y, a = _C.ternary_gemm_int8(q1, s1, wt, scale, bias, k, dt, True, res, True)
        assert _same(y, y_ref) and torch.equal(a, a_ref)
        tiled = _C.retile_weights(wt, k, False)
        assert torch.equal(_C.untile_weights(tiled, n, k), wt)
        for oo, (q, s) in ((False, (q0, s0)), (True, (q1, s1))):
            y, a = _C.ternary_gemm_int8_tiled(q, s, tiled, scale, bias, k, n, dt, True, res, oo)
            assert _same(y, y_ref) and torch.equal(a, a_ref)
        if k % 128 == 0:
            pairs = bool(n % 32 == 0 and rng.random() < 0.5)
            fields = _C.retile_fields(_C.retile_weights(wt, k, pairs), k, n)
            y, a = _C.ternary_gemm_int8_fields(q1, s1, rs, fields, scale, bias, k, n, dt, True, res, True, pairs)
            assert _same(y, y_ref) and torch.equal(a, a_ref)


@pytest.mark.parametrize("seed", [1, 2])
def test_float_family_on_random_shapes(seed):
    from bittorch_amd import _C
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(seed)
    torch.manual_seed(seed)
    for it in range(20):
        m = _pick_m(rng) if rng.random() < 0.7 else 1
        n, k = 4 * int(rng.integers(1, 800)), int(rng.integers(1, 3000))
        if rng.random() < 0.6:
            k = 16 * int(rng.integers(1, 260))
        xdt = [torch.float32, torch.bfloat16, torch.float16][int(rng.integers(0, 3))]
        announce("random float", seed, it, m, n, k, xdt)
        wt = _rand_wt(n, k, dev)
        w_dense = _C.unpack_dequant(wt, k, None, torch.int8).double()
        x = torch.randn(m, k, device=dev).to(xdt)
        scale = torch.rand(n, device=dev) * 0.05 + 0.01
        bias = (torch.randn(n, device=dev) * 0.1).to(xdt) if rng.random() < 0.5 else None
        acc64 = x.double() @ w_dense.t()
        ref = acc64 * scale.double() + (0 if bias is None else bias.double())
        floor = (acc64.abs().mean() + 1e-3) * scale.double().mean()
        tol = {torch.float32: 2e-5, torch.bfloat16: 1.2e-2, torch.float16: 2e-3}[xdt]
        y = _C.ternary_linear_packed_forward(x, wt, scale, bias, k)
        yt = _C.ternary_linear_tiled_forward(x, _C.retile_weights(wt, k, False), scale, bias, k, n)
        for out in (y, yt):
            assert float(((out.double() - ref).abs() / (ref.abs() + floor)).max()) < tol
        if m <= 32:  # both layouts take the same kernel
            assert _same(y, yt)
        if m == 1 and xdt == torch.float16 and k % 16 == 0:
            # the exact GEMV: the float64 sum is the exact sum here, rounded once to fp32, then the fp32 epilogue
            exact = (acc64.float() * scale + (0 if bias is None else bias.float())).half()
            assert _same(exact, y)


@pytest.mark.parametrize("seed", [1, 2])
def test_row_kernels_on_random_shapes(oracle, seed):
    from bittorch_amd import _C
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(seed)
    torch.manual_seed(seed)
    for it in range(24):
        b = int(rng.choice([1, 3, 17, 511, 2047, 2048, 2049, 4095, 4096, 4097])) if rng.random() < 0.5 else int(rng.integers(1, 6000))
        k = 8 * int(rng.integers(1, 900)) if rng.random() < 0.8 else int(rng.integers(1, 5000))
        if rng.random() < 0.3:
            k = int(rng.choice([512, 1024, 1536, 2048, 2056, 2560, 3072, 3080, 4096, 6912]))
        dt = [torch.float32, torch.float16, torch.bfloat16][int(rng.integers(0, 3))]
        announce("random rows", seed, it, b, k, dt)
        g = (torch.randn(b, k, device=dev) * (1 + 5 * torch.rand(b, 1, device=dev))).to(dt)
        u = torch.randn(b, k, device=dev).to(dt)
        if b > 2:
            u[1] = 0
        w = (1 + 0.1 * torch.randn(k, device=dev)).to(dt)
        oo = bool(k % 16 == 0 and rng.random() < 0.5)
        q, s, rs = _C.act_quant_int8(g, oo, True)
        qn, sn = _C.act_quant_int8(g, False)
        assert torch.equal(rs, qn.int().sum(1).int()) and torch.equal(s, sn)
        if oo:
            assert torch.equal(q.view(b, k // 16, 4, 4), qn.view(b, k // 16, 4, 4).transpose(2, 3))
        if b * k <= 1_500_000:
            oq, os_ = oracle.act_quant_i8(g.float().cpu().numpy())
            assert np.array_equal(qn.cpu().numpy(), oq) and np.array_equal(sn.cpu().numpy(), os_)
        fast = (_C.swiglu(g, u, store=True, quantize=True, operand_order=oo, return_rowsum=True),
                _C.rmsnorm(g, w, 1e-5, store=True, quantize=True, operand_order=oo, return_rowsum=True))
        plain = (_C.swiglu(g, u), _C.rmsnorm(g, w, 1e-5))
        set_option("ROWOP_GENERIC", "1")
        try:
            generic = (_C.swiglu(g, u, store=True, quantize=True, operand_order=oo, return_rowsum=True),
                       _C.rmsnorm(g, w, 1e-5, store=True, quantize=True, operand_order=oo, return_rowsum=True))
        finally:
            set_option("ROWOP_GENERIC", None)
        for a, c, p_ in zip(fast, generic, plain):
            assert all(_same(x_, y_) for x_, y_ in zip(a, c)) and _same(p_, a[0])
