"""GPU parity: packed fp32-accumulate forward (decode GEMV / small batch / generic)
vs the CPU oracle.  Tolerances: <= 1e-3 (fp32 out), <= 1e-2 (fp16/bf16 out),
relative to the largest output magnitude; the float64 oracle is the truth the
fp32-accumulate oracle itself is also measured against."""
import os

import numpy as np
import pytest
import torch

from conftest import announce
from _util import assert_close_like_reference, f32np, random_ternary, rel_err, seeded_acts, seeded_weights, set_option

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-3, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def _case(oracle, b, n, k, dtype, bias=True, seed=0, scale_dtype=None, per_tensor=False):
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    w = random_ternary(n, k, seed=seed)
    g = torch.Generator().manual_seed(seed + 7)
    scale = (torch.rand(1 if per_tensor else n, generator=g) * 0.05 + 0.01)
    bias_t = (torch.randn(n, generator=g) * 0.01) if bias else None
    x = seeded_acts(b, k, seed=seed + 3, dtype=dtype)
    packed, _ = pack_ternary_transposed(w)
    sdt = scale_dtype or dtype
    scale_d = scale.to(sdt)
    bias_d = None if bias_t is None else bias_t.to(dtype)
    y = _C.ternary_linear_packed_forward(x.cuda(), packed.cuda(), scale_d.cuda(),
                                         None if bias_d is None else bias_d.cuda(), k)
    torch.cuda.synchronize()
    assert y.dtype == dtype and tuple(y.shape) == (b, n)
    args = (f32np(x), packed.numpy(), f32np(scale_d), k, None if bias_d is None else f32np(bias_d))
    truth = oracle.linear_packed(*args, f64=True)
    ref = oracle.linear_packed(*args)
    got = f32np(y)
    # the oracle's own distance from the truth bounds what fp32 accumulation may cost
    assert rel_err(ref, truth) < 1e-5
    assert rel_err(got, truth) < TOL[dtype], (b, n, k, dtype)
    assert_close_like_reference(got, truth, dtype)
    return got, ref.astype(np.float32)


def test_config2_decode_gemv_fp16(oracle):
    """x fp16 [1,4096] x W [4096,4096], per-tensor fp32 scale, fp16 bias."""
    announce("config2 gemv fp16")
    from bittorch_amd import _C
    w = seeded_weights(4096, 4096, seed=0).cuda()
    packed, scale, _ = _C.ternary_quantize_pack(w, 0.05, per_channel=False)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, 4096, generator=g).half()
    bias = (torch.randn(4096, generator=g) * 0.01).half()
    y = _C.ternary_linear_packed_forward(x.cuda(), packed, scale.reshape(1), bias.cuda(), 4096)
    torch.cuda.synchronize()
    truth = oracle.linear_packed(f32np(x), packed.cpu().numpy(), f32np(scale.reshape(1)), 4096,
                                 f32np(bias), f64=True)
    assert rel_err(f32np(y), truth) < 1e-2
    # fp16 output of the exactly rounded result differs from ours by at most 1 ulp-ish
    exact16 = torch.from_numpy(truth).to(torch.float16).float().numpy()
    assert np.mean(exact16 != f32np(y)) < 0.02


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("b,n,k", [(1, 64, 64), (4, 16, 8), (8, 32, 64), (1, 4096, 4096), (16, 1024, 4096),
                                   (3, 256, 11008), (16, 512, 512), (33, 128, 256), (64, 256, 768),
                                   (2, 48, 100), (5, 40, 36)])
def test_packed_forward_shapes(oracle, dtype, b, n, k):
    announce("packed_forward", dtype, b, n, k)
    _case(oracle, b, n, k, dtype, seed=b + n + k)


@pytest.mark.parametrize("k", [1, 2, 3, 5, 6, 7, 9, 13, 17, 31, 65])
@pytest.mark.parametrize("n", [4, 32, 67])
def test_packed_forward_ragged_k_and_n(oracle, k, n):
    announce("packed_forward ragged", n, k)
    for dtype in (torch.float32, torch.float16):
        _case(oracle, 3, n, k, dtype, seed=k)


@pytest.mark.parametrize("b", [1, 2, 4, 8, 15, 16, 17, 32, 64])
def test_packed_forward_batch_sizes(oracle, b):
    announce("packed_forward batch", b)
    _case(oracle, b, 128, 256, torch.float16, seed=b)
    _case(oracle, b, 128, 256, torch.bfloat16, seed=b)


@pytest.mark.parametrize("route", ["auto", "gemm"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("b,n,k", [(128, 256, 64), (33, 128, 256), (200, 260, 72), (129, 512, 1000), (512, 1024, 4096),
                                   (130, 36, 8), (257, 300, 136), (64, 256, 768)])
def test_packed_forward_tall_batches_use_the_tiled_kernel(oracle, dtype, b, n, k, route, monkeypatch):
    """Batches above the streaming kernel's limit go to the 16-bit matrix-core GEMM: partial row
    and column tiles, K tails that are not a multiple of the 64-wide stage, odd last stages."""
    if route == "gemm":  # batches beyond 32 rows to the tiled GEMM whatever their size (the default rule streams small outputs)
        set_option("STREAM_MAX_ROWS", "32")
    announce("packed_forward tall", dtype, b, n, k)
    _case(oracle, b, n, k, dtype, seed=b + n + k)


def test_packed_forward_tall_batch_matches_streaming_kernel(oracle):
    """The tiled kernel and the streaming kernel (forced by splitting the batch into 16-row
    calls) see the same exact products; they differ by fp32 summation order only."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("packed_forward tall vs stream")
    g = torch.Generator().manual_seed(5)
    n, k, b = 512, 2048, 256
    w = torch.randint(-1, 2, (n, k), generator=g).float()
    packed = pack_ternary_transposed(w)[0].cuda()
    scale = (torch.rand(n, generator=g) + 0.5).cuda()
    for dtype in (torch.float16, torch.bfloat16):
        x = torch.randn(b, k, generator=g).to(dtype).cuda()
        y_tiled = _C.ternary_linear_packed_forward(x, packed, scale, None, k)
        y_stream = torch.cat([_C.ternary_linear_packed_forward(x[i:i + 16].contiguous(), packed, scale, None, k)
                              for i in range(0, b, 16)])
        ref = (x.double() @ w.double().cuda().T) * scale.double()
        denom = ref.abs().max()
        assert ((y_tiled.double() - ref).abs().max() / denom) < 1e-2
        assert ((y_tiled.double() - y_stream.double()).abs().max() / denom) < 1e-2


def test_packed_forward_any_number_of_rows(oracle, monkeypatch):
    """The shape-generic kernel takes any batch, more rows than a grid dimension holds included (fp32, the
    reference's MNIST layer 784 -> 256 cut to 16 columns), and is bit-exact against the oracle.  The streaming
    kernel serves a call beyond its 65535 row blocks in slices."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("packed_forward many rows")
    n, k = 16, 784
    w = random_ternary(n, k, seed=1)
    packed = pack_ternary_transposed(w)[0]
    scale = torch.rand(n) * 0.05 + 0.01
    bias = torch.randn(n) * 0.01
    monkeypatch.setenv("BITTORCH_KERNEL", "generic")
    for b in (3, 70000):
        x = seeded_acts(b, k, seed=b)
        y = _C.ternary_linear_packed_forward(x.cuda(), packed.cuda(), scale.cuda(), bias.cuda(), k)
        ref = oracle.linear_packed(f32np(x), packed.numpy(), f32np(scale), k, f32np(bias))
        np.testing.assert_array_equal(f32np(y), ref)
    # dense int8 weights on the generic route, same batch
    x = seeded_acts(70000, k, seed=5)
    y = _C.ternary_linear_forward(x.cuda(), w.cuda(), scale.cuda(), bias.cuda())
    np.testing.assert_array_equal(f32np(y), oracle.linear_unpacked(f32np(x), w.numpy(), f32np(scale), f32np(bias)))
    monkeypatch.delenv("BITTORCH_KERNEL")
    # streaming kernel, 16 * 65535 + 40 rows
    set_option("STREAM_MAX_ROWS", "2000000")
    b, k2 = 16 * 65535 + 40, 64
    packed2 = pack_ternary_transposed(random_ternary(n, k2, seed=2))[0].cuda()
    xb = torch.randn(b, k2, device="cuda").bfloat16()
    yb = _C.ternary_linear_packed_forward(xb, packed2, scale.cuda(), bias.cuda(), k2)
    for r0 in (0, 16 * 65535 - 8, b - 24):
        part = _C.ternary_linear_packed_forward(xb[r0:r0 + 24].contiguous(), packed2, scale.cuda(), bias.cuda(), k2)
        assert torch.equal(yb[r0:r0 + 24], part)


@pytest.mark.parametrize("b,n,k", [(1, 256, 784), (64, 256, 784), (3, 16, 20), (17, 100, 1), (5, 36, 63), (40, 64, 65),
                                   (2, 8, 130), (1200, 256, 784), (70000, 16, 784), (4096, 512, 1000)])
def test_packed_forward_fp32_any_k_on_the_matrix_cores(oracle, b, n, k):
    """fp32 activations whose K is not a multiple of 64 (the reference's MNIST layer, 784 -> 256) run the matrix-core
    kernels on zero-padded bf16 planes: every element within the reference tests' fp32 thresholds
    (tests/test_packed_kernel.py:44-50) of the oracle's k-ordered fp32 sum, both weight layouts, the streaming kernel
    and the tiled GEMM; equal to the float64 dot product to a few fp32 roundings."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("packed_forward fp32 padded planes", b, n, k)
    w = random_ternary(n, k, seed=n + k)
    packed = pack_ternary_transposed(w)[0]
    g = torch.Generator().manual_seed(b + k)
    scale = torch.rand(n, generator=g) * 0.05 + 0.01
    bias = torch.randn(n, generator=g) * 0.01
    x = seeded_acts(b, k, seed=b + 1)
    xd, pd, sd, bd = x.cuda(), packed.cuda(), scale.cuda(), bias.cuda()
    y = _C.ternary_linear_packed_forward(xd, pd, sd, bd, k)
    rows = slice(0, b) if b <= 4096 else slice(b - 100, b)
    ref = oracle.linear_packed(f32np(x[rows]), packed.numpy(), f32np(scale), k, f32np(bias))
    assert_close_like_reference(f32np(y[rows]), ref, torch.float32)
    exact = (x.double() @ w.double().T) * scale.double() + bias.double()
    assert float((y.cpu().double() - exact).abs().max()) <= 4e-6 * float(exact.abs().max()) + 1e-7
    tiled = _C.retile_weights(pd, k)
    y_t = _C.ternary_linear_tiled_forward(xd, tiled, sd, bd, k, n)
    # (the same kernel on either layout gives the same bits; where the dispatch picks the GEMM for one layout and the
    # streaming kernel for the other, the sums differ in their order)
    assert float((y_t.cpu().double() - exact).abs().max()) <= 4e-6 * float(exact.abs().max()) + 1e-7
    assert_close_like_reference(f32np(y_t[rows]), ref, torch.float32)
    # an unaligned activation base (a view one element into a buffer): element-wise plane split
    if b * k < 1 << 20:
        buf = torch.zeros(b * k + 1, device="cuda")
        buf[1:] = xd.reshape(-1)
        y_u = _C.ternary_linear_packed_forward(buf[1:].view(b, k), pd, sd, bd, k)
        assert torch.equal(y_u, y)


def test_packed_forward_fp32_generic_is_bit_exact(oracle, monkeypatch):
    """The generic kernel accumulates in the reference's k order: equal to the oracle bit for bit
    (shapes whose K is a multiple of 64 take the matrix-core route by default, so it is forced)."""
    announce("packed_forward fp32 bit exact")
    monkeypatch.setenv("BITTORCH_KERNEL", "generic")
    for (b, n, k) in [(32, 256, 512), (7, 33, 17), (1, 1, 1), (2, 100, 1000)]:
        got, ref = _case(oracle, b, n, k, torch.float32, seed=11)
        np.testing.assert_array_equal(got, ref)


@pytest.mark.parametrize("route", ["auto", "gemm"])
@pytest.mark.parametrize("b,n,k", [(1, 4096, 4096), (1, 64, 64), (5, 100, 128), (16, 512, 1024), (33, 256, 192),
                                   (200, 260, 448), (512, 1024, 4096)])
def test_packed_forward_fp32_on_the_matrix_cores(oracle, b, n, k, monkeypatch, route):
    """fp32 activations with K % 64 == 0 are split into three exact bf16 planes and run on the bf16
    kernels (streaming kernel up to 32 rows, tiled kernel above): every product is exact, only the
    fp32 summation order differs from the generic kernel - far inside the 1e-3 budget for fp32."""
    if route == "gemm":  # batches beyond 32 rows to the tiled GEMM whatever their size (the default rule streams small outputs)
        set_option("STREAM_MAX_ROWS", "32")
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("packed_forward fp32 planes", b, n, k)
    w = random_ternary(n, k, seed=k + n)
    g = torch.Generator().manual_seed(b + 1)
    scale = torch.rand(n, generator=g) * 0.05 + 0.01
    bias = torch.randn(n, generator=g) * 0.01
    # activations spanning many binades, so that all three planes carry information
    x = torch.randn(b, k, generator=g) * torch.exp(torch.randn(b, k, generator=g) * 3)
    packed = pack_ternary_transposed(w)[0]
    y = _C.ternary_linear_packed_forward(x.cuda(), packed.cuda(), scale.cuda(), bias.cuda(), k)
    assert y.dtype == torch.float32
    truth = oracle.linear_packed(f32np(x), packed.numpy(), f32np(scale), k, f32np(bias), f64=True)
    assert rel_err(f32np(y), truth) < 1e-5
    monkeypatch.setenv("BITTORCH_KERNEL", "generic")
    y_gen = _C.ternary_linear_packed_forward(x.cuda(), packed.cuda(), scale.cuda(), bias.cuda(), k)
    assert rel_err(f32np(y), f32np(y_gen)) < 1e-5


def test_f32_plane_split_is_exact():
    """hi + mid + lo reproduces every fp32 activation exactly: with identity-like weights
    (one +1 per output) the matrix-core route returns the inputs themselves."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("packed_forward fp32 planes exact")
    k = n = 128
    g = torch.Generator().manual_seed(3)
    x = torch.randn(8, k, generator=g) * torch.exp(torch.randn(8, k, generator=g) * 6)
    x[0, :4] = torch.tensor([0.0, -0.0, 1.0, -1.0])
    x[1, :4] = torch.tensor([3.4028235e38, -3.4028235e38, 1e-30, -7e-25])
    perm = torch.randperm(k, generator=g)
    w = torch.zeros(n, k)
    w[torch.arange(n), perm] = 1.0
    packed = pack_ternary_transposed(w)[0].cuda()
    y = _C.ternary_linear_packed_forward(x.cuda(), packed, torch.ones(n).cuda(), None, k)
    assert torch.equal(y.cpu(), x[:, perm])


def test_packed_forward_mixed_scale_dtypes(oracle):
    announce("packed_forward scale dtypes")
    _case(oracle, 1, 256, 512, torch.float16, scale_dtype=torch.float32, per_tensor=True)
    _case(oracle, 4, 256, 512, torch.bfloat16, scale_dtype=torch.float32)
    _case(oracle, 4, 256, 512, torch.float16, bias=False)


def test_packed_forward_known_answers(oracle):
    """All-zero weights give the bias; all-ones weights give row sums; reserved code 3 is zero."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("packed_forward known answers")
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        x = seeded_acts(4, 64, seed=2, dtype=dtype).cuda()
        bias = torch.linspace(-1, 1, 32).to(dtype).cuda()
        ones_scale = torch.ones(32, dtype=dtype).cuda()
        zeros = pack_ternary_transposed(torch.zeros(32, 64))[0].cuda()
        y = _C.ternary_linear_packed_forward(x, zeros, ones_scale, bias, 64)
        assert torch.equal(y, bias.expand(4, 32))
        threes = torch.full_like(zeros, 0xFF)
        y = _C.ternary_linear_packed_forward(x, threes, ones_scale, bias, 64)
        assert torch.equal(y, bias.expand(4, 32))
        ones = pack_ternary_transposed(torch.ones(32, 64))[0].cuda()
        y = _C.ternary_linear_packed_forward(x, ones, ones_scale, None, 64)
        ref = x.float().sum(dim=1, keepdim=True).expand(4, 32)
        assert torch.allclose(y.float(), ref, rtol=1e-2, atol=1e-2)
    # the reference's JS known-answer vectors
    wts = torch.tensor([[1, -1, 0, 0], [-1, 1, 0, 0]], dtype=torch.float32)
    p = pack_ternary_transposed(wts)[0].cuda()
    x = torch.tensor([[10.0, 3.0, 0.0, 0.0]]).cuda()
    y = _C.ternary_linear_packed_forward(x, p, torch.ones(2).cuda(), None, 4)
    assert y.tolist() == [[7.0, -7.0]]
    wts = torch.tensor([[1, 0, 0, 0], [0, 1, 0, 0]], dtype=torch.float32)
    p = pack_ternary_transposed(wts)[0].cuda()
    x = torch.tensor([[4.0, 8.0, 0.0, 0.0]]).cuda()
    y = _C.ternary_linear_packed_forward(x, p, torch.tensor([2.0, 0.5]).cuda(), None, 4)
    assert y.tolist() == [[8.0, 4.0]]


def test_packed_forward_stream_configs_agree(oracle):
    """Every tile width / wave count of the streaming kernel gives the same sums
    (exact decode; fp32 sums differ only by association)."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("packed_forward stream configs")
    w = random_ternary(512, 1024, seed=4)
    packed = pack_ternary_transposed(w)[0].cuda()
    x = seeded_acts(5, 1024, seed=5, dtype=torch.float16).cuda()
    scale = torch.ones(512, dtype=torch.float16).cuda()
    truth = oracle.linear_packed(f32np(x), packed.cpu().numpy(), f32np(scale), 1024, f64=True)
    try:
        for cfg in ("16,4", "16,1", "8,8", "8,2", "4,4", "4,16", "2,8", "2,16", "1,1", "1,4", "1,16"):
            set_option("STREAM_CFG", cfg)
            y = _C.ternary_linear_packed_forward(x, packed, scale, None, 1024)
            torch.cuda.synchronize()
            assert rel_err(f32np(y), truth) < 2e-3, cfg
    finally:
        set_option("STREAM_CFG", None)


def test_unpacked_forward_matches_oracle(oracle, monkeypatch):
    """Dense int8 weights: by default they are packed on the device and take the packed kernels
    (exact products, fp32 sums in a different order); the dense generic kernel sums in the
    reference's k order, bit for bit."""
    from bittorch_amd import _C
    announce("unpacked forward")
    for (b, n, k) in [(4, 8, 16), (1, 1, 1), (17, 67, 123), (32, 256, 512), (200, 128, 192)]:
        w = random_ternary(n, k, seed=k)
        g = torch.Generator().manual_seed(1)
        scale = torch.rand(n, generator=g)
        bias = torch.randn(n, generator=g)
        x = seeded_acts(b, k, seed=2)
        ref = oracle.linear_unpacked(f32np(x), w.numpy(), f32np(scale), f32np(bias))
        ref16 = oracle.linear_unpacked(f32np(x.half()), w.numpy(), f32np(scale.half()), None)
        for forced in (False, True):
            if forced:
                monkeypatch.setenv("BITTORCH_KERNEL", "generic")
            else:
                monkeypatch.delenv("BITTORCH_KERNEL", raising=False)
            y = _C.ternary_linear_forward(x.cuda(), w.cuda(), scale.cuda(), bias.cuda())
            if forced:
                np.testing.assert_array_equal(f32np(y), ref)
            else:
                assert rel_err(f32np(y), ref) < 1e-5
            y16 = _C.ternary_linear_forward(x.half().cuda(), w.cuda(), scale.half().cuda(), None)
            assert y16.dtype == torch.float16
            assert rel_err(f32np(y16), ref16) < 1e-2


def test_device_pack_of_dense_ternary_weights():
    """bt_pack_ternary_i8 writes the bytes of pack_ternary_transposed, for ragged shapes too."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("pack_ternary_int8")
    for (n, k) in [(1, 1), (16, 4), (33, 17), (67, 123), (256, 512), (100, 1000), (4096, 1024)]:
        w = random_ternary(n, k, seed=n + k)
        got = _C.pack_ternary_int8(w.cuda())
        want, _ = pack_ternary_transposed(w)
        assert torch.equal(got.cpu(), want), (n, k)
