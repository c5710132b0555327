"""GPU parity of the fused block glue: SwiGLU, RMSNorm (each with the optional per-row int8
quantization) and the residual folded into the GEMM epilogues.

* against the CPU oracle: bit-exact (values on the dtype's grid, int8 codes, activation scales);
* against torch's own unfused ops on the GPU: equal up to one unit in the last place of the
  tensor dtype (torch's silu uses the device library's exp, this library a fixed polynomial);
* the residual: bit-exact against "linear, then add" on every kernel path.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import announce
from _util import BT_DT, f32np, random_ternary, seeded_acts, set_option

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# fast path (row in registers), K % 8 != 0 (generic), largest fast K, beyond it (generic)
SHAPES = [(1, 8), (3, 7), (5, 520), (16, 4096), (4, 6912), (2, 16384), (2, 20000)]


def _ulp_close(got, ref, dtype, ulps=1):
    got, ref = got.float(), ref.float()
    if dtype == torch.float32:
        tol = torch.abs(ref) * (ulps * 2.0 ** -23) + 1e-37
    elif dtype == torch.float16:
        tol = torch.clamp(torch.abs(ref) * (ulps * 2.0 ** -10), min=ulps * 2.0 ** -24)
    else:
        tol = torch.abs(ref) * (ulps * 2.0 ** -7) + 1e-37
    bad = torch.abs(got - ref) > tol
    return int(bad.sum())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("b,k", SHAPES)
def test_swiglu_matches_oracle_bit_for_bit(oracle, dtype, b, k):
    from bittorch_amd import _C
    announce("swiglu", dtype, b, k)
    g = seeded_acts(b, k, seed=b + k, dtype=dtype, outliers=True) * 3
    u = seeded_acts(b, k, seed=b + k + 1, dtype=dtype)
    if b > 2:
        u[1] = 0  # all-zero product row: scale 1, codes 0
    h, q, s = _C.swiglu(g.cuda(), u.cuda(), store=True, quantize=True)
    torch.cuda.synchronize()
    oh, oq, os_ = oracle.swiglu(f32np(g), f32np(u), BT_DT[dtype])
    np.testing.assert_array_equal(f32np(h), oh)
    np.testing.assert_array_equal(s.cpu().numpy(), os_)
    np.testing.assert_array_equal(q.cpu().numpy(), oq)
    # the quantized output alone, and the stored output alone, are the same values
    q2, s2 = _C.swiglu(g.cuda(), u.cuda(), store=False, quantize=True)
    h2 = _C.swiglu(g.cuda(), u.cuda())
    assert torch.equal(q2, q) and torch.equal(s2, s) and torch.equal(h2, h)


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_against_torch_ops(dtype):
    from bittorch_amd import _C
    announce("swiglu vs torch", dtype)
    g = (seeded_acts(64, 6912, seed=3, dtype=dtype, outliers=True) * 3).cuda()
    u = seeded_acts(64, 6912, seed=4, dtype=dtype).cuda()
    ref = F.silu(g) * u
    got = _C.swiglu(g, u)
    # fp32: two different exp implementations (each below 1 ulp), one add, one divide, one multiply
    assert _ulp_close(got, ref, dtype, ulps=4 if dtype == torch.float32 else 1) == 0
    # and the fused quantization is the stand-alone quantizer applied to the stored product
    q, s = _C.swiglu(g, u, store=False, quantize=True)
    q_ref, s_ref = _C.act_quant_int8(got)
    assert torch.equal(q, q_ref) and torch.equal(s, s_ref)


def test_swiglu_special_values():
    from bittorch_amd import _C
    g = torch.tensor([[0.0, -0.0, 100.0, -100.0, 1e-30, float("inf"), -float("inf"), float("nan")]]).cuda()
    u = torch.ones_like(g)
    h = _C.swiglu(g, u).cpu()[0]
    assert h[0] == 0 and h[1] == 0 and h[2] == 100.0
    assert h[3] == 0                         # -100 / (1 + inf): exp(100) overflows fp32, as in torch
    assert float(h[4]) == pytest.approx(0.5e-30, rel=1e-6)
    assert h[5] == float("inf")
    assert torch.isnan(h[6]) or h[6] == 0    # -inf * 0
    assert torch.isnan(h[7])


def test_swiglu_reads_halves_of_one_wide_matrix_in_place(oracle):
    from bittorch_amd import _C
    announce("swiglu strided")
    gu = seeded_acts(33, 2 * 1024, seed=9, dtype=torch.bfloat16).cuda()
    g, u = gu[:, :1024], gu[:, 1024:]
    h = _C.swiglu(g, u)
    assert torch.equal(h, _C.swiglu(g.contiguous(), u.contiguous()))
    oh, _, _ = oracle.swiglu(f32np(g), f32np(u), BT_DT[torch.bfloat16])
    np.testing.assert_array_equal(f32np(h), oh)
    # 3-D inputs keep their leading shape
    h3, q3, s3 = _C.swiglu(g.contiguous().view(3, 11, 1024), u.contiguous().view(3, 11, 1024), True, True)
    assert h3.shape == (3, 11, 1024) and q3.shape == (3, 11, 1024) and s3.shape == (3, 11)
    assert torch.equal(h3.view(33, 1024), h)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("b,k", SHAPES)
@pytest.mark.parametrize("with_weight", [True, False])
def test_rmsnorm_matches_oracle_bit_for_bit(oracle, dtype, b, k, with_weight):
    from bittorch_amd import _C
    announce("rmsnorm", dtype, b, k, with_weight)
    x = seeded_acts(b, k, seed=b + k + 5, dtype=dtype, outliers=True)
    if b > 2:
        x[1] = 0  # all-zero row: rsqrt(eps), outputs 0
    w = (1 + 0.1 * torch.randn(k, generator=torch.Generator().manual_seed(k))).to(dtype) if with_weight else None
    eps = 1e-5
    y, q, s = _C.rmsnorm(x.cuda(), None if w is None else w.cuda(), eps, store=True, quantize=True)
    torch.cuda.synchronize()
    oy, oq, os_ = oracle.rmsnorm(f32np(x), None if w is None else f32np(w), eps, BT_DT[dtype])
    np.testing.assert_array_equal(f32np(y), oy)
    np.testing.assert_array_equal(s.cpu().numpy(), os_)
    np.testing.assert_array_equal(q.cpu().numpy(), oq)
    q2, s2 = _C.rmsnorm(x.cuda(), None if w is None else w.cuda(), eps, store=False, quantize=True)
    assert torch.equal(q2, q) and torch.equal(s2, s)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_against_torch(dtype):
    from bittorch_amd import _C
    announce("rmsnorm vs torch", dtype)
    x = seeded_acts(64, 2560, seed=7, dtype=dtype, outliers=True).cuda()
    w = (1 + 0.1 * torch.randn(2560, generator=torch.Generator().manual_seed(1))).to(dtype).cuda()
    got = _C.rmsnorm(x, w, 1e-5)
    ref64 = (x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + 1e-5) * w.double())
    assert _ulp_close(got, ref64.to(dtype), dtype, ulps=2 if dtype == torch.float32 else 1) == 0
    ref_t = F.rms_norm(x, (2560,), w, 1e-5)
    assert _ulp_close(got, ref_t, dtype, ulps=4 if dtype == torch.float32 else 2) == 0


def _packed_case(n, k, seed=0):
    from bittorch_amd.quant import pack_ternary_transposed
    w = random_ternary(n, k, seed=seed)
    packed = pack_ternary_transposed(w)[0].cuda()
    g = torch.Generator().manual_seed(seed + 1)
    scale = (torch.rand(n, generator=g) * 0.05 + 0.01).cuda()
    bias = (torch.randn(n, generator=g) * 0.01).cuda()
    return packed, scale, bias


# (B, N, K): streaming kernel, tiled 16-bit GEMM (whole and ragged tiles), generic shapes
RES_SHAPES = [(1, 4096, 4096), (16, 1000, 520), (33, 256, 128), (200, 520, 192), (130, 260, 70), (5, 37, 23)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("b,n,k", RES_SHAPES)
def test_residual_in_packed_forward_equals_linear_then_add(dtype, b, n, k):
    from bittorch_amd import _C
    announce("residual packed", dtype, b, n, k)
    packed, scale, bias = _packed_case(n, k, seed=b + n)
    x = seeded_acts(b, k, seed=3, dtype=dtype).cuda()
    res = seeded_acts(b, n, seed=4, dtype=dtype).cuda()
    y = _C.ternary_linear_packed_forward(x, packed, scale, bias, k)
    fused = _C.ternary_linear_packed_forward(x, packed, scale, bias, k, res)
    assert torch.equal(fused, y + res)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("b,n,k", [(1, 4096, 4096), (16, 1000, 520), (200, 520, 256), (130, 260, 80)])
def test_residual_in_int8_gemm_equals_linear_then_add(out_dtype, b, n, k):
    from bittorch_amd import _C
    announce("residual int8", out_dtype, b, n, k)
    packed, scale, bias = _packed_case(n, k, seed=b + n)
    x = seeded_acts(b, k, seed=5, dtype=torch.bfloat16, outliers=True).cuda()
    res = seeded_acts(b, n, seed=6, dtype=out_dtype).cuda()
    q, s = _C.act_quant_int8(x)
    y = _C.ternary_gemm_int8(q, s, packed, scale, bias, k, out_dtype)
    fused = _C.ternary_gemm_int8(q, s, packed, scale, bias, k, out_dtype, residual=res)
    assert torch.equal(fused, y + res)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("b,n,k", [(256, 512, 256), (300, 520, 192), (384, 260, 128)])
def test_residual_in_the_tiled_gemms_full_and_ragged_tiles(dtype, b, n, k, monkeypatch):
    """Both matrix-core GEMMs forced (batches beyond 32 rows leave the streaming kernel), on both weight layouts: full
    128-row tiles take the epilogue that requests the residual of all their rows at once (16-bit outputs), ragged ones
    and fp32 outputs the row-by-row one; every output equals linear-then-add bit for bit, and the int8 GEMM's two
    epilogues agree."""
    from bittorch_amd import _C
    announce("residual tiled gemms", dtype, b, n, k)
    set_option("STREAM_MAX_ROWS", "32")
    packed, scale, bias = _packed_case(n, k, seed=b + n + 1)
    tiled = _C.retile_weights(packed, k)
    x = seeded_acts(b, k, seed=7, dtype=dtype).cuda()
    res = seeded_acts(b, n, seed=8, dtype=dtype).cuda()
    y = _C.ternary_linear_packed_forward(x, packed, scale, bias, k)
    assert torch.equal(_C.ternary_linear_packed_forward(x, packed, scale, bias, k, res), y + res)
    assert torch.equal(_C.ternary_linear_tiled_forward(x, tiled, scale, bias, k, n, residual=res), y + res)
    q, s_x = _C.act_quant_int8(x)
    y8 = _C.ternary_gemm_int8(q, s_x, packed, scale, bias, k, dtype)
    assert torch.equal(_C.ternary_gemm_int8(q, s_x, packed, scale, bias, k, dtype, residual=res), y8 + res)
    assert torch.equal(_C.ternary_gemm_int8_tiled(q, s_x, tiled, scale, bias, k, n, dtype, residual=res), y8 + res)
    set_option("GEMM_LONG_EPILOGUE", "1")
    assert torch.equal(_C.ternary_gemm_int8_tiled(q, s_x, tiled, scale, bias, k, n, dtype, residual=res), y8 + res)


def test_residual_on_the_generic_kernel(monkeypatch):
    from bittorch_amd import _C
    monkeypatch.setenv("BITTORCH_KERNEL", "generic")
    packed, scale, bias = _packed_case(260, 70, seed=2)
    x = seeded_acts(9, 70, seed=3).cuda()
    res = seeded_acts(9, 260, seed=4).cuda()
    y = _C.ternary_linear_packed_forward(x, packed, scale, bias, 70)
    assert torch.equal(_C.ternary_linear_packed_forward(x, packed, scale, bias, 70, res), y + res)


def test_residual_argument_errors():
    from bittorch_amd import _C
    packed, scale, bias = _packed_case(64, 32)
    x = seeded_acts(4, 32, dtype=torch.float16).cuda()
    with pytest.raises(RuntimeError, match="residual shape"):
        _C.ternary_linear_packed_forward(x, packed, scale, bias, 32, torch.zeros(4, 63, dtype=torch.float16).cuda())
    with pytest.raises(RuntimeError, match="residual must have the output's dtype"):
        _C.ternary_linear_packed_forward(x, packed, scale, bias, 32, torch.zeros(4, 64).cuda())
    with pytest.raises(RuntimeError, match="nothing to compute"):
        _C.swiglu(x, x, store=False, quantize=False)
    with pytest.raises(RuntimeError, match="gate and up must match"):
        _C.swiglu(x, x[:, :16])


@pytest.mark.parametrize("compute", ["float", "int8"])
def test_ternary_swiglu_module_equals_its_unfused_composition(compute):
    import bittorch_amd as bt
    from bittorch_amd import _C
    announce("TernarySwiGLU", compute)
    d, ffn, tokens = 256, 640, 48
    mk = lambda i, o, seed: bt.nn.create_ternary_linear_inference(
        i, o, (torch.randn(o, i, generator=torch.Generator().manual_seed(seed)) * 0.02).cuda())
    gate, up, down = mk(d, ffn, 1), mk(d, ffn, 2), mk(ffn, d, 3)
    mlp = bt.nn.TernarySwiGLU(gate, up, down, compute=compute)
    x = seeded_acts(tokens, d, seed=8, dtype=torch.bfloat16).cuda()
    nw = (1 + 0.1 * torch.randn(d, generator=torch.Generator().manual_seed(4))).bfloat16().cuda()
    got = mlp(x, nw, 1e-5, residual=x)
    h = _C.rmsnorm(x, nw, 1e-5)
    if compute == "float":
        ref = down(_C.swiglu(gate(h), up(h))) + x
    else:
        q, s = _C.act_quant_int8(h)
        g = _C.ternary_gemm_int8(q, s, gate.weight_packed, gate.scale, None, d, torch.bfloat16)
        u = _C.ternary_gemm_int8(q, s, up.weight_packed, up.scale, None, d, torch.bfloat16)
        q2, s2 = _C.act_quant_int8(_C.swiglu(g, u))
        ref = _C.ternary_gemm_int8(q2, s2, down.weight_packed, down.scale, None, ffn, torch.bfloat16) + x
    assert torch.equal(got, ref)
    # and against plain torch glue around the same layers, to bf16 accuracy
    ht = F.rms_norm(x, (d,), nw, 1e-5)
    ref_t = down(F.silu(gate(ht)) * up(ht)) + x
    err = (got.float() - ref_t.float()).abs().max() / ref_t.float().abs().max()
    assert err < (2e-2 if compute == "float" else 6e-2)
    # without a norm the input itself is the activation
    got2 = mlp(x)
    assert got2.shape == (tokens, d) and torch.isfinite(got2.float()).all()


def test_fused_layers_equal_the_separate_layers_bit_for_bit():
    import bittorch_amd as bt
    announce("fuse_ternary_linear_inference")
    d, tokens = 256, 70
    mk = lambda o, seed: bt.nn.create_ternary_linear_inference(
        d, o, (torch.randn(o, d, generator=torch.Generator().manual_seed(seed)) * 0.02).cuda(),
        (torch.randn(o, generator=torch.Generator().manual_seed(seed + 9)) * 0.01).cuda())
    q, k, v = mk(256, 1), mk(128, 2), mk(64, 3)
    qkv = bt.utils.fuse_ternary_linear_inference(q, k, v)
    assert qkv.out_features == 448 and qkv.weight_packed.shape == (64, 448)
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        x = seeded_acts(tokens, d, seed=5, dtype=dtype).cuda()
        y = qkv(x)
        assert torch.equal(y[:, :256], q(x)) and torch.equal(y[:, 256:384], k(x)) and torch.equal(y[:, 384:], v(x))
    x1 = seeded_acts(1, d, seed=6, dtype=torch.float16).cuda()   # decode shape: streaming kernel
    y1 = qkv(x1)
    assert torch.equal(y1[:, :256], q(x1)) and torch.equal(y1[:, 384:], v(x1))
    other = bt.nn.create_ternary_linear_inference(128, 32, (torch.randn(32, 128) * 0.02).cuda())
    with pytest.raises(ValueError, match="share in_features"):
        bt.utils.fuse_ternary_linear_inference(q, other)


@pytest.mark.parametrize("compute", ["float", "int8"])
def test_swiglu_module_with_fused_gate_up_equals_the_unfused_module(compute):
    import bittorch_amd as bt
    announce("TernarySwiGLU fused gate_up", compute)
    d, ffn = 256, 640
    mk = lambda i, o, seed: bt.nn.create_ternary_linear_inference(
        i, o, (torch.randn(o, i, generator=torch.Generator().manual_seed(seed)) * 0.02).cuda())
    gate, up, down = mk(d, ffn, 1), mk(d, ffn, 2), mk(ffn, d, 3)
    a = bt.nn.TernarySwiGLU(gate, up, down, compute=compute)
    b = bt.nn.TernarySwiGLU(gate, up, down, compute=compute, fuse_gate_up=True)
    x = seeded_acts(3 * 16, d, seed=8, dtype=torch.bfloat16).cuda().view(3, 16, d)
    nw = torch.ones(d).bfloat16().cuda()
    assert torch.equal(a(x, nw, 1e-5, residual=x), b(x, nw, 1e-5, residual=x))


def test_block_glue_at_config5_sizes():
    """Full-size shapes of the block stack (4096 tokens, d 2560, FFN 6912, bf16) through properties that
    need no CPU pass: the fused quantization equals the stand-alone quantizer on the stored tensor, the
    stored tensor agrees with torch's operators to one unit in the last place, RMSNorm rows have unit
    RMS, and the residual epilogue of a tall GEMM equals linear-then-add."""
    from bittorch_amd import _C
    announce("block glue, full size")
    g = torch.Generator(device="cuda").manual_seed(0)
    gate = torch.randn(4096, 6912, device="cuda", generator=g).bfloat16() * 2
    up = torch.randn(4096, 6912, device="cuda", generator=g).bfloat16()
    h, q, s = _C.swiglu(gate, up, True, True)
    q_ref, s_ref = _C.act_quant_int8(h)
    assert torch.equal(q, q_ref) and torch.equal(s, s_ref)
    assert _ulp_close(h, F.silu(gate) * up, torch.bfloat16, ulps=1) == 0
    del gate, up, h, q, q_ref

    x = torch.randn(4096, 2560, device="cuda", generator=g).bfloat16() * 3
    y, q, s = _C.rmsnorm(x, None, 1e-6, True, True)
    q_ref, s_ref = _C.act_quant_int8(y)
    assert torch.equal(q, q_ref) and torch.equal(s, s_ref)
    rms = y.float().pow(2).mean(-1).sqrt()
    assert torch.allclose(rms, torch.ones_like(rms), atol=5e-3)

    packed, scale, _ = _packed_case(2560, 2560, seed=11)
    lin = _C.ternary_linear_packed_forward(y, packed, scale, None, 2560)
    assert torch.equal(_C.ternary_linear_packed_forward(y, packed, scale, None, 2560, x), lin + x)
    lin8 = _C.ternary_gemm_int8(q, s, packed, scale, None, 2560, torch.bfloat16)
    assert torch.equal(_C.ternary_gemm_int8(q, s, packed, scale, None, 2560, torch.bfloat16, residual=x), lin8 + x)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("b,n,k", [(1, 4096, 4096), (16, 1000, 528), (33, 256, 128), (200, 520, 272), (130, 260, 80)])
def test_operand_order_activations_give_the_same_results(oracle, dtype, b, n, k):
    """Q written in the matrix cores' operand order is the row-major Q with every 16-byte group
    transposed 4x4, and both int8 GEMM kernels return the same bits from either layout."""
    from bittorch_amd import _C
    announce("operand order", dtype, b, n, k)
    packed, scale, bias = _packed_case(n, k, seed=b + n)
    x = seeded_acts(b, k, seed=5, dtype=dtype, outliers=True).cuda()
    q, s = _C.act_quant_int8(x)
    qo, so = _C.act_quant_int8(x, operand_order=True)
    assert torch.equal(s, so)
    assert torch.equal(qo.view(b, k // 16, 4, 4), q.view(b, k // 16, 4, 4).transpose(2, 3))
    res = seeded_acts(b, n, seed=6, dtype=torch.bfloat16).cuda()
    y, acc = _C.ternary_gemm_int8(q, s, packed, scale, bias, k, torch.bfloat16, return_acc=True)
    yo, acco = _C.ternary_gemm_int8(qo, so, packed, scale, bias, k, torch.bfloat16, return_acc=True, q_operand_order=True)
    assert torch.equal(acc, acco) and torch.equal(y, yo)
    yr = _C.ternary_gemm_int8(qo, so, packed, scale, bias, k, torch.bfloat16, residual=res, q_operand_order=True)
    assert torch.equal(yr, y + res)
    # the fused producers write the same layout
    g2 = seeded_acts(b, k, seed=7, dtype=dtype).cuda()
    qs, ss = _C.swiglu(x, g2, False, True)
    qso, sso = _C.swiglu(x, g2, False, True, operand_order=True)
    assert torch.equal(ss, sso) and torch.equal(qso.view(b, k // 16, 4, 4), qs.view(b, k // 16, 4, 4).transpose(2, 3))
    qn, sn = _C.rmsnorm(x, None, 1e-5, False, True)
    qno, sno = _C.rmsnorm(x, None, 1e-5, False, True, operand_order=True)
    assert torch.equal(sn, sno) and torch.equal(qno.view(b, k // 16, 4, 4), qn.view(b, k // 16, 4, 4).transpose(2, 3))


def test_operand_order_needs_whole_groups():
    from bittorch_amd import _C
    x = seeded_acts(4, 40, dtype=torch.bfloat16).cuda()
    with pytest.raises(RuntimeError, match="operand-order layout needs K % 16 == 0"):
        _C.act_quant_int8(x, operand_order=True)
    with pytest.raises(RuntimeError, match="operand-order layout needs K % 16 == 0"):
        _C.swiglu(x, x, False, True, operand_order=True)


def test_operand_order_on_the_generic_row_kernels(monkeypatch):
    from bittorch_amd import _C
    set_option("ROWOP_GENERIC", "1")
    x = seeded_acts(5, 64, dtype=torch.float16).cuda()
    qn, _ = _C.rmsnorm(x, None, 1e-5, False, True)
    qo, _ = _C.rmsnorm(x, None, 1e-5, False, True, operand_order=True)
    assert torch.equal(qo.view(5, 4, 4, 4), qn.view(5, 4, 4, 4).transpose(2, 3))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("b,n,k", [(1, 4096, 4096), (1, 2560, 6912), (1, 1000, 520), (1, 260, 72), (3, 512, 256), (40, 520, 192)])
def test_forward_with_prologue_equals_the_separate_kernels(dtype, b, n, k):
    """RMSNorm / SwiGLU applied inside the packed forward (inside the GEMV kernel for one 16-bit row,
    as a kernel of its own otherwise) give the bits of the unfused sequence."""
    from bittorch_amd import _C
    announce("prologue", dtype, b, n, k)
    packed, scale, bias = _packed_case(n, k, seed=n + k)
    x = (seeded_acts(b, k, seed=3, dtype=dtype, outliers=True) * 2).cuda()
    u = seeded_acts(b, k, seed=4, dtype=dtype).cuda()
    w = (1 + 0.1 * torch.randn(k, generator=torch.Generator().manual_seed(k))).to(dtype).cuda()
    res = seeded_acts(b, n, seed=5, dtype=dtype).cuda()
    for norm_w in (w, None):
        ref = _C.ternary_linear_packed_forward(_C.rmsnorm(x, norm_w, 1e-5), packed, scale, bias, k, res)
        got = _C.ternary_linear_packed_forward_fused(x, packed, scale, bias, k, res, norm=(norm_w, 1e-5))
        assert torch.equal(got, ref)
    ref = _C.ternary_linear_packed_forward(_C.swiglu(x, u), packed, scale, bias, k)
    got = _C.ternary_linear_packed_forward_fused(x, packed, scale, bias, k, swiglu_up=u)
    assert torch.equal(got, ref)


def test_prologue_on_halves_of_a_wide_row_and_argument_errors():
    from bittorch_amd import _C
    packed, scale, bias = _packed_case(512, 1024, seed=1)
    gu = seeded_acts(1, 2048, seed=2, dtype=torch.bfloat16).cuda()
    g, u = gu[:, :1024], gu[:, 1024:]
    assert torch.equal(_C.ternary_linear_packed_forward_fused(g, packed, scale, None, 1024, swiglu_up=u),
                       _C.ternary_linear_packed_forward(_C.swiglu(g, u), packed, scale, None, 1024))
    with pytest.raises(RuntimeError, match="exactly one of norm and swiglu_up"):
        _C.ternary_linear_packed_forward_fused(g, packed, scale, None, 1024)
    with pytest.raises(RuntimeError, match="gate and up must match"):
        _C.ternary_linear_packed_forward_fused(g, packed, scale, None, 1024, swiglu_up=u[:, :512])


def test_swiglu_module_decode_token_equals_batched_rows():
    """One token through TernarySwiGLU (prologues inside the GEMV kernels) equals the same row taken
    from a batch (prologues as separate kernels, tiled GEMMs have another summation order: compare to
    bf16 accuracy) and equals its own unfused composition exactly."""
    import bittorch_amd as bt
    from bittorch_amd import _C
    d, ffn = 512, 1280
    mk = lambda i, o, seed: bt.nn.create_ternary_linear_inference(
        i, o, (torch.randn(o, i, generator=torch.Generator().manual_seed(seed)) * 0.02).cuda())
    gate, up, down = mk(d, ffn, 1), mk(d, ffn, 2), mk(ffn, d, 3)
    nw = (1 + 0.1 * torch.randn(d, generator=torch.Generator().manual_seed(4))).bfloat16().cuda()
    x = seeded_acts(1, d, seed=8, dtype=torch.bfloat16).cuda()
    for fuse in (False, True):
        mlp = bt.nn.TernarySwiGLU(gate, up, down, fuse_gate_up=fuse)
        got = mlp(x, nw, 1e-5, residual=x)
        h = _C.rmsnorm(x, nw, 1e-5)
        ref = down(_C.swiglu(gate(h), up(h))) + x
        assert torch.equal(got, ref)


@pytest.mark.parametrize("tiled", [False, True])
def test_rmsnorm_prologue_without_weight_gives_the_same_bits_with_and_without_workspace(tiled):
    """One fp16 row under RMSNorm with no norm weight (ones), through the raw C ABI: the exact GEMV applies the
    prologue itself whether or not the caller passes a workspace, so both calls return the bits of
    "row kernel, then forward"."""
    from bittorch_amd import _C, _lib
    lib = _lib.load()
    n, k = 1024, 512
    packed, scale, bias = _packed_case(n, k, seed=9)
    w = _C.retile_weights(packed, k) if tiled else packed
    x = (seeded_acts(1, k, seed=3, dtype=torch.float16, outliers=True) * 2).cuda()
    ref = _C.ternary_linear_packed_forward(_C.rmsnorm(x, None, 1e-5), packed, scale, bias, k)
    st = torch.cuda.current_stream().cuda_stream
    outs = []
    for with_ws in (False, True):
        announce("null norm weight", tiled, with_ws)
        y = torch.full((1, n), float("nan"), dtype=torch.float16, device="cuda")
        nbytes = lib.bt_packed_forward_fused_workspace_bytes(1, n, k, 1) if with_ws else 0
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device="cuda")
        args = (x.data_ptr(), k, 1, 1, None, 0, 1e-5, w.data_ptr(), scale.data_ptr(), BT_DT[scale.dtype], n,
                bias.data_ptr(), BT_DT[bias.dtype], None)
        tail = (y.data_ptr(), 1, n, k, ws.data_ptr() if with_ws else None, nbytes, st)
        if tiled:
            rc = lib.bt_ternary_linear_tiled_forward(*args, 0, *tail)
        else:
            rc = lib.bt_ternary_linear_packed_forward_fused(*args, *tail)
        assert rc == 0, _lib.last_error()
        torch.cuda.synchronize()
        outs.append(y)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("b,k", [(1, 16), (5, 528), (16, 4096), (3, 6912), (2, 16384), (2, 20000), (3, 7)])
def test_fused_quantizers_return_the_row_sums_of_their_codes(dtype, b, k):
    """SwiGLU and RMSNorm with the per-row quantizer can also write, per row, the sum of the int8 codes they emit (what
    the prefill copy's GEMM starts its accumulators from): equal to summing the stored codes, in both storage orders,
    on the register kernel and on the generic one, and nothing else of the result changes."""
    from bittorch_amd import _C
    announce("row sums of the fused quantizers", dtype, b, k)
    g = (seeded_acts(b, k, seed=b + k, dtype=dtype, outliers=True) * 3).cuda()
    u = seeded_acts(b, k, seed=b + k + 1, dtype=dtype).cuda()
    if b > 2:
        u[1] = 0
    w = (1 + 0.1 * torch.randn(k, generator=torch.Generator().manual_seed(k))).to(dtype).cuda()
    for oo in ([False, True] if k % 16 == 0 else [False]):
        q, s = _C.swiglu(g, u, store=False, quantize=True, operand_order=oo)
        q1, s1, rs = _C.swiglu(g, u, store=False, quantize=True, operand_order=oo, return_rowsum=True)
        assert rs.dtype == torch.int32 and rs.shape == (b,)
        assert torch.equal(q1, q) and torch.equal(s1, s)
        assert torch.equal(rs, q.view(b, -1).to(torch.int32).sum(1, dtype=torch.int32))
        h, q2, s2, rs2 = _C.swiglu(g, u, store=True, quantize=True, operand_order=oo, return_rowsum=True)
        assert torch.equal(q2, q) and torch.equal(rs2, rs) and torch.equal(h, _C.swiglu(g, u))
        q, s = _C.rmsnorm(g, w, 1e-5, store=False, quantize=True, operand_order=oo)
        q1, s1, rs = _C.rmsnorm(g, w, 1e-5, store=False, quantize=True, operand_order=oo, return_rowsum=True)
        assert torch.equal(q1, q) and torch.equal(s1, s)
        assert torch.equal(rs, q.view(b, -1).to(torch.int32).sum(1, dtype=torch.int32))
    # row sums belong to the quantizer: without it there is nothing to sum
    with pytest.raises(RuntimeError, match="return_rowsum needs quantize"):
        _C.swiglu(g, u, store=True, quantize=False, return_rowsum=True)


@pytest.mark.parametrize("fuse_gate_up", [False, True])
def test_swiglu_module_with_prefill_copies_changes_no_bits(fuse_gate_up):
    """TernarySwiGLU.prepare_prefill(): every projection gets its field-layout copy, the quantizers hand their row
    sums on, and prefill-sized batches run on the copies: the same bits as without, with and without the norm, and
    decode-sized batches never touch the copies."""
    import bittorch_amd as bt
    from bittorch_amd.nn.ternary_linear_infer import PREFILL_ROWS
    announce("TernarySwiGLU prefill copies", fuse_gate_up)
    d, ffn = 512, 1280
    mk = lambda i, o, seed: bt.nn.create_ternary_linear_inference(
        i, o, (torch.randn(o, i, generator=torch.Generator().manual_seed(seed)) * 0.02).cuda())
    mlp = bt.nn.TernarySwiGLU(mk(d, ffn, 1), mk(d, ffn, 2), mk(ffn, d, 3), compute="int8", fuse_gate_up=fuse_gate_up)
    nw = (1 + 0.1 * torch.randn(d, generator=torch.Generator().manual_seed(4))).bfloat16().cuda()
    xs = {rows: seeded_acts(rows, d, seed=rows, dtype=torch.bfloat16).cuda() for rows in (PREFILL_ROWS + 37, 24)}
    ref = {rows: (mlp(x, nw, 1e-5, residual=x), mlp(x)) for rows, x in xs.items()}
    before = sum(m.resident_weight_bytes() for m in mlp._linears())
    assert mlp.prepare_prefill() is mlp
    assert all(m._prefill_copy() is not None for m in mlp._linears())
    assert sum(m.resident_weight_bytes() for m in mlp._linears()) > before
    assert mlp._wants_rowsum(PREFILL_ROWS) and not mlp._wants_rowsum(PREFILL_ROWS - 1)
    for rows, x in xs.items():
        assert torch.equal(mlp(x, nw, 1e-5, residual=x), ref[rows][0])
        assert torch.equal(mlp(x), ref[rows][1])
    mlp.drop_prefill()
    assert not mlp._wants_rowsum(PREFILL_ROWS) and sum(m.resident_weight_bytes() for m in mlp._linears()) == before
    assert torch.equal(mlp(xs[24]), ref[24][1])


def test_swiglu_module_on_prefill_copies_replays_in_a_graph():
    """The int8 MLP on its prefill copies (row sums from the RMSNorm and SwiGLU quantizers, GEMMs on the field layout)
    captured once and replayed on new inputs, with eager work between the replays: every replay equals the eager call."""
    import bittorch_amd as bt
    from bittorch_amd.nn.ternary_linear_infer import PREFILL_ROWS
    announce("TernarySwiGLU prefill copies under graph replay")
    d, ffn, rows = 512, 1280, PREFILL_ROWS + 128
    mk = lambda i, o, seed: bt.nn.create_ternary_linear_inference(
        i, o, (torch.randn(o, i, generator=torch.Generator().manual_seed(seed)) * 0.02).cuda())
    mlp = bt.nn.TernarySwiGLU(mk(d, ffn, 1), mk(d, ffn, 2), mk(ffn, d, 3), compute="int8", fuse_gate_up=True).prepare_prefill()
    nw = (1 + 0.1 * torch.randn(d, generator=torch.Generator().manual_seed(4))).bfloat16().cuda()
    xs = [seeded_acts(rows, d, seed=s_, dtype=torch.bfloat16, outliers=True).cuda() for s_ in (11, 12, 13)]
    eager = [mlp(xi, nw, 1e-5, residual=xi) for xi in xs]
    x = xs[0].clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        mlp(x, nw, 1e-5, residual=x)  # warm-up on a side stream, as torch asks before a capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = mlp(x, nw, 1e-5, residual=x)
    for xi, want in zip(xs, eager):
        _ = mlp(xi[:24], nw, 1e-5)  # eager work between the replays (a decode-sized call on the same layers)
        x.copy_(xi)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("b,k", [(2050, 520), (2048, 2560), (4099, 1032), (2051, 3072), (4096, 24), (4100, 2056)])
def test_many_short_rows_match_the_oracle_bit_for_bit(oracle, dtype, b, k):
    """Launches of thousands of short rows run one wave per row (rows that would leave a quarter of a workgroup's lanes
    idle): the same values, codes, scales and row sums as the oracle's, for every iteration count the kernel is built
    with, in both storage orders, with the row count not a multiple of the four rows a workgroup takes."""
    from bittorch_amd import _C
    announce("one wave per row", dtype, b, k)
    g = (seeded_acts(b, k, seed=b + k, dtype=dtype, outliers=True) * 3)
    u = seeded_acts(b, k, seed=b + k + 1, dtype=dtype)
    u[1] = 0
    w = (1 + 0.1 * torch.randn(k, generator=torch.Generator().manual_seed(k))).to(dtype)
    oh, oq, os_ = oracle.swiglu(f32np(g), f32np(u), BT_DT[dtype])
    h, q, s, rs = _C.swiglu(g.cuda(), u.cuda(), store=True, quantize=True, return_rowsum=True)
    np.testing.assert_array_equal(f32np(h), oh)
    np.testing.assert_array_equal(s.cpu().numpy(), os_)
    np.testing.assert_array_equal(q.cpu().numpy(), oq)
    np.testing.assert_array_equal(rs.cpu().numpy(), oq.astype(np.int32).sum(1))
    assert torch.equal(_C.swiglu(g.cuda(), u.cuda()), h)
    oy, oq, os_ = oracle.rmsnorm(f32np(g), f32np(w), 1e-5, BT_DT[dtype])
    y, q, s = _C.rmsnorm(g.cuda(), w.cuda(), 1e-5, store=True, quantize=True)
    np.testing.assert_array_equal(f32np(y), oy)
    np.testing.assert_array_equal(s.cpu().numpy(), os_)
    np.testing.assert_array_equal(q.cpu().numpy(), oq)
    assert torch.equal(_C.rmsnorm(g.cuda(), w.cuda(), 1e-5), y)
    if k % 16 == 0:  # operand order: the same codes, every aligned 16 of them 4 x 4 transposed
        q2, s2 = _C.rmsnorm(g.cuda(), w.cuda(), 1e-5, store=False, quantize=True, operand_order=True)
        assert torch.equal(s2, s)
        assert torch.equal(q2.view(b, k // 16, 4, 4).transpose(2, 3).reshape(b, k), q)
    # the generic kernel (element-wise passes) agrees
    set_option("ROWOP_GENERIC", "1")
    try:
        y3, q3, s3 = _C.rmsnorm(g.cuda(), w.cuda(), 1e-5, store=True, quantize=True)
    finally:
        set_option("ROWOP_GENERIC", None)
    assert torch.equal(y3, y) and torch.equal(q3, q) and torch.equal(s3, s)
