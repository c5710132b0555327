"""GPU parity: int8 activation quantizer and int8 x ternary matrix-core GEMM vs the
CPU oracle.  int8 activations, activation scales and int32 accumulators are
bit-exact; float outputs are bit-exact in fp32 and equal after the same final
rounding in bf16/fp16 (the epilogue performs the oracle's operations one by one)."""
import numpy as np
import pytest
import torch

from conftest import announce
from _util import f32np, random_ternary, rel_err, seeded_acts, set_option

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("b,k", [(1, 1), (3, 7), (16, 4096), (5, 11008), (64, 520), (2, 100000)])
def test_act_quant_bit_exact(oracle, dtype, b, k):
    from bittorch_amd import _C
    announce("act_quant", dtype, b, k)
    x = seeded_acts(b, k, seed=b + k, dtype=dtype, outliers=True)
    if b > 2:
        x[1] = 0  # all-zero row: scale 1
    q, s = _C.act_quant_int8(x.cuda())
    torch.cuda.synchronize()
    oq, os_ = oracle.act_quant_i8(f32np(x))
    np.testing.assert_array_equal(s.cpu().numpy(), os_)
    np.testing.assert_array_equal(q.cpu().numpy(), oq)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("b,k", [(2050, 520), (2048, 2560), (4099, 1032), (2051, 3072), (4096, 24), (2049, 2000)])
def test_act_quant_of_many_short_rows_bit_exact(oracle, dtype, b, k):
    """Thousands of short rows take the quantizer's one-wave-per-row kernel: codes and scales equal the oracle's, the
    row sums equal the codes' sums, and the operand order holds the same codes 4 x 4 transposed."""
    from bittorch_amd import _C
    announce("act_quant, a wave per row", dtype, b, k)
    x = seeded_acts(b, k, seed=b + k, dtype=dtype, outliers=True)
    x[1] = 0
    q, s, rs = _C.act_quant_int8(x.cuda(), False, True)
    oq, os_ = oracle.act_quant_i8(f32np(x))
    np.testing.assert_array_equal(s.cpu().numpy(), os_)
    np.testing.assert_array_equal(q.cpu().numpy(), oq)
    np.testing.assert_array_equal(rs.cpu().numpy(), oq.astype(np.int32).sum(1))
    if k % 16 == 0:
        qo, so = _C.act_quant_int8(x.cuda(), True)
        assert torch.equal(so, s) and torch.equal(qo.view(b, k // 16, 4, 4), q.view(b, k // 16, 4, 4).transpose(2, 3))


def _gemm_case(oracle, b, n, k, out_dtype, seed=0, bias=True, outliers=False):
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    w = random_ternary(n, k, seed=seed)
    packed = pack_ternary_transposed(w)[0]
    g = torch.Generator().manual_seed(seed + 1)
    scale = torch.rand(n, generator=g) * 0.05 + 0.01
    bias_t = torch.randn(n, generator=g) * 0.01 if bias else None
    x = seeded_acts(b, k, seed=seed + 2, dtype=out_dtype, outliers=outliers)
    oq, os_, oacc, oy = oracle.linear_i8(f32np(x), packed.numpy(), f32np(scale), k,
                                         None if bias_t is None else f32np(bias_t))
    q, s = _C.act_quant_int8(x.cuda())
    y, acc = _C.ternary_gemm_int8(q, s, packed.cuda(), scale.cuda(),
                                  None if bias_t is None else bias_t.cuda(), k, out_dtype=out_dtype,
                                  return_acc=True)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(q.cpu().numpy(), oq)
    np.testing.assert_array_equal(acc.cpu().numpy(), oacc)
    expect = torch.from_numpy(oy).to(out_dtype)
    assert torch.equal(y.cpu(), expect), (b, n, k, out_dtype)
    # fused entry point (quantize + GEMM in one call) gives the same output
    y2 = _C.ternary_linear_tensor_core_forward(x.cuda(), packed.cuda(), scale.cuda(),
                                               None if bias_t is None else bias_t.cuda(), k, 2)
    assert torch.equal(y2.cpu(), expect)
    return x, packed, scale, bias_t, oy


# streaming (decode-shape) kernel: B <= 32
@pytest.mark.parametrize("b,n,k", [(1, 64, 64), (16, 256, 4096), (16, 1024, 11008), (5, 48, 100),
                                   (32, 128, 512), (17, 512, 1000), (2, 16, 20)])
def test_gemm_i8_small_batch_bit_exact(oracle, b, n, k):
    announce("gemm_i8 small", b, n, k)
    _gemm_case(oracle, b, n, k, torch.bfloat16, seed=b + n)
    _gemm_case(oracle, b, n, k, torch.float32, seed=b + n + 1, bias=False)


# prefill kernel: B > 32, including ragged M / N / K tiles
@pytest.mark.parametrize("route", ["auto", "gemm"])
@pytest.mark.parametrize("b,n,k", [(128, 256, 128), (256, 512, 1024), (33, 64, 64), (130, 260, 132),
                                   (64, 4, 16), (200, 1024, 4096), (129, 300, 1000), (2048, 256, 512)])
def test_gemm_i8_prefill_bit_exact(oracle, b, n, k, route, monkeypatch):
    if route == "gemm":  # batches beyond 32 rows to the tiled GEMM whatever their size (the default rule streams small outputs)
        set_option("STREAM_MAX_ROWS", "32")
    announce("gemm_i8 prefill", b, n, k)
    _gemm_case(oracle, b, n, k, torch.bfloat16, seed=n + k, outliers=True)
    _gemm_case(oracle, b, n, k, torch.float16, seed=n + k + 1)
    _gemm_case(oracle, b, n, k, torch.float32, seed=n + k + 2, bias=False)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_gemm_i8_epilogue_paths_agree_for_any_row_scale(oracle, out_dtype, monkeypatch):
    """The prefill kernel has a short epilogue (full tiles, no residual, no accumulator output: division by 127 in two
    operations) and a long one.  The short one is exact only while float(127 acc) * s_x stays out of 2^-122 .. 2^-113, so
    a tile with a row scale below 2^-119 must take the long one: caller-made s_x with tiny, subnormal, huge, negative and
    zero entries, every output against the oracle's true division, both epilogues forced and compared."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("gemm_i8 epilogue paths", out_dtype)
    set_option("STREAM_MAX_ROWS", "32")
    b, n, k = 384, 512, 256
    w = random_ternary(n, k, seed=3)
    packed = pack_ternary_transposed(w)[0]
    g = torch.Generator().manual_seed(4)
    q = torch.randint(-127, 128, (b, k), generator=g, dtype=torch.int8)
    scale = torch.rand(n, generator=g) * 0.05 + 0.01
    bias = torch.randn(n, generator=g) * 0.01
    s_x = torch.rand(b, generator=g) * 0.05 + 1e-3           # rows 0..127: ordinary scales -> short epilogue
    s_x[128:256] = torch.tensor(2.0) ** torch.randint(-126, -100, (128,), generator=g).float()  # around the bad range
    s_x[130] = 2.0 ** -119                                    # exactly the threshold (still the short division's range)
    s_x[140] = 1e-42                                          # subnormal
    s_x[150] = 0.0
    s_x[256:] = torch.rand(128, generator=g) * 1e30           # third row tile: huge, one negative
    s_x[300] = -0.37
    _, oy = oracle.gemm_i8(q.numpy(), f32np(s_x), packed.numpy(), f32np(scale), k, f32np(bias))
    expect = torch.from_numpy(oy).to(out_dtype)
    args = (q.cuda(), s_x.cuda(), packed.cuda(), scale.cuda(), bias.cuda(), k)
    y_short = _C.ternary_gemm_int8(*args, out_dtype=out_dtype)
    set_option("GEMM_LONG_EPILOGUE", "1")
    y_long = _C.ternary_gemm_int8(*args, out_dtype=out_dtype)
    torch.cuda.synchronize()
    assert torch.equal(y_long.cpu().view(torch.int16 if out_dtype != torch.float32 else torch.int32),
                       expect.view(torch.int16 if out_dtype != torch.float32 else torch.int32))
    assert torch.equal(y_short.cpu().view(torch.int16 if out_dtype != torch.float32 else torch.int32),
                       expect.view(torch.int16 if out_dtype != torch.float32 else torch.int32))
    # without a bias the reference still adds 0.0f, which turns a -0 product into +0: zero, negative and tiny column
    # scales and the negative row scale above must come out the same, sign of zero included
    set_option("GEMM_LONG_EPILOGUE", None)
    scale2 = scale.clone()
    scale2[0:64] = 0.0
    scale2[64:128] = -0.03
    scale2[256:320] = 1e-30
    q2 = q.clone()
    q2[:, :] = torch.where(torch.rand(b, k, generator=g) < 0.5, q2, torch.zeros_like(q2))
    q2[5] = 0                                                  # a zero accumulator row
    s_ok = torch.rand(b, generator=g) * 0.05 + 1e-3
    for sx_case in (s_ok, s_x):
        _, oy2 = oracle.gemm_i8(q2.numpy(), f32np(sx_case), packed.numpy(), f32np(scale2), k, None)
        e2 = torch.from_numpy(oy2).to(out_dtype)
        y2 = _C.ternary_gemm_int8(q2.cuda(), sx_case.cuda(), packed.cuda(), scale2.cuda(), None, k, out_dtype=out_dtype)
        torch.cuda.synchronize()
        iv = torch.int16 if out_dtype != torch.float32 else torch.int32
        assert torch.equal(y2.cpu().view(iv), e2.view(iv))


def test_gemm_i8_close_to_float_path(oracle):
    """int8 path vs the unquantized float product: inside the int8 quantisation error."""
    announce("gemm_i8 vs float")
    x, packed, scale, bias, oy = _gemm_case(oracle, 64, 256, 1024, torch.float32, seed=5)
    truth = oracle.linear_packed(f32np(x), packed.numpy(), f32np(scale), 1024, f32np(bias), f64=True)
    assert rel_err(oy, truth) < 2e-2


def test_gemm_i8_full_size_properties(oracle):
    """Config-4 shape [2048,4096] x [4096,4096]: linearity in the weights' sign, agreement of two independent
    kernels (streaming rows vs prefill tiles), and the variant the benchmark times -- decode-tiled weights with
    operand-order activations -- against the row-major entry point (accumulators and outputs) and against the oracle
    on a 64 x 256 slice."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("gemm_i8 full size")
    w = random_ternary(4096, 4096, seed=1)
    packed = pack_ternary_transposed(w)[0].cuda()
    packed_neg = pack_ternary_transposed(-w)[0].cuda()
    x = seeded_acts(2048, 4096, seed=2, dtype=torch.bfloat16, outliers=True).cuda()
    scale = torch.ones(4096, device="cuda")
    q, s = _C.act_quant_int8(x)
    _, acc = _C.ternary_gemm_int8(q, s, packed, scale, None, 4096, return_acc=True)
    _, acc_neg = _C.ternary_gemm_int8(q, s, packed_neg, scale, None, 4096, return_acc=True)
    assert torch.equal(acc, -acc_neg)
    # rows 100..115 through the streaming kernel
    _, acc_rows = _C.ternary_gemm_int8(q[100:116].contiguous(), s[100:116].contiguous(), packed, scale,
                                       None, 4096, return_acc=True)
    assert torch.equal(acc_rows, acc[100:116])
    # against torch integer matmul on a slice (CPU, exact)
    w127 = (w[:64].to(torch.int32) * 127)
    ref = q[:32].cpu().to(torch.int32) @ w127.t()
    assert torch.equal(acc[:32, :64].cpu(), ref)
    # the benchmarked pair: decode-tiled weights, activations in operand order, bf16 outputs with scale and bias
    g = torch.Generator().manual_seed(3)
    scale_cpu = torch.rand(4096, generator=g) * 0.05 + 0.01
    bias_cpu = torch.randn(4096, generator=g) * 0.01
    scale2, bias2 = scale_cpu.cuda(), bias_cpu.cuda()
    tiled = _C.retile_weights(packed, 4096)
    q_oo, s_oo = _C.act_quant_int8(x, True)
    assert torch.equal(s_oo, s)
    y_rm, acc_rm = _C.ternary_gemm_int8(q, s, packed, scale2, bias2, 4096, out_dtype=torch.bfloat16, return_acc=True)
    assert torch.equal(acc_rm, acc)
    y_t, acc_t = _C.ternary_gemm_int8_tiled(q_oo, s, tiled, scale2, bias2, 4096, 4096, torch.bfloat16, True, None, True)
    assert torch.equal(acc_t, acc) and torch.equal(y_t, y_rm)
    y_t2 = _C.ternary_gemm_int8_tiled(q_oo, s, tiled, scale2, bias2, 4096, 4096, torch.bfloat16, False, None, True)
    assert torch.equal(y_t2, y_rm)  # (without the accumulator output the epilogue takes its short path)
    r0, c0 = 1984, 3840  # the last row tile and column tile of the 128 x 256 tiling
    packed_cpu = packed.cpu().numpy()
    oq, os_, oacc, oy = oracle.linear_i8(f32np(x[r0:r0 + 64].cpu()), np.ascontiguousarray(packed_cpu[:, c0:c0 + 256]),
                                         f32np(scale_cpu[c0:c0 + 256]), 4096, f32np(bias_cpu[c0:c0 + 256]))
    np.testing.assert_array_equal(q[r0:r0 + 64].cpu().numpy(), oq)
    np.testing.assert_array_equal(acc_t[r0:r0 + 64, c0:c0 + 256].cpu().numpy(), oacc)
    assert torch.equal(y_t2[r0:r0 + 64, c0:c0 + 256].cpu(), torch.from_numpy(oy).bfloat16())
