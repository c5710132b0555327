"""GPU parity over seeded random shapes: odd sizes, ragged tails and every kernel family in one sweep
(quantize+pack bit-exact, int8 path bit-exact, float path against the float64 truth, fused residual)."""
import numpy as np
import pytest
import torch

from conftest import announce
from _util import BT_DT, f32np, random_ternary, rel_err, seeded_acts, seeded_weights, assert_close_like_reference

pytestmark = pytest.mark.gpu

_rng = np.random.default_rng(20240607)


def _shape():
    b = int(_rng.choice([1, 2, 5, 16, 17, 31, 33, 48, 130, 257]))
    n = int(_rng.choice([1, 3, 4, 37, 64, 100, 128, 260, 516, 1000]))
    k = int(_rng.choice([1, 3, 4, 16, 23, 64, 70, 128, 192, 528, 1040]))
    return b, n, k


CASES = [(*_shape(), [torch.float32, torch.float16, torch.bfloat16][i % 3], i) for i in range(36)]


@pytest.mark.parametrize("b,n,k,dtype,seed", CASES)
def test_random_shape_sweep(oracle, b, n, k, dtype, seed):
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed
    announce("random shape", b, n, k, dtype, seed)
    # quantize + pack: bytes and scales bit-exact
    w = seeded_weights(n, k, seed=seed, dtype=dtype)
    packed, scale, _ = _C.ternary_quantize_pack(w.cuda(), 0.05, True)
    o_tern, o_scale = oracle.ternary_quantize(f32np(w), 0.05, True, BT_DT[dtype])
    o_packed, _ = oracle.pack_ternary_transposed(o_tern)
    np.testing.assert_array_equal(packed.cpu().numpy(), o_packed)
    np.testing.assert_array_equal(f32np(scale), o_scale)

    # float path (whatever kernel the shape selects) against the float64 truth, plus the residual
    x = seeded_acts(b, k, seed=seed + 1, dtype=dtype)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(seed + 2)) * 0.01).to(dtype)
    y = _C.ternary_linear_packed_forward(x.cuda(), packed, scale, bias.cuda(), k)
    truth = oracle.linear_packed(f32np(x), o_packed, o_scale, k, f32np(bias), f64=True)
    assert rel_err(f32np(y), truth) < (1e-3 if dtype == torch.float32 else 1e-2)
    assert_close_like_reference(f32np(y), truth, dtype)
    res = seeded_acts(b, n, seed=seed + 3, dtype=dtype).cuda()
    assert torch.equal(_C.ternary_linear_packed_forward(x.cuda(), packed, scale, bias.cuda(), k, res), y + res)

    # int8 path: activations, scales, accumulators and outputs bit-exact; both activation layouts
    xq = x.cuda()
    q, s = _C.act_quant_int8(xq)
    oq, os_, oacc, oy = oracle.linear_i8(f32np(x), o_packed, o_scale, k, f32np(bias))
    np.testing.assert_array_equal(q.cpu().numpy(), oq)
    np.testing.assert_array_equal(s.cpu().numpy(), os_)
    y8, acc = _C.ternary_gemm_int8(q, s, packed, scale, bias.cuda(), k, out_dtype=dtype, return_acc=True)
    np.testing.assert_array_equal(acc.cpu().numpy(), oacc)
    assert torch.equal(y8.cpu(), torch.from_numpy(oy).to(dtype))
    if k % 16 == 0:
        qo, so = _C.act_quant_int8(xq, operand_order=True)
        y8o = _C.ternary_gemm_int8(qo, so, packed, scale, bias.cuda(), k, out_dtype=dtype, q_operand_order=True)
        assert torch.equal(y8o, y8)
    yt = _C.ternary_linear_tensor_core_forward(xq, packed, scale, bias.cuda(), k, 2)
    assert torch.equal(yt, y8)

    # the decode-tiled copy of the weights: layout against the oracle, int8 path bit-exact at every
    # batch size (streaming kernel up to 32 rows, tiled GEMM beyond), float path equal to the
    # row-major streaming kernel where that is what the row-major call runs
    tiled = _C.retile_weights(packed, k)
    np.testing.assert_array_equal(tiled.cpu().numpy(), oracle.retile_weights(o_packed, k))
    y8t, acct = _C.ternary_gemm_int8_tiled(q, s, tiled, scale, bias.cuda(), k, n, dtype, True)
    np.testing.assert_array_equal(acct.cpu().numpy(), oacc)
    assert torch.equal(y8t, y8)
    if dtype != torch.float32 or k % 64 == 0:
        yt_f = _C.ternary_linear_tiled_forward(x.cuda(), tiled, scale, bias.cuda(), k, n)
        assert rel_err(f32np(yt_f), truth) < (1e-3 if dtype == torch.float32 else 1e-2)
        assert_close_like_reference(f32np(yt_f), truth, dtype)
        if dtype != torch.float32 and b <= 32:  # (beyond, the plans may split K over different numbers of waves)
            assert torch.equal(yt_f, y)
