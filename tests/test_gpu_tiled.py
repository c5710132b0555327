"""GPU parity of the decode-tiled copy of the packed weights.

* the layout: ``retile_weights`` against the oracle's numpy restatement, byte for byte, and
  ``untile_weights`` as its exact inverse (ragged N and K included);
* the kernels: every forward on the tiled copy equals the same forward on the row-major ``W_T``
  bit for bit (which the other GPU tests hold against the oracle), on decode shapes, batches that
  span several 16-row launches, all dtypes, with bias / residual / prologues, and the int8 path
  with its int32 accumulators;
* one direct comparison with the oracle, so that this file stands on its own.
"""
import os

import numpy as np
import pytest
import torch

from conftest import announce
from _util import f32np, random_ternary, rel_err, seeded_acts, set_option

pytestmark = pytest.mark.gpu

# (N, K): config-2 shape, ragged columns (N % 16 != 0, N % 4 != 0), ragged K, tiny, wide
LAYOUT_SHAPES = [(4096, 4096), (100, 64), (37, 100), (16, 4), (1, 1), (250, 1030), (11008, 512)]


def _packed(oracle, n, k, seed=0):
    w = random_ternary(n, k, seed=seed)
    packed_t, _ = oracle.pack_ternary_transposed(w.numpy())
    return w, torch.from_numpy(packed_t).cuda()


@pytest.mark.parametrize("n,k", LAYOUT_SHAPES)
def test_retile_layout_and_inverse(oracle, n, k):
    from bittorch_amd import _C
    announce("retile", n, k)
    _, wt = _packed(oracle, n, k, seed=n + k)
    tiled = _C.retile_weights(wt, k)
    torch.cuda.synchronize()
    assert tiled.numel() == ((n + 15) // 16) * (((k + 3) // 4 + 15) // 16) * 256
    np.testing.assert_array_equal(tiled.cpu().numpy(), oracle.retile_weights(wt.cpu().numpy(), k))
    back = _C.untile_weights(tiled, n, k)
    assert torch.equal(back, wt)


FWD_SHAPES = [(4096, 4096), (2560, 2560), (6912, 2560), (2560, 6912), (100, 64), (37, 100), (250, 1030), (16, 8),
              (11008, 4096)]


@pytest.mark.parametrize("route", ["auto", "gemm"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,k", FWD_SHAPES)
def test_tiled_forward_equals_row_major(oracle, dtype, n, k, route, monkeypatch):
    if route == "gemm":  # batches beyond 32 rows to the tiled GEMM whatever their size (the default rule streams small outputs)
        set_option("STREAM_MAX_ROWS", "32")
    from bittorch_amd import _C
    _, wt = _packed(oracle, n, k, seed=1)
    tiled = _C.retile_weights(wt, k)
    g = torch.Generator().manual_seed(n + k)
    scale = (torch.rand(n, generator=g) + 0.5).cuda()
    bias = (torch.randn(n, generator=g) * 0.01).to(dtype).cuda()
    for b in (1, 2, 5, 16, 17, 32, 40, 200):
        announce("tiled forward", dtype, n, k, b)
        x = seeded_acts(b, k, seed=b, dtype=dtype).cuda()
        res = seeded_acts(b, n, seed=b + 1, dtype=dtype).cuda()
        ref = _C.ternary_linear_packed_forward(x, wt, scale, bias, k, residual=res)
        got = _C.ternary_linear_tiled_forward(x, tiled, scale, bias, k, n, residual=res)
        if b <= 32 or route == "gemm":  # (the tiled GEMMs sum in one order on either layout)
            assert torch.equal(got, ref)
        else:  # same kernel family on either layout, but the plans may split K over different numbers of waves
            assert rel_err(f32np(got), f32np(ref)) <= 2e-3
    x = seeded_acts(1, k, seed=9, dtype=dtype).cuda()
    assert torch.equal(_C.ternary_linear_tiled_forward(x, tiled, scale[:1], None, k, n),
                       _C.ternary_linear_packed_forward(x, wt, scale[:1], None, k))


@pytest.mark.parametrize("route", ["auto", "gemm"])
@pytest.mark.parametrize("n,k", [(4096, 4096), (100, 64), (2560, 6912)])
def test_tiled_forward_fp32_planes(oracle, n, k, route, monkeypatch):
    if route == "gemm":  # batches beyond 32 rows to the tiled GEMM whatever their size (the default rule streams small outputs)
        set_option("STREAM_MAX_ROWS", "32")
    from bittorch_amd import _C
    _, wt = _packed(oracle, n, k, seed=2)
    tiled = _C.retile_weights(wt, k)
    scale = (torch.rand(n) + 0.5).cuda()
    for b in (1, 3, 20, 70):
        announce("tiled forward fp32", n, k, b)
        x = seeded_acts(b, k, seed=b, dtype=torch.float32).cuda()
        assert torch.equal(_C.ternary_linear_tiled_forward(x, tiled, scale, None, k, n),
                           _C.ternary_linear_packed_forward(x, wt, scale, None, k))


def test_tiled_forward_fp32_ragged_k(oracle):
    """fp32 rows whose K is not a multiple of 64 run on zero-padded planes: same bits as the row-major entry point
    (N = 37 is not a multiple of 4, so both take the streaming kernel's general column path)."""
    from bittorch_amd import _C
    _, wt = _packed(oracle, 37, 100)
    tiled = _C.retile_weights(wt, 100)
    x = seeded_acts(2, 100, dtype=torch.float32).cuda()
    scale = torch.ones(37).cuda()
    y = _C.ternary_linear_tiled_forward(x, tiled, scale, None, 100, 37)
    ref = oracle.linear_packed(f32np(x.cpu()), wt.cpu().numpy(), f32np(scale.cpu()), 100, None)
    np.testing.assert_allclose(f32np(y), ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,k", [(4096, 4096), (7680, 2560), (2560, 6912), (100, 64)])
def test_tiled_prologues_equal_row_major(oracle, dtype, n, k):
    from bittorch_amd import _C
    _, wt = _packed(oracle, n, k, seed=3)
    tiled = _C.retile_weights(wt, k)
    scale = (torch.rand(n) + 0.5).cuda()
    nw = (torch.rand(k) + 0.5).to(dtype).cuda()
    for b in (1, 3):
        announce("tiled prologue", dtype, n, k, b)
        x = seeded_acts(b, k, seed=b, dtype=dtype).cuda()
        u = seeded_acts(b, k, seed=b + 5, dtype=dtype).cuda()
        res = seeded_acts(b, n, seed=b + 7, dtype=dtype).cuda()
        for kw in (dict(norm=(nw, 1e-5)), dict(norm=(None, 1e-6)), dict(swiglu_up=u)):
            ref = _C.ternary_linear_packed_forward_fused(x, wt, scale, None, k, residual=res, **kw)
            got = _C.ternary_linear_tiled_forward(x, tiled, scale, None, k, n, residual=res, **kw)
            assert torch.equal(got, ref)


@pytest.mark.parametrize("route", ["auto", "gemm"])
@pytest.mark.parametrize("n,k", [(4096, 4096), (11008, 4096), (4096, 11008), (100, 64), (37, 100), (260, 192), (520, 1040)])
def test_tiled_int8_equals_row_major(oracle, n, k, route, monkeypatch):
    if route == "gemm":  # batches beyond 32 rows to the tiled GEMM whatever their size (the default rule streams small outputs)
        set_option("STREAM_MAX_ROWS", "32")
    from bittorch_amd import _C
    _, wt = _packed(oracle, n, k, seed=4)
    tiled = _C.retile_weights(wt, k)
    scale = (torch.rand(n) + 0.5).cuda()
    bias = (torch.randn(n) * 0.01).cuda()
    for b in (1, 16, 33, 200):  # up to 32 rows the streaming kernel, beyond it the tiled GEMM
        for oo in ((False, True) if k % 16 == 0 else (False,)):
            announce("tiled int8", n, k, b, oo)
            x = seeded_acts(b, k, seed=b, dtype=torch.bfloat16, outliers=True).cuda()
            q, s = _C.act_quant_int8(x, oo)
            res = seeded_acts(b, n, seed=b + 1, dtype=torch.bfloat16).cuda()
            y0, a0 = _C.ternary_gemm_int8(q, s, wt, scale, bias, k, torch.bfloat16, True, res, oo)
            y1, a1 = _C.ternary_gemm_int8_tiled(q, s, tiled, scale, bias, k, n, torch.bfloat16, True, res, oo)
            assert torch.equal(a1, a0) and torch.equal(y1, y0)


# ---- the prefill-only field layout of the tiled copy ------------------------------------------------------------------
@pytest.mark.parametrize("n,k", LAYOUT_SHAPES + [(520, 1024)])
def test_field_layout_against_the_oracle(oracle, n, k):
    """`retile_fields` byte for byte against the numpy restatement, on natural and pair-ordered tiled copies."""
    from bittorch_amd import _C
    announce("field layout", n, k)
    _, wt = _packed(oracle, n, k, seed=n + 2 * k)
    for pairs in ((False, True) if n % 32 == 0 else (False,)):
        tiled = _C.retile_weights(wt, k, pairs)
        fields = _C.retile_fields(tiled, k, n)
        np.testing.assert_array_equal(fields.cpu().numpy(), oracle.retile_fields(tiled.cpu().numpy(), n, k))


def test_act_quant_row_sums(oracle):
    """The quantizer's third output: the rows' sums of q, with q and s_x unchanged, in both layouts and on both of its
    kernels (rows in registers / the generic one for ragged K)."""
    from bittorch_amd import _C
    for (b, k, dtype) in [(5, 64, torch.float32), (33, 4096, torch.bfloat16), (7, 11008, torch.float16), (3, 100, torch.float32),
                          (2, 20000, torch.bfloat16)]:
        announce("row sums", b, k, dtype)
        x = seeded_acts(b, k, seed=b + k, dtype=dtype, outliers=True).cuda()
        for oo in ((False, True) if k % 16 == 0 else (False,)):
            q0, s0 = _C.act_quant_int8(x, oo)
            q, s, rs = _C.act_quant_int8(x, oo, return_rowsum=True)
            assert torch.equal(q, q0) and torch.equal(s, s0)
            assert rs.dtype == torch.int32 and torch.equal(rs, q.to(torch.int32).sum(dim=1, dtype=torch.int32))
        oq, _ = oracle.act_quant_i8(f32np(x.cpu()))
        np.testing.assert_array_equal(_C.act_quant_int8(x, False, return_rowsum=True)[2].cpu().numpy(), oq.astype(np.int64).sum(axis=1))


# (M, N, K): whole tiles, ragged rows and columns, K of one to many whole stages, a launch that cuts its remainder finer
# (320 and 128 tiles), and config 4's second shape
FIELD_SHAPES = [(128, 256, 128), (100, 200, 256), (130, 260, 384), (257, 520, 1024), (40, 1028, 128), (4096, 2560, 256),
                (1024, 4096, 128), (2048, 11008, 4096)]


@pytest.mark.parametrize("m,n,k", FIELD_SHAPES)
def test_field_layout_gemm_equals_tiled_gemm(oracle, m, n, k):
    """The prefill GEMM on the field layout (one AND per operand dword, accumulators started at minus the rows' sums
    of q, the factor 4^t taken out in the epilogue's multiplication): the int32 accumulators and the output bits of
    the GEMM on the decode-tiled copy, with both activation layouts, bias, residual, every output type, natural and
    pair-ordered copies; and the oracle's on row slices."""
    from bittorch_amd import _C
    set_option("STREAM_MAX_ROWS", "32")
    _, wt = _packed(oracle, n, k, seed=(m + k) % 13)
    g = torch.Generator().manual_seed(m + n + k)
    scale = torch.rand(n, generator=g) * 0.05 + 0.01
    bias = torch.randn(n, generator=g) * 0.01
    x = seeded_acts(m, k, seed=m + k, dtype=torch.bfloat16, outliers=True)
    res = seeded_acts(m, n, seed=m + 1, dtype=torch.bfloat16).cuda()
    for pairs in ((False, True) if n % 32 == 0 and m <= 300 else (False,)):
        tiled = _C.retile_weights(wt, k, pairs)
        fields = _C.retile_fields(tiled, k, n)
        ref_tiled = _C.retile_weights(wt, k)
        for oo in (False, True):
            announce("field layout gemm", m, n, k, pairs, oo)
            q, sx, rs = _C.act_quant_int8(x.cuda(), oo, return_rowsum=True)
            for out_dtype, r, b in ((torch.bfloat16, res, bias), (torch.float32, None, None), (torch.float16, None, bias)):
                bb = None if b is None else b.cuda()
                y0, a0 = _C.ternary_gemm_int8_tiled(q, sx, ref_tiled, scale.cuda(), bb, k, n, out_dtype, True, r, oo)
                y0n = _C.ternary_gemm_int8_tiled(q, sx, ref_tiled, scale.cuda(), bb, k, n, out_dtype, False, r, oo)
                y1, a1 = _C.ternary_gemm_int8_fields(q, sx, rs, fields, scale.cuda(), bb, k, n, out_dtype, True, r, oo, pairs)
                y1n = _C.ternary_gemm_int8_fields(q, sx, rs, fields, scale.cuda(), bb, k, n, out_dtype, False, r, oo, pairs)
                assert torch.equal(a1, a0) and torch.equal(y1, y0) and torch.equal(y1n, y0n)
    q, sx, rs = _C.act_quant_int8(x.cuda(), False, return_rowsum=True)
    fields = _C.retile_fields(_C.retile_weights(wt, k), k, n)
    y1, a1 = _C.ternary_gemm_int8_fields(q, sx, rs, fields, scale.cuda(), bias.cuda(), k, n, torch.float32, True)
    oq, os_ = oracle.act_quant_i8(f32np(x))
    for lo, hi in ((0, min(m, 24)), (max(0, m - 24), m)):
        oacc, oy = oracle.gemm_i8(oq[lo:hi], os_[lo:hi], wt.cpu().numpy(), f32np(scale), k, f32np(bias))
        np.testing.assert_array_equal(a1[lo:hi].cpu().numpy(), oacc)
        np.testing.assert_array_equal(y1[lo:hi].cpu().numpy(), oy)


def test_layer_prefill_copy_is_opt_in_and_changes_no_bits(oracle):
    """`prepare_prefill()` adds the field-layout copy; `forward_int8` with row sums and a prefill-sized batch runs on it
    (natural and gate/up pair-ordered layers), gives the bits of the same call without it, is not used below the row
    threshold or without row sums, stops being used when the layer is re-tiled, and `drop_prefill()` releases it."""
    import bittorch_amd as bt
    from bittorch_amd.nn import TernaryLinearInference
    from bittorch_amd.nn.ternary_linear_infer import PREFILL_ROWS
    n, k = 512, 1024
    w = random_ternary(n, k, seed=77)
    packed, _ = oracle.pack_ternary_transposed(w.numpy())
    gen = torch.Generator().manual_seed(5)
    mk = lambda: TernaryLinearInference(k, n, torch.from_numpy(packed), torch.rand(n, generator=gen) * 0.05 + 0.01,
                                        torch.randn(n, generator=gen) * 0.01).cuda()
    for order in ("natural", "gate_up_pairs"):
        announce("layer prefill copy", order)
        gen.manual_seed(5)
        plain = mk()
        gen.manual_seed(5)
        layer = mk()
        layer.tile_order = order
        x = seeded_acts(PREFILL_ROWS + 40, k, seed=3, dtype=torch.bfloat16, outliers=True).cuda()
        q, s, rs = bt.ops.act_quant_int8(x, True, return_rowsum=True)
        want = plain.forward_int8(q, s, torch.bfloat16, None, True)
        one_copy = layer.prepare_decode().resident_weight_bytes()
        layer.prepare_prefill()
        assert layer.resident_weight_bytes() == 2 * one_copy
        assert torch.equal(layer.forward_int8(q, s, torch.bfloat16, None, True, q_rowsum=rs), want)
        res = seeded_acts(x.shape[0], n, seed=4, dtype=torch.bfloat16).cuda()
        assert torch.equal(layer.forward_int8(q, s, torch.bfloat16, res, True, q_rowsum=rs),
                           plain.forward_int8(q, s, torch.bfloat16, res, True))
        # too few rows, or no row sums: the usual route, the same bits
        assert torch.equal(layer.forward_int8(q[:64], s[:64], torch.bfloat16, None, True, q_rowsum=rs[:64]), want[:64])
        assert torch.equal(layer.forward_int8(q, s, torch.bfloat16, None, True), want)
        # a wrong row-sum vector would show: the copy really is in use
        assert not torch.equal(layer.forward_int8(q, s, torch.bfloat16, None, True, q_rowsum=rs + 1), want)
        held = layer.resident_weight_bytes()  # (a pair-ordered layer holds weight_packed by now: its plain int8 calls need it)
        layer.drop_prefill()
        assert layer.resident_weight_bytes() == held - one_copy
        assert torch.equal(layer.forward_int8(q, s, torch.bfloat16, None, True, q_rowsum=rs + 1), want)
    # re-tiling (a tile order change) orphans the copy instead of reading stale bytes
    gen.manual_seed(5)
    layer = mk().prepare_prefill()
    layer.tile_order = "gate_up_pairs"
    layer.prepare_decode()
    assert layer._prefill_copy() is None
    assert torch.equal(layer.forward_int8(q, s, torch.bfloat16, None, True, q_rowsum=rs), want)


def test_field_layout_gemm_argument_errors(oracle):
    from bittorch_amd import _C
    _, wt = _packed(oracle, 64, 192)
    fields = _C.retile_fields(_C.retile_weights(wt, 192), 192, 64)
    q, sx, rs = _C.act_quant_int8(torch.randn(4, 192, device="cuda"), False, return_rowsum=True)
    with pytest.raises(RuntimeError, match="multiple of 128"):
        _C.ternary_gemm_int8_fields(q, sx, rs, fields, torch.ones(64, device="cuda"), None, 192, 64)
    with pytest.raises(RuntimeError, match="q_rowsum must be int32"):
        _C.ternary_gemm_int8_fields(q, sx, rs.float(), fields, torch.ones(64, device="cuda"), None, 192, 64)


# (M, N, K) whose 128 x 256 tiles leave most of a 256-unit chip idle in their last round, so that the launch cuts
# the remainder finer: 320 tiles (256 whole + 64 as 256 tiles of 32 rows), 128 tiles (as 256 of 64 rows), 64 tiles (as
# 256 of 32 rows); the same with ragged last row tiles, ragged columns and several stages of K
REMAINDER_SHAPES = [(4096, 2560, 256), (1024, 4096, 128), (512, 4096, 384), (1000, 4096, 256), (500, 4096, 128),
                    (512, 4000, 128), (4090, 2560, 128)]


# ... and config 5's two projections of 1.25 rounds at their full size
@pytest.mark.parametrize("m,n,k", REMAINDER_SHAPES + [(4096, 2560, 2560), (4096, 2560, 6912)])
def test_tiled_int8_remainder_in_finer_tiles(oracle, m, n, k, monkeypatch):
    """The prefill GEMM computes the column tiles of a mostly empty last round in tiles of 64 or 32 rows
    (a second launch behind the whole tiles).  Same bits as one launch of whole tiles -- outputs and int32
    accumulators, both activation layouts, bias, residual, 16-bit and fp32 outputs -- and equal to the oracle on
    row slices at the start, across tile borders and at the ragged end."""
    from bittorch_amd import _C
    set_option("STREAM_MAX_ROWS", "32")
    _, wt = _packed(oracle, n, k, seed=m % 7)
    tiled = _C.retile_weights(wt, k)
    g = torch.Generator().manual_seed(m + n)
    scale = torch.rand(n, generator=g) * 0.05 + 0.01
    bias = torch.randn(n, generator=g) * 0.01
    x = seeded_acts(m, k, seed=m + k, dtype=torch.bfloat16, outliers=True)
    res = seeded_acts(m, n, seed=m + 1, dtype=torch.bfloat16).cuda()
    oq, os_ = oracle.act_quant_i8(f32np(x))
    slices = [(0, min(m, 40)), (max(0, m // 2 - 20), min(m, m // 2 + 20)), (max(0, m - 40), m)]
    for oo in (False, True):
        announce("remainder tiles", m, n, k, oo)
        q, s = _C.act_quant_int8(x.cuda(), oo)
        outs = {}
        for split in ("0", "1"):
            set_option("GEMM_TAIL_SPLIT", split)
            y32, acc = _C.ternary_gemm_int8_tiled(q, s, tiled, scale.cuda(), bias.cuda(), k, n, torch.float32, True, None, oo)
            y16 = _C.ternary_gemm_int8_tiled(q, s, tiled, scale.cuda(), None, k, n, torch.bfloat16, False, res, oo)
            y16b = _C.ternary_gemm_int8_tiled(q, s, tiled, scale.cuda(), bias.cuda(), k, n, torch.float16, False, None, oo)
            outs[split] = (y32, acc, y16, y16b)
        torch.cuda.synchronize()
        for a, b in zip(outs["0"], outs["1"]):
            assert torch.equal(a, b)
        y32, acc = outs["1"][0].cpu().numpy(), outs["1"][1].cpu().numpy()
        for r0, r1 in slices:
            oacc, oy = oracle.gemm_i8(oq[r0:r1], os_[r0:r1], wt.cpu().numpy(), f32np(scale), k, f32np(bias))
            np.testing.assert_array_equal(acc[r0:r1], oacc)
            np.testing.assert_array_equal(y32[r0:r1], oy)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("m,n,k", REMAINDER_SHAPES)
def test_tiled_forward_remainder_in_finer_tiles(oracle, dtype, m, n, k, monkeypatch):
    """The same for the 16-bit matrix-core GEMM (fp32 rows: three bf16 planes): finer tiles for the remainder give the
    bits of one launch of whole tiles, with bias and with a residual, and agree with the oracle's float64-free
    restatement of the reference's loop within the rounding of 16-bit products summed in fp32."""
    from bittorch_amd import _C
    set_option("STREAM_MAX_ROWS", "32")
    _, wt = _packed(oracle, n, k, seed=m % 5)
    tiled = _C.retile_weights(wt, k)
    g = torch.Generator().manual_seed(m + n + 1)
    scale = torch.rand(n, generator=g) + 0.5
    bias = (torch.randn(n, generator=g) * 0.01).to(dtype)
    x = seeded_acts(m, k, seed=m + k + 1, dtype=dtype)
    res = seeded_acts(m, n, seed=m + 2, dtype=dtype).cuda()
    announce("remainder tiles, float", dtype, m, n, k)
    outs = {}
    for split in ("0", "1"):
        set_option("GEMM_TAIL_SPLIT", split)
        outs[split] = (_C.ternary_linear_tiled_forward(x.cuda(), tiled, scale.cuda(), bias.cuda(), k, n),
                       _C.ternary_linear_tiled_forward(x.cuda(), tiled, scale.cuda(), None, k, n, residual=res))
    torch.cuda.synchronize()
    for a, b in zip(outs["0"], outs["1"]):
        assert torch.equal(a, b)
    y = f32np(outs["1"][0])
    for r0, r1 in [(0, min(m, 40)), (max(0, m // 2 - 20), min(m, m // 2 + 20)), (max(0, m - 40), m)]:
        ref = oracle.linear_packed(f32np(x[r0:r1]), wt.cpu().numpy(), scale.numpy(), k, f32np(bias))
        assert rel_err(y[r0:r1], ref) <= (1e-3 if dtype == torch.float32 else 1e-2)  # output rounding of the 16-bit dtypes


def test_remainder_tiles_replay_in_a_graph(oracle, monkeypatch):
    """The two launches of a call with finer remainder tiles are captured like any other: every replay of the graph,
    with eager work and synchronizations between the replays, gives the eager result."""
    from bittorch_amd import _C
    set_option("STREAM_MAX_ROWS", "32")
    m, n, k = 4096, 2560, 256
    _, wt = _packed(oracle, n, k, seed=3)
    tiled = _C.retile_weights(wt, k)
    scale = (torch.rand(n) * 0.05 + 0.01).cuda()
    xs = [seeded_acts(m, k, seed=s_, dtype=torch.bfloat16, outliers=True).cuda() for s_ in (1, 2, 3)]
    x = xs[0].clone()
    q, s = _C.act_quant_int8(x, True)
    eager = []
    for xi in xs:
        qi, si = _C.act_quant_int8(xi, True)
        eager.append(_C.ternary_gemm_int8_tiled(qi, si, tiled, scale, None, k, n, torch.bfloat16, False, None, True))
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _C.ternary_gemm_int8_tiled(q, s, tiled, scale, None, k, n, torch.bfloat16, False, None, True)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = _C.ternary_gemm_int8_tiled(q, s, tiled, scale, None, k, n, torch.bfloat16, False, None, True)
    for xi, want in zip(xs, eager):
        qi, si = _C.act_quant_int8(xi, True)  # eager work between the replays
        q.copy_(qi)
        s.copy_(si)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want)


def test_tiled_forward_against_oracle(oracle):
    from bittorch_amd import _C
    n, k = 300, 520
    w, wt = _packed(oracle, n, k, seed=5)
    tiled = _C.retile_weights(wt, k)
    scale = torch.rand(n) + 0.5
    bias = torch.randn(n) * 0.01
    x = seeded_acts(4, k, seed=6, dtype=torch.float16)
    got = _C.ternary_linear_tiled_forward(x.cuda(), tiled, scale.cuda(), bias.half().cuda(), k, n)
    ref = oracle.linear_packed(f32np(x), wt.cpu().numpy(), scale.numpy(), k, f32np(bias.half()))
    assert rel_err(f32np(got), ref) <= 1e-3  # fp16 output rounding on fp32 sums


def test_tiled_size_mismatch_is_refused(oracle):
    from bittorch_amd import _C
    _, wt = _packed(oracle, 64, 64)
    tiled = _C.retile_weights(wt, 64)
    x = seeded_acts(1, 64, dtype=torch.float16).cuda()
    with pytest.raises(RuntimeError, match="W_tiled size"):
        _C.ternary_linear_tiled_forward(x, tiled, torch.ones(80).cuda(), None, 64, 80)


def _layer(oracle, n, k, seed=0, **kw):
    from bittorch_amd.nn import TernaryLinearInference
    w = random_ternary(n, k, seed=seed)
    packed_t, _ = oracle.pack_ternary_transposed(w.numpy())
    g = torch.Generator().manual_seed(seed)
    return TernaryLinearInference(k, n, torch.from_numpy(packed_t), torch.rand(n, generator=g) + 0.5,
                                  torch.randn(n, generator=g) * 0.01, **kw).cuda()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_module_uses_tiled_copy_for_decode_shapes(oracle, dtype):
    announce("module tiled", dtype)
    a = _layer(oracle, 640, 512, seed=3)                      # default: tiled copy on first decode call
    b = _layer(oracle, 640, 512, seed=3, decode_tiled=False)  # weight_packed only
    assert a.decode_tiled and a._tiled is None
    for shape in ((512,), (1, 512), (2, 3, 512), (32, 512), (70, 512)):
        x = seeded_acts(1, int(np.prod(shape)), seed=len(shape), dtype=dtype).reshape(shape).cuda()
        ya, yb = a(x), b(x)
        assert ya.shape == yb.shape == (*shape[:-1], 640)
        if x.numel() // 512 <= 32:
            assert torch.equal(ya, yb)
        else:  # (the two layouts' plans may split K over different numbers of waves)
            assert rel_err(f32np(ya), f32np(yb)) <= (1e-5 if dtype == torch.float32 else 2e-3)
    assert a._tiled is not None and b._tiled is None
    assert "_tiled" not in a.state_dict() and set(a.state_dict()) == set(b.state_dict())
    # prologues, residual and the int8 path go the same way
    x = seeded_acts(1, 512, seed=8, dtype=dtype).cuda()
    r = seeded_acts(1, 640, seed=9, dtype=dtype).cuda()
    assert torch.equal(a(x, r, norm=(None, 1e-6)), b(x, r, norm=(None, 1e-6)))
    assert torch.equal(a(x, swiglu_up=x.flip(-1)), b(x, swiglu_up=x.flip(-1)))
    from bittorch_amd import _C
    q, s = _C.act_quant_int8(x, True)
    assert torch.equal(a.forward_int8(q, s, torch.bfloat16, None, True), b.forward_int8(q, s, torch.bfloat16, None, True))


def test_module_holds_one_copy_of_its_weights(oracle):
    """After its first GPU call the layer holds the decode-tiled copy only (2 bits per weight: the 16x of the
    reference's tests/test_packed_ternary.py:131-141 holds on the device), while state_dict(), .cpu(), pickling and
    load_state_dict still see `weight_packed` in the reference's layout, bit for bit."""
    import copy
    import pickle
    announce("module single copy")
    n, k = 4096, 4096
    w = random_ternary(n, k, seed=5)
    packed_t, _ = oracle.pack_ternary_transposed(w.numpy())
    from bittorch_amd.nn import TernaryLinearInference
    from bittorch_amd.utils import get_model_memory_bytes
    a = TernaryLinearInference(k, n, torch.from_numpy(packed_t), torch.rand(n) + 0.5).cuda()
    assert a._has_row_major() and a.resident_weight_bytes() == n * k // 4
    x = seeded_acts(1, k, dtype=torch.float16).cuda()
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    y = a(x)
    assert not a._has_row_major() and "weight_packed" not in dict(a.named_buffers())
    assert a.resident_weight_bytes() == n * k // 4                       # 0.25 bytes per weight
    assert get_model_memory_bytes(a)["packed_ternary"] == n * k // 4
    assert 4 * n * k / a.resident_weight_bytes() == 16.0
    del y
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() <= base + (1 << 20)              # the row-major buffer was released
    sd = a.state_dict()
    assert list(sd) == ["weight_packed", "scale"]
    np.testing.assert_array_equal(sd["weight_packed"].cpu().numpy(), packed_t)
    np.testing.assert_array_equal(a.packed_weights().cpu().numpy(), packed_t)
    assert not a._has_row_major()                                         # neither call changed what the layer holds
    for clone in (copy.deepcopy(a), pickle.loads(pickle.dumps(a))):
        assert clone._tiled is None and torch.equal(clone.weight_packed, sd["weight_packed"])
        assert torch.equal(clone(x), a(x))
    c = copy.deepcopy(a).cpu()
    np.testing.assert_array_equal(c.weight_packed.numpy(), packed_t)
    assert rel_err(f32np(c(x.cpu().float())), f32np(a(x))) < 2e-3
    # reading the attribute brings the buffer back for good: in-place edits keep their meaning
    wp = a.weight_packed
    assert a._has_row_major() and a.keep_row_major and a.resident_weight_bytes() == 2 * n * k // 4
    np.testing.assert_array_equal(wp.cpu().numpy(), packed_t)
    wp.zero_()
    assert torch.equal(a(x).float(), torch.zeros(1, n, device="cuda"))
    a.load_state_dict(sd)
    assert torch.equal(a(x), c.cuda()(x))
    a.drop_row_major()
    assert not a._has_row_major() and a.resident_weight_bytes() == n * k // 4
    # fp32 rows of any K read the tiled copy too; a call only the row-major kernels serve (the shape-generic
    # kernel) keeps both from then on
    b = _layer(oracle, 48, 100, seed=2)
    b(seeded_acts(1, 100, dtype=torch.float16).cuda())
    assert not b._has_row_major()
    y32 = b(seeded_acts(2, 100, dtype=torch.float32).cuda())
    assert not b._has_row_major()
    os.environ["BITTORCH_KERNEL"] = "generic"
    try:
        y_gen = b(seeded_acts(2, 100, dtype=torch.float32).cuda())
    finally:
        os.environ.pop("BITTORCH_KERNEL")
    assert b._has_row_major() and b.keep_row_major
    np.testing.assert_allclose(f32np(y32), f32np(y_gen), rtol=1e-4, atol=1e-4)


def test_module_invalidate_after_a_write_through_data(oracle):
    a = _layer(oracle, 64, 64, seed=3)
    x = seeded_acts(1, 64, dtype=torch.float16).cuda()
    a(x)
    wp = a.weight_packed                       # brings the buffer back; the layer holds both copies now
    a(x)
    wp.data.zero_()                            # not seen by the version counter
    a.invalidate_packed_cache()
    assert torch.equal(a(x).float(), a.bias.half().float().expand(1, -1))


def test_module_rebuilds_tiled_copy_when_weights_change(oracle):
    a = _layer(oracle, 64, 64, seed=1)
    x = seeded_acts(1, 64, dtype=torch.float16).cuda()
    y0 = a(x)
    first = a._tiled
    a.weight_packed.zero_()                      # in-place write: the copy is stale
    assert torch.equal(a(x).float(), a.bias.half().float().expand(1, -1))
    assert a._tiled is not first
    other = _layer(oracle, 64, 64, seed=1)
    a.load_state_dict(other.state_dict())        # copy_ into the buffers: stale again
    assert torch.equal(a(x), y0)


def test_module_never_builds_the_copy_inside_a_capture(oracle):
    a = _layer(oracle, 256, 256, seed=2)
    x = seeded_acts(1, 256, dtype=torch.bfloat16).cuda()
    ref = _layer(oracle, 256, 256, seed=2, decode_tiled=False)(x)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        with torch.cuda.graph(g, stream=s):
            y = a(x)
    torch.cuda.current_stream().wait_stream(s)
    assert a._tiled is None                      # fell back to weight_packed
    g.replay()
    torch.cuda.synchronize()
    assert torch.equal(y, ref)
    a.prepare_decode()
    assert a._tiled is not None and torch.equal(a(x), ref)


@pytest.mark.parametrize("n,k", [(64, 64), (96, 100), (13824, 2560), (32, 4)])
def test_retile_gate_up_pair_order(oracle, n, k):
    from bittorch_amd import _C
    announce("retile pairs", n, k)
    _, wt = _packed(oracle, n, k, seed=n + k)
    tiled = _C.retile_weights(wt, k, True)
    np.testing.assert_array_equal(tiled.cpu().numpy(), oracle.retile_weights(wt.cpu().numpy(), k, True))
    assert torch.equal(_C.untile_weights(tiled, n, k, True), wt)
    with pytest.raises(RuntimeError, match="N % 32"):
        _C.retile_weights(wt[:, :n - 16].contiguous(), k, True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,k", [(13824, 2560), (64, 64), (96, 100), (8192, 4096), (320, 1030)])
def test_swiglu_output_stage_equals_projection_then_swiglu(oracle, dtype, n, k):
    """Y = swiglu(gate(x), up(x)) from the GEMV's output stage against the stored projections fed to the
    SwiGLU kernel (which the fused-glue tests hold against the oracle bit for bit)."""
    from bittorch_amd import _C
    _, wt = _packed(oracle, n, k, seed=7)
    tiled = _C.retile_weights(wt, k, True)
    g = torch.Generator().manual_seed(n)
    scale = (torch.rand(n, generator=g) + 0.5).cuda() * 0.05
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype).cuda()
    nw = (torch.rand(k, generator=g) + 0.5).to(dtype).cuda()
    for b in (1, 3, 16, 20):
        x = seeded_acts(b, k, seed=b, dtype=dtype).cuda()
        for norm in (None, (nw, 1e-5)):
            for bs in (None, bias):
                announce("swiglu stage", dtype, n, k, b, norm is not None, bs is not None)
                if norm is None:
                    gu = _C.ternary_linear_packed_forward(x, wt, scale, bs, k)
                else:
                    gu = _C.ternary_linear_packed_forward_fused(x, wt, scale, bs, k, norm=norm)
                ref = _C.swiglu(gu[:, :n // 2], gu[:, n // 2:])
                got = _C.ternary_linear_tiled_forward(x, tiled, scale, bs, k, n, None, norm, None, True)
                assert got.shape == (b, n // 2)
                assert torch.equal(got, ref)
    x = seeded_acts(1, k, dtype=dtype).cuda()
    with pytest.raises(RuntimeError):
        _C.ternary_linear_tiled_forward(x, tiled, scale, None, k, n, torch.zeros(1, n, dtype=dtype).cuda(), None, None, True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_ternary_swiglu_decode_uses_the_output_stage(oracle, dtype):
    from bittorch_amd.nn import TernarySwiGLU
    d, ffn = 256, 704
    gate, up, down = _layer(oracle, ffn, d, seed=1), _layer(oracle, ffn, d, seed=2), _layer(oracle, d, ffn, seed=3)
    for L in (gate, up, down):
        L.scale.mul_(0.05)
    fused = TernarySwiGLU(gate, up, down, compute="float", fuse_gate_up=True)
    assert fused.gate_up.tile_order == "gate_up_pairs"
    plain = TernarySwiGLU(gate, up, down, compute="float", fuse_gate_up=False)
    nw = (torch.rand(d) + 0.5).to(dtype).cuda()
    for rows in (1, 5, 40, 70):
        announce("TernarySwiGLU decode", dtype, rows)
        x = seeded_acts(rows, d, seed=rows, dtype=dtype).cuda()
        if rows <= 32:
            assert torch.equal(fused(x, nw, 1e-5, residual=x), plain(x, nw, 1e-5, residual=x))
            assert torch.equal(fused(x), plain(x))
        else:  # (wider fused layers may split K over another number of waves: same values up to output rounding)
            assert rel_err(f32np(fused(x, nw, 1e-5, residual=x)), f32np(plain(x, nw, 1e-5, residual=x))) <= 1e-2
            assert rel_err(f32np(fused(x)), f32np(plain(x))) <= 1e-2
    assert fused.gate_up._tiled is not None
    # the fused layer called as an ordinary linear layer still gives [gate | up] in natural order
    x = seeded_acts(1, d, dtype=dtype).cuda()
    assert torch.equal(fused.gate_up(x), torch.cat([gate(x), up(x)], dim=-1))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,k", [(13824, 2560), (64, 64), (96, 100), (320, 1030), (8192, 4096)])
def test_pair_ordered_copy_read_in_natural_order(oracle, dtype, n, k):
    """A copy in gate/up pair order read as a plain linear layer (every kernel looks its column tiles up where the pair
    order put them) gives the bits of the natural-order copy: exact GEMV, streaming kernel, tiled GEMM, fp32 planes,
    with bias, residual and the RMSNorm prologue."""
    from bittorch_amd import _C
    _, wt = _packed(oracle, n, k, seed=11)
    nat, pairs = _C.retile_weights(wt, k), _C.retile_weights(wt, k, True)
    g = torch.Generator().manual_seed(n + k)
    scale = (torch.rand(n, generator=g) + 0.5).cuda() * 0.05
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype).cuda()
    nw = (torch.rand(k, generator=g) + 0.5).to(dtype).cuda()
    for b, route in ((1, None), (3, None), (16, None), (40, None), (200, "32"), (200, "2000000")):
        if route is not None:
            set_option("STREAM_MAX_ROWS", route)  # 32: the tiled GEMM; 2000000: the streaming kernel
        x = seeded_acts(b, k, seed=b, dtype=dtype).cuda()
        res = seeded_acts(b, n, seed=b + 1, dtype=dtype).cuda()
        for norm in (None, (nw, 1e-5)):
            for bs, rs in ((None, None), (bias, res)):
                announce("natural from pairs", dtype, n, k, b, route, norm is not None, bs is not None)
                want = _C.ternary_linear_tiled_forward(x, nat, scale, bs, k, n, rs, norm)
                got = _C.ternary_linear_tiled_forward(x, pairs, scale, bs, k, n, rs, norm, None, False, True)
                assert torch.equal(got, want)
        set_option("STREAM_MAX_ROWS", None)
    x = seeded_acts(1, k, dtype=dtype).cuda()
    if n % 32:
        with pytest.raises(RuntimeError):
            _C.ternary_linear_tiled_forward(x, pairs, scale, None, k, n, None, None, None, False, True)


def test_fused_gate_up_layer_keeps_one_copy_through_prefill_and_capture(oracle):
    """A TernarySwiGLU in its float default stores gate|up in pair order.  Decode, prefill (more rows than the decode
    kernels take), fp32 activations and calls recorded into a HIP graph all read that one copy: the row-major buffer
    never comes back, and the outputs equal those of the unfused MLP."""
    from bittorch_amd.nn import TernarySwiGLU
    d, ffn = 256, 704
    gate, up, down = _layer(oracle, ffn, d, seed=1), _layer(oracle, ffn, d, seed=2), _layer(oracle, d, ffn, seed=3)
    for L in (gate, up, down):
        L.scale.mul_(0.05)
    fused = TernarySwiGLU(gate, up, down, compute="float", fuse_gate_up=True)
    plain = TernarySwiGLU(gate, up, down, compute="float", fuse_gate_up=False)
    gu = fused.gate_up
    one_copy = gu.packed_size_bytes
    nw = (torch.rand(d) + 0.5).bfloat16().cuda()
    fused(seeded_acts(1, d, dtype=torch.bfloat16).cuda())  # first call builds the copy and releases weight_packed
    assert gu.resident_weight_bytes() == ((2 * ffn + 15) // 16) * (((d + 3) // 4 + 15) // 16) * 256 and not gu._has_row_major()
    tiled_bytes = gu.resident_weight_bytes()
    assert tiled_bytes < 2 * one_copy
    for dtype, rows in ((torch.bfloat16, 300), (torch.float16, 150), (torch.float32, 1), (torch.float32, 200)):
        announce("fused gate|up one copy", dtype, rows)
        x = seeded_acts(rows, d, seed=rows, dtype=dtype).cuda()
        y, ref = fused(x, nw.to(dtype), 1e-5, residual=x), plain(x, nw.to(dtype), 1e-5, residual=x)
        assert rel_err(f32np(y), f32np(ref)) <= (1e-5 if dtype == torch.float32 else 1e-2)
        assert gu.resident_weight_bytes() == tiled_bytes and not gu._has_row_major() and not gu.keep_row_major
    # a prefill recorded into a graph: same copy, nothing rebuilt inside the capture
    x = seeded_acts(300, d, seed=5, dtype=torch.bfloat16).cuda()
    want = fused(x, nw, 1e-5, residual=x)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = fused(x, nw, 1e-5, residual=x)
    for _ in range(2):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want)
    assert gu.resident_weight_bytes() == tiled_bytes and not gu._has_row_major()
    # the fused layer called as a plain linear layer: natural column order from the pair-ordered copy, bit for bit
    x1 = seeded_acts(1, d, dtype=torch.float16).cuda()
    assert torch.equal(gu(x1), torch.cat([gate(x1), up(x1)], dim=-1))
    assert gu.resident_weight_bytes() == tiled_bytes


def test_row_major_fallback_keeps_its_promises(oracle):
    """(1) A layer whose first call is recorded into a graph runs that call on weight_packed without marking the buffer
    as one to keep: prepare_decode() afterwards still leaves one copy.  (2) A call that needs a released weight_packed
    inside a capture is refused instead of recording the kernel that would rebuild it."""
    a = _layer(oracle, 256, 256, seed=2)
    x = seeded_acts(1, 256, dtype=torch.bfloat16).cuda()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        with torch.cuda.graph(g, stream=s):
            a(x)
    torch.cuda.current_stream().wait_stream(s)
    assert not a.keep_row_major and a._has_row_major()
    del g
    a.prepare_decode()
    assert not a._has_row_major() and a.resident_weight_bytes() == a._tiled.numel()
    # (2) int8 activations on a pair-ordered copy are served by the row-major kernels
    from bittorch_amd import _C
    b = _layer(oracle, 256, 256, seed=3)
    b.tile_order = "gate_up_pairs"
    b.prepare_decode()
    assert not b._has_row_major()
    q, sx = _C.act_quant_int8(x, False)
    s.wait_stream(torch.cuda.current_stream())
    g2 = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="before capturing"):
        with torch.cuda.stream(s):
            with torch.cuda.graph(g2, stream=s):
                b.forward_int8(q, sx)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    want = _layer(oracle, 256, 256, seed=3, decode_tiled=False).forward_int8(q, sx)
    assert torch.equal(b.forward_int8(q, sx), want)   # outside a capture: rebuilt, both copies held from here on
    assert b.keep_row_major and b._has_row_major()
