"""GPU parity of the exact single-row fp16 GEMV (int8 matrix cores, six base-128 digit rows) and of the grouped
launch that runs G such GEMVs at once.

Bar: bit-exact against `oracle.linear_packed_exact_f16` (the dot product summed as an integer and rounded to
fp32 once, then the reference's epilogue `acc * scale + bias`, csrc/kernels/ternary_gemm_production.cu:139-141),
on both weight layouts; against the reference's own fp32-accumulate arithmetic (`oracle.linear_packed`) within
its tests' thresholds (tests/test_packed_kernel.py:44-50: element-wise rtol = atol = 1e-2 for fp16); every unit
of a grouped launch bit-identical to the single call.
"""
import numpy as np
import pytest
import torch

from conftest import announce
from _util import f32np, random_ternary, seeded_acts, set_option

pytestmark = pytest.mark.gpu


def _setup(n, k, seed, per_tensor=False, bias=True, wide=False):
    from bittorch_amd.quant import pack_ternary_transposed
    w = random_ternary(n, k, seed=seed)
    g = torch.Generator().manual_seed(seed + 7)
    scale = torch.rand(1 if per_tensor else n, generator=g) * 0.05 + 0.01
    bias_t = (torch.randn(n, generator=g) * 0.01).half() if bias else None
    x = seeded_acts(1, k, seed=seed + 3, dtype=torch.float32)
    if wide:  # the whole dynamic range of fp16, subnormals included
        x = x * torch.exp2(torch.randint(-24, 12, (1, k), generator=g).float())
    x = x.half()
    packed, _ = pack_ternary_transposed(w)
    return x, packed, scale, bias_t


def _expect(oracle, x, packed, scale, bias, k):
    y = oracle.linear_packed_exact_f16(f32np(x), packed.numpy(), f32np(scale), k, None if bias is None else f32np(bias))
    return torch.from_numpy(y).half()


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("n,k", [(4096, 4096), (64, 64), (16, 16), (100, 144), (2560, 2560), (7680, 2560), (2560, 6912),
                                 (36, 8192), (11008, 4096), (260, 1040), (4, 48), (48, 16384), (2048, 11008)])
def test_single_row_fp16_is_exact_on_both_layouts(oracle, n, k, wide):
    from bittorch_amd import _C
    announce("exact gemv", n, k, wide)
    x, packed, scale, bias, = _setup(n, k, seed=n + k, wide=wide)
    expect = _expect(oracle, x, packed, scale, bias, k)
    xd, pd, sd, bd = x.cuda(), packed.cuda(), scale.cuda(), bias.cuda()
    y_rm = _C.ternary_linear_packed_forward(xd, pd, sd, bd, k)
    tiled = _C.retile_weights(pd, k)
    y_t = _C.ternary_linear_tiled_forward(xd, tiled, sd, bd, k, n)
    torch.cuda.synchronize()
    assert torch.equal(y_rm.cpu(), expect)
    assert torch.equal(y_t.cpu(), expect)
    # the reference's arithmetic (fp32 accumulation in k order), at its own tests' fp16 thresholds
    ref = oracle.linear_packed(f32np(x), packed.numpy(), f32np(scale), k, f32np(bias))
    if not wide:
        np.testing.assert_allclose(f32np(y_t), ref, rtol=1e-2, atol=1e-2)


def test_single_row_fp16_variants(oracle):
    """Per-tensor scale, fp16 scale, no bias, a residual, tile widths of the kernel, ties and extreme values."""
    import os
    from bittorch_amd import _C
    announce("exact gemv variants")
    n, k = 512, 1024
    x, packed, scale, bias = _setup(n, k, seed=3, per_tensor=True)
    xd, pd = x.cuda(), packed.cuda()
    tiled = _C.retile_weights(pd, k)
    expect = _expect(oracle, x, packed, scale, bias, k)
    assert torch.equal(_C.ternary_linear_tiled_forward(xd, tiled, scale.cuda(), bias.cuda(), k, n).cpu(), expect)
    assert torch.equal(_C.ternary_linear_packed_forward(xd, pd, scale.cuda(), bias.cuda(), k).cpu(), expect)
    s16 = scale.half()
    expect16 = _expect(oracle, x, packed, s16.float(), None, k)
    assert torch.equal(_C.ternary_linear_tiled_forward(xd, tiled, s16.cuda(), None, k, n).cpu(), expect16)
    res = seeded_acts(1, n, seed=9, dtype=torch.float16)
    got = _C.ternary_linear_tiled_forward(xd, tiled, scale.cuda(), bias.cuda(), k, n, residual=res.cuda())
    assert torch.equal(got.cpu(), expect + res)
    try:
        for nacc in ("1", "2", "4"):
            set_option("PLANES_NACC", nacc)
            assert torch.equal(_C.ternary_linear_tiled_forward(xd, tiled, scale.cuda(), bias.cuda(), k, n).cpu(), expect)
            assert torch.equal(_C.ternary_linear_packed_forward(xd, pd, scale.cuda(), bias.cuda(), k).cpu(), expect)
    finally:
        set_option("PLANES_NACC", None)
    # one matrix through the contiguous-walk kernel (what a very wide layer takes by itself), residual included
    try:
        set_option("GROUP_WALK", "1")
        for (n2, k2) in ((4096, 4096), (96, 2560), (1000, 1536), (20, 3600)):
            x2, packed2, scale2, bias2 = _setup(n2, k2, seed=n2 + k2 + 1)
            tiled2 = _C.retile_weights(packed2.cuda(), k2)
            expect2 = _expect(oracle, x2, packed2, scale2, bias2, k2)
            got2 = _C.ternary_linear_tiled_forward(x2.cuda(), tiled2, scale2.cuda(), bias2.cuda(), k2, n2)
            assert torch.equal(got2.cpu(), expect2), (n2, k2)
            res2 = seeded_acts(1, n2, seed=5, dtype=torch.float16)
            got2 = _C.ternary_linear_tiled_forward(x2.cuda(), tiled2, scale2.cuda(), bias2.cuda(), k2, n2, residual=res2.cuda())
            assert torch.equal(got2.cpu(), expect2 + res2), (n2, k2)
    finally:
        set_option("GROUP_WALK", None)
    # ties of the final rounding and the largest magnitudes: all-ones weights, crafted activations
    from bittorch_amd.quant import pack_ternary_transposed
    ones = pack_ternary_transposed(torch.ones(16, 16, dtype=torch.int8))[0]
    u = 2.0 ** -24
    for vals in ([1.0, u], [1.0, u, u, u], [-1.0, -u], [65504.0] * 16, [65504.0, u, -65504.0], [-0.0, 0.0]):
        xv = torch.zeros(1, 16, dtype=torch.float16)
        xv[0, :len(vals)] = torch.tensor(vals, dtype=torch.float64).half()
        e = _expect(oracle, xv, ones, torch.ones(16), None, 16)
        assert torch.equal(_C.ternary_linear_packed_forward(xv.cuda(), ones.cuda(), torch.ones(16).cuda(), None, 16).cpu(), e)
    # an infinity or a NaN in the row: column by column what the reference's float loop leaves (the oracle restates it)
    for pos, val in (((5,), float("inf")), ((5, k - 1), float("-inf")), ((0,), float("nan"))):
        xv = x.clone()
        for q_ in pos:
            xv[0, q_] = val
        e = _expect(oracle, xv, packed, scale, bias, k)
        assert torch.isnan(e).any() and (torch.isinf(e).any() or val != val)
        got_t = _C.ternary_linear_tiled_forward(xv.cuda(), tiled, scale.cuda(), bias.cuda(), k, n).cpu()
        got_r = _C.ternary_linear_packed_forward(xv.cuda(), packed.cuda(), scale.cuda(), bias.cuda(), k).cpu()
        for got in (got_t, got_r):
            assert torch.equal(torch.isnan(got), torch.isnan(e))
            assert torch.equal(torch.nan_to_num(got, nan=0.0), torch.nan_to_num(e, nan=0.0))


def _tables(_C, xs, tiles, scales, biases, ys):
    return (_C.pointer_table(xs), _C.pointer_table(tiles), _C.pointer_table(scales),
            None if biases is None else _C.pointer_table(biases), _C.pointer_table(ys))


@pytest.mark.parametrize("g,n,k,per_tensor,bias", [(1, 4096, 4096, True, True), (5, 256, 512, False, True),
                                                   (37, 1024, 1024, False, False), (3, 100, 144, False, True),
                                                   (9, 2560, 6912, True, True), (130, 128, 64, False, True),
                                                   (4, 36, 8192, False, True), (3, 64, 11008, False, True),
                                                   (2, 32, 16384, True, True),
                                                   # K of 3..8 steps per wave: the contiguous-walk kernel
                                                   (7, 96, 2560, False, True), (3, 2560, 2560, True, True),
                                                   (5, 64, 1536, False, False), (11, 4128, 3008, False, True),
                                                   (6, 48, 3600, True, True), (4, 32, 4080, False, True),
                                                   (70, 544, 4096, False, True), (2, 20, 1104, False, True),
                                                   (600, 32, 2048, False, True)])
def test_grouped_launch_equals_single_calls(oracle, g, n, k, per_tensor, bias):
    import os
    from bittorch_amd import _C
    announce("grouped gemv", g, n, k)
    xs, tiles, scales, biases, singles = [], [], [], [], []
    for u in range(g):
        x, packed, scale, b = _setup(n, k, seed=100 * u + n, per_tensor=per_tensor, bias=bias, wide=(u % 2 == 1))
        xs.append(x.cuda())
        tiles.append(_C.retile_weights(packed.cuda(), k))
        scales.append(scale.cuda())
        biases.append(b.cuda() if bias else None)
        singles.append(_C.ternary_linear_tiled_forward(xs[-1], tiles[-1], scales[-1], biases[-1], k, n))
        if u == 0:
            assert torch.equal(singles[0].cpu(), _expect(oracle, x, packed, scale, b, k))
    # the library's own choice of kernel, then the contiguous-walk kernel (where the shape allows it), the
    # one-stream-per-wave kernel in its three widths and the one-matrix kernel over (unit, tile) workgroups
    try:
        for walk, nacc, units in ((None, None, None), ("1", None, "0"), ("0", "1", "0"), ("0", "2", "0"), ("0", "4", "0"),
                                  (None, None, "1")):
            for name, val in (("GROUP_WALK", walk), ("GROUP_NACC", nacc), ("GROUP_UNITS", units)):
                set_option(name, val)
            ys = [torch.full((1, n), float("nan"), dtype=torch.float16, device="cuda") for _ in range(g)]
            tabs = _tables(_C, xs, tiles, scales, biases if bias else None, ys)
            _C.ternary_gemv_grouped(*tabs, k, n, scale_len=1 if per_tensor else n)
            torch.cuda.synchronize()
            for u in range(g):
                assert torch.equal(ys[u], singles[u]), (u, walk, nacc, units)
    finally:
        set_option("GROUP_NACC", None)
        set_option("GROUP_WALK", None)
        set_option("GROUP_UNITS", None)


def test_grouped_launch_config2_units_and_shared_operands(oracle):
    """G = 24 config-2 units (x fp16 [1,4096], W [4096,4096], per-tensor fp32 scale, fp16 bias), some units
    sharing their activations or their weights; second call on the same tables gives the same result."""
    from bittorch_amd import _C
    announce("grouped gemv config 2")
    n = k = 4096
    base = [_setup(n, k, seed=s, per_tensor=True) for s in range(4)]
    xs_, tiles_, scales_, biases_ = [], [], [], []
    for (x, packed, scale, b) in base:
        xs_.append(x.cuda()); tiles_.append(_C.retile_weights(packed.cuda(), k)); scales_.append(scale.cuda()); biases_.append(b.cuda())
    units = [(u % 4, (u // 4) % 4) for u in range(24)]  # (activation, weight) index pairs
    xs = [xs_[a] for a, _ in units]
    tiles = [tiles_[w] for _, w in units]
    scales = [scales_[w] for _, w in units]
    biases = [biases_[w] for _, w in units]
    ys = [torch.empty(1, n, dtype=torch.float16, device="cuda") for _ in units]
    tabs = _tables(_C, xs, tiles, scales, biases, ys)
    for _ in range(2):
        for y in ys:
            y.fill_(float("nan"))
        _C.ternary_gemv_grouped(*tabs, k, n, scale_len=1)
        torch.cuda.synchronize()
        for (a, w), y in zip(units, ys):
            x, packed, scale, b = base[a][0], base[w][1], base[w][2], base[w][3]
            assert torch.equal(y, _C.ternary_linear_tiled_forward(xs_[a], tiles_[w], scales_[w], biases_[w], k, n))
    x, packed, scale, b = base[1][0], base[2][1], base[2][2], base[2][3]
    assert torch.equal(ys[units.index((1, 2))].cpu(), _expect(oracle, x, packed, scale, b, k))


def test_grouped_launch_non_finite_row_and_large_group(oracle, monkeypatch):
    """160 units of 2048 x 2048 (the contiguous-walk kernel by the library's own rule): one unit's row holds an
    infinity and gets what the reference's float loop leaves (NaN on zero weights, the signed infinity elsewhere), its
    neighbours are untouched."""
    from bittorch_amd import _C
    announce("grouped gemv non-finite")
    n = k = 2048
    base = [_setup(n, k, seed=s, per_tensor=False) for s in range(3)]
    tiles_ = [_C.retile_weights(b[1].cuda(), k) for b in base]
    g = 160
    xs = [base[u % 3][0].clone().cuda() for u in range(g)]
    xs[77][0, 1999] = float("inf")
    tiles = [tiles_[u % 3] for u in range(g)]
    scales = [base[u % 3][2].cuda() for u in range(g)]
    biases = [base[u % 3][3].cuda() for u in range(g)]
    ys = [torch.empty(1, n, dtype=torch.float16, device="cuda") for _ in range(g)]
    _C.ternary_gemv_grouped(*_tables(_C, xs, tiles, scales, biases, ys), k, n, scale_len=n)
    torch.cuda.synchronize()
    xe = base[77 % 3][0].clone()
    xe[0, 1999] = float("inf")
    e77 = _expect(oracle, xe, base[77 % 3][1], base[77 % 3][2], base[77 % 3][3], k)
    assert torch.isnan(e77).any() and torch.isinf(e77).any()   # zero weights and +-1 weights at that position
    assert torch.equal(torch.isnan(ys[77].cpu()), torch.isnan(e77))
    assert torch.equal(torch.nan_to_num(ys[77].cpu(), nan=0.0), torch.nan_to_num(e77, nan=0.0))
    for u in (0, 76, 78, 159):
        b = base[u % 3]
        assert torch.equal(ys[u].cpu(), _expect(oracle, b[0], b[1], b[2], b[3], k))


def test_grouped_launch_argument_errors():
    from bittorch_amd import _C, _lib
    lib = _lib.load()
    t = torch.zeros(8, dtype=torch.int64, device="cuda")
    p = t.data_ptr()
    assert lib.bt_ternary_gemv_grouped(None, 1, p, p, 0, 16, None, 1, p, 8, 16, 16, None) == -1
    assert "null" in _lib.last_error()
    assert lib.bt_ternary_gemv_grouped(p, 0, p, p, 0, 16, None, 1, p, 8, 16, 16, None) == -1
    assert "fp16" in _lib.last_error()
    assert lib.bt_ternary_gemv_grouped(p, 1, p, p, 0, 16, None, 1, p, 8, 16, 24, None) == -1
    assert "multiple of 16" in _lib.last_error()
    assert lib.bt_ternary_gemv_grouped(p, 1, p, p, 0, 5, None, 1, p, 8, 16, 16, None) == -1
    assert "scale" in _lib.last_error()
    assert lib.bt_ternary_gemv_grouped(p, 1, p, p, 0, 16, None, 1, p, 0, 16, 16, None) == -1


_grp_rng = np.random.default_rng(977)
_GROUP_CASES = [(int(_grp_rng.integers(1, 40)), int(_grp_rng.integers(1, 80)) * 4,
                 int(_grp_rng.integers(65, 257)) * 16, bool(_grp_rng.integers(0, 2)), bool(_grp_rng.integers(0, 2)), i)
                for i in range(24)]


@pytest.mark.parametrize("g,n,k,per_tensor,bias,seed", _GROUP_CASES)
def test_grouped_launch_random_shapes(oracle, g, n, k, per_tensor, bias, seed):
    """Seeded random G, N (any multiple of 4) and K (1040 .. 4096, the range of the contiguous-walk kernel), units
    drawn from three weight matrices and three activation rows: the walk kernel where the shape allows it, the
    one-stream-per-wave kernel and the one-matrix kernel over (unit, tile) workgroups all equal the single calls, and
    those the oracle."""
    import os
    from bittorch_amd import _C
    announce("grouped gemv random", g, n, k, per_tensor, bias, seed)
    base = [_setup(n, k, seed=1000 + 7 * seed + s, per_tensor=per_tensor, bias=bias, wide=(s == 1)) for s in range(3)]
    xs_ = [b[0].cuda() for b in base]
    tiles_ = [_C.retile_weights(b[1].cuda(), k) for b in base]
    units = [(int(_grp_rng.integers(0, 3)), int(_grp_rng.integers(0, 3))) for _ in range(g)]
    xs = [xs_[a] for a, _ in units]
    tiles = [tiles_[w] for _, w in units]
    scales = [base[w][2].cuda() for _, w in units]
    biases = [base[w][3].cuda() for _, w in units] if bias else None
    singles = {}
    for (a, w) in set(units):
        singles[(a, w)] = _C.ternary_linear_tiled_forward(xs_[a], tiles_[w], base[w][2].cuda(),
                                                          base[w][3].cuda() if bias else None, k, n)
    a0, w0 = units[0]
    assert torch.equal(singles[(a0, w0)].cpu(), _expect(oracle, base[a0][0], base[w0][1], base[w0][2], base[w0][3], k))
    try:
        for walk, one_matrix in (("1", "0"), ("0", "0"), ("0", "1")):
            set_option("GROUP_WALK", walk)
            set_option("GROUP_UNITS", one_matrix)
            ys = [torch.full((1, n), float("nan"), dtype=torch.float16, device="cuda") for _ in range(g)]
            _C.ternary_gemv_grouped(*_tables(_C, xs, tiles, scales, biases, ys), k, n, scale_len=1 if per_tensor else n)
            torch.cuda.synchronize()
            for u in range(g):
                assert torch.equal(ys[u], singles[units[u]]), (u, walk, one_matrix)
    finally:
        set_option("GROUP_WALK", None)
        set_option("GROUP_UNITS", None)


# ---- bf16 rows: scaled by the row's largest exponent, summed exactly ---------------------------------------------------
def _setup_bf16(n, k, seed, per_tensor=False, bias=True, spread=0):
    from bittorch_amd.quant import pack_ternary_transposed
    w = random_ternary(n, k, seed=seed)
    g = torch.Generator().manual_seed(seed + 7)
    scale = torch.rand(1 if per_tensor else n, generator=g) * 0.05 + 0.01
    x = seeded_acts(1, k, seed=seed + 3, dtype=torch.float32)
    if spread:  # elements down to `spread` binades below the largest, and a row exponent far from 0
        x = x * torch.exp2(-torch.randint(0, spread, (1, k), generator=g).float()) * (2.0 ** ((seed % 7) * 11 - 30))
    x = x.bfloat16()
    bias_t = (torch.randn(n, generator=g) * 0.01 * float(x.abs().max())).bfloat16() if bias else None
    packed, _ = pack_ternary_transposed(w)
    return x, packed, scale, bias_t


def _expect_bf16(oracle, x, packed, scale, bias, k):
    y = oracle.linear_packed_rowscaled_bf16(f32np(x), packed.numpy(), f32np(scale), k, None if bias is None else f32np(bias))
    return torch.from_numpy(y).bfloat16()


@pytest.mark.parametrize("g,n,k,per_tensor,bias,spread", [(1, 4096, 4096, True, True, 0), (7, 96, 2560, False, True, 20),
                                                          (3, 2560, 2560, True, False, 45), (5, 64, 1536, False, True, 38),
                                                          (11, 4128, 3008, False, True, 0), (140, 512, 2048, False, True, 30),
                                                          (4, 32, 4080, False, True, 60),
                                                          # shapes outside the contiguous walk: the one-stream-per-wave kernel
                                                          (3, 100, 144, False, True, 10), (2, 36, 8192, False, True, 50),
                                                          (5, 2560, 6912, True, True, 0), (2, 48, 16384, False, False, 33),
                                                          (40, 16, 64, False, True, 5), (3, 520, 1024, False, True, 25)])
def test_grouped_bf16_units_against_the_oracle(oracle, g, n, k, per_tensor, bias, spread):
    """bf16 units of a grouped launch: bit-exact against the oracle's restatement of the row-scaled integer sum, and
    within the reference tests' 16-bit thresholds (tests/test_packed_kernel.py:44-50) of the fp32-accumulate arithmetic.
    Where the shape allows both kernels, both run."""
    import os
    from bittorch_amd import _C
    announce("grouped gemv bf16", g, n, k, spread)
    sets = [_setup_bf16(n, k, seed=50 * u + n, per_tensor=per_tensor, bias=bias, spread=spread) for u in range(min(g, 5))]
    tiles_ = [_C.retile_weights(s_[1].cuda(), k) for s_ in sets]
    idx = [u % len(sets) for u in range(g)]
    xs = [sets[i][0].cuda() for i in idx]
    tiles = [tiles_[i] for i in idx]
    scales = [sets[i][2].cuda() for i in idx]
    biases = [sets[i][3].cuda() for i in idx] if bias else None
    expects = [_expect_bf16(oracle, *s_, k) for s_ in sets]
    try:
        for walk in (None, "0"):
            set_option("GROUP_WALK", None)
            if walk:
                set_option("GROUP_WALK", walk)
            ys = [torch.full((1, n), float("nan"), dtype=torch.bfloat16, device="cuda") for _ in range(g)]
            _C.ternary_gemv_grouped(*_tables(_C, xs, tiles, scales, biases, ys), k, n, scale_len=1 if per_tensor else n,
                                    bias_dtype=torch.bfloat16, x_dtype=torch.bfloat16)
            torch.cuda.synchronize()
            for u in range(g):
                assert torch.equal(ys[u].cpu(), expects[idx[u]]), (u, walk)
    finally:
        set_option("GROUP_WALK", None)
    x, packed, scale, b = sets[0]
    ref = oracle.linear_packed(f32np(x), packed.numpy(), f32np(scale), k, None if b is None else f32np(b))
    np.testing.assert_allclose(f32np(ys[0]), ref, rtol=1e-2, atol=1e-2 * float(np.abs(ref).max()))


def test_bf16_row_times_a_wide_matrix_and_argument_errors(oracle):
    """One bf16 row through the single-matrix entry point takes the same kernel where the matrix is wide enough
    (forced here on a small one); a non-finite row gets the float loop's answer; bad arguments of the grouped entry point are refused."""
    import os
    from bittorch_amd import _C, _lib
    announce("bf16 wide row")
    n, k = 1024, 2560
    x, packed, scale, bias = _setup_bf16(n, k, seed=5, spread=25)
    tiled = _C.retile_weights(packed.cuda(), k)
    y_stream = _C.ternary_linear_tiled_forward(x.cuda(), tiled, scale.cuda(), bias.cuda(), k, n)
    try:
        set_option("GROUP_WALK", "1")
        y = _C.ternary_linear_tiled_forward(x.cuda(), tiled, scale.cuda(), bias.cuda(), k, n)
        assert torch.equal(y.cpu(), _expect_bf16(oracle, x, packed, scale, bias, k))
        res = seeded_acts(1, n, seed=9, dtype=torch.bfloat16)
        y_r = _C.ternary_linear_tiled_forward(x.cuda(), tiled, scale.cuda(), bias.cuda(), k, n, residual=res.cuda())
        assert torch.equal(y_r.cpu(), y.cpu() + res)
        xb = x.clone()
        xb[0, 77] = float("nan")
        assert torch.isnan(_C.ternary_linear_tiled_forward(xb.cuda(), tiled, scale.cuda(), bias.cuda(), k, n)).all()
        xb[0, 77] = float("inf")
        e = _expect_bf16(oracle, xb, packed, scale, bias, k)
        got = _C.ternary_linear_tiled_forward(xb.cuda(), tiled, scale.cuda(), bias.cuda(), k, n).cpu()
        assert torch.isinf(e).any() and torch.equal(torch.isnan(got), torch.isnan(e))
        assert torch.equal(torch.nan_to_num(got, nan=0.0), torch.nan_to_num(e, nan=0.0))
    finally:
        set_option("GROUP_WALK", None)
    # the 16-bit matrix-core kernel (what a narrow matrix takes) agrees within bf16 rounding
    np.testing.assert_allclose(f32np(y_stream), f32np(y), rtol=2e-2, atol=2e-2 * float(f32np(y).__abs__().max()))
    lib = _lib.load()
    t = torch.zeros(8, dtype=torch.int64, device="cuda")
    p = t.data_ptr()
    assert lib.bt_ternary_gemv_grouped(p, 2, p, p, 0, 64, None, 2, p, 1, 64, 16400, None) == -1   # K beyond 16384
    assert "at most 16384" in _lib.last_error()
    assert lib.bt_ternary_gemv_grouped(p, 2, p, p, 0, 48, None, 2, p, 1, 48, 4104, None) == -1    # K % 16 != 0
    assert "multiple of 16" in _lib.last_error()


def test_ops_ternary_linear_grouped_equals_the_single_calls(oracle):
    """The caller the kept API offers for the grouped launch: `ops.ternary_linear_grouped(layers, xs)` returns, row
    by row, the bits of `layer(x_row)` for fp16 rows (and the row-scaled exact sums for bf16 rows), with a shared
    row, per-layer rows, an `out=` buffer, cached pointer tables that notice a layer whose buffers moved, and the
    single-call fallback for what the grouped kernel does not take."""
    import bittorch_amd as bt
    from bittorch_amd.nn import TernaryLinearInference
    n, k, g = 384, 512, 6
    layers = []
    for u in range(g):
        w = random_ternary(n, k, seed=40 + u)
        packed, _ = oracle.pack_ternary_transposed(w.numpy())
        gen = torch.Generator().manual_seed(u)
        layers.append(TernaryLinearInference(k, n, torch.from_numpy(packed), torch.rand(n, generator=gen) * 0.05 + 0.01,
                                             (torch.randn(n, generator=gen) * 0.01).half()).cuda())
    xs = seeded_acts(g, k, seed=3, dtype=torch.float16).cuda()
    announce("ops.ternary_linear_grouped fp16")
    want = torch.cat([L(xs[u:u + 1]) for u, L in enumerate(layers)])
    got = bt.ops.ternary_linear_grouped(layers, xs)
    assert got.shape == (g, n) and torch.equal(got, want)
    # again (cached tables), into a caller's buffer, from a list of rows, and one row shared by every layer
    out = torch.empty(g, n, dtype=torch.float16, device="cuda")
    assert bt.ops.ternary_linear_grouped(layers, xs, out=out) is out and torch.equal(out, want)
    assert torch.equal(bt.ops.ternary_linear_grouped(layers, [xs[u] for u in range(g)]), want)
    shared = torch.cat([L(xs[:1]) for L in layers])
    assert torch.equal(bt.ops.ternary_linear_grouped(layers, xs[0]), shared)
    # a layer whose buffers moved: the cached tables are rebuilt
    layers[2].scale = layers[2].scale.clone() * 2
    want2 = torch.cat([L(xs[u:u + 1]) for u, L in enumerate(layers)])
    assert torch.equal(bt.ops.ternary_linear_grouped(layers, xs), want2) and not torch.equal(want2, want)
    # bf16 rows: exact row-scaled sums, within the single call's fp32 rounding
    for L in layers:
        L.bias = L.bias.bfloat16()
    xb = xs.bfloat16()
    got_b = bt.ops.ternary_linear_grouped(layers, xb)
    want_b = torch.cat([L(xb[u:u + 1]) for u, L in enumerate(layers)])
    np.testing.assert_allclose(f32np(got_b), f32np(want_b), rtol=1e-2, atol=1e-2)
    # fallbacks: fp32 rows and CPU tensors run the single calls
    xf = xs.float()
    for L in layers:
        L.bias = L.bias.float()
    assert torch.equal(bt.ops.ternary_linear_grouped(layers, xf), torch.cat([L(xf[u:u + 1]) for u, L in enumerate(layers)]))
    cpu_layers = [TernaryLinearInference(k, n, L.packed_weights().cpu(), L.scale.cpu(), L.bias.cpu()) for L in layers[:2]]
    yc = bt.ops.ternary_linear_grouped(cpu_layers, xf[:2].cpu())
    assert yc.shape == (2, n) and not yc.is_cuda
    # argument errors in the reference's style
    with pytest.raises(RuntimeError, match="doesn't match in_features"):
        bt.ops.ternary_linear_grouped(layers, xs[:, :k - 16])
    other = TernaryLinearInference(k, n + 16, torch.zeros(k // 4, n + 16, dtype=torch.uint8), torch.ones(n + 16)).cuda()
    with pytest.raises(ValueError, match="same in_features and out_features"):
        bt.ops.ternary_linear_grouped(layers + [other], xs[0])


def _same_with_nans(a, b):
    return torch.equal(torch.isnan(a), torch.isnan(b)) and torch.equal(torch.nan_to_num(a, nan=0.0), torch.nan_to_num(b, nan=0.0))


def test_non_finite_rows_through_prologues_and_the_swiglu_stage(oracle):
    """Rows that are (or become, inside an activation prologue) non-finite: the fused calls still equal the unfused
    sequences -- row kernel, then the exact GEMV, then the SwiGLU kernel -- NaN for NaN and infinity for infinity."""
    from bittorch_amd import _C
    n, k = 256, 512
    x, packed, scale, bias = _setup(n, k, seed=21)
    pd, sd, bd = packed.cuda(), scale.cuda(), bias.cuda()
    nat, pairs = _C.retile_weights(pd, k), _C.retile_weights(pd, k, True)
    g = torch.Generator().manual_seed(5)
    nw = (torch.rand(k, generator=g) + 0.5).half().cuda()
    up = seeded_acts(1, k, seed=6, dtype=torch.float16).cuda()
    cases = []
    xi = x.clone(); xi[0, 7] = float("inf"); cases.append(("inf", xi, nw))
    xn = x.clone(); xn[0, 300] = float("nan"); cases.append(("nan", xn, nw))
    xo = x.clone(); xo[0, 11] = 60000.0; cases.append(("overflows in the norm", xo, (nw * 6000).half()))  # finite in, Inf after the norm
    for name, xc, w in cases:
        announce("non-finite through prologues", name)
        xc = xc.cuda()
        normed = _C.rmsnorm(xc, w, 1e-5)
        assert not torch.isfinite(normed.float()).all()
        for tiled_, kw in ((nat, {}), (pairs, dict(natural_from_pairs=True))):
            want = _C.ternary_linear_tiled_forward(normed, tiled_, sd, bd, k, n, **kw)
            got = _C.ternary_linear_tiled_forward(xc, tiled_, sd, bd, k, n, norm=(w, 1e-5), **kw)
            assert _same_with_nans(got, want), name
        assert _same_with_nans(_C.ternary_linear_packed_forward_fused(xc, pd, sd, bd, k, norm=(w, 1e-5)),
                               _C.ternary_linear_packed_forward(normed, pd, sd, bd, k)), name
        # SwiGLU prologue: silu(x) * up
        h = _C.swiglu(xc, up)
        assert _same_with_nans(_C.ternary_linear_tiled_forward(xc, nat, sd, bd, k, n, swiglu_up=up),
                               _C.ternary_linear_tiled_forward(h, nat, sd, bd, k, n)), name
        # SwiGLU output stage on the pair-ordered copy (with and without the norm prologue)
        for norm in (None, (w, 1e-5)):
            xin = xc if norm is None else normed
            gu = _C.ternary_linear_tiled_forward(xin, nat, sd, bd, k, n)
            want = _C.swiglu(gu[:, :n // 2], gu[:, n // 2:])
            got = _C.ternary_linear_tiled_forward(xc, pairs, sd, bd, k, n, None, norm, None, True)
            assert _same_with_nans(got, want), (name, norm is not None)
