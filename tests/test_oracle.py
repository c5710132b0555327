"""Pins the CPU oracle (oracle/bt_oracle.c) without the GPU:
reference-held known answers (tests/golden/known_answers.json), brute force in
pure Python on tiny inputs, closed forms / invariants, and torch's CPU ops
executing the reference's formula as an independent library routine."""
import json
import os

import numpy as np
import pytest
import torch

from _util import random_ternary, seeded_acts, seeded_weights

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "known_answers.json")) as fh:
    GOLD = json.load(fh)


def _filled(spec):
    return np.full(spec["shape"], spec["value"], dtype=np.float32)


# ---------------------------------------------------------------- quantizer (a1)
@pytest.mark.parametrize("case", GOLD["quantize"], ids=lambda c: c["cite"])
def test_quantize_known_answers(oracle, case):
    w = np.array(case["weight"], dtype=np.float32) if "weight" in case else _filled(case["weight_fill"])
    w_tern, scale = oracle.ternary_quantize(w, case["tf"], case["per_channel"])
    if "scale" in case:
        np.testing.assert_allclose(scale, np.array(case["scale"], dtype=np.float32), rtol=1e-6)
        np.testing.assert_array_equal(w_tern, np.array(case["w_tern"]))
    else:
        assert (scale == case["scale_fill"]).all() and (w_tern == case["w_tern_fill"]).all()


def test_quantize_brute_force(oracle):
    """Element-by-element Python evaluation of the definition on small tensors."""
    rng = np.random.default_rng(0)
    for per_channel in (True, False):
        w = rng.standard_normal((5, 7)).astype(np.float32)
        w[2, 3] = 0.0
        w[4] = 0.0
        got_t, got_s = oracle.ternary_quantize(w, 0.3, per_channel)
        tf = np.float32(0.3)
        for n in range(5):
            s = np.abs(w[n]).max() if per_channel else np.abs(w).max()
            s = max(np.float32(s), np.float32(1e-8))
            assert got_s[n if per_channel else 0] == s
            thr = np.float32(tf * s)
            for k in range(7):
                expect = 0 if not (abs(w[n, k]) > thr) else (1 if w[n, k] > 0 else -1)
                assert got_t[n, k] == expect


def test_quantize_edge_semantics(oracle):
    # tf = 0: only true zeros map to 0 (reference tests/test_ternary_quant.py:180-189)
    w = seeded_weights(32, 64, seed=1, std=1.0).numpy()
    w[0, 0] = 0.0
    t, _ = oracle.ternary_quantize(w, 0.0)
    assert (t == 0).sum() == (w == 0).sum()
    # tf = 1: nothing exceeds its own row maximum (tests/test_ternary_quant.py:191-197)
    t, _ = oracle.ternary_quantize(w, 1.0)
    assert (t == 0).all()
    # signs are preserved, values are ternary (:17-27, :80-87)
    t, _ = oracle.ternary_quantize(w, 0.05)
    assert set(np.unique(t)) <= {-1, 0, 1}
    assert ((t == 0) | (np.sign(w) == t)).all()
    # all-zero row: scale is the floor, codes are zero
    z = np.zeros((2, 8), dtype=np.float32)
    t, s = oracle.ternary_quantize(z, 0.05)
    assert (t == 0).all() and (s == np.float32(1e-8)).all()
    # threshold compare is strict: an element equal to the threshold is dropped
    w2 = np.array([[1.0, 0.5, -0.5, 0.25]], dtype=np.float32)
    t, _ = oracle.ternary_quantize(w2, 0.5)
    np.testing.assert_array_equal(t, [[1, 0, 0, 0]])


@pytest.mark.parametrize("dtype,tag", [(torch.float32, 0), (torch.float16, 1), (torch.bfloat16, 2)])
@pytest.mark.parametrize("per_channel", [True, False])
def test_quantize_matches_torch_ops(oracle, dtype, tag, per_channel):
    """torch's CPU kernels evaluating abs/max/clamp/mul/gt/sign/where fix the rounding of
    the threshold (fl(0.05f * scale) in the weight dtype); the oracle must agree bit for bit."""
    from bittorch_amd.quant import ternary_quantize
    for seed, (n, k), std in ((0, (64, 128), 0.02), (1, (7, 33), 1.0), (2, (16, 1000), 1e-4)):
        w = seeded_weights(n, k, seed=seed, std=std, dtype=dtype)
        ref_t, ref_s = ternary_quantize(w, 0.05, per_channel)
        got_t, got_s = oracle.ternary_quantize(w.float().numpy(), 0.05, per_channel, dtype=tag)
        np.testing.assert_array_equal(got_t, ref_t.float().numpy().astype(np.int8))
        np.testing.assert_array_equal(got_s.reshape(-1), ref_s.float().reshape(-1).numpy())


# ---------------------------------------------------------------- codec (a3-a5)
@pytest.mark.parametrize("case", GOLD["pack"], ids=lambda c: c["cite"])
def test_pack_known_answers(oracle, case):
    w = np.array(case["w_tern"], dtype=np.int8) if "w_tern" in case else _filled(case["w_tern_fill"]).astype(np.int8)
    packed, k = oracle.pack_ternary(w)
    assert packed.dtype == np.uint8 and k == w.shape[1]
    if "packed" in case:
        np.testing.assert_array_equal(packed, np.array(case["packed"], dtype=np.uint8))
    if "packed_fill" in case:
        assert (packed == case["packed_fill"]).all()
    if "packed_shape" in case:
        assert list(packed.shape) == case["packed_shape"]
    np.testing.assert_array_equal(oracle.unpack_ternary(packed, k), w)
    packed_t, _ = oracle.pack_ternary_transposed(w)
    np.testing.assert_array_equal(packed_t, packed.T)
    np.testing.assert_array_equal(oracle.unpack_ternary_transposed(packed_t, k), w)


def test_pack_brute_force_and_roundtrip(oracle):
    for (n, k) in [(1, 1), (3, 5), (7, 13), (4, 8), (32, 64), (9, 31)]:
        w = random_ternary(n, k, seed=n * 17 + k).numpy()
        packed, _ = oracle.pack_ternary(w)
        assert packed.shape == (n, (k + 3) // 4)
        for r in range(n):
            for kb in range((k + 3) // 4):
                byte = 0
                for i in range(4):
                    kk = 4 * kb + i
                    v = int(w[r, kk]) if kk < k else 0
                    byte |= {0: 0, 1: 1, -1: 2}[v] << (2 * i)
                assert packed[r, kb] == byte
        np.testing.assert_array_equal(oracle.unpack_ternary(packed, k), w)


def test_unpack_reserved_code_is_zero(oracle):
    packed = np.array([[0xFF, 0b11100100]], dtype=np.uint8)  # codes 3,3,3,3 | 0,1,2,3
    np.testing.assert_array_equal(oracle.unpack_ternary(packed, 8), [[0, 0, 0, 0, 0, 1, -1, 0]])


def test_codec_matches_torch_host_functions(oracle):
    from bittorch_amd.quant import pack_ternary, pack_ternary_transposed, unpack_ternary_transposed
    for (n, k) in [(256, 512), (17, 123), (5, 6)]:
        w = random_ternary(n, k, seed=3)
        np.testing.assert_array_equal(oracle.pack_ternary(w.numpy())[0], pack_ternary(w)[0].numpy())
        pt = pack_ternary_transposed(w)[0]
        np.testing.assert_array_equal(oracle.pack_ternary_transposed(w.numpy())[0], pt.numpy())
        np.testing.assert_array_equal(oracle.unpack_ternary_transposed(pt.numpy(), k),
                                      unpack_ternary_transposed(pt, k).numpy())


@pytest.mark.parametrize("case", GOLD["sizes"], ids=lambda c: c["cite"])
def test_packed_size_known_answers(case):
    from bittorch_amd.quant import get_packed_size
    assert get_packed_size(case["out_features"], case["in_features"]) == case["packed_size"]


# ---------------------------------------------------------------- float linear (a6)
@pytest.mark.parametrize("case", GOLD["matmul"], ids=lambda c: c["cite"])
def test_linear_known_answers(oracle, case):
    w = np.array(case["weights"], dtype=np.int8)
    packed_t, k = oracle.pack_ternary_transposed(w)
    x = np.array(case["input"], dtype=np.float32)
    scale = np.array(case["scales"], dtype=np.float32)
    expect = np.array(case["output"], dtype=np.float32)
    np.testing.assert_array_equal(oracle.linear_packed(x, packed_t, scale, k), expect)
    np.testing.assert_array_equal(oracle.linear_unpacked(x, w, scale), expect)
    np.testing.assert_array_equal(oracle.linear_packed(x, packed_t, scale, k, f64=True), expect)


def test_linear_textbook_and_special_cases(oracle):
    for (b, n, k) in [(4, 8, 16), (3, 33, 17), (1, 1, 1), (8, 64, 130)]:
        w = random_ternary(n, k, seed=k).numpy()
        x = seeded_acts(b, k, seed=1).numpy()
        rng = np.random.default_rng(k)
        scale = rng.random(n).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32)
        packed_t, _ = oracle.pack_ternary_transposed(w)
        truth = x.astype(np.float64) @ (w.astype(np.float64) * scale[:, None].astype(np.float64)).T + bias
        y64 = oracle.linear_packed(x, packed_t, scale, k, bias, f64=True)
        np.testing.assert_allclose(y64, truth, rtol=1e-12, atol=1e-12)
        y32 = oracle.linear_packed(x, packed_t, scale, k, bias)
        np.testing.assert_allclose(y32, truth, rtol=1e-4, atol=1e-4)
        np.testing.assert_array_equal(oracle.linear_unpacked(x, w, scale, bias), y32)
        # per-tensor scale broadcasts
        y1 = oracle.linear_packed(x, packed_t, scale[:1], k, bias)
        np.testing.assert_array_equal(y1, oracle.linear_packed(x, packed_t, np.full(n, scale[0], np.float32), k, bias))
    # all-zero weights give the bias, all-ones weights give the row sums
    # (reference tests/test_ternary_cuda.py:216-247)
    x = seeded_acts(4, 16, seed=2).numpy()
    bias = np.arange(8, dtype=np.float32)
    z, _ = oracle.pack_ternary_transposed(np.zeros((8, 16), np.int8))
    np.testing.assert_array_equal(oracle.linear_packed(x, z, np.ones(8, np.float32), 16, bias), np.tile(bias, (4, 1)))
    o1, _ = oracle.pack_ternary_transposed(np.ones((8, 16), np.int8))
    got = oracle.linear_packed(x, o1, np.ones(8, np.float32), 16)
    np.testing.assert_allclose(got, np.tile(x.sum(1, keepdims=True), (1, 8)), rtol=1e-5, atol=1e-5)


def test_linear_sequential_fp32_order(oracle):
    """The fp32 path adds in ascending k: a case where the order is visible."""
    x = np.array([[1e8, 1.0, -1e8, 1.0]], dtype=np.float32)
    w = np.ones((1, 4), dtype=np.int8)
    p, _ = oracle.pack_ternary_transposed(w)
    # ((1e8 + 1) - 1e8) + 1 = 1 in fp32 (the first +1 is absorbed), 2 in exact arithmetic
    assert oracle.linear_packed(x, p, np.ones(1, np.float32), 4)[0, 0] == 1.0
    assert oracle.linear_packed(x, p, np.ones(1, np.float32), 4, f64=True)[0, 0] == 2.0


def test_linear_exact_f16_is_the_correctly_rounded_dot_product(oracle):
    """The exact variant against float64: fp16 operands times +-1 are exact in float64 and so is their sum while
    it stays below 2^53 units of 2^-24, hence float64 dot -> one rounding to fp32 is the correctly rounded result.
    Plus the cases a wrong rounding, a dropped digit or a sign error would show: ties, subnormals, 65504, the
    order-dependent example of the fp32 loop, the reference's known-answer vectors, non-finite rows."""
    rng = np.random.default_rng(0)
    for (b, n, k) in [(1, 8, 16), (3, 33, 64), (2, 64, 4096), (1, 5, 20)]:
        w = random_ternary(n, k, seed=k + 1).numpy()
        # wide dynamic range: random sign, 11-bit significand, exponents over the whole fp16 range incl. subnormals
        x = (rng.standard_normal((b, k)) * np.exp2(rng.integers(-24, 15, (b, k)))).astype(np.float16).astype(np.float32)
        x[np.abs(x) > 60000] = 1.0
        packed_t, _ = oracle.pack_ternary_transposed(w)
        ones = np.ones(n, np.float32)
        acc64 = x.astype(np.float64) @ w.astype(np.float64).T
        assert np.abs(acc64).max() * 2.0 ** 24 < 2.0 ** 53
        np.testing.assert_array_equal(oracle.linear_packed_exact_f16(x, packed_t, ones, k), acc64.astype(np.float32))
        # epilogue: one fp32 multiply, one fp32 add
        scale = rng.random(n).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32)
        expect = acc64.astype(np.float32) * scale[None, :] + bias[None, :]
        np.testing.assert_array_equal(oracle.linear_packed_exact_f16(x, packed_t, scale, k, bias), expect)
        np.testing.assert_array_equal(oracle.linear_packed_exact_f16(x, packed_t, scale[:1], k, bias),
                                      acc64.astype(np.float32) * scale[0] + bias[None, :])
    one = np.ones(1, np.float32)
    p4, _ = oracle.pack_ternary_transposed(np.ones((1, 4), np.int8))
    u = np.float32(2.0 ** -24)  # the smallest fp16 subnormal
    # ties go to even: 1 + 2^-24 -> 1;  1 + 3 * 2^-24 -> 1 + 4 * 2^-24 = 1 + 2^-22;  -(1 + 2^-24) -> -1
    assert oracle.linear_packed_exact_f16(np.array([[1.0, u, 0, 0]], np.float32), p4, one, 4)[0, 0] == 1.0
    assert oracle.linear_packed_exact_f16(np.array([[1.0, u, u, u]], np.float32), p4, one, 4)[0, 0] == np.float32(1 + 2.0 ** -22)
    assert oracle.linear_packed_exact_f16(np.array([[-1.0, -u, 0, 0]], np.float32), p4, one, 4)[0, 0] == -1.0
    # what the fp32 loop loses, the exact sum keeps: 2048 + 1 - 2048 + 1 (fp16 values) is 2 either way, but
    # 65504 + 2^-24 - 65504 is 2^-24 exactly here and 0 in the fp32 loop
    x = np.array([[65504.0, u, -65504.0, 0]], np.float32)
    assert oracle.linear_packed_exact_f16(x, p4, one, 4)[0, 0] == u
    assert oracle.linear_packed(x, p4, one, 4)[0, 0] == 0.0
    # sign of the weights, and the largest magnitudes on every term
    m4, _ = oracle.pack_ternary_transposed(-np.ones((1, 4), np.int8))
    x = np.full((1, 4), 65504.0, np.float32)
    assert oracle.linear_packed_exact_f16(x, p4, one, 4)[0, 0] == np.float32(4 * 65504.0)
    assert oracle.linear_packed_exact_f16(x, m4, one, 4)[0, 0] == np.float32(-4 * 65504.0)
    # the reference's own known-answer vectors (small integers and halves: exact in fp16)
    for case in GOLD["matmul"]:
        w = np.array(case["weights"], dtype=np.int8)
        packed_t, k = oracle.pack_ternary_transposed(w)
        x = np.array(case["input"], dtype=np.float32)
        if not np.array_equal(x.astype(np.float16).astype(np.float32), x):
            continue
        np.testing.assert_array_equal(oracle.linear_packed_exact_f16(x, packed_t, np.array(case["scales"], np.float32), k),
                                      np.array(case["output"], dtype=np.float32))
    # a row with an infinity: +inf where it meets +1 weights (the float loop's answer, pinned in its own test below),
    # other rows are untouched; non-fp16 inputs are refused
    x = np.array([[1.0, np.inf, 0, 0], [1.0, 2.0, 3.0, 4.0]], np.float32)
    y = oracle.linear_packed_exact_f16(x, p4, one, 4)
    assert y[0, 0] == np.inf and y[1, 0] == 10.0
    with pytest.raises(ValueError):
        oracle.linear_packed_exact_f16(np.array([[1.0 + 2.0 ** -20, 0, 0, 0]], np.float32), p4, one, 4)


def _float_loop(x, w, n):
    """the reference's accumulation (ternary_gemm_production.cu:126-133) for one column, in plain fp32 arithmetic"""
    acc = np.float32(0.0)
    with np.errstate(invalid="ignore", over="ignore"):
        for k in range(x.shape[0]):
            acc = np.float32(acc + np.float32(x[k] * np.float32(w[n, k])))
    return acc


@pytest.mark.parametrize("fn", ["linear_packed_exact_f16", "linear_packed_rowscaled_bf16"])
def test_exact_linears_on_non_finite_rows_follow_the_float_loop(oracle, fn):
    """A row that holds an infinity or a NaN: every column gets what the reference's fp32 loop leaves -- NaN where a
    NaN, an infinity on a zero weight, or infinities of both signs meet; otherwise the infinity with the sign of its
    products -- and the other rows of the call are untouched.  Pinned by running that loop in numpy."""
    f = getattr(oracle, fn)
    w = np.array([[1, 1, 0, -1, 1, 0, 1, -1],     # column 0: inf meets +1 (k=1): +inf
                  [1, -1, 0, 1, 1, 0, 1, 1],      # column 1: inf meets -1: -inf
                  [1, 0, 1, 1, -1, 0, 1, 1],      # column 2: inf meets 0: NaN
                  [0, 1, 1, -1, -1, 1, 0, 1]], dtype=np.int8)  # column 3: +inf * 1, and (row 2) +inf * -1 as well
    packed_t, k = oracle.pack_ternary_transposed(w)
    one = np.ones(4, np.float32)
    rows = np.array([[1.0, np.inf, 2.0, 0.5, -3.0, 4.0, 1.0, 1.0],       # one +inf at k = 1
                     [1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0],           # finite: untouched
                     [1.0, np.inf, 2.0, 0.5, np.inf, 0.0, 1.0, 1.0],     # +inf at k = 1 and at k = 4
                     [np.nan, 1.0, 2.0, 3.0, 1.0, 1.0, 1.0, 1.0],        # a NaN: NaN wherever it goes
                     [1.0, -np.inf, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0]], np.float32)
    y = f(rows, packed_t, one, k)
    for b in range(rows.shape[0]):
        for n in range(4):
            want = _float_loop(rows[b], w, n)
            if np.isnan(want):
                assert np.isnan(y[b, n]), (b, n, y[b, n])
            else:
                assert y[b, n] == want, (b, n, y[b, n], want)
    assert y[0, 0] == np.inf and y[0, 1] == -np.inf and np.isnan(y[0, 2]) and y[0, 3] == np.inf
    assert y[2, 0] == np.inf and np.isnan(y[2, 1]) and np.isnan(y[2, 3])  # same sign twice; opposite signs meet
    assert np.isnan(y[3]).all() and y[4, 1] == np.inf
    # the epilogue applies as ever: scale and bias (a negative scale flips the infinity)
    y2 = f(rows[:1], packed_t, np.array([-2.0, 1.0, 1.0, 1.0], np.float32), k, np.full(4, 5.0, np.float32))
    assert y2[0, 0] == -np.inf and y2[0, 1] == -np.inf and np.isnan(y2[0, 2])


def _bf16(a):
    """float32 array rounded to bf16 values (round to nearest even), still float32"""
    u = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000
    return u.astype(np.uint32).view(np.float32)


def test_linear_rowscaled_bf16_is_the_correctly_rounded_dot_product(oracle):
    """The bf16 variant against float64.  While every element of a row lies within 32 binades of the row's largest,
    each is represented exactly and the result is the float64 dot product (exact for such rows) rounded once to fp32;
    elements further down are rounded to the row's grid (half up in magnitude), which crafted rows pin, as they pin the
    scaling by the row's exponent over the whole bf16 range, signs, ties of the final rounding and non-finite rows."""
    rng = np.random.default_rng(1)
    for (b, n, k) in [(1, 8, 16), (3, 33, 64), (2, 64, 4096), (1, 5, 48)]:
        w = random_ternary(n, k, seed=k + 2).numpy()
        # per row a base exponent anywhere in the bf16 range, elements spread over 30 binades below it
        base = rng.integers(-100, 100, (b, 1))
        x = _bf16(rng.standard_normal((b, k)) * np.exp2(base + rng.integers(-28, 1, (b, k))))
        for r in range(b):  # make sure the row's largest element sits at the top of the spread
            x[r, 0] = _bf16(np.float32(1.5) * np.exp2(np.float32(base[r, 0] + 1)))
        packed_t, _ = oracle.pack_ternary_transposed(w)
        ones = np.ones(n, np.float32)
        acc64 = x.astype(np.float64) @ w.astype(np.float64).T   # exact: 8-bit significands within 31 binades, 4096 terms
        np.testing.assert_array_equal(oracle.linear_packed_rowscaled_bf16(x, packed_t, ones, k), acc64.astype(np.float32))
        scale = rng.random(n).astype(np.float32)
        bias = (rng.standard_normal(n) * np.exp2(base[0, 0])).astype(np.float32)
        expect = acc64.astype(np.float32) * scale[None, :] + bias[None, :]
        np.testing.assert_array_equal(oracle.linear_packed_rowscaled_bf16(x, packed_t, scale, k, bias), expect)
    one = np.ones(1, np.float32)
    p4, _ = oracle.pack_ternary_transposed(np.ones((1, 4), np.int8))
    m4, _ = oracle.pack_ternary_transposed(-np.ones((1, 4), np.int8))
    f = lambda vals, p=p4: oracle.linear_packed_rowscaled_bf16(np.array([vals], np.float32), p, one, 4)[0, 0]
    # ties of the final rounding go to even: 1 + 2^-24 -> 1; 1 + 3 * 2^-24 -> 1 + 2^-22 (all terms exact on the grid)
    u = np.float32(2.0 ** -24)
    assert f([1.0, u, 0, 0]) == 1.0 and f([1.0, u, u, u]) == np.float32(1 + 2.0 ** -22) and f([-1.0, -u, 0, 0]) == -1.0
    # what an fp32 loop loses: 2^100 + 1 * 2^70 - 2^100 keeps the small term (30 binades down: exact)
    assert f([2.0 ** 100, 2.0 ** 70, -(2.0 ** 100), 0]) == np.float32(2.0 ** 70)
    # the grid: with the largest element 1.0 (e1 = 127) the unit is 2^-39 ... an element of 1.5 * 2^-39 rounds half up
    # to 2 units, 1.25 * 2^-39 to 1 unit, 2^-41 (a quarter unit) to 0; signs follow the element
    g = np.float32(2.0 ** -39)
    assert f([1.0, 1.5 * g, -1.0, 0]) == np.float32(2 * g) and f([1.0, 1.25 * g, -1.0, 0]) == g
    assert f([1.0, 2.0 ** -41, -1.0, 0]) == 0.0 and f([1.0, -1.5 * g, -1.0, 0]) == np.float32(-2 * g)
    assert f([1.0, 0.5 * g, -1.0, 0]) == g               # exactly half a unit: up in magnitude
    # the row's exponent scales the grid: the same row times 2^-100 and times 2^90 gives the same bits scaled
    row = [1.0, 0.75, -0.375, 2.0 ** -20]
    for e in (-100, -60, 0, 90):
        sc = np.float32(2.0) ** e
        assert f([v * sc for v in row]) == np.float32((1.0 + 0.75 - 0.375 + 2.0 ** -20) * 2.0 ** e)
        assert f([v * sc for v in row], m4) == np.float32(-(1.0 + 0.75 - 0.375 + 2.0 ** -20) * 2.0 ** e)
    # subnormal bf16 values (biased exponent 0) and an all-zero row
    tiny = np.float32(2.0 ** -133)
    assert f([tiny, tiny, 3 * tiny, 0]) == np.float32(5 * tiny) and f([0, 0, 0, 0]) == 0.0
    # the largest bf16 value on every term stays finite in fp32 only up to the fp32 range
    big = _bf16(np.float32(3.3e38))[()]
    assert f([big, 0, 0, 0]) == big and np.isinf(f([big, big, big, big]))
    # the reference's own known-answer vectors that are bf16 values
    for case in GOLD["matmul"]:
        w = np.array(case["weights"], dtype=np.int8)
        packed_t, k = oracle.pack_ternary_transposed(w)
        x = np.array(case["input"], dtype=np.float32)
        if not np.array_equal(_bf16(x), x):
            continue
        np.testing.assert_array_equal(oracle.linear_packed_rowscaled_bf16(x, packed_t, np.array(case["scales"], np.float32), k),
                                      np.array(case["output"], dtype=np.float32))
    # non-finite rows: the float loop's answer (own test below), other rows untouched; inputs that are not bf16 values
    # are refused
    x = np.array([[1.0, np.inf, 0, 0], [1.0, 2.0, 3.0, 4.0]], np.float32)
    y = oracle.linear_packed_rowscaled_bf16(x, p4, one, 4)
    assert y[0, 0] == np.inf and y[1, 0] == 10.0
    with pytest.raises(ValueError):
        oracle.linear_packed_rowscaled_bf16(np.array([[1.0 + 2.0 ** -10, 0, 0, 0]], np.float32), p4, one, 4)


# ---------------------------------------------------------------- int8 path (a7)
def test_act_quant_brute_force(oracle):
    import math
    x = np.array([[0.5, -1.0, 2.0, 0.0], [0.0, 0.0, 0.0, 0.0], [1e-7, -1e-7, 0.0, 5e-8],
                  [127.0, 63.5, -63.5, 0.4999]], dtype=np.float32)
    q, s = oracle.act_quant_i8(x)
    for r in range(x.shape[0]):
        amax = np.float32(np.abs(x[r]).max())
        se = np.float32(amax / np.float32(127.0)) if amax > np.float32(1e-6) else np.float32(1.0)
        assert s[r] == se
        inv = np.float32(1.0) / se
        for c in range(x.shape[1]):
            v = float(np.float32(x[r, c] * inv))
            rounded = math.floor(abs(v) + 0.5) * (1 if v >= 0 else -1)  # half away from zero
            assert q[r, c] == max(-127, min(127, rounded))
    # the row maximum always maps to +-127; halves round away from zero
    np.testing.assert_array_equal(q[0], [32, -64, 127, 0])
    np.testing.assert_array_equal(q[3], [127, 64, -64, 0])
    np.testing.assert_array_equal(q[1], [0, 0, 0, 0])
    assert s[1] == 1.0 and s[2] == 1.0  # amax <= 1e-6 -> scale 1


def test_gemm_i8_brute_force_and_identities(oracle):
    rng = np.random.default_rng(5)
    b, n, k = 3, 6, 10
    q = rng.integers(-127, 128, size=(b, k)).astype(np.int8)
    s_x = rng.random(b).astype(np.float32) + 0.1
    w = random_ternary(n, k, seed=8).numpy()
    scale = rng.random(n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    p, _ = oracle.pack_ternary_transposed(w)
    acc, y = oracle.gemm_i8(q, s_x, p, scale, k, bias)
    for i in range(b):
        for j in range(n):
            a = sum(int(q[i, kk]) * 127 * int(w[j, kk]) for kk in range(k))
            assert acc[i, j] == a
            r = np.float32(np.float32(a) * s_x[i])
            r = np.float32(r / np.float32(127.0))
            r = np.float32(r * scale[j])
            r = np.float32(r + bias[j])
            assert y[i, j] == r
    # integer GEMM equals numpy's exact integer product; sign flip of W negates it
    np.testing.assert_array_equal(acc, q.astype(np.int64) @ (127 * w.astype(np.int64)).T)
    pn, _ = oracle.pack_ternary_transposed(-w)
    np.testing.assert_array_equal(oracle.gemm_i8(q, s_x, pn, scale, k)[0], -acc)


def test_int8_path_tracks_float_path(oracle):
    """The whole int8 route stays inside the quantisation error of 8-bit activations."""
    b, n, k = 8, 64, 512
    x = seeded_acts(b, k, seed=4).numpy()
    w = random_ternary(n, k, seed=2).numpy()
    p, _ = oracle.pack_ternary_transposed(w)
    scale = np.full(n, 0.03, np.float32)
    _, _, _, y8 = oracle.linear_i8(x, p, scale, k)
    y = oracle.linear_packed(x, p, scale, k, f64=True)
    assert np.abs(y8 - y).max() / np.abs(y).max() < 2e-2


def test_round_helpers_match_torch(oracle):
    vals = [1e-8, 6e-8, 3e-8, 65519.0, 65520.0, 0.05, 0.1, 1.0009765625, 3.14159, 1e-40, -2.5e-5]
    for v in vals:
        assert oracle.round_to_dtype(v, 1) == float(torch.tensor(v, dtype=torch.float32).half().float())
        assert oracle.round_to_dtype(v, 2) == float(torch.tensor(v, dtype=torch.float32).bfloat16().float())


# ---- fused row operations (this library's own glue; pinned by float64 closed forms) ------------

def test_exp_fixed_is_within_one_ulp_of_exp(oracle):
    rng = np.random.default_rng(0)
    xs = np.concatenate([np.linspace(-87, 88.72, 4001), rng.normal(0, 4, 4000), [0.0, -0.0, 1.0, -1.0]])
    xs = xs.astype(np.float32)
    got = np.array([oracle.exp_fixed(float(x)) for x in xs], dtype=np.float64)
    ref = np.exp(xs.astype(np.float64))
    ulp = np.spacing(ref.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got - ref) / ulp) < 1.0
    assert oracle.exp_fixed(0.0) == 1.0
    assert np.isnan(oracle.exp_fixed(float("nan")))
    # overflows like exp; saturates at exp(-87) below (callers only ever add it to 1)
    assert oracle.exp_fixed(1000.0) == float("inf") and oracle.exp_fixed(88.8) == float("inf")
    assert oracle.exp_fixed(88.72) < np.finfo(np.float32).max
    assert oracle.exp_fixed(-1000.0) == oracle.exp_fixed(-87.0) > 0


@pytest.mark.parametrize("dtype,rel", [(0, 3e-7), (1, 1.0 / 1024), (2, 1.0 / 128)])
def test_swiglu_oracle_against_float64_closed_form(oracle, dtype, rel):
    rng = np.random.default_rng(1)
    g = (rng.normal(0, 3, (7, 130))).astype(np.float32)
    u = rng.normal(0, 1, (7, 130)).astype(np.float32)
    if dtype:
        td = torch.float16 if dtype == 1 else torch.bfloat16
        g = torch.from_numpy(g).to(td).float().numpy()
        u = torch.from_numpy(u).to(td).float().numpy()
    h, q, s = oracle.swiglu(g, u, dtype)
    ref = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.all(np.abs(h - ref) <= rel * np.abs(ref) + 1e-30)
    # a swapped operand or a missing silu would fail this: silu(g)*u != silu(u)*g in general
    assert not np.allclose(h, u / (1 + np.exp(-u)) * g, rtol=1e-2)
    # the quantization is the stand-alone quantizer applied to h
    q_ref, s_ref = oracle.act_quant_i8(h)
    np.testing.assert_array_equal(q, q_ref)
    np.testing.assert_array_equal(s, s_ref)
    # exact special cases: g = 0 gives 0; u = 0 gives 0
    h0, _, s0 = oracle.swiglu(np.zeros((1, 8), np.float32), np.ones((1, 8), np.float32), dtype)
    assert np.all(h0 == 0) and s0[0] == 1.0


@pytest.mark.parametrize("dtype,rel", [(0, 3e-7), (1, 1.0 / 1024), (2, 1.0 / 128)])
def test_rmsnorm_oracle_against_float64_closed_form(oracle, dtype, rel):
    rng = np.random.default_rng(2)
    x = rng.normal(0, 2, (5, 257)).astype(np.float32)
    w = (1 + 0.1 * rng.normal(0, 1, 257)).astype(np.float32)
    if dtype:
        td = torch.float16 if dtype == 1 else torch.bfloat16
        x = torch.from_numpy(x).to(td).float().numpy()
        w = torch.from_numpy(w).to(td).float().numpy()
    eps = 1e-5
    y, q, s = oracle.rmsnorm(x, w, eps, dtype)
    x64 = x.astype(np.float64)
    ref = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + eps) * w
    assert np.all(np.abs(y - ref) <= rel * np.abs(ref) + 1e-30)
    y1, _, _ = oracle.rmsnorm(x, None, eps, dtype)
    ref1 = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + eps)
    assert np.all(np.abs(y1 - ref1) <= rel * np.abs(ref1) + 1e-30)
    # invariant: without weight the output rows have unit RMS (up to eps and rounding)
    assert np.allclose(np.sqrt((y1.astype(np.float64) ** 2).mean(-1)), 1.0, rtol=5 * rel + 1e-5)
    # a constant row c maps to sign(c) * w (eps negligible)
    yc, _, _ = oracle.rmsnorm(np.full((1, 257), -3.0, np.float32), w, 1e-12, 0)
    assert np.allclose(yc[0], -w, rtol=1e-6)
    q_ref, s_ref = oracle.act_quant_i8(y)
    np.testing.assert_array_equal(q, q_ref)
    np.testing.assert_array_equal(s, s_ref)


# ---- property tests over arbitrary small shapes (hypothesis) ------------------------------------

def test_codec_and_quantizer_properties_over_random_shapes(oracle):
    from hypothesis import given, settings, strategies as st

    @settings(max_examples=60, deadline=None)
    @given(n=st.integers(1, 9), k=st.integers(1, 37), seed=st.integers(0, 2 ** 16), tf=st.sampled_from([0.0, 0.05, 0.3, 1.0]),
           per_channel=st.booleans())
    def run(n, k, seed, tf, per_channel):
        rng = np.random.default_rng(seed)
        w = (rng.normal(0, 0.02, (n, k)) * rng.choice([0.0, 1.0, 50.0], (n, 1))).astype(np.float32)
        tern, scale = oracle.ternary_quantize(w, tf, per_channel)
        # codes are ternary; the scale is the (row or tensor) absmax floored at 1e-8; an entry is kept
        # exactly when its magnitude exceeds fl32(tf * scale) and then carries the sign of the weight
        assert set(np.unique(tern)).issubset({-1, 0, 1})
        amax = np.abs(w).max(axis=1) if per_channel else np.full(n, np.abs(w).max())
        np.testing.assert_array_equal(np.broadcast_to(scale.reshape(-1), (n,)) if per_channel else np.full(n, scale.reshape(-1)[0]),
                                      np.maximum(amax, np.float32(1e-8)).astype(np.float32))
        thr = (np.float32(tf) * np.maximum(amax, np.float32(1e-8)).astype(np.float32)).astype(np.float32)
        keep = np.abs(w) > thr[:, None]
        np.testing.assert_array_equal(tern, (np.sign(w) * keep).astype(np.int8))
        # pack -> unpack is the identity for every K (padding codes are zero and sliced off), and the
        # transposed layout is the transpose of the row-major one
        packed, kk = oracle.pack_ternary(tern)
        assert kk == k and packed.shape == (n, (k + 3) // 4)
        np.testing.assert_array_equal(oracle.unpack_ternary(packed, k), tern)
        packed_t, _ = oracle.pack_ternary_transposed(tern)
        np.testing.assert_array_equal(packed_t, packed.T)
        np.testing.assert_array_equal(oracle.unpack_ternary_transposed(packed_t, k), tern)
        if k % 4:
            assert not np.any(packed[:, -1] >> (2 * (k % 4)))  # padding slots hold code 0

    run()


def test_epilogue_as_written_and_contracted_differ_by_one_ulp_at_most(oracle):
    """The reference's epilogue line `acc * s + b_val` (csrc/kernels/ternary_gemm_production.cu:139-141) is compiled by
    nvcc with floating-point contraction on by default, i.e. possibly as one fused multiply-add; the oracle and the
    library round the product first.  Both readings are computed here: they differ in a minority of the outputs, and
    never by more than one unit in the last place at the magnitude of the product (its rounding error, half a unit, is all
    that separates the two before the final rounding)."""
    rng = np.random.default_rng(7)
    n, k, b = 257, 512, 5
    w = rng.integers(-1, 2, size=(n, k)).astype(np.int8)
    packed, _ = oracle.pack_ternary_transposed(w)
    x = rng.standard_normal((b, k)).astype(np.float32)
    scale = (rng.random(n) * 0.05 + 0.01).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    y0 = oracle.linear_packed(x, packed, scale, k, bias)
    y1 = oracle.linear_packed(x, packed, scale, k, bias, fused_epilogue=True)
    differing = int((y0 != y1).sum())
    assert 0 < differing < y0.size // 2
    # the unit: the spacing of fp32 numbers at the larger of product and sum (where the sum cancels below the product, one
    # unit of the product is several of the sum)
    prod = np.abs(y0.astype(np.float64) - bias)
    ulp = np.spacing(np.maximum(prod, np.abs(y0)).astype(np.float32))
    assert float((np.abs(y0.astype(np.float64) - y1) / ulp).max()) <= 1.0
    # without a bias the two readings are the same operation
    z0 = oracle.linear_packed(x, packed, scale, k, None)
    z1 = oracle.linear_packed(x, packed, scale, k, None, fused_epilogue=True)
    np.testing.assert_array_equal(z0, z1)


def test_field_layout_means_what_it_says(oracle):
    """The field layout of the tiled copy, read back by its definition with plain loops: field t of byte b of dword c
    of a group is column 4 q + t of the group's tile at k = 64 s + 16 g + 4 b + c, stored as w + 1 (t < 3) or as w in
    two's complement (t = 3); positions outside the matrix read as weight 0."""
    for (n, k) in ((20, 70), (16, 64), (37, 130)):
        w = random_ternary(n, k, seed=n + k).numpy()
        packed, _ = oracle.pack_ternary_transposed(w)
        tiled = oracle.retile_weights(packed, k)
        fields = oracle.retile_fields(tiled, n, k)
        assert fields.dtype == np.uint8 and fields.size == tiled.size
        steps, tiles = ((k + 3) // 4 + 15) // 16, (n + 15) // 16
        f = fields.reshape(tiles, steps, 4, 4, 4, 4)   # [tile][step s][row group g][quad q][dword c][byte b]
        for tile in range(tiles):
            for s in range(steps):
                for g in range(4):
                    for q in range(4):
                        for c in range(4):
                            for b in range(4):
                                byte = int(f[tile, s, g, q, c, b])
                                for t in range(4):
                                    field = (byte >> (2 * t)) & 3
                                    got = field - 1 if t < 3 else (field if field < 2 else field - 4)
                                    col, kk = 16 * tile + 4 * q + t, 64 * s + 16 * g + 4 * b + c
                                    want = int(w[col, kk]) if col < n and kk < k else 0
                                    assert got == want, (n, k, tile, s, g, q, c, b, t)
