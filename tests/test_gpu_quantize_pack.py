"""GPU parity: fused quantize + 2-bit pack kernel vs the CPU oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from conftest import announce
from _util import BT_DT, f32np, seeded_weights

pytestmark = pytest.mark.gpu


def _run(oracle, w_cpu, tf, per_channel, want_tern=True):
    from bittorch_amd import _C
    w = w_cpu.cuda()
    packed, scale, tern = _C.ternary_quantize_pack(w, tf, per_channel, want_packed=True, want_tern=want_tern)
    torch.cuda.synchronize()
    o_tern, o_scale = oracle.ternary_quantize(f32np(w_cpu), tf, per_channel, dtype=BT_DT[w_cpu.dtype])
    o_packed, _ = oracle.pack_ternary_transposed(o_tern)
    np.testing.assert_array_equal(f32np(scale).reshape(-1), o_scale.reshape(-1))
    np.testing.assert_array_equal(packed.cpu().numpy(), o_packed)
    if want_tern:
        np.testing.assert_array_equal(tern.cpu().numpy(), o_tern)
    return packed, scale


# (N, K): config shapes, ragged N (not a multiple of 16), K % 4 != 0, tiny, each ITERS variant
SHAPES = [(256, 512), (16, 64), (1, 1), (3, 4), (7, 33), (17, 123), (33, 5), (64, 1024), (40, 1028),
          (48, 2048), (32, 4096), (24, 5000), (16, 8192), (16, 11008), (16, 12288), (8, 12292), (4, 20000)]


@pytest.mark.parametrize("n,k", SHAPES)
@pytest.mark.parametrize("per_channel", [True, False])
def test_quantize_pack_matches_oracle_fp32(oracle, n, k, per_channel):
    announce("quantize_pack fp32", n, k, per_channel)
    _run(oracle, seeded_weights(n, k, seed=n * 131 + k), 0.05, per_channel)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,k", [(256, 512), (7, 33), (32, 4096), (16, 11008)])
def test_quantize_pack_matches_oracle_16bit(oracle, n, k, dtype):
    announce("quantize_pack", dtype, n, k)
    _run(oracle, seeded_weights(n, k, seed=5, dtype=dtype), 0.05, True)
    _run(oracle, seeded_weights(n, k, seed=6, dtype=dtype), 0.05, False)


# The one-read kernel (packed output only, K % 256 == 0, N % 16 == 0): a row per wave up to K = 4096, a row over two
# waves up to 8192 and over four up to 16384 -- every registers-per-lane variant of each, with rows that fill the last
# wave's share only partly (5120 = 20 chunks over two waves of 10; 11008 = 43 over four of 11; 9216 = 36 over four of 10).
FAST_SHAPES = [(32, 256), (64, 1024), (32, 2048), (32, 4096), (96, 4096), (32, 4352), (32, 5120), (48, 6144),
               (32, 6912), (16, 8192), (32, 9216), (32, 11008), (16, 12288), (16, 14336), (16, 16384)]


@pytest.mark.parametrize("n,k", FAST_SHAPES)
def test_quantize_pack_one_read_kernel_matches_oracle(oracle, n, k):
    announce("quantize_pack one-read kernel", n, k)
    for dtype, seed in ((torch.float32, 1), (torch.bfloat16, 2), (torch.float16, 3)):
        w = seeded_weights(n, k, seed=seed * 1000 + n + k, dtype=dtype)
        w[n // 2, k - 1] = w.abs().max() * 2   # the row's maximum in the last wave's share
        w[1, 0] = -w.abs().max() * 3           # ... and in the first's
        _run(oracle, w, 0.05, True, want_tern=False)
        _run(oracle, w, 0.05, False, want_tern=False)


@pytest.mark.parametrize("tf", [0.0, 0.01, 0.1, 0.5, 1.0])
def test_quantize_pack_threshold_factors(oracle, tf):
    announce("quantize_pack tf", tf)
    w = seeded_weights(64, 256, seed=9, std=1.0)
    w[3, 7] = 0.0
    w[5] = 0.0  # all-zero row: scale floors at 1e-8, all codes zero
    _run(oracle, w, tf, True)
    _run(oracle, w, tf, False)


def test_quantize_pack_extreme_magnitudes(oracle):
    announce("quantize_pack magnitudes")
    for mag in (1e-10, 1e10):
        _run(oracle, seeded_weights(32, 64, seed=3, std=1.0) * mag, 0.05, True)


def test_quantize_pack_matches_torch_ops_full_size(oracle):
    """Config-2 shape: kernel vs the torch op chain on the same GPU tensor (bit-exact)."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed, ternary_quantize
    announce("quantize_pack 4096x4096 vs torch ops")
    w = seeded_weights(4096, 4096, seed=0).cuda()
    for per_channel in (True, False):
        packed, scale, _ = _C.ternary_quantize_pack(w, 0.05, per_channel)
        w_tern, s_ref = ternary_quantize(w, 0.05, per_channel)
        p_ref, _ = pack_ternary_transposed(w_tern)
        assert torch.equal(scale, s_ref)
        assert torch.equal(packed, p_ref)
    # the 11008-wide rows of config 3
    w = seeded_weights(256, 11008, seed=1).cuda()
    packed, scale, _ = _C.ternary_quantize_pack(w, 0.05, True)
    w_tern, s_ref = ternary_quantize(w, 0.05, True)
    assert torch.equal(scale, s_ref)
    assert torch.equal(packed, pack_ternary_transposed(w_tern)[0])


def test_unpack_dequant_roundtrip(oracle):
    from bittorch_amd import _C
    announce("unpack_dequant")
    for n, k in [(64, 128), (17, 123), (256, 512), (100, 4096)]:
        w = seeded_weights(n, k, seed=n + k).cuda()
        packed, scale, tern = _C.ternary_quantize_pack(w, 0.05, True, want_tern=True)
        back = _C.unpack_dequant(packed, k, out_dtype=torch.int8)
        assert torch.equal(back, tern)
        np.testing.assert_array_equal(back.cpu().numpy(),
                                      oracle.unpack_ternary_transposed(packed.cpu().numpy(), k))
        deq = _C.unpack_dequant(packed, k, scale, out_dtype=torch.float32)
        assert torch.equal(deq, tern.float() * scale.unsqueeze(1))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_threshold_ties_in_16_bit_weights(oracle, dtype):
    """``threshold_factor * scale`` on 16-bit weights is a float product rounded to fp32 and then to the weights' dtype.
    With threshold_factor = 0.7 the fp32 product is now and then exactly half way between two 16-bit values, and a
    weight equal to the upper one survives or not depending on which way the tie goes: the kernel, the oracle and the
    torch path of ``quant.ternary_quantize`` on either device must all take the two roundings (torch's ROCm kernel
    for ``scalar * half_tensor`` alone would round the exact product once and keep such a weight)."""
    from bittorch_amd import _C
    from bittorch_amd.quant import pack_ternary_transposed, ternary_quantize
    announce("threshold ties", dtype)
    ties = 0
    for seed in (1, 2, 3, 4):
        torch.manual_seed(seed)
        w = (torch.randn(800, 800) * 0.02).to(dtype)
        packed, scale, tern = _C.ternary_quantize_pack(w.cuda(), 0.7, True, True, True)
        o_tern, o_scale = oracle.ternary_quantize(f32np(w), 0.7, True, dtype=BT_DT[dtype])
        np.testing.assert_array_equal(tern.cpu().numpy(), o_tern)
        for dev in ("cpu", "cuda"):
            w_t, s = ternary_quantize(w.to(dev), 0.7, True)
            assert torch.equal(s.cpu().float(), torch.from_numpy(o_scale))
            np.testing.assert_array_equal(w_t.cpu().float().numpy(), o_tern.astype(np.float32))
            if dev == "cuda":
                assert torch.equal(pack_ternary_transposed(w_t)[0], packed)
        if dtype == torch.float16:  # how many rows of this matrix have such a tie (the test must meet the case)
            prod = o_scale.astype(np.float32) * np.float32(0.7)
            near = prod.astype(np.float16)
            away = np.nextafter(near, np.where(prod > near.astype(np.float32), np.float16(np.inf), np.float16(-np.inf)))
            ties += int(((near.astype(np.float64) + away.astype(np.float64)) / 2 == prod.astype(np.float64)).sum())
    assert dtype != torch.float16 or ties > 0
