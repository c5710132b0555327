"""Shared helpers for the parity tests."""
import numpy as np
import torch

BT_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def set_option(name, value):
    """Overrides a run-time option of the HIP library for the rest of the test (tests/conftest.py un-sets every
    override when the test ends); value None un-sets it."""
    from bittorch_amd import _lib
    _lib.set_option(name, value)


def seeded_weights(n, k, seed=0, std=0.02, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, k, generator=g) * std).to(dtype)


def seeded_acts(b, k, seed=1, dtype=torch.float32, outliers=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(b, k, generator=g)
    if outliers:
        mask = torch.rand(b, k, generator=g) < 0.001
        x = torch.where(mask, x * 20, x)
    return x.to(dtype)


def random_ternary(n, k, seed=0, p_zero=0.2):
    g = torch.Generator().manual_seed(seed)
    r = torch.rand(n, k, generator=g)
    w = torch.zeros(n, k, dtype=torch.int8)
    w[r > p_zero] = 1
    w[r > p_zero + (1 - p_zero) / 2] = -1
    return w


def f32np(t):
    return t.detach().to(torch.float32).cpu().numpy()


def rel_err(got, ref):
    """max |got-ref| / max |ref| (scale-relative error of a whole output tensor)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))


# element-wise thresholds of the reference's own kernel tests (tests/test_packed_kernel.py:44-50: rtol = atol =
# 1e-4 for fp32; :159-199: 1e-2 for fp16; bf16, which the reference does not take, is held to the fp16 figure)
REF_ELEMENTWISE = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def assert_close_like_reference(got, ref, dtype):
    """Every output element within the reference tests' `allclose(rtol, atol)` of `ref`: unlike `rel_err`, which
    is relative to the largest output, this also holds the small-magnitude outputs."""
    thr = REF_ELEMENTWISE[dtype]
    np.testing.assert_allclose(np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64), rtol=thr, atol=thr)
