"""The entry point that allocates nothing (`bt_ternary_linear_tensor_core_forward_static`): called through the
C ABI with raw device pointers, its output must equal that of `bt_ternary_linear_tensor_core_forward` (which
takes the same scratch from a caller-provided workspace) bit for bit -- on two calls in a row, the second on a
smaller input, so that what the first call left in the library's device array cannot leak into the second."""
import pytest
import torch

from conftest import announce
from _util import BT_DT, random_ternary, seeded_acts

pytestmark = pytest.mark.gpu

_WARM = {"done": False}  # the first call of the process is allowed to move the driver's free-memory figure


def _both(lib, x, packed, scale, bias, n, k, warmed=True):
    """(static entry point's output, workspace entry point's output) for activations x [B, K]"""
    b = x.shape[0]
    dt = BT_DT[x.dtype]
    st = torch.cuda.current_stream().cuda_stream
    y_ws = torch.empty(b, n, dtype=x.dtype, device=x.device)
    nbytes = lib.bt_tensor_core_workspace_bytes(b, n, k)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    rc = lib.bt_ternary_linear_tensor_core_forward(x.data_ptr(), dt, packed.data_ptr(), scale.data_ptr(), 0, n,
                                                   bias.data_ptr(), 0, y_ws.data_ptr(), b, n, k, ws.data_ptr(), nbytes, st)
    assert rc == 0
    y_st = torch.full((b, n), float("nan"), dtype=x.dtype, device=x.device)
    torch.cuda.synchronize()
    # what the driver itself reports as free (a hipMalloc / hipFree inside the library would move it; torch's own
    # counter only sees torch's allocator)
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    rc = lib.bt_ternary_linear_tensor_core_forward_static(x.data_ptr(), dt, packed.data_ptr(), scale.data_ptr(), 0, n,
                                                          bias.data_ptr(), 0, y_st.data_ptr(), b, n, k, st)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    if warmed:  # (the very first call on a device may load the code object that holds the array)
        assert torch.cuda.mem_get_info()[0] == free_before
    return y_st, y_ws


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_static_scratch_entry_point_matches_workspace_entry_point(dtype):
    from bittorch_amd import _lib
    from bittorch_amd.quant import pack_ternary_transposed
    lib = _lib.load()
    g = torch.Generator().manual_seed(5)
    # first call: a prefill shape on the tiled GEMM; second call: fewer, shorter rows on another layer
    for (b, n, k, seed) in ((300, 512, 1024, 1), (7, 256, 208, 2)):
        announce("static scratch", dtype, b, n, k)
        packed = pack_ternary_transposed(random_ternary(n, k, seed=seed))[0].cuda()
        scale = (torch.rand(n, generator=g) * 0.05 + 0.01).cuda()
        bias = (torch.randn(n, generator=g) * 0.01).cuda()
        x = seeded_acts(b, k, seed=seed + 10, dtype=dtype, outliers=True).cuda()
        y_st, y_ws = _both(lib, x, packed, scale, bias, n, k, warmed=_WARM["done"])
        _WARM["done"] = True
        assert torch.equal(y_st, y_ws), (dtype, b, n, k)


def test_static_scratch_entry_point_inside_a_graph_capture():
    """The use the entry point is for: after one call outside a capture (which looks the array's address up), the
    call is recorded into a HIP graph and replayed, with eager work between the replays; every replay equals the
    workspace entry point on the same inputs."""
    from bittorch_amd import _lib
    from bittorch_amd.quant import pack_ternary_transposed
    lib = _lib.load()
    b, n, k = 40, 512, 1024
    g = torch.Generator().manual_seed(7)
    packed = pack_ternary_transposed(random_ternary(n, k, seed=4))[0].cuda()
    scale = (torch.rand(n, generator=g) * 0.05 + 0.01).cuda()
    bias = (torch.randn(n, generator=g) * 0.01).cuda()
    xs = [seeded_acts(b, k, seed=20 + i, dtype=torch.bfloat16, outliers=True).cuda() for i in range(3)]
    want = [_both(lib, xi, packed, scale, bias, n, k, warmed=_WARM["done"])[1] for xi in xs]
    _WARM["done"] = True
    x = xs[0].clone()
    y = torch.empty(b, n, dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.bt_ternary_linear_tensor_core_forward_static(
            x.data_ptr(), 2, packed.data_ptr(), scale.data_ptr(), 0, n, bias.data_ptr(), 0, y.data_ptr(), b, n, k,
            torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.last_error()
    for xi, w in zip(xs, want):
        announce("static scratch replay")
        x.copy_(xi)  # eager work between the replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, w)


def test_static_scratch_entry_point_rejects_oversized_calls():
    from bittorch_amd import _lib
    lib = _lib.load()
    t = torch.zeros(256, dtype=torch.uint8, device="cuda")
    p = t.data_ptr()
    # B * K beyond the 16 MiB of int8 activations the library holds; B beyond its 65536 row scales
    assert lib.bt_ternary_linear_tensor_core_forward_static(p, 2, p, p, 0, 16, None, 0, p, 4097, 16, 4096, None) == -2
    assert "static scratch" in _lib.last_error()
    assert lib.bt_ternary_linear_tensor_core_forward_static(p, 2, p, p, 0, 16, None, 0, p, 65537, 16, 16, None) == -2
