"""Model conversion, accounting and checkpoints (mirror of bittorch/utils/convert.py; the
reference ships no test for these, so the checks are the definitions themselves: a converted
layer computes what the training layer's plain-torch forward computes, counts follow from the
shapes, and a checkpoint round trip reproduces every buffer bit for bit)."""
import numpy as np
import pytest
import torch
import torch.nn as nn

import bittorch_amd as bt
from bittorch_amd.nn import TernaryLinear, TernaryLinearInference
from bittorch_amd.quant import pack_ternary_transposed, ternary_quantize
from bittorch_amd.utils import (convert_linear_layers, count_ternary_params, fp_linear_to_ternary_infer,
                                get_model_memory_bytes, load_ternary_checkpoint, load_ternary_safetensors,
                                save_ternary_checkpoint, save_ternary_safetensors, ternary_linear_to_infer)


def _mlp():
    torch.manual_seed(0)
    return nn.Sequential(nn.Linear(64, 32), nn.ReLU(), TernaryLinear(32, 16, backend="python"), nn.ReLU(),
                         nn.Linear(16, 10))


def test_fp_linear_to_ternary_infer_matches_definition():
    torch.manual_seed(1)
    lin = nn.Linear(70, 33)  # K not a multiple of 4
    inf = fp_linear_to_ternary_infer(lin, threshold_factor=0.07)
    assert isinstance(inf, TernaryLinearInference)
    assert (inf.in_features, inf.out_features) == (70, 33)
    w_tern, scale = ternary_quantize(lin.weight.data, threshold_factor=0.07)
    packed, k = pack_ternary_transposed(w_tern)
    assert k == 70 and torch.equal(inf.weight_packed, packed) and torch.equal(inf.scale, scale)
    assert inf.weight_packed.shape == (18, 33) and inf.weight_packed.dtype == torch.uint8
    x = torch.randn(5, 70)
    ref = x @ (w_tern * scale[:, None]).T + lin.bias
    assert torch.allclose(inf(x), ref, atol=1e-5)
    assert not any(p.requires_grad for p in inf.parameters())


def test_ternary_linear_to_infer_uses_the_layers_own_settings():
    torch.manual_seed(2)
    for per_channel in (True, False):
        layer = TernaryLinear(48, 24, threshold_factor=0.1, per_channel=per_channel, backend="python")
        inf = ternary_linear_to_infer(layer)
        x = torch.randn(7, 48)
        assert torch.allclose(inf(x), layer(x), atol=1e-5)
        assert inf.scale.shape == (24,)
    layer = TernaryLinear(8, 4, bias=False, backend="python")
    assert ternary_linear_to_infer(layer).bias is None


def test_convert_linear_layers_copy_skip_and_inplace():
    model = _mlp()
    x = torch.randn(3, 64)
    conv = convert_linear_layers(model, skip_names=["4"])
    assert isinstance(model[0], nn.Linear) and isinstance(model[2], TernaryLinear)  # original untouched
    assert isinstance(conv[0], TernaryLinearInference) and isinstance(conv[2], TernaryLinearInference)
    assert isinstance(conv[4], nn.Linear)
    # the converted model equals the model whose first layer is quantized the same way
    w_tern, scale = ternary_quantize(model[0].weight.data, threshold_factor=0.05)
    h = torch.relu(x @ (w_tern * scale[:, None]).T + model[0].bias)
    ref = model[4](torch.relu(model[2](h)))
    assert torch.allclose(conv(x), ref, atol=1e-5)
    same = convert_linear_layers(model, inplace=True)
    assert same is model and all(isinstance(model[i], TernaryLinearInference) for i in (0, 2, 4))

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.attn = nn.ModuleDict({"q_proj": nn.Linear(8, 8), "proj": nn.Linear(8, 8)})
            self.lm_head = nn.Linear(8, 20)

    blk = convert_linear_layers(Block(), skip_names=["head"])
    assert isinstance(blk.attn["q_proj"], TernaryLinearInference) and isinstance(blk.lm_head, nn.Linear)


def test_counts_and_memory():
    model = _mlp()
    c = count_ternary_params(model)
    assert c == {"fp32": 64 * 32 + 32 * 16 + 16 * 10, "fp16": 0, "packed_ternary": 0, "total": 64 * 32 + 32 * 16 + 160}
    conv = convert_linear_layers(model, skip_names=["4"])
    c = count_ternary_params(conv)
    assert c["packed_ternary"] == 64 * 32 + 32 * 16 and c["fp32"] == 160 and c["total"] == 64 * 32 + 32 * 16 + 160
    m = get_model_memory_bytes(conv)
    assert m["packed_ternary"] == 16 * 32 + 8 * 16          # ceil(K/4) * N bytes
    assert m["scales"] == 4 * (32 + 16) and m["fp32"] == 4 * 160
    assert m["total"] == m["packed_ternary"] + m["scales"] + m["fp32"] + 4 * (32 + 16 + 10)
    half = nn.Sequential(nn.Linear(8, 4).half())
    assert count_ternary_params(half)["fp16"] == 32 and get_model_memory_bytes(half)["fp16"] == 64


def test_checkpoint_round_trips(tmp_path):
    conv = convert_linear_layers(_mlp())
    x = torch.randn(4, 64)
    y = conv(x)
    path = str(tmp_path / "m.pt")
    save_ternary_checkpoint(conv, path, metadata={"note": "unit test", "layers": 3})
    torch.manual_seed(9)
    fresh = convert_linear_layers(nn.Sequential(nn.Linear(64, 32), nn.ReLU(), nn.Linear(32, 16), nn.ReLU(),
                                                nn.Linear(16, 10)))
    assert not torch.equal(fresh(x), y)
    meta = load_ternary_checkpoint(path, fresh)
    assert meta == {"note": "unit test", "layers": 3}
    assert torch.equal(fresh(x), y)
    for k, v in conv.state_dict().items():
        assert torch.equal(v, fresh.state_dict()[k]), k
    assert sorted(conv.state_dict()) == ["0.bias", "0.scale", "0.weight_packed", "2.bias", "2.scale",
                                         "2.weight_packed", "4.bias", "4.scale", "4.weight_packed"]

    st = str(tmp_path / "m.safetensors")
    save_ternary_safetensors(conv, st, metadata={"format": "bittorch"})
    again = convert_linear_layers(nn.Sequential(nn.Linear(64, 32), nn.ReLU(), nn.Linear(32, 16), nn.ReLU(),
                                                nn.Linear(16, 10)))
    assert load_ternary_safetensors(st, again)["format"] == "bittorch"
    assert torch.equal(again(x), y)
    from safetensors import safe_open
    with safe_open(st, framework="pt") as fh:
        t = fh.get_tensor("0.weight_packed")
        assert t.dtype == torch.uint8 and tuple(t.shape) == (16, 32)       # [inBytes, outFeatures]
        assert fh.get_tensor("0.scale").dtype == torch.float32


@pytest.mark.gpu
def test_gpu_conversion_equals_cpu_conversion():
    """On the GPU the fused quantize+pack kernel does the conversion: same bytes, same scales."""
    from conftest import announce
    announce("convert on gpu")
    torch.manual_seed(3)
    model = nn.Sequential(nn.Linear(256, 128), nn.ReLU(), TernaryLinear(128, 64, threshold_factor=0.08), nn.ReLU(),
                          TernaryLinear(64, 32, per_channel=False))
    cpu = convert_linear_layers(model)
    gpu = convert_linear_layers(model.cuda())
    for k, v in cpu.state_dict().items():
        assert torch.equal(v, gpu.state_dict()[k].cpu()), k
    x = torch.randn(9, 256)
    assert torch.allclose(gpu(x.cuda()).cpu(), cpu(x), atol=1e-4, rtol=1e-4)


def test_fused_layers_on_the_cpu_path_equal_the_separate_layers():
    import bittorch_amd as bt
    torch.manual_seed(0)
    mk = lambda o: bt.nn.create_ternary_linear_inference(64, o, torch.randn(o, 64) * 0.02, torch.randn(o) * 0.01)
    a, b = mk(48), mk(16)
    ab = bt.utils.fuse_ternary_linear_inference(a, b)
    assert ab.in_features == 64 and ab.out_features == 64 and ab.weight_packed.shape == (16, 64)
    x = torch.randn(5, 64)
    y = ab(x)
    assert torch.equal(y[:, :48], a(x)) and torch.equal(y[:, 48:], b(x))
    with pytest.raises(ValueError, match="share in_features"):
        bt.utils.fuse_ternary_linear_inference(a, bt.nn.create_ternary_linear_inference(32, 8, torch.randn(8, 32)))
    with pytest.raises(ValueError, match="bias"):
        bt.utils.fuse_ternary_linear_inference(a, bt.nn.create_ternary_linear_inference(64, 8, torch.randn(8, 64)))


def test_ternary_swiglu_cpu_path_and_argument_checks():
    import torch.nn.functional as F
    import bittorch_amd as bt
    torch.manual_seed(1)
    mk = lambda i, o: bt.nn.create_ternary_linear_inference(i, o, torch.randn(o, i) * 0.02)
    gate, up, down = mk(32, 80), mk(32, 80), mk(80, 32)
    x = torch.randn(7, 32)
    nw = torch.ones(32)
    for fuse in (False, True):
        mlp = bt.nn.TernarySwiGLU(gate, up, down, fuse_gate_up=fuse)
        h = F.rms_norm(x, (32,), nw, 1e-5)
        ref = down(F.silu(gate(h)) * up(h)) + x
        assert torch.allclose(mlp(x, nw, 1e-5, residual=x), ref, rtol=1e-5, atol=1e-6)
        assert torch.allclose(mlp(x), down(F.silu(gate(x)) * up(x)), rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError, match="compute must be"):
        bt.nn.TernarySwiGLU(gate, up, down, compute="fp8")
    with pytest.raises(ValueError, match="do not form an MLP"):
        bt.nn.TernarySwiGLU(gate, up, mk(64, 32))


class _Blk(nn.Module):
    """A block in the shape the exporter reads: seven ternary layers and two RMSNorms."""
    def __init__(self, d=64, kv=32, ffn=96, layer=None):
        super().__init__()
        mk = layer or (lambda i, o: TernaryLinear(i, o, bias=False))
        self.q, self.k, self.v, self.o = mk(d, d), mk(d, kv), mk(d, kv), mk(d, d)
        self.gate, self.up, self.down = mk(d, ffn), mk(d, ffn), mk(ffn, d)
        self.n1, self.n2 = nn.RMSNorm(d), nn.RMSNorm(d)


def test_js_runtime_export_names_shapes_and_round_trip(tmp_path):
    """The file the reference's browser runtime loads (js/src/models/TernaryTransformer.ts:124-188): names, dtypes,
    [inBytes, outFeatures] shapes, k|v fused as kv_proj, bytes equal to the layers' own packing."""
    import bittorch_amd as bt
    from safetensors import safe_open
    torch.manual_seed(0)
    blocks = nn.ModuleList([_Blk(), _Blk()])
    for b in blocks:
        nn.init.normal_(b.n1.weight)
    emb, head, norm = torch.randn(50, 64), torch.randn(50, 64), torch.rand(64)
    path = str(tmp_path / "model.safetensors")
    bt.utils.export_js_safetensors(blocks, path, emb, head, norm, metadata={"format": "pt"})
    with safe_open(path, framework="pt") as fh:
        keys = set(fh.keys())
        expect = {"tok.weight", "head.weight", "norm.weight"}
        for i in range(2):
            expect |= {f"blocks.{i}.norm1.weight", f"blocks.{i}.norm2.weight"}
            for name in ("attn.q_proj", "attn.kv_proj", "attn.proj", "mlp.w_gate", "mlp.w_up", "mlp.w_down"):
                expect |= {f"blocks.{i}.{name}.weight_packed", f"blocks.{i}.{name}.scale"}
        assert keys == expect
        assert fh.get_tensor("blocks.0.attn.kv_proj.weight_packed").shape == (16, 64)     # [64 / 4, 32 + 32]
        assert fh.get_tensor("blocks.1.mlp.w_down.weight_packed").shape == (24, 64)
        assert fh.get_tensor("blocks.0.mlp.w_gate.weight_packed").dtype == torch.uint8
        assert fh.get_tensor("blocks.0.mlp.w_gate.scale").dtype == torch.float32
        assert fh.get_tensor("blocks.0.mlp.w_gate.scale").shape == (96,)
        assert torch.equal(fh.get_tensor("blocks.0.norm1.weight"), blocks[0].n1.weight.detach())
        # the bytes are the layers' own packing (reference layout), k then v along the columns
        k_inf, v_inf = bt.utils.ternary_linear_to_infer(blocks[0].k), bt.utils.ternary_linear_to_infer(blocks[0].v)
        kv = fh.get_tensor("blocks.0.attn.kv_proj.weight_packed")
        assert torch.equal(kv[:, :32], k_inf.weight_packed) and torch.equal(kv[:, 32:], v_inf.weight_packed)
        assert torch.equal(fh.get_tensor("blocks.0.attn.kv_proj.scale"), torch.cat([k_inf.scale, v_inf.scale]))
    loaded, extras, meta = bt.utils.load_js_safetensors(path)
    assert meta == {"format": "pt"} and len(loaded) == 2 and torch.equal(extras["tok.weight"], emb)
    x = torch.randn(3, 64)
    blk = loaded[1]
    ref = bt.utils.convert_linear_layers(blocks[1])
    assert torch.equal(blk["attn.q_proj"](x), ref.q(x))
    assert torch.equal(blk["attn.kv_proj"](x), torch.cat([ref.k(x), ref.v(x)], dim=-1))
    h = torch.randn(3, 96)
    assert torch.equal(blk["mlp.w_down"](h), ref.down(h))
    with pytest.raises(ValueError, match="no bias"):
        bt.utils.export_js_safetensors([_Blk(layer=lambda i, o: TernaryLinear(i, o, bias=True))], path)
    with pytest.raises(ValueError, match="multiple of 4"):
        bt.utils.export_js_safetensors([_Blk(d=66, layer=lambda i, o: TernaryLinear(i, o, bias=False))], path)


@pytest.mark.gpu
def test_gpu_converted_block_round_trips_through_the_js_file(tmp_path):
    """GPU-converted block (fused quantize+pack kernel, decode-tiled resident weights) -> file -> reload on the GPU:
    identical bytes, identical forward of every layer."""
    import bittorch_amd as bt
    from conftest import announce
    announce("js export on gpu")
    torch.manual_seed(1)
    d, kv, ffn = 256, 128, 704
    blocks = nn.ModuleList([_Blk(d, kv, ffn) for _ in range(2)]).cuda()
    infer = bt.utils.convert_linear_layers(blocks)
    x = torch.randn(5, d, device="cuda").half()
    h = torch.randn(5, ffn, device="cuda").half()
    before = [{n: getattr(b, n)(h if n == "down" else x) for n in ("q", "k", "v", "o", "gate", "up", "down")} for b in infer]
    for b in infer:   # decode-shape calls have made the tiled copy the layers' only one
        assert not b.q._has_row_major() and b.q.resident_weight_bytes() == b.q._tiled.numel()
    path = str(tmp_path / "model.safetensors")
    bt.utils.export_js_safetensors(infer, path)
    cpu_path = str(tmp_path / "cpu.safetensors")
    bt.utils.export_js_safetensors(bt.utils.convert_linear_layers(blocks.cpu()), cpu_path)
    assert open(path, "rb").read() == open(cpu_path, "rb").read()        # byte-identical files
    loaded, _, _ = bt.utils.load_js_safetensors(path, device="cuda")
    for b, blk, ref in zip(infer, loaded, before):
        assert torch.equal(blk["attn.q_proj"].packed_weights(), b.q.packed_weights())
        assert torch.equal(blk["attn.q_proj"](x), ref["q"])
        assert torch.equal(blk["attn.kv_proj"](x), torch.cat([ref["k"], ref["v"]], dim=-1))
        assert torch.equal(blk["attn.proj"](x), ref["o"])
        assert torch.equal(blk["mlp.w_gate"](x), ref["gate"]) and torch.equal(blk["mlp.w_up"](x), ref["up"])
        assert torch.equal(blk["mlp.w_down"](h), ref["down"])
