"""The config-5 harness: a BitNet-b1.58-like decoder stack whose seven projections per block are ternary layers.

Not a model zoo entry: the workload the benchmark times and the GPU tests compare, in every variant of the ternary
path (training modules, converted inference modules, inference modules with the block glue fused, the int8 path).
Block structure of the reference's JS runtime (js/src/models/TernaryTransformer.ts:366-423, :489-521): pre-norm,
causal attention, SwiGLU MLP; attention, norms and the embedding stay in PyTorch.
"""

from __future__ import annotations

import torch


class BlockStack:
    """Config 5: a 2B-parameter BitNet-b1.58-like stack.  q/k/v/o/gate/up/down are TernaryLinear
    (random N(0,0.02) masters, no bias); RMSNorm, rotary-free causal SDPA and the embedding stay in
    PyTorch-ROCm; bf16 activations, a seeded token batch of batch x seq.  The same stack runs in the
    variants the benchmark times (and the GPU tests compare): training modules, converted inference
    modules, inference modules with the glue fused, and the int8 path."""

    def __init__(self, dev, layers=30, d_model=2560, heads=20, ffn=6912, batch=8, seq=512, vocab=32000,
                 backend="auto", act_dtype=None, fake_quant=False, attn_scale=None, master_std=0.02):
        """``attn_scale``: the softmax scale of the attention (default 1/sqrt(head_dim)).  ``master_std``: standard
        deviation of the random master weights, one number or a dict by projection name (``q k v o gate up down``;
        missing names take 0.02).  With the defaults (N(0, 0.02) masters everywhere) the attention logits of a block
        have a standard deviation near 15 and the MLP branch is some 70 times the residual stream; a test that wants
        every branch of order one, so that element-wise bounds bite, passes smaller values."""
        import torch.nn as nn
        import torch.nn.functional as F
        import bittorch_amd as bt

        self.torch, self.F, self.bt = torch, F, bt
        self.attn_scale = attn_scale
        self.prefill_copy = False  # prepare_prefill(): the int8 path on the layers' field-layout copies
        std_of = (lambda name: master_std.get(name, 0.02)) if isinstance(master_std, dict) else (lambda name: master_std)
        self.d_model, self.heads, self.ffn = d_model, heads, ffn
        act_dtype = act_dtype or torch.bfloat16
        self.act_dtype = act_dtype

        def fq(t):
            """fake_quant: the int8 path's per-token activation quantizer (whole-row absmax / 127, halves away
            from zero, clamp) applied in the tensor's own dtype ahead of every ternary layer, in plain torch"""
            if not fake_quant:
                return t
            amax = t.abs().amax(dim=-1, keepdim=True).float()
            s = torch.where(amax > 1e-6, amax / 127.0, torch.ones_like(amax))
            v = t.float() * (1.0 / s)
            q = torch.clamp(torch.sign(v) * torch.floor(v.abs() + 0.5), -127, 127)
            return (q * s).to(t.dtype)

        class Block(nn.Module):
            def __init__(self):
                super().__init__()
                mk = lambda i, o: bt.nn.TernaryLinear(i, o, bias=False, backend=backend)
                self.q, self.k, self.v, self.o = mk(d_model, d_model), mk(d_model, d_model), mk(d_model, d_model), mk(d_model, d_model)
                self.gate, self.up, self.down = mk(d_model, ffn), mk(d_model, ffn), mk(ffn, d_model)
                self.n1 = nn.RMSNorm(d_model, eps=1e-5)
                self.n2 = nn.RMSNorm(d_model, eps=1e-5)

            def forward(self, x):
                b, t, _ = x.shape
                h = fq(self.n1(x))
                q = self.q(h).view(b, t, heads, -1).transpose(1, 2)
                k = self.k(h).view(b, t, heads, -1).transpose(1, 2)
                v = self.v(h).view(b, t, heads, -1).transpose(1, 2)
                a = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=attn_scale).transpose(1, 2).reshape(b, t, -1)
                x = x + self.o(fq(a))
                h = fq(self.n2(x))
                return x + self.down(fq(F.silu(self.gate(h)) * self.up(h)))

        torch.manual_seed(0)
        with torch.device(dev):
            self.emb = nn.Embedding(vocab, d_model).to(act_dtype)
            self.blocks = nn.ModuleList([Block() for _ in range(layers)])
            self.final = nn.RMSNorm(d_model, eps=1e-5)
        for name, m in self.blocks.named_modules():
            if isinstance(m, bt.nn.TernaryLinear):
                nn.init.normal_(m.weight, std=std_of(name.rsplit(".", 1)[-1]))
            elif isinstance(m, nn.RMSNorm):
                m.to(act_dtype)
        self.final.to(act_dtype)
        self.tokens = torch.randint(0, vocab, (batch, seq), generator=torch.Generator().manual_seed(0)).to(dev)
        self.n_tern = sum(m.weight.numel() for m in self.blocks.modules() if isinstance(m, bt.nn.TernaryLinear))
        self.infer = None

    def forward(self, stack=None):
        """Unfused forward of `stack` (the training modules by default, or the converted modules)."""
        torch = self.torch
        with torch.no_grad():
            x = self.emb(self.tokens)
            for blk in (self.blocks if stack is None else stack):
                x = blk(x)
            return self.final(x)

    def drop_packed_caches(self):
        for m in self.blocks.modules():
            if isinstance(m, self.bt.nn.TernaryLinear):
                m._packed.clear()

    def convert(self, inplace=True):
        """TernaryLinear -> TernaryLinearInference, then q|k|v and gate|up each as one layer."""
        bt = self.bt
        self.infer = bt.utils.convert_linear_layers(self.blocks, inplace=inplace)
        if inplace:
            self.blocks = None  # (the masters are freed layer by layer)
        return self.infer

    def fuse(self):
        bt = self.bt
        for blk in self.infer:
            blk.qkv = bt.utils.fuse_ternary_linear_inference(blk.q, blk.k, blk.v)
            blk.mlp = bt.nn.TernarySwiGLU(blk.gate, blk.up, blk.down, compute="float", fuse_gate_up=True)

    def _fused_block(self, blk, x, int8):
        torch, F, bt = self.torch, self.F, self.bt
        from bittorch_amd.ops import fused
        heads, d_model = self.heads, self.d_model
        b, s, _ = x.shape
        heads_of = lambda t: t.view(b, s, heads, -1).transpose(1, 2)
        if int8:  # BitNet-style: every projection on the int8 matrix cores from activations that leave the
            # norm / SwiGLU kernels already quantized per token
            # (row sums of the quantized rows ride along where the layers hold a prefill copy: prepare_prefill)
            pre = self.prefill_copy
            qh, sh, *rs = fused.rmsnorm(x, blk.n1.weight, blk.n1.eps or torch.finfo(x.dtype).eps, store=False, quantize=True,
                                        operand_order=True, return_rowsum=pre)
            qkv = blk.qkv.forward_int8(qh, sh, x.dtype, None, True, rs[0] if rs else None)
        else:
            qkv = blk.qkv(fused.rmsnorm(x, blk.n1.weight, blk.n1.eps or torch.finfo(x.dtype).eps))
        q, k, v = qkv.split(d_model, dim=-1)  # one GEMM over the concatenated q|k|v columns
        a = F.scaled_dot_product_attention(heads_of(q), heads_of(k), heads_of(v), is_causal=True, scale=self.attn_scale)
        a = a.transpose(1, 2).reshape(b, s, -1)
        if int8:
            qa, sa, *rs = bt._C.act_quant_int8(a.reshape(b * s, -1), True, self.prefill_copy)
            x = blk.o.forward_int8(qa, sa, x.dtype, x.reshape(b * s, -1), True, rs[0] if rs else None).view(b, s, -1)
        else:
            x = blk.o(a, x)
        return blk.mlp(x, blk.n2.weight, blk.n2.eps or torch.finfo(x.dtype).eps, residual=x)

    def prepare_prefill(self, on: bool = True):
        """Give every fused inference layer its prefill-only second weight copy (or release it): the int8 path then
        runs its GEMMs on the field layout, with the same results."""
        self.prefill_copy = bool(on)
        for blk in self.infer:
            for m in (blk.qkv, blk.o):
                m.prepare_prefill() if on else m.drop_prefill()
            blk.mlp.prepare_prefill() if on else blk.mlp.drop_prefill()
        return self

    def forward_fused(self, int8):
        """The converted stack with the glue between the ternary layers fused: residual adds in the GEMM
        epilogues, silu(gate)*up in one kernel, RMSNorm from this library, q|k|v and gate|up each one GEMM
        over concatenated columns; int8: every projection on the int8 matrix cores."""
        torch = self.torch
        for blk in self.infer:
            blk.mlp.compute = "int8" if int8 else "float"
        with torch.no_grad():
            x = self.emb(self.tokens)
            for blk in self.infer:
                x = self._fused_block(blk, x, int8)
            return self.final(x)


