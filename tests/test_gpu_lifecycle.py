"""GPU: the module life cycle -- quantize, forward / backward, merge + re-quantise, inject into a model, load a
pre-quantized checkpoint, merge scheduling with optimizer reset.  The assertions restate the contracts of the
reference's own module tests (tests/qlora/test_qlora.py:101-560) on this package's classes; the numeric checks
of the kernels themselves are in the parity tests."""

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from xorl_amd import quantize as Q
from xorl_amd.qlora import (BlockFP8QLoRALinear, QLoRALinear, inject_qlora_into_model, maybe_merge_lora,
                            maybe_requant_qlora, reset_lora_optimizer_states)

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(300)]
FP4_MAX, FP8_MAX = 6.0, 448.0


def _bf16_linear(dev, k=256, n=512, seed=0):
    torch.manual_seed(seed)
    return nn.Linear(k, n, bias=False, device=dev, dtype=torch.bfloat16)


class _MLP(nn.Module):
    def __init__(self):
        super().__init__()
        self.gate_proj, self.up_proj, self.down_proj = nn.Linear(256, 512, bias=False), nn.Linear(256, 512, bias=False), nn.Linear(512, 256, bias=False)

    def forward(self, x):
        return self.down_proj(F.silu(self.gate_proj(x)) * self.up_proj(x))


class _Attn(nn.Module):
    def __init__(self):
        super().__init__()
        for n in ("q_proj", "k_proj", "v_proj", "o_proj"):
            setattr(self, n, nn.Linear(256, 256, bias=False))

    def forward(self, x):
        q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
        att = torch.softmax(torch.bmm(q, k.transpose(-1, -2)) / 16.0, -1)
        return self.o_proj(torch.bmm(att, v))


class _Layer(nn.Module):
    def __init__(self):
        super().__init__()
        self.self_attn, self.mlp = _Attn(), _MLP()

    def forward(self, x):
        return x + self.mlp(self.self_attn(x))


class _Model(nn.Module):
    def __init__(self):
        super().__init__()
        self.layers = nn.ModuleList([_Layer()])

    def forward(self, x):
        for layer in self.layers:
            x = layer(x)
        return x


def _make_model(dev):
    torch.manual_seed(3)
    return _Model().to(dev).to(torch.bfloat16)


def _fill_injected(model):
    g = torch.Generator(device="cuda").manual_seed(4)
    for m in model.modules():
        if isinstance(m, QLoRALinear) and m._is_prequantized:
            w = torch.randn(m.out_features, m.in_features, device="cuda", generator=g) * 0.05
            m._quantize_and_store(w.to(torch.bfloat16))


@pytest.mark.parametrize("fmt,group", [("nvfp4", 16), ("block_fp8", 128), ("nf4", 64), ("int4", 128)])
def test_quantize_forward_backward_memory(hip_device, fmt, group):
    lin = _bf16_linear(hip_device)
    m = QLoRALinear.from_module(lin, r=16, lora_alpha=16, quant_format=fmt, quant_group_size=group)
    assert m.packed_weight_f32.dtype == torch.float32 and not m.packed_weight_f32.requires_grad
    assert m.lora_A.requires_grad and m.lora_B.requires_grad and m.weight is None
    x = torch.randn(2, 10, 256, device=hip_device, dtype=torch.bfloat16)
    out = m(x)
    assert out.shape == (2, 10, 512)
    out.sum().backward()
    assert m.lora_A.grad is not None and m.lora_B.grad is not None and m.packed_weight_f32.grad is None
    nbytes = m.packed_weight_f32.numel() * 4
    for name in ("weight_block_scales", "weight_global_scale", "weight_scales"):
        s = getattr(m, name, None)
        if s is not None:
            nbytes += s.numel() * s.element_size()
    assert nbytes < lin.weight.numel() * 2


def test_dequantize_roundtrip_bounds(hip_device):
    for fmt, group in (("nvfp4", 16), ("nf4", 64), ("block_fp8", 128)):
        lin = _bf16_linear(hip_device, seed=1)
        w = lin.weight.detach().clone()
        m = QLoRALinear.from_module(lin, r=16, lora_alpha=16, quant_format=fmt, quant_group_size=group)
        deq = m._dequantize_weight().float()
        if fmt == "nvfp4":
            torch.testing.assert_close(w, deq.to(torch.bfloat16), atol=0.05, rtol=0.05)
        else:
            rel = (w.float() - deq).abs().mean() / w.float().abs().mean()
            assert rel < (0.10 if fmt == "nf4" else 0.03)


def test_from_quantized_nvfp4(hip_device):
    torch.manual_seed(2)
    w = torch.randn(512, 256, device=hip_device, dtype=torch.bfloat16)
    packed, bs, gs = Q.nvfp4_quantize(w, 16)
    m = QLoRALinear.from_quantized(packed_weight=packed, weight_block_scales=bs, weight_global_scale=gs, in_features=256,
                                   out_features=512, quant_format="nvfp4", quant_group_size=16, device=hip_device)
    assert m.packed_weight_f32.dtype == torch.float32
    # the module decodes what the codec decodes
    ref = Q.nvfp4_dequantize(packed, bs, gs, 512 * 256, 16).reshape(512, 256)
    assert torch.equal(m._dequantize_weight(), ref.to(torch.bfloat16))
    out = m(torch.randn(2, 10, 256, device=hip_device, dtype=torch.bfloat16))
    out.sum().backward()
    assert out.shape == (2, 10, 512) and m.lora_A.grad is not None and m.lora_B.grad is not None


def test_ema_amax_and_nvfp4_scale_convention(hip_device):
    lin = _bf16_linear(hip_device, seed=5)
    amax = lin.weight.float().abs().max().item()
    m = QLoRALinear.from_module(lin, r=16, lora_alpha=16, quant_format="nvfp4", quant_group_size=16)
    assert m._ema_amax is not None and m._ema_amax.shape == (1,) and abs(m._ema_amax.item() - amax) < 1e-4
    with torch.no_grad():
        m.lora_A.fill_(0.5)
        m.lora_B.fill_(0.5)
    m.merge_weights(ema_decay=0.5)
    # merged weight = w + 0.5*0.5*16 = w + 4 everywhere: amax ~ 4 + amax; the EMA moves half way
    assert abs(m._ema_amax.item() - (0.5 * amax + 0.5 * (4.0 + amax))) < 0.1
    gs = m._recover_tensor(m.weight_global_scale, m._scale_dtypes["weight_global_scale"]).item()
    want = m._ema_amax.item() / (FP4_MAX * FP8_MAX)
    assert abs(gs - want) / want < 0.01

    w2 = torch.randn(512, 256, device=hip_device, dtype=torch.bfloat16) * 2.0
    packed, bs, gs2 = Q.nvfp4_quantize(w2, 16)
    assert bs.float().max().item() > 1.0                       # block scales span the fp8 range, not [0, 1]
    deq = Q.nvfp4_dequantize(packed, bs, gs2, 512 * 256, 16).reshape(512, 256)
    assert (w2.float() - deq.float()).abs().mean() / w2.float().abs().mean() < 0.15
    w3 = torch.randn(512, 256, device=hip_device, dtype=torch.bfloat16) * 3.0
    _, _, gs3 = Q.nvfp4_quantize(w3, 16)
    assert gs3.item() * FP4_MAX * FP8_MAX >= w3.float().abs().max().item() * 0.99


def test_merge_weights_and_requant(hip_device):
    m = QLoRALinear.from_module(_bf16_linear(hip_device, seed=6), r=16, lora_alpha=16, quant_format="nvfp4", quant_group_size=16)
    with torch.no_grad():
        m.lora_A.fill_(0.1)
        m.lora_B.fill_(0.1)
    before = m._dequantize_weight().clone()
    m.merge_weights()
    assert (m._dequantize_weight() - before).float().abs().mean() > 0.001
    assert not torch.all(m.lora_A == 0) and torch.all(m.lora_B == 0)       # A re-drawn, B zero

    m2 = QLoRALinear.from_module(_bf16_linear(hip_device, seed=7), r=16, lora_alpha=16, quant_format="nvfp4", quant_group_size=16)
    with torch.no_grad():
        m2.lora_A.fill_(0.05)
        m2.lora_B.fill_(0.05)
    before = m2._dequantize_weight().clone()
    expected = before + m2.get_delta_weight().to(before.dtype)
    m2.merge_weights()
    assert (m2._dequantize_weight() - expected).float().abs().mean() < 0.1
    sd = m2.get_quantized_state_dict()
    assert all(k in sd for k in ("packed_weight_f32", "weight_block_scales", "weight_global_scale"))

    m3 = QLoRALinear.from_module(_bf16_linear(hip_device, seed=8), r=16, lora_alpha=16, quant_format="nvfp4", quant_group_size=16)
    amax = m3._ema_amax.item()
    with torch.no_grad():
        m3.lora_A.fill_(1.0)
        m3.lora_B.fill_(1.0)
    before = m3._dequantize_weight().clone()
    assert maybe_requant_qlora(nn.ModuleList([m3]), ema_decay=0.5) == 1
    assert not torch.equal(before, m3._dequantize_weight()) and m3._ema_amax.item() != amax and torch.all(m3.lora_B == 0)


def test_injected_model_trains(hip_device):
    model = _make_model(hip_device)
    inject_qlora_into_model(model, r=16, lora_alpha=16, quant_format="nvfp4", quant_group_size=16,
                            target_modules=["q_proj", "k_proj", "v_proj", "o_proj"])
    _fill_injected(model)
    layer = model.layers[0]
    assert isinstance(layer.self_attn.q_proj, QLoRALinear) and not isinstance(layer.mlp.gate_proj, QLoRALinear)
    assert layer.self_attn.q_proj.packed_weight_f32.device.type == "cuda"
    x = torch.randn(2, 10, 256, device=hip_device, dtype=torch.bfloat16)
    model(x).sum().backward()
    for name, m in model.named_modules():
        if isinstance(m, QLoRALinear):
            assert m.lora_A.grad is not None and m.lora_B.grad is not None, name
            assert torch.isfinite(m.lora_A.grad).all() and torch.count_nonzero(m.lora_B.grad) > 0, name

    model = _make_model(hip_device)
    inject_qlora_into_model(model, r=16, lora_alpha=16, quant_format="block_fp8", quant_group_size=128,
                            checkpoint_quant_format="block_fp8", target_modules=["q_proj", "o_proj", "down_proj"])
    mods = [m for m in model.modules() if isinstance(m, QLoRALinear)]
    assert len(mods) == 3 and all(m._source_quant_format == "block_fp8" and m.quant_format == "block_fp8" for m in mods)


def _load_fp8(m, fqn, parts, dev):
    data = {}
    torch.manual_seed(9)
    ws = []
    for name, rows in parts:
        w = torch.randn(rows, m.in_features, device=dev, dtype=torch.bfloat16)
        b, s = Q.block_fp8_quantize_gkn(w.float(), 128)
        data[f"{fqn}{name}.weight"], data[f"{fqn}{name}.weight_scale_inv"] = b.cpu(), s.cpu()
        ws.append(w)
    m._is_prequantized, m._source_quant_format = True, "block_fp8"
    m._load_prequantized(lambda key: data[key])
    return torch.cat(ws, 0)


def test_prequantized_block_fp8_load_forward_merge(hip_device):
    m = BlockFP8QLoRALinear(256, 256, r=16, lora_alpha=16, device=torch.device(hip_device))
    m._merge_sources, m._source_fqn = None, "model.layers.0.self_attn.o_proj"
    w = _load_fp8(m, "model.layers.0.self_attn.o_proj", [("", 256)], hip_device)
    assert m.packed_weight_f32 is not None and m._ema_amax is None
    deq = m._dequantize_weight().to(torch.bfloat16)
    assert (w - deq).float().abs().mean() / w.float().abs().mean() < 0.03
    out = m(torch.randn(2, 10, 256, device=hip_device, dtype=torch.bfloat16))
    out.sum().backward()
    assert out.shape == (2, 10, 256) and m.lora_A.grad is not None

    qkv = BlockFP8QLoRALinear(256, 256 + 128 + 128, r=16, lora_alpha=16, device=torch.device(hip_device))
    qkv._merge_sources, qkv._source_fqn = ("q_proj", "k_proj", "v_proj"), "model.layers.0.self_attn"
    w = _load_fp8(qkv, "model.layers.0.self_attn.", [("q_proj", 256), ("k_proj", 128), ("v_proj", 128)], hip_device)
    assert qkv.packed_weight_f32.numel() * 4 == 512 * 256
    deq = qkv._dequantize_weight().to(torch.bfloat16)
    assert (w - deq).float().abs().mean() / w.float().abs().mean() < 0.03      # the rows landed in source order

    with torch.no_grad():
        m.lora_A.fill_(0.1)
        m.lora_B.fill_(0.1)
    before = m._dequantize_weight().clone()
    m.merge_weights()
    assert (m._dequantize_weight() - before).float().abs().mean() > 0.001 and m._ema_amax is None


def test_optimizer_reset_and_merge_schedule(hip_device):
    m = QLoRALinear.from_module(_bf16_linear(hip_device, seed=10), r=16, lora_alpha=16, quant_format="block_fp8", quant_group_size=128)
    m.train()
    opt = torch.optim.AdamW([m.lora_A, m.lora_B], lr=1e-3)
    x = torch.randn(4, 8, 256, device=hip_device, dtype=torch.bfloat16)
    tgt = torch.randn(4, 8, 512, device=hip_device, dtype=torch.bfloat16)

    def step():
        opt.zero_grad()
        ((m(x) - tgt) ** 2).mean().backward()
        opt.step()

    step()
    assert m.lora_A in opt.state and "exp_avg" in opt.state[m.lora_A] and m.lora_B in opt.state
    assert reset_lora_optimizer_states(nn.ModuleList([m]), opt) == 2
    assert m.lora_A not in opt.state and m.lora_B not in opt.state
    step()
    assert m.lora_A in opt.state and m.lora_B in opt.state

    # only the factors' state goes; other trainable parameters keep theirs
    model = _make_model(hip_device)
    inject_qlora_into_model(model, r=16, lora_alpha=16, quant_format="block_fp8", quant_group_size=128,
                            target_modules=["q_proj", "k_proj", "v_proj", "o_proj"])
    _fill_injected(model)
    opt2 = torch.optim.AdamW(list(model.parameters()), lr=1e-3)
    xs = torch.randn(2, 8, 256, device=hip_device, dtype=torch.bfloat16)
    opt2.zero_grad()
    model(xs).sum().backward()
    opt2.step()
    kept = {n: opt2.state[p]["exp_avg"].clone() for n, p in model.named_parameters() if "lora_" not in n and p in opt2.state}
    assert kept and reset_lora_optimizer_states(model, opt2) == 8
    for n, p in model.named_parameters():
        if n in kept:
            assert torch.equal(opt2.state[p]["exp_avg"], kept[n])

    # scheduling: nothing off the interval; merge + re-quantise + reset on it
    model = _make_model(hip_device)
    inject_qlora_into_model(model, r=16, lora_alpha=16, quant_format="block_fp8", quant_group_size=128,
                            target_modules=["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"])
    _fill_injected(model)
    model.train()
    opt3 = torch.optim.AdamW([p for p in model.parameters() if p.requires_grad], lr=1e-3)
    opt3.zero_grad()
    model(xs).sum().backward()
    opt3.step()
    mods = [q for q in model.modules() if isinstance(q, QLoRALinear)]
    assert len(mods) == 7 and all(q.lora_A in opt3.state and q.lora_B in opt3.state for q in mods)
    with torch.no_grad():
        for q in mods:
            q.lora_A.fill_(0.25)
            q.lora_B.fill_(0.25)
    packed = [q.packed_weight_f32.clone() for q in mods]
    maybe_merge_lora(model, enable_lora=False, enable_qlora=True, merge_interval=10, global_step=9, optimizer=opt3, reset_optimizer=True)
    assert all(torch.equal(q.packed_weight_f32, b) for q, b in zip(mods, packed))
    assert all(q.lora_A in opt3.state for q in mods) and all(torch.all(q.lora_B == 0.25) for q in mods)
    maybe_merge_lora(model, enable_lora=False, enable_qlora=True, merge_interval=10, global_step=10, optimizer=opt3, reset_optimizer=True)
    assert all(not torch.equal(q.packed_weight_f32, b) for q, b in zip(mods, packed))
    assert all(q.lora_A not in opt3.state and q.lora_B not in opt3.state for q in mods)
    assert all(torch.count_nonzero(q.lora_B) == 0 for q in mods)
    # and the model still trains after the merge
    opt3.zero_grad()
    model(xs).sum().backward()
    opt3.step()
    assert all(q.lora_A in opt3.state for q in mods)


class _Router(nn.Module):
    """Top-k softmax router + experts call with the reference block's calling convention
    (hidden_states, routing_weights, selected_experts)."""

    def __init__(self, E, h, i, topk):
        super().__init__()
        self.gate = nn.Linear(h, E, bias=False)
        self.experts = nn.Module()
        for n, shape in (("gate_proj", (E, h, i)), ("up_proj", (E, h, i)), ("down_proj", (E, i, h))):
            self.experts.register_parameter(n, nn.Parameter(torch.empty(*shape, device="meta")))
        self.topk = topk

    def route(self, x):
        w, sel = torch.topk(torch.softmax(self.gate(x).float(), -1), self.topk, -1)
        return (w / w.sum(-1, keepdim=True)).to(x.dtype), sel.to(torch.int32)

    def forward(self, x):
        w, sel = self.route(x)
        return self.experts(x, w, sel)


def test_injected_moe_model_loads_a_checkpoint_and_trains(hip_device, tmp_path):
    """The whole switch: a model whose expert weights are still on the meta device gets QLoRA modules, fills them
    from a block-fp8 checkpoint directory and trains; its output matches a bf16 torch model built from the
    checkpoint's own decoded tensors."""
    import json
    import os

    import safetensors.torch

    from xorl_amd.qlora import BlockFP8QLoRAMoeExperts, maybe_load_prequantized_qlora

    E, h, i, topk, T = 8, 256, 128, 2, 192
    dev = hip_device
    g = torch.Generator().manual_seed(12)
    tensors, deq = {}, {}

    def add(key, rows, cols):
        b, s = Q.block_fp8_quantize_gkn(torch.randn(rows, cols, generator=g) * 0.05, 128)
        tensors[f"{key}.weight"], tensors[f"{key}.weight_scale_inv"] = b, s
        deq[key] = (b.float().view(rows // 128, 128, cols // 128, 128) * s.view(rows // 128, 1, cols // 128, 1)).view(rows, cols).to(torch.bfloat16)

    add("blk.o_proj", h, h)
    for e in range(E):
        add(f"blk.moe.experts.{e}.gate_proj", i, h)
        add(f"blk.moe.experts.{e}.up_proj", i, h)
        add(f"blk.moe.experts.{e}.down_proj", h, i)
    safetensors.torch.save_file(tensors, os.path.join(tmp_path, "model.safetensors"))
    json.dump({"weight_map": {k: "model.safetensors" for k in tensors}}, open(os.path.join(tmp_path, "model.safetensors.index.json"), "w"))

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.o_proj = nn.Linear(h, h, bias=False)
            self.moe = _Router(E, h, i, topk)

        def forward(self, x):
            return self.moe(self.o_proj(x))

    class Model(nn.Module):
        def __init__(self):
            super().__init__()
            self.blk = Block()

        def forward(self, x):
            return self.blk(x)

    torch.manual_seed(13)
    model = Model()
    model.blk.o_proj.to(dev)
    model.blk.moe.gate.to(dev).to(torch.bfloat16)
    inject_qlora_into_model(model, r=8, lora_alpha=16, quant_format="block_fp8", checkpoint_quant_format="block_fp8",
                            target_modules=["o_proj", "gate_proj", "up_proj", "down_proj"])
    ex = model.blk.moe.experts
    assert isinstance(ex, BlockFP8QLoRAMoeExperts) and not ex._weights_loaded
    assert maybe_load_prequantized_qlora(model, str(tmp_path)) == 2
    assert ex._weights_loaded and ex.gate_packed.device.type == "cuda" and ex.gate_proj_lora_A.device.type == "cuda"
    with torch.no_grad():                                       # non-zero B factors so every term contributes
        for p in (model.blk.o_proj.lora_B, ex.gate_proj_lora_B, ex.up_proj_lora_B, ex.down_proj_lora_B):
            p.copy_(torch.randn(p.shape, generator=g).to(dev) * 0.05)

    x = (torch.randn(T, h, generator=g)).to(dev).to(torch.bfloat16)
    y = model(x)
    y.float().pow(2).sum().backward()
    for n, p in model.named_parameters():
        if "lora_" in n:
            assert p.grad is not None and torch.isfinite(p.grad).all() and torch.count_nonzero(p.grad) > 0, n

    # bf16 torch model from the decoded checkpoint tensors + the same factors, float32 accumulation
    def lin(xx, w, A, B, s):
        return (xx.float() @ w.to(dev).float().t() + s * (xx.float() @ A.float().t()) @ B.float().t())

    with torch.no_grad():
        o = model.blk.o_proj
        hdn = lin(x, deq["blk.o_proj"], o.lora_A, o.lora_B, o.scaling).to(torch.bfloat16)
        w, sel = model.blk.moe.route(hdn)
        ref = torch.zeros(T, h, device=dev)
        for e in range(E):
            tok, slot = (sel == e).nonzero(as_tuple=True)
            if tok.numel() == 0:
                continue
            xe = hdn[tok]

            def proj(name, inp):
                A, B = getattr(ex, f"{name}_lora_A"), getattr(ex, f"{name}_lora_B")
                A = A[e if A.shape[0] > 1 else 0]
                B = B[e if B.shape[0] > 1 else 0]
                return inp.float() @ deq[f"blk.moe.experts.{e}.{name}"].to(dev).float().t() + ex.scaling * (inp.float() @ A.float()) @ B.float()

            act = (F.silu(proj("gate_proj", xe)) * proj("up_proj", xe)).to(torch.bfloat16)
            ref.index_add_(0, tok, proj("down_proj", act) * w[tok, slot].float().unsqueeze(1))
    err = (y.float() - ref).abs().max() / ref.abs().max()
    assert err <= 2e-2, float(err)
