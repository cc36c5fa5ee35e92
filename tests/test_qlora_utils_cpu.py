"""Host logic: model-level QLoRA helpers (no GPU).  The contracts are those of the reference's own tests
(tests/qlora/test_qlora.py:283-330 injection, :17-62 scale convention) restated on the package's modules."""

import json
import os

import pytest
import torch
import torch.nn as nn

from xorl_amd.qlora import (BlockFP8QLoRALinear, BlockFP8QLoRAMoeExperts, NF4QLoRALinear, NF4QLoRAMoeExperts,
                            NvFP4QLoRALinear, QLoRALinear, QLoRAMoeExperts, detect_prequantized_block_fp8,
                            detect_prequantized_nvfp4, inject_qlora_into_model, maybe_load_prequantized_qlora,
                            maybe_quantize_qlora, save_qlora_checkpoint)


class _Attn(nn.Module):
    def __init__(self, h, fused):
        super().__init__()
        if fused:
            self.qkv_proj = nn.Linear(h, 2 * h, bias=False)
        else:
            self.q_proj, self.k_proj, self.v_proj = nn.Linear(h, h, bias=False), nn.Linear(h, h // 2, bias=False), nn.Linear(h, h // 2, bias=False)
        self.o_proj = nn.Linear(h, h, bias=True)


class _Experts(nn.Module):
    def __init__(self, E, h, i):
        super().__init__()
        self.gate_proj = nn.Parameter(torch.randn(E, h, i) * 0.05)
        self.up_proj = nn.Parameter(torch.randn(E, h, i) * 0.05)
        self.down_proj = nn.Parameter(torch.randn(E, i, h) * 0.05)
        self.act_fn = nn.SiLU()


class _MoeBlock(nn.Module):
    def __init__(self, E, h, i):
        super().__init__()
        self.gate = nn.Linear(h, E, bias=False)          # the router: never quantized
        self.experts = _Experts(E, h, i)


class _Layer(nn.Module):
    def __init__(self, h, fused, moe):
        super().__init__()
        self.self_attn = _Attn(h, fused)
        self.mlp = _MoeBlock(4, h, 128) if moe else nn.ModuleDict({"gate_proj": nn.Linear(h, 2 * h, bias=False),
                                                                  "down_proj": nn.Linear(2 * h, h, bias=False)})


class _Model(nn.Module):
    def __init__(self, h=256, fused=False, moe=False):
        super().__init__()
        self.model = nn.ModuleDict({"layers": nn.ModuleList([_Layer(h, fused, moe) for _ in range(2)])})
        self.lm_head = nn.Linear(h, 512, bias=False)


def test_injection_replaces_only_the_targets():
    model = _Model()
    inject_qlora_into_model(model, r=16, lora_alpha=16, quant_format="nvfp4", quant_group_size=16,
                            target_modules=["q_proj", "k_proj", "v_proj", "o_proj"])
    layer = model.model["layers"][0]
    assert isinstance(layer.self_attn.q_proj, NvFP4QLoRALinear) and isinstance(layer.self_attn.o_proj, QLoRALinear)
    assert not isinstance(layer.mlp["gate_proj"], QLoRALinear) and not isinstance(model.lm_head, QLoRALinear)
    q, o = layer.self_attn.q_proj, layer.self_attn.o_proj
    assert q._is_prequantized and q._source_fqn == "model.layers.0.self_attn.q_proj" and q._merge_sources is None
    assert q._qlora_expected_skip_keys == {"weight"} and q.weight is None
    assert o.bias is not None and (q.in_features, q.out_features, q.r) == (256, 256, 16)
    assert q.packed_weight_f32.dtype == torch.float32 and not q.packed_weight_f32.requires_grad
    assert q.lora_A.requires_grad and q.lora_B.requires_grad
    # a second call finds nothing left to replace among these targets
    with pytest.raises(ValueError, match="No nn.Linear modules found"):
        inject_qlora_into_model(model, target_modules=["q_proj"])
    with pytest.raises(ValueError, match="Supported QLoRA formats"):
        inject_qlora_into_model(_Model(), quant_format="mxfp4")


def test_injection_default_targets_fused_modules_and_checkpoint_format():
    model = _Model(fused=True)
    inject_qlora_into_model(model, r=8, lora_alpha=16, quant_format="block_fp8", quant_group_size=128,
                            checkpoint_quant_format="block_fp8", exclude_modules=["down_proj"])
    attn = model.model["layers"][1].self_attn
    assert isinstance(attn.qkv_proj, BlockFP8QLoRALinear) and isinstance(attn.o_proj, BlockFP8QLoRALinear)
    assert attn.qkv_proj._merge_sources == ("q_proj", "k_proj", "v_proj")
    assert attn.qkv_proj._source_fqn == "model.layers.1.self_attn"            # the parent: sources hang below it
    assert attn.o_proj._merge_sources is None and attn.o_proj._source_fqn == "model.layers.1.self_attn.o_proj"
    for m in model.modules():
        if isinstance(m, QLoRALinear):
            assert m._source_quant_format == "block_fp8" and m.quant_format == "block_fp8" and m.quant_group_size == 128
    assert not isinstance(model.model["layers"][0].mlp["down_proj"], QLoRALinear)   # excluded by name
    assert not isinstance(model.lm_head, QLoRALinear)


def test_injection_nf4_quantizes_at_once_and_experts_follow():
    model = _Model(moe=True)
    w_o = model.model["layers"][0].self_attn.o_proj.weight.detach().clone()
    inject_qlora_into_model(model, r=8, lora_alpha=8, quant_format="nf4",
                            target_modules=["o_proj", "gate_proj", "up_proj", "down_proj"])
    layer = model.model["layers"][0]
    o = layer.self_attn.o_proj
    assert isinstance(o, NF4QLoRALinear) and not o._is_prequantized
    # storage: 4 bits per weight + one fp32 absmax per 64
    assert o.packed_weight_f32.numel() * 4 == w_o.numel() // 2 and o.weight_scales.numel() == w_o.numel() // 64 * 4
    assert isinstance(layer.mlp.gate, nn.Linear) and not isinstance(layer.mlp.gate, QLoRALinear)   # router untouched
    ex = layer.mlp.experts
    assert isinstance(ex, NF4QLoRAMoeExperts) and ex._weights_loaded and ex.hybrid_shared
    assert ex.target_modules == ("gate_proj", "up_proj", "down_proj")
    assert ex.gate_packed.shape == (4, 128, 128) and ex.down_packed.shape == (4, 64, 256)
    assert ex.gate_proj_lora_A.shape == (1, 256, 8) and ex.down_proj_lora_A.shape == (4, 128, 8)


def test_injection_prequantized_experts_wait_for_the_checkpoint():
    model = _Model(moe=True)
    inject_qlora_into_model(model, quant_format="block_fp8", target_modules=["gate_proj", "up_proj", "down_proj"],
                            checkpoint_quant_format="block_fp8")
    ex = model.model["layers"][1].mlp.experts
    assert isinstance(ex, BlockFP8QLoRAMoeExperts) and not ex._weights_loaded
    assert ex._source_fqn == "model.layers.1.mlp.experts" and ex._source_quant_format == "block_fp8"
    with pytest.raises(ValueError, match="quant_group_size=128"):
        QLoRAMoeExperts.from_module(_Experts(2, 128, 128), quant_format="block_fp8", quant_group_size=16)
    with pytest.raises(TypeError):
        QLoRAMoeExperts.from_module(nn.Linear(4, 4), quant_format="block_fp8", quant_group_size=128)


def test_inject_then_load_from_a_checkpoint_directory(tmp_path):
    """inject -> maybe_load_prequantized_qlora on a block-fp8 checkpoint with separate q/k/v: the fused module's
    rows are the sources' rows in order."""
    import safetensors.torch

    from xorl_amd import quantize as Q

    h = 256
    model = _Model(h=h, fused=True)
    inject_qlora_into_model(model, r=4, lora_alpha=4, quant_format="block_fp8", target_modules=["qkv_proj", "o_proj"],
                            checkpoint_quant_format="block_fp8")
    tensors, want = {}, {}
    g = torch.Generator().manual_seed(1)
    for layer in range(2):
        rows = []
        for name, n in (("q_proj", h), ("k_proj", h // 2), ("v_proj", h // 2), ("o_proj", h)):
            b, s = Q.block_fp8_quantize_gkn(torch.randn(n, h, generator=g) * 0.05, 128)
            tensors[f"model.layers.{layer}.self_attn.{name}.weight"] = b
            tensors[f"model.layers.{layer}.self_attn.{name}.weight_scale_inv"] = s
            if name != "o_proj":
                rows.append(b.view(torch.uint8))
        want[layer] = torch.cat(rows, 0)
    safetensors.torch.save_file(tensors, os.path.join(tmp_path, "model.safetensors"))
    json.dump({"weight_map": {k: "model.safetensors" for k in tensors}},
              open(os.path.join(tmp_path, "model.safetensors.index.json"), "w"))
    json.dump({"quantization_config": {"quant_method": "fp8", "weight_block_size": [128, 128]}},
              open(os.path.join(tmp_path, "config.json"), "w"))
    assert detect_prequantized_block_fp8(str(tmp_path)) and not detect_prequantized_nvfp4(str(tmp_path))
    assert maybe_load_prequantized_qlora(model, str(tmp_path)) == 4
    for layer in range(2):
        qkv = model.model["layers"][layer].self_attn.qkv_proj
        got = qkv.packed_weight_f32.detach().contiguous().view(torch.uint8).reshape(2 * h, h)
        assert torch.equal(got.cpu(), want[layer])
    # and back out: the saved files hold every module's packed state and factors
    out = save_qlora_checkpoint(model, str(tmp_path / "saved"))
    qs = safetensors.torch.load_file(os.path.join(out, "quantized_weights.safetensors"))
    ls = safetensors.torch.load_file(os.path.join(out, "lora_weights.safetensors"))
    assert "model.layers.0.self_attn.qkv_proj.packed_weight_f32" in qs and "model.layers.1.self_attn.o_proj.weight_block_scales" in qs
    assert "model.layers.0.self_attn.o_proj.bias" in ls and ls["model.layers.1.self_attn.qkv_proj.lora_A"].shape == (4, h)


def test_detection_signals(tmp_path):
    d = tmp_path / "nv"
    d.mkdir()
    assert not detect_prequantized_nvfp4(str(d)) and not detect_prequantized_block_fp8(str(d)) and not detect_prequantized_nvfp4(None)
    json.dump({"quantization": {"quant_algo": "NVFP4"}}, open(d / "hf_quant_config.json", "w"))
    assert detect_prequantized_nvfp4(str(d))
    e = tmp_path / "idx"
    e.mkdir()
    json.dump({"weight_map": {"a.weight": "s", "a.weight_scale": "s", "a.weight_scale_2": "s"}},
              open(e / "model.safetensors.index.json", "w"))
    assert detect_prequantized_nvfp4(str(e)) and not detect_prequantized_block_fp8(str(e))
    f = tmp_path / "fp8"
    f.mkdir()
    json.dump({"weight_map": {"a.weight": "s", "a.weight_scale_inv": "s"}}, open(f / "model.safetensors.index.json", "w"))
    assert detect_prequantized_block_fp8(str(f)) and not detect_prequantized_nvfp4(str(f))


def test_deferred_quantization_of_a_materialised_weight():
    """A module created on the meta device receives its bf16 weight later; maybe_quantize_qlora packs and drops it."""
    with torch.device("meta"):
        lin = nn.Linear(128, 64, bias=False)
    m = NF4QLoRALinear.from_module(lin, r=4, lora_alpha=4)
    assert m.weight is not None and m.weight.device.type == "meta"
    m.weight = nn.Parameter(torch.randn(64, 128) * 0.05, requires_grad=False)
    holder = nn.ModuleList([m])
    assert maybe_quantize_qlora(holder) == 1 and m.weight is None
    assert maybe_quantize_qlora(holder) == 0
