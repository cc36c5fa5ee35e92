"""Host-side checks that need no GPU: the C ABI library loads and exports every
symbol include/xq.h declares; module construction, state names/dtypes/shapes and
error behaviour match the reference's QLoRA modules; nothing runs on CPU tensors."""

import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from xorl_amd import _C

    hdr = open(os.path.join(ROOT, "include", "xq.h")).read()
    declared = set(re.findall(r"\b(xq_[a-z0-9_]+)\s*\(", hdr))
    assert declared, "no declarations found"
    L = ctypes.CDLL(_C.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(L, name), f"{name} declared in xq.h but not exported"
    assert declared == set(_C.EXPORTS)
    assert b"gfx950" in _C.lib().xq_version()


def test_product_never_imports_the_oracle():
    for base, _, files in os.walk(os.path.join(ROOT, "xorl_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                src = open(os.path.join(base, f)).read()
                assert "oracle" not in src.replace("oracle's", ""), f"{f} mentions the oracle package"


def test_dense_module_state_matches_reference_contract():
    from xorl_amd.qlora import BlockFP8QLoRALinear, Int4QLoRALinear, NF4QLoRALinear, NvFP4QLoRALinear, QLoRALinear

    with pytest.raises(TypeError):
        QLoRALinear(8, 8)
    m = BlockFP8QLoRALinear(576, 384, r=16, lora_alpha=32)      # 576: partial edge tile of scales
    assert m.packed_weight_f32.dtype == torch.float32 and tuple(m.packed_weight_f32.shape) == (384, 144)
    assert not m.packed_weight_f32.requires_grad
    assert m.weight_block_scales.dtype == torch.uint8 and tuple(m.weight_block_scales.shape) == (3, 5 * 4)
    assert m.lora_A.dtype == torch.float32 and tuple(m.lora_A.shape) == (16, 576)
    assert tuple(m.lora_B.shape) == (384, 16) and torch.count_nonzero(m.lora_B) == 0
    assert m.weight is None and m.bias is None and m.scaling == 2.0
    assert m.quant_format == "block_fp8" and m.quant_group_size == 128
    assert m.adapter_gradient_producer_family == "module_managed" and m.fsdp_requires_full_precision
    assert set(m.get_quantized_state_dict()) == {"packed_weight_f32", "weight_block_scales"}
    assert set(m.get_lora_state_dict()) == {"lora_A", "lora_B"}
    n = NvFP4QLoRALinear(64, 32)
    assert tuple(n.packed_weight_f32.shape) == (32, 8) and tuple(n.weight_global_scale.shape) == (4,)
    assert tuple(n.weight_block_scales.shape) == (32, 16)
    i4 = Int4QLoRALinear(256, 32)
    assert tuple(i4.weight_scales.shape) == (32, 4) and i4._scale_dtypes["weight_scales"] == torch.bfloat16
    n4 = NF4QLoRALinear(256, 32)
    assert n4.quant_group_size == 64 and tuple(n4.packed_weight_f32.shape) == (32, 32)
    assert tuple(n4.weight_scales.shape) == (32, 16) and n4._scale_dtypes["weight_scales"] == torch.float32
    with pytest.raises(NotImplementedError):
        n4._load_prequantized(lambda k: None)
    with pytest.raises(ValueError):
        m.set_runtime_lora_config(17, 1)


def test_from_module_roundtrip_and_model_dtype_move():
    from xorl_amd.qlora import QLoRALinear

    lin = torch.nn.Linear(256, 128, bias=True)
    for fmt in ("block_fp8", "nvfp4", "int4", "nf4"):
        q = QLoRALinear.from_module(lin, r=8, lora_alpha=16, quant_format=fmt)
        assert q.quant_format == fmt and torch.equal(q.bias, lin.bias)
        packed = q.packed_weight_f32.detach().clone()
        q.to(torch.bfloat16)                              # must not touch packed bytes / fp32 masters
        assert q.packed_weight_f32.dtype == torch.float32
        assert torch.equal(q.packed_weight_f32.detach().view(torch.int32), packed.view(torch.int32))   # bytes, NaN-safe
        assert q.lora_A.dtype == torch.float32
        assert q._read_packed_weight_uint8().dtype == torch.uint8
        q.packed_weight_f32.data = q.packed_weight_f32.data.to(torch.bfloat16)
        with pytest.raises(RuntimeError, match="expected float32"):
            q._read_packed_weight_uint8()
    with pytest.raises(ValueError):
        QLoRALinear.from_module(lin, quant_format="mxfp4")


def test_from_quantized_and_delta_weight():
    from xorl_amd import quantize as Q
    from xorl_amd.qlora import QLoRALinear

    w = torch.randn(128, 256) * 0.02
    fp8, s = Q.block_fp8_quantize_gkn(w)
    q = QLoRALinear.from_quantized(fp8, weight_block_scales=s, in_features=256, out_features=128, r=4, lora_alpha=8,
                                   quant_format="block_fp8")
    assert q._is_prequantized and q._scale_dtypes["weight_block_scales"] == torch.float32
    assert torch.equal(q._read_packed_weight_uint8().reshape(128, 256), fp8.view(torch.uint8))
    with torch.no_grad():
        q.lora_B.normal_()
    d = q.get_delta_weight()
    assert torch.allclose(d, (q.lora_B @ q.lora_A) * 2.0)


def test_no_cpu_fallback():
    from xorl_amd import quantize as Q
    from xorl_amd.qlora import BlockFP8QLoRALinear

    m = BlockFP8QLoRALinear(128, 64)
    with pytest.raises((RuntimeError, NotImplementedError)):
        m(torch.zeros(2, 128, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError):
        Q.block_fp8_dequantize_gkn(torch.zeros(128, 128).to(torch.float8_e4m3fn), torch.ones(1, 1))


def test_moe_module_state_matches_reference_contract():
    from xorl_amd.qlora import BlockFP8QLoRAMoeExperts, NvFP4QLoRAMoeExperts, QLoRAMoeExperts

    with pytest.raises(TypeError):
        QLoRAMoeExperts(2, 2, 64, 64)
    m = BlockFP8QLoRAMoeExperts(4, 4, 128, 256, r=8, lora_alpha=16)
    shapes = {n: tuple(p.shape) for n, p in m.named_parameters()}
    assert shapes == {"gate_proj_lora_A": (1, 256, 8), "gate_proj_lora_B": (4, 8, 128),
                      "up_proj_lora_A": (1, 256, 8), "up_proj_lora_B": (4, 8, 128),
                      "down_proj_lora_A": (4, 128, 8), "down_proj_lora_B": (1, 8, 256)}
    assert m._skip_fsdp and m._qlora_expected_skip_keys == {"gate_proj", "up_proj", "down_proj"}
    assert m.gated and m.hidden_act == "silu" and m.hidden_dim == 256 and m.swiglu_limit == 0.0
    m.load_weights(torch.randn(4, 256, 128) * 0.02, torch.randn(4, 256, 128) * 0.02, torch.randn(4, 128, 256) * 0.02)
    assert m.gate_packed.dtype == torch.uint8 and tuple(m.gate_packed.shape) == (4, 256, 128)
    assert tuple(m.down_block_scales.shape) == (4, 1, 2 * 4)
    n = NvFP4QLoRAMoeExperts(4, 4, 128, 256, hybrid_shared=False, target_modules=["down_proj"])
    assert [k for k, _ in n.named_parameters()] == ["down_proj_lora_A", "down_proj_lora_B"]
    assert tuple(n.gate_proj_lora_A.shape) == (4, 256, 16) and not n.gate_proj_lora_A.requires_grad
    with pytest.raises(ValueError):
        BlockFP8QLoRAMoeExperts(4, 4, 128, 256, target_modules=["q_proj"])
    with pytest.raises(ValueError):
        BlockFP8QLoRAMoeExperts(2, 4, 128, 256)          # expert parallel shards are out of scope
