"""Host logic: expert banks filled from HF-style per-expert checkpoint tensors (no GPU).

The contracts are those of the reference's own loader test (tests/qlora/test_moe_load_experts.py:15-140):
the bank is the per-expert transpose of the checkpoint's bytes and scales, nvfp4's global scale is folded
into fp32 block scales (stored global = 1) and seeds the amax EMA with global * 6 * 448."""

import json
import os

import numpy as np
import pytest
import torch

from oracle import cdecode as C
from oracle import decode_np as NP
from xorl_amd import quantize as Q
from xorl_amd.qlora import BlockFP8QLoRAMoeExperts, NF4QLoRAMoeExperts, NvFP4QLoRAMoeExperts

HF = ("gate_proj", "up_proj", "down_proj")


def _nvfp4_tensors(E, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    codes = [torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=g) for _ in range(E)]
    bs = [torch.rand(N, K // 16, generator=g).to(torch.float8_e4m3fn) for _ in range(E)]
    gs = [torch.tensor(0.001 + torch.rand(1, generator=g).item() * 0.01) for _ in range(E)]
    return codes, bs, gs


def _fp8_tensors(E, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    w = [(torch.rand(N, K, generator=g) * 2 - 1).to(torch.float8_e4m3fn) for _ in range(E)]
    sc = [torch.rand(N // 128, K // 128, generator=g) for _ in range(E)]
    return w, sc


@pytest.mark.parametrize("E,I,H", [(4, 768, 2048), (8, 512, 1024), (1, 256, 512)])
def test_nvfp4_prequantized_load_is_a_transpose(E, I, H):
    codes, bs, gs = _nvfp4_tensors(E, I, H, seed=E)
    data = {}
    for hf in HF:
        for e in range(E):
            data[f"layer.{e}.{hf}.weight"] = codes[e]
            data[f"layer.{e}.{hf}.weight_scale"] = bs[e]
            data[f"layer.{e}.{hf}.weight_scale_2"] = gs[e]
    m = NvFP4QLoRAMoeExperts(E, E, I, H, r=4, lora_alpha=4)
    m._source_fqn = "layer"
    m._load_experts(lambda k: data[k], {})
    ref_packed = torch.stack([c.t().contiguous() for c in codes])
    ref_scales = torch.stack([(b.float() * g.float()).t().contiguous().view(torch.uint8) for b, g in zip(bs, gs)])
    for p in ("gate", "up", "down"):
        assert torch.equal(getattr(m, f"{p}_packed"), ref_packed), p
        assert torch.equal(getattr(m, f"{p}_block_scales"), ref_scales), p
        g1 = m._recover_tensor(getattr(m, f"{p}_global_scale"), torch.float32)
        assert torch.equal(g1, torch.ones_like(g1))
        for got, g in zip(m._ema_amax[p].tolist(), gs):
            assert abs(got - g.item() * 6.0 * 448.0) < 1e-5
        assert m._scale_dtypes[p] == {"weight_block_scales": torch.float32, "weight_global_scale": torch.float32}
    # the bank decodes to the transpose of what the checkpoint's own layout decodes to (oracle on both sides)
    e = E - 1
    hf_dec = NP.nvfp4_decode_flat(codes[e].numpy(), C.e4m3_scales_to_f32(bs[e].view(torch.uint8).numpy()) * np.float32(gs[e].item()),
                                  1.0, I, H)
    bank_sc = m.gate_block_scales[e].contiguous().view(torch.float32).numpy()
    gkn_dec = NP.nvfp4_decode_gkn(m.gate_packed[e].numpy(), bank_sc, 1.0, H, I)
    assert np.array_equal(gkn_dec, hf_dec.T)


def test_block_fp8_prequantized_load_is_a_transpose():
    for E, I, H in ((4, 768, 2048), (2, 256, 512)):
        w, sc = _fp8_tensors(E, I, H, seed=E)
        data = {}
        for hf in HF:
            for e in range(E):
                data[f"layer.{e}.{hf}.weight"] = w[e]
                data[f"layer.{e}.{hf}.weight_scale_inv"] = sc[e].to(torch.bfloat16) if e % 2 else sc[e]
        m = BlockFP8QLoRAMoeExperts(E, E, I, H, r=4, lora_alpha=4)
        m._source_fqn = "layer"
        m._load_experts(lambda k: data[k], {})
        ref_packed = torch.stack([x.t().contiguous().view(torch.uint8) for x in w])
        ref_scales = torch.stack([data[f"layer.{e}.gate_proj.weight_scale_inv"].float().t().contiguous().view(torch.uint8)
                                  for e in range(E)])
        for p in ("gate", "up", "down"):
            assert torch.equal(getattr(m, f"{p}_packed"), ref_packed), p
            assert torch.equal(getattr(m, f"{p}_block_scales"), ref_scales), p
            assert m._scale_dtypes[p] == {"weight_block_scales": torch.float32}
        e = 0
        hf_dec = NP.fp8_decode(w[e].view(torch.uint8).numpy(), sc[e].numpy(), I, H)[1]
        gkn_dec = NP.fp8_decode(m.gate_packed[e].numpy().reshape(H, I),
                                m.gate_block_scales[e].contiguous().view(torch.float32).numpy(), H, I)[1]
        assert np.array_equal(gkn_dec, hf_dec.T)


def test_bf16_checkpoints_are_quantized_on_load_and_safetensors_round_trip(tmp_path):
    import safetensors.torch

    E, I, H = 3, 128, 256
    g = torch.Generator().manual_seed(5)
    hf_w = {(e, hf): (torch.randn(*((H, I) if hf == "down_proj" else (I, H)), generator=g) * 0.05).to(torch.bfloat16)
            for e in range(E) for hf in HF}
    # two shard files + an index, as a HF checkpoint directory holds them
    shards = {"model-00001-of-00002.safetensors": {}, "model-00002-of-00002.safetensors": {}}
    weight_map = {}
    for (e, hf), t in hf_w.items():
        key = f"model.layers.0.mlp.experts.{e}.{hf}.weight"
        shard = "model-00001-of-00002.safetensors" if e < 2 else "model-00002-of-00002.safetensors"
        shards[shard][key] = t
        weight_map[key] = shard
    for name, tensors in shards.items():
        safetensors.torch.save_file(tensors, os.path.join(tmp_path, name))
    json.dump({"weight_map": weight_map}, open(os.path.join(tmp_path, "model.safetensors.index.json"), "w"))

    for cls in (NvFP4QLoRAMoeExperts, NF4QLoRAMoeExperts):
        m = cls(E, E, I, H, r=4, lora_alpha=4)
        m._source_fqn = "model.layers.0.mlp.experts"
        cache = {}
        m.load_and_quantize_weights(str(tmp_path), weight_map=weight_map, shard_cache=cache)
        assert m._weights_loaded and cache == {}                     # shards are dropped as soon as they are consumed
        for p, hf in (("gate", "gate_proj"), ("up", "up_proj"), ("down", "down_proj")):
            K, N = m._proj_dims(p)
            for e in range(E):
                w_gkn = hf_w[(e, hf)].t().contiguous()               # [in, out] = [K, N]
                if cls is NF4QLoRAMoeExperts:
                    pk, sc = Q.nf4_quantize_gkn(w_gkn.float(), 64)
                    assert torch.equal(getattr(m, f"{p}_packed")[e], pk)
                    assert torch.equal(getattr(m, f"{p}_scales")[e].contiguous().view(torch.float32), sc)
                else:
                    a = w_gkn.float().abs().max().reshape(1)
                    pk, bs, gs = Q.nvfp4_quantize_gkn(w_gkn, 16, global_amax=a)
                    assert torch.equal(getattr(m, f"{p}_packed")[e], pk)
                    assert torch.equal(getattr(m, f"{p}_block_scales")[e].contiguous().view(torch.float32), bs.float() * gs.float())
                    assert abs(m._ema_amax[p][e].item() - a.item()) < 1e-7
        m.load_and_quantize_weights("/nonexistent")                  # second call is a no-op
    # a key missing from the index is reported as the reference reports it
    m = BlockFP8QLoRAMoeExperts(E, E, I, H, r=4, lora_alpha=4)
    m._source_fqn = "model.layers.0.mlp.experts"
    with pytest.raises(RuntimeError, match="not found in checkpoint index"):
        m.load_and_quantize_weights(str(tmp_path), weight_map=weight_map)
    # no source name: nothing to do (module built from tensors instead)
    m2 = BlockFP8QLoRAMoeExperts(E, E, I, H, r=4, lora_alpha=4)
    m2.load_and_quantize_weights(str(tmp_path))
    assert not m2._weights_loaded


def test_model_level_prequantized_load_and_requant(tmp_path):
    """maybe_load_prequantized_qlora fills dense (single and merged q/k/v sources) and expert modules from a
    sharded checkpoint directory, reading only each module's keys; the dense state decodes to what the
    checkpoint's own tensors decode to."""
    import safetensors.torch

    from xorl_amd.qlora import BlockFP8QLoRALinear, NvFP4QLoRALinear
    from xorl_amd.qlora.utils import maybe_load_prequantized_qlora, prequantized_module_keys

    g = torch.Generator().manual_seed(11)
    K = 256
    tensors = {}
    # dense block_fp8 o_proj [256, 256]
    wo, so = _fp8_tensors(1, 256, K, seed=21)
    tensors["model.layers.0.self_attn.o_proj.weight"] = wo[0]
    tensors["model.layers.0.self_attn.o_proj.weight_scale_inv"] = so[0]
    # nvfp4 q/k/v merged into one module: rows 128 + 64 + 64
    parts = {"q_proj": 128, "k_proj": 64, "v_proj": 64}
    nv = {}
    for name, n in parts.items():
        codes, bs, gs = _nvfp4_tensors(1, n, K, seed=len(name) + n)
        nv[name] = (codes[0], bs[0], gs[0])
        tensors[f"model.layers.0.self_attn.{name}.weight"] = codes[0]
        tensors[f"model.layers.0.self_attn.{name}.weight_scale"] = bs[0]
        tensors[f"model.layers.0.self_attn.{name}.weight_scale_2"] = gs[0]
    # fp8 experts
    E, I, H = 2, 128, 256
    we, se = _fp8_tensors(E, I, H, seed=31)
    for e in range(E):
        for hf in HF:
            tensors[f"model.layers.0.mlp.experts.{e}.{hf}.weight"] = (we[e] if hf != "down_proj" else we[e].t()).contiguous().clone()
            tensors[f"model.layers.0.mlp.experts.{e}.{hf}.weight_scale_inv"] = (se[e] if hf != "down_proj" else se[e].t()).contiguous().clone()
    tensors["model.embed_tokens.weight"] = torch.zeros(4, 4)      # a key no module asks for
    keys = sorted(tensors)
    weight_map = {}
    for i, shard in enumerate(("a.safetensors", "b.safetensors")):
        sel = {k: tensors[k] for k in keys[i::2]}
        safetensors.torch.save_file(sel, os.path.join(tmp_path, shard))
        weight_map.update({k: shard for k in sel})
    json.dump({"weight_map": weight_map}, open(os.path.join(tmp_path, "model.safetensors.index.json"), "w"))

    class Layer(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.o = BlockFP8QLoRALinear(K, 256, r=4, lora_alpha=4)
            self.o._is_prequantized, self.o._source_fqn = True, "model.layers.0.self_attn.o_proj"
            self.qkv = NvFP4QLoRALinear(K, 256, r=4, lora_alpha=4)
            self.qkv._is_prequantized, self.qkv._source_fqn = True, "model.layers.0.self_attn"
            self.qkv._merge_sources = ("q_proj", "k_proj", "v_proj")
            self.experts = BlockFP8QLoRAMoeExperts(E, E, I, H, r=4, lora_alpha=4)
            self.experts._source_fqn = "model.layers.0.mlp.experts"

    model = Layer()
    assert len(prequantized_module_keys(model.qkv, weight_map)) == 9
    assert maybe_load_prequantized_qlora(model, str(tmp_path)) == 3
    assert maybe_load_prequantized_qlora(model, str(tmp_path)) == 2 and model.experts._weights_loaded   # dense reload, banks kept

    # dense fp8: same bytes and scales
    o_bytes = model.o.packed_weight_f32.detach().contiguous().view(torch.uint8).reshape(256, K)
    assert torch.equal(o_bytes, wo[0].view(torch.uint8))
    assert torch.equal(model.o.weight_block_scales.contiguous().view(torch.float32).reshape(2, 2), so[0])
    # merged nvfp4: each part decodes (global folded into fp32 block scales, stored global 1) to its own checkpoint decode
    packed = model.qkv.packed_weight_f32.detach().contiguous().view(torch.uint8).reshape(256, K // 2).numpy()
    sc = model.qkv.weight_block_scales.contiguous().view(torch.float32).reshape(256, K // 16).numpy()
    assert model.qkv.weight_global_scale.contiguous().view(torch.float32).item() == 1.0
    got = NP.nvfp4_decode_flat(packed, sc, 1.0, 256, K)
    row = 0
    for name, n in parts.items():
        codes, bs, gs = nv[name]
        s = (bs.float() * gs.float()).numpy()                         # fl(e4m3 * global), as the loader folds it
        want = NP.nvfp4_decode_flat(codes.numpy(), s, 1.0, n, K)
        assert np.array_equal(got[row:row + n], want), name
        row += n
    assert abs(model.qkv._ema_amax.item() - max(v[2].item() for v in nv.values()) * 6.0 * 448.0) < 1e-4
    # experts: the transpose contract
    assert torch.equal(model.experts.gate_packed[1], we[1].t().contiguous().view(torch.uint8))
    assert torch.equal(model.experts.down_packed[1], we[1].view(torch.uint8))
    # a module whose keys are missing from the index is reported with its name
    model.o._source_fqn = "model.layers.9.self_attn.o_proj"
    with pytest.raises(RuntimeError, match="not in the index"):
        maybe_load_prequantized_qlora(model, str(tmp_path))
    with pytest.raises(RuntimeError, match="model.safetensors.index.json"):
        maybe_load_prequantized_qlora(model, str(tmp_path / "nowhere"))


# ---------------------------------------------------------------------------------------------------------
# streaming ("inline") buffers: the same packed state as the module-at-a-time loader, whatever order the keys
# arrive in (the reference's contracts: checkpoint_handlers/buffers.py:617-776 dense, :925-1200 experts)
def _dense_model(K):
    from xorl_amd.qlora import BlockFP8QLoRALinear, NvFP4QLoRALinear

    class Layer(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.o_proj = BlockFP8QLoRALinear(K, 256, r=4, lora_alpha=4)
            self.o_proj._is_prequantized, self.o_proj._source_fqn = True, "model.layers.0.self_attn.o_proj"
            self.o_proj._source_quant_format = "block_fp8"
            self.qkv_proj = NvFP4QLoRALinear(K, 256, r=4, lora_alpha=4)
            self.qkv_proj._is_prequantized, self.qkv_proj._source_fqn = True, "model.layers.0.self_attn"
            self.qkv_proj._merge_sources = ("q_proj", "k_proj", "v_proj")
            self.qkv_proj._source_quant_format = "nvfp4"

    return Layer()


@pytest.mark.parametrize("order_seed", [0, 1, 2])
def test_inline_dense_buffers_match_the_deferred_loader(order_seed):
    from xorl_amd.qlora.inline_buffers import BlockFP8WeightBuffer, NvFP4WeightBuffer, QLoRAWeightBuffer

    K = 256
    tensors = {}
    wo, so = _fp8_tensors(1, 256, K, seed=21)
    tensors["model.layers.0.self_attn.o_proj.weight"] = wo[0]
    tensors["model.layers.0.self_attn.o_proj.weight_scale_inv"] = so[0]
    for name, n in {"q_proj": 128, "k_proj": 64, "v_proj": 64}.items():
        codes, bs, gs = _nvfp4_tensors(1, n, K, seed=len(name) + n)
        tensors[f"model.layers.0.self_attn.{name}.weight"] = codes[0]
        tensors[f"model.layers.0.self_attn.{name}.weight_scale"] = bs[0]
        tensors[f"model.layers.0.self_attn.{name}.weight_scale_2"] = gs[0]
        tensors[f"model.layers.0.self_attn.{name}.input_scale"] = torch.ones(1)      # not a piece of the format
    tensors["model.norm.weight"] = torch.ones(4)

    # expected: the module-at-a-time loader on a twin model
    twin = _dense_model(K)
    for mod in (twin.o_proj, twin.qkv_proj):
        mod._load_prequantized(lambda k: tensors[k])

    model = _dense_model(K)
    # the factory picks the format of the first pre-quantized module; each format gets its own buffer
    assert isinstance(QLoRAWeightBuffer(model), BlockFP8WeightBuffer)
    bufs = [BlockFP8WeightBuffer(model), NvFP4WeightBuffer(model)]
    keys = list(tensors)
    order = torch.randperm(len(keys), generator=torch.Generator().manual_seed(order_seed)).tolist()
    got, complete = {}, 0
    for i in order:
        key = keys[i]
        claimed = [b.try_consume(key, tensors[key]) for b in bufs if b.is_qlora_key(key)]
        if key.endswith("input_scale") or key == "model.norm.weight":
            assert claimed == [] and all(b.try_consume(key, tensors[key]) is None for b in bufs)
            continue
        assert len(claimed) == 1                      # exactly one buffer owns a quantized key
        if claimed[0]:
            complete += 1
            got.update(dict(claimed[0]))
    assert complete == 2
    assert set(got) == {"o_proj.packed_weight_f32", "o_proj.weight_block_scales", "qkv_proj.packed_weight_f32",
                        "qkv_proj.weight_block_scales", "qkv_proj.weight_global_scale"}
    sd = dict(twin.named_parameters()) | dict(twin.named_buffers())
    for name, t in got.items():
        want = sd[name]
        assert t.dtype == want.dtype and t.shape == want.shape, name
        assert torch.equal(t.contiguous().view(torch.uint8), want.detach().contiguous().view(torch.uint8)), name
    # a reader dispatches the pairs into the module, then the buffers record what the bytes mean
    with torch.no_grad():
        for name, t in got.items():
            mod, attr = name.split(".")
            tgt = getattr(getattr(model, mod), attr)
            if tgt.shape == t.shape:
                tgt.copy_(t)
            else:
                setattr(getattr(model, mod), attr, t)
    for b in bufs:
        b.set_inline_metadata()
    assert model.qkv_proj._inline_loaded and not model.o_proj._inline_loaded       # block_fp8 is filled again from disk
    assert model.qkv_proj._scale_dtypes == twin.qkv_proj._scale_dtypes
    assert torch.equal(model.qkv_proj._ema_amax, twin.qkv_proj._ema_amax) and model.o_proj._ema_amax is None


@pytest.mark.parametrize("fmt", ["block_fp8", "nvfp4"])
def test_inline_expert_buffer_fills_the_local_range(fmt):
    """Two ranks' worth of experts stream by in a shuffled order; rank 1 keeps experts [2, 4), counts the others
    (some offered as tensors, some reported as skipped) and ends with the bank the module-at-a-time loader builds."""
    from xorl_amd.qlora.inline_buffers import QLoRAExpertBuffer, parse_expert_full_key

    E, I, H = 4, 128, 256
    cls = BlockFP8QLoRAMoeExperts if fmt == "block_fp8" else NvFP4QLoRAMoeExperts
    tensors = {}
    for hf in HF:
        N, K = (H, I) if hf == "down_proj" else (I, H)
        if fmt == "block_fp8":
            w, sc = _fp8_tensors(E, N, K, seed=len(hf))
            for e in range(E):
                tensors[f"model.layers.3.mlp.experts.{e}.{hf}.weight"] = w[e]
                tensors[f"model.layers.3.mlp.experts.{e}.{hf}.weight_scale_inv"] = sc[e]
        else:
            codes, bs, gs = _nvfp4_tensors(E, N, K, seed=len(hf))
            for e in range(E):
                tensors[f"model.layers.3.mlp.experts.{e}.{hf}.weight"] = codes[e]
                tensors[f"model.layers.3.mlp.experts.{e}.{hf}.weight_scale"] = bs[e]
                tensors[f"model.layers.3.mlp.experts.{e}.{hf}.weight_scale_2"] = gs[e]
                tensors[f"model.layers.3.mlp.experts.{e}.{hf}.input_scale"] = torch.ones(1)
    assert parse_expert_full_key("model.layers.3.mlp.experts.2.up_proj.weight_scale") == (3, 2, "up", "weight_scale")
    assert parse_expert_full_key("model.layers.3.mlp.gate.weight") is None

    def make():
        class Model(torch.nn.Module):
            def __init__(self):
                super().__init__()
                self.layers = torch.nn.ModuleList([torch.nn.Identity() for _ in range(4)])
                m = cls(2, 2, I, H, r=4, lora_alpha=4)      # this rank's two experts
                m.expert_offset, m._source_fqn = 2, "model.layers.3.mlp.experts"
                self.layers[3] = m
        return Model()

    twin = make()
    twin.layers[3]._load_experts(lambda k: tensors[k], {})
    model = make()
    buf = QLoRAExpertBuffer(model, ep_rank=1, ep_size=2, num_experts=E)
    assert buf is not None and (buf.expert_start, buf.expert_end) == (2, 4)
    keys = list(tensors)
    order = torch.randperm(len(keys), generator=torch.Generator().manual_seed(5)).tolist()
    assert buf.try_consume("model.layers.0.mlp.experts.0.gate_proj.weight", torch.zeros(1)) is None   # no module there
    for n, i in enumerate(order):
        key = keys[i]
        expert = parse_expert_full_key(key)[1]
        if expert < 2 and n % 2:
            assert buf.count_skipped(key) == []                   # the reader never loaded this tensor
        else:
            assert buf.try_consume(key, tensors[key]) == []
        if n == len(order) // 2:
            assert buf.get_pending() and not model.layers[3]._weights_loaded
    assert buf.get_pending() == [] and model.layers[3]._weights_loaded
    got, want = model.layers[3], twin.layers[3]
    for p in ("gate", "up", "down"):
        assert torch.equal(getattr(got, f"{p}_packed"), getattr(want, f"{p}_packed")), p
        assert torch.equal(getattr(got, f"{p}_block_scales"), getattr(want, f"{p}_block_scales")), p
        assert got._scale_dtypes[p] == want._scale_dtypes[p]
        if fmt == "nvfp4":
            assert torch.equal(getattr(got, f"{p}_global_scale"), getattr(want, f"{p}_global_scale"))
            assert torch.equal(got._ema_amax[p], want._ema_amax[p])
    # a model whose expert modules are all loaded needs no buffer
    assert QLoRAExpertBuffer(model, 1, 2, E) is None
