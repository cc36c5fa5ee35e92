"""Model-level helpers of the QLoRA path on one GPU: fill every QLoRA module of a model from a
HF safetensors checkpoint, and merge + re-quantise all of them between optimizer steps.

Counterparts of ``xorl.qlora.utils.maybe_load_prequantized_qlora`` (qlora/utils.py:747-922) and
``maybe_requant_qlora`` (:925-953) without the multi-rank fan-out: every module reads exactly the
checkpoint keys it consumes, one module's shards at a time, so host memory holds at most the
shards of one module.
"""

from __future__ import annotations

import json
import math
import os
from typing import Dict, Tuple

import torch
import torch.nn as nn

from .linear import QLoRALinear, deregister_qlora_weights_from_fsdp
from .moe_experts import QLoRAMoeExperts

SAFE_WEIGHTS_INDEX_NAME = "model.safetensors.index.json"


def prequantized_module_keys(module: nn.Module, weight_map: dict) -> Tuple[str, ...]:
    """The checkpoint keys one deferred module consumes (qlora/utils.py:596-640)."""
    src = getattr(module, "_source_fqn", None)
    if not src:
        raise RuntimeError(f"{type(module).__name__} has no checkpoint source FQN")
    if isinstance(module, QLoRALinear):
        fmt = getattr(module, "_source_quant_format", None) or module.quant_format
        if fmt == "block_fp8":
            suffixes = ("weight", "weight_scale_inv")
        elif fmt == "nvfp4":
            suffixes = ("weight", "weight_scale", "weight_scale_2")
        else:
            raise RuntimeError(f"Unsupported pre-quantized QLoRA source format: {fmt!r}")
        merge = getattr(module, "_merge_sources", None)
        prefixes = (src,) if merge is None else tuple(f"{src}.{p}" for p in merge)
        keys = tuple(f"{p}.{s}" for p in prefixes for s in suffixes)
    elif isinstance(module, QLoRAMoeExperts):
        first = f"{src}.{module.expert_offset}.gate_proj"
        if f"{first}.weight_scale_inv" in weight_map:
            suffixes = ("weight", "weight_scale_inv")
        elif f"{first}.weight_scale" in weight_map:
            suffixes = ("weight", "weight_scale", "weight_scale_2")
        else:
            suffixes = ("weight",)          # bf16 experts, quantized on load
        keys = tuple(f"{src}.{e}.{p}.{s}" for p in ("gate_proj", "up_proj", "down_proj")
                     for e in range(module.expert_offset, module.expert_offset + module.num_local_experts)
                     for s in suffixes)
    else:
        raise TypeError(f"Unsupported deferred QLoRA module: {type(module).__name__}")
    missing = [k for k in keys if k not in weight_map]
    if missing:
        raise RuntimeError(f"{len(missing)} checkpoint key(s) of {src} are not in the index, e.g. {missing[0]}")
    return keys


def _load_selected_shards(keys, weight_map: dict, weights_path: str) -> Dict[str, Dict[str, torch.Tensor]]:
    """shard file -> {key: tensor} holding only the requested keys of each shard."""
    from safetensors import safe_open

    by_shard: Dict[str, list] = {}
    for k in keys:
        by_shard.setdefault(weight_map[k], []).append(k)
    cache = {}
    for shard, ks in by_shard.items():
        path = os.path.join(weights_path, shard)
        if not os.path.exists(path):
            from transformers.utils import cached_file

            path = cached_file(weights_path, shard)
        with safe_open(path, framework="pt", device="cpu") as f:
            cache[shard] = {k: f.get_tensor(k) for k in ks}
    return cache


def _materialize_lora(module: nn.Module, device: torch.device) -> None:
    """LoRA parameters still on the meta device get real storage: A kaiming-uniform, B zero."""
    for name, p in list(module.named_parameters(recurse=False)):
        if p.device.type != "meta":
            continue
        t = torch.zeros(p.shape, dtype=p.dtype, device=device)
        if name.endswith("_A") or name == "lora_A":
            for i in range(t.shape[0]) if t.dim() == 3 else (None,):
                nn.init.kaiming_uniform_(t if i is None else t[i], a=math.sqrt(5))
        setattr(module, name, nn.Parameter(t, requires_grad=p.requires_grad))


def maybe_load_prequantized_qlora(model: nn.Module, weights_path: str, load_mode: str = "all_ranks") -> int:
    """Fill every deferred QLoRALinear (`_is_prequantized`, not loaded inline) and every QLoRAMoeExperts that has
    not loaded its banks yet from the checkpoint directory `weights_path`; returns the number of modules filled."""
    index = os.path.join(weights_path, SAFE_WEIGHTS_INDEX_NAME)
    if not os.path.exists(index):
        try:
            from transformers.utils import cached_file

            index = cached_file(weights_path, SAFE_WEIGHTS_INDEX_NAME)
        except Exception:
            index = None
    if not index or not os.path.exists(index):
        raise RuntimeError(f"Could not load weight index from {weights_path}. "
                           "Pre-quantized loading requires model.safetensors.index.json.")
    with open(index) as f:
        weight_map = json.load(f).get("weight_map", {})
    device = torch.device("cuda") if torch.cuda.is_available() else torch.device("cpu")

    n_linear = 0
    for module in model.modules():
        if isinstance(module, QLoRALinear) and module._is_prequantized and not getattr(module, "_inline_loaded", False):
            cache = _load_selected_shards(prequantized_module_keys(module, weight_map), weight_map, weights_path)
            try:
                with torch.no_grad():
                    module.load_prequantized_weights(weight_map, cache, weights_path)
            finally:
                cache.clear()
            _materialize_lora(module, device)
            n_linear += 1
    n_moe = 0
    for module in model.modules():
        if isinstance(module, QLoRAMoeExperts) and not module._weights_loaded and module._source_fqn is not None:
            cache = _load_selected_shards(prequantized_module_keys(module, weight_map), weight_map, weights_path)
            try:
                module.load_and_quantize_weights(weights_path, weight_map=weight_map, shard_cache=cache)
            finally:
                cache.clear()
            _materialize_lora(module, device)
            n_moe += 1
    if n_linear + n_moe:
        deregister_qlora_weights_from_fsdp(model, param_names=("packed_weight_f32",))
    return n_linear + n_moe


def maybe_requant_qlora(model: nn.Module, ema_decay: float = 0.1) -> int:
    """Merge the LoRA update into the base weight of every QLoRA module and re-quantise it (between
    optimizer.step() and the next forward); returns the number of modules touched."""
    count = 0
    for module in model.modules():
        if isinstance(module, (QLoRALinear, QLoRAMoeExperts)):
            module.merge_weights(ema_decay=ema_decay)
            count += 1
    return count
