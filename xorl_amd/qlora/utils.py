"""Model-level helpers of the QLoRA path on one GPU: put QLoRA modules into a model, fill them from a HF
safetensors checkpoint, merge + re-quantise all of them between optimizer steps, save them.

Counterparts of ``xorl.qlora.utils`` -- ``inject_qlora_into_model`` (qlora/utils.py:68-305),
``save_qlora_checkpoint`` (:308-343), ``maybe_quantize_qlora`` (:346-374), ``maybe_load_and_quantize_moe_qlora``
(:377-487), ``detect_prequantized_nvfp4`` / ``detect_prequantized_block_fp8`` (:545-576),
``maybe_load_prequantized_qlora`` (:747-922) and ``maybe_requant_qlora`` (:925-953), and of the merge
scheduling that calls the latter from the training loop (trainers/training_utils.py:308-372) -- without the multi-rank
fan-out: every module reads exactly the checkpoint keys it consumes, one module's shards at a time, so host
memory holds at most the shards of one module.
"""

from __future__ import annotations

import json
import math
import os
from typing import Collection, Dict, List, Optional, Tuple

import torch
import torch.nn as nn

from .linear import (BlockFP8QLoRALinear, LoraModule, NF4QLoRALinear, NvFP4QLoRALinear, QLoRALinear,
                     deregister_qlora_weights_from_fsdp)

# the name the reference's callers and tests import (qlora/utils.py:490-542)
_deregister_qlora_weights_from_fsdp = deregister_qlora_weights_from_fsdp
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
    weight_map = _read_weight_map(weights_path, "Pre-quantized loading")
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


def reset_lora_optimizer_states(model: nn.Module, optimizer: torch.optim.Optimizer) -> int:
    """Drop the optimizer's state (moments, step count) of every LoRA factor: after a merge the factors are
    re-initialised, so what the optimizer remembers of them is stale (trainers/training_utils.py:308-343).
    Returns the number of parameters whose state was dropped; other parameters keep theirs."""
    lora_ids = {id(p) for m in model.modules() if isinstance(m, LoraModule) for p in m.get_lora_parameters()}
    count = 0
    for group in optimizer.param_groups:
        for p in group["params"]:
            if id(p) in lora_ids and p in optimizer.state:
                del optimizer.state[p]
                count += 1
    return count


def maybe_merge_lora(model: nn.Module, enable_lora: bool, enable_qlora: bool, merge_interval: int, global_step: int,
                     optimizer: Optional[torch.optim.Optimizer] = None, reset_optimizer: bool = False) -> None:
    """Every ``merge_interval`` steps fold the factors into the base weights -- re-quantising for QLoRA modules --
    and optionally reset the factors' optimizer state (trainers/training_utils.py:346-372).  Off the interval,
    or with ``merge_interval <= 0``, nothing is touched."""
    if merge_interval <= 0 or global_step % merge_interval != 0:
        return
    if enable_qlora:
        maybe_requant_qlora(model)
    elif enable_lora:
        for m in model.modules():
            if isinstance(m, LoraModule) and not isinstance(m, (QLoRALinear, QLoRAMoeExperts)):
                m.merge_weights()
    if reset_optimizer and optimizer is not None:
        reset_lora_optimizer_states(model, optimizer)


# ---------------------------------------------------------------------------------------------------------
# putting QLoRA modules into a model
DEFAULT_TARGET_MODULES = ("qkv_proj", "o_proj", "gate_up_proj", "down_proj")
# a fused module of the model is assembled from these separate projections of the checkpoint
PREQUANT_MERGE_SOURCES = {"qkv_proj": ("q_proj", "k_proj", "v_proj"), "gate_up_proj": ("gate_proj", "up_proj")}
_EXPERT_PROJECTIONS = frozenset({"gate_proj", "up_proj", "down_proj"})
_FORMAT_GROUP = {"block_fp8": 128, "nvfp4": 16, "nf4": 64}
_NEVER_QUANTIZED = frozenset({"lm_head", "gate"})          # output head and MoE router


def _expert_weights(experts: nn.Module) -> Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]]:
    """(gate, up, down) [E, in, out] views of an experts container that keeps 3-D parameters, else None."""
    if isinstance(experts, QLoRAMoeExperts):
        return None
    down = getattr(experts, "down_proj", None)
    if not (isinstance(down, nn.Parameter) and down.dim() == 3):
        return None
    fused = getattr(experts, "gate_up_proj", None)
    if isinstance(fused, nn.Parameter) and fused.dim() == 3:
        half = fused.shape[2] // 2
        return fused[:, :, :half], fused[:, :, half:], down
    gate, up = getattr(experts, "gate_proj", None), getattr(experts, "up_proj", None)
    if isinstance(gate, nn.Parameter) and isinstance(up, nn.Parameter) and gate.dim() == 3:
        return gate, up, down
    return None


def inject_qlora_into_model(model: nn.Module, r: int = 16, lora_alpha: int = 16, quant_format: str = "nvfp4",
                            quant_group_size: int = 16, target_modules: Optional[List[str]] = None,
                            checkpoint_quant_format: Optional[str] = None, merge_qkv: bool = True,
                            exclude_modules: Optional[Collection[str]] = None, enable_aqn: bool = False,
                            aqn_alpha: float = 1.0) -> nn.Module:
    """Replace the targeted nn.Linear modules of `model` by QLoRA modules and, when expert projections are
    targeted, the 3-D expert containers of its MoE blocks by packed-bank expert modules.

    nvfp4 / block_fp8 modules are created empty and marked for loading from a pre-quantized checkpoint
    (`maybe_load_prequantized_qlora`, or the streaming buffers); nf4 modules quantize the weights they replace at
    once (or after those have been materialised, when the model is still on the meta device).  `merge_qkv` is
    accepted for signature parity: whether q/k/v are fused is a property of the model that is passed in."""
    if quant_format not in _FORMAT_GROUP:
        raise ValueError(f"Supported QLoRA formats: 'nvfp4', 'block_fp8', 'nf4'. Got quant_format={quant_format!r}")
    quant_group_size = _FORMAT_GROUP[quant_format]
    targets = list(DEFAULT_TARGET_MODULES if target_modules is None else target_modules)
    excluded = set(_NEVER_QUANTIZED) | set(exclude_modules or ())
    paths = [name for name, mod in model.named_modules()
             if isinstance(mod, nn.Linear) and not isinstance(mod, QLoRALinear)
             and name.rsplit(".", 1)[-1] in targets and name.rsplit(".", 1)[-1] not in excluded]
    expert_targets = [t for t in targets if t in _EXPERT_PROJECTIONS]
    if not paths and not expert_targets:
        names = [n.rsplit(".", 1)[-1] for n, _ in model.named_modules() if n][:20]
        raise ValueError(f"No nn.Linear modules found matching target_modules={targets}. Available: {names}...")

    for path in paths:
        parent_path, _, attr = path.rpartition(".")
        parent = model.get_submodule(parent_path) if parent_path else model
        old = getattr(parent, attr)
        if quant_format == "nf4":
            new = NF4QLoRALinear.from_module(old, r=r, lora_alpha=lora_alpha, enable_aqn=enable_aqn, aqn_alpha=aqn_alpha)
        else:
            cls = BlockFP8QLoRALinear if quant_format == "block_fp8" else NvFP4QLoRALinear
            new = cls(in_features=old.in_features, out_features=old.out_features, r=r, lora_alpha=lora_alpha,
                      bias=old.bias is not None, device=old.weight.device, enable_aqn=enable_aqn, aqn_alpha=aqn_alpha)
            new._is_prequantized = True
            new._source_quant_format = checkpoint_quant_format
            new._merge_sources = PREQUANT_MERGE_SOURCES.get(attr)
            # a fused module reads `<parent>.<source projection>.*`, a plain one `<its own path>.*`
            new._source_fqn = parent_path if new._merge_sources is not None else path
            new._qlora_expected_skip_keys = {"weight"}
        setattr(parent, attr, new)

    if not expert_targets:
        return model
    for name, block in list(model.named_modules()):
        if not (hasattr(block, "gate") and hasattr(block, "experts")):
            continue
        weights = _expert_weights(block.experts)
        if weights is None:
            continue
        new = QLoRAMoeExperts.from_module(block.experts, r=r, lora_alpha=lora_alpha, quant_format=quant_format,
                                          quant_group_size=quant_group_size, hybrid_shared=True,
                                          target_modules=expert_targets)
        fqn = name if name.endswith(".experts") else f"{name}.experts" if name else "experts"
        if quant_format == "nf4" and weights[0].device.type != "meta":
            with torch.no_grad():
                for proj, w in zip(("gate", "up", "down"), weights):
                    new._quantize_proj(proj, w.detach().float())
            new._weights_loaded = True
        else:
            new._source_fqn = fqn
            if quant_format != "nf4":
                new._source_quant_format = checkpoint_quant_format
        block.experts = new
    return model


def maybe_quantize_qlora(model: nn.Module) -> int:
    """Quantize the bf16 `weight` that deferred (meta-initialised) QLoRA modules received from a checkpoint
    and drop it; returns the number of modules quantized."""
    pending = [m for m in model.modules() if isinstance(m, QLoRALinear) and m.weight is not None]
    if not pending:
        return 0
    deregister_qlora_weights_from_fsdp(model, param_names=("weight",))
    for m in pending:
        m.quantize_weight()
    return len(pending)


def _read_weight_map(weights_path: str, what: str) -> dict:
    index = os.path.join(weights_path, SAFE_WEIGHTS_INDEX_NAME) if weights_path else None
    if index and not os.path.exists(index):
        try:
            from transformers.utils import cached_file

            index = cached_file(weights_path, SAFE_WEIGHTS_INDEX_NAME)
        except Exception:
            index = None
    if not index or not os.path.exists(index):
        raise RuntimeError(f"Could not load weight index from {weights_path}. {what} requires {SAFE_WEIGHTS_INDEX_NAME}.")
    with open(index) as f:
        return json.load(f).get("weight_map", {})


def maybe_load_and_quantize_moe_qlora(model: nn.Module, weights_path: str, load_mode: str = "grouped") -> int:
    """Fill the expert modules that have no banks yet from the bf16 (or pre-quantized) per-expert tensors of the
    checkpoint, quantizing on the device where the format has no checkpoint form (nf4); returns their number."""
    pending = [m for m in model.modules()
               if isinstance(m, QLoRAMoeExperts) and not m._weights_loaded and m._source_fqn is not None]
    if not pending:
        return 0
    weight_map = _read_weight_map(weights_path, "MoE expert loading")
    device = torch.device("cuda") if torch.cuda.is_available() else torch.device("cpu")
    for m in pending:
        cache = _load_selected_shards(prequantized_module_keys(m, weight_map), weight_map, weights_path)
        try:
            m.load_and_quantize_weights(weights_path, weight_map=weight_map, shard_cache=cache)
        finally:
            cache.clear()
        _materialize_lora(m, device)
    return len(pending)


def save_qlora_checkpoint(model: nn.Module, save_path: str) -> str:
    """`quantized_weights.safetensors` (packed bytes and scale buffers of every dense QLoRA module) and
    `lora_weights.safetensors` (their factors and biases) under `save_path`."""
    from safetensors.torch import save_file

    os.makedirs(save_path, exist_ok=True)
    quantized, lora = {}, {}
    for name, m in model.named_modules():
        if not isinstance(m, QLoRALinear):
            continue
        for key, t in m.get_quantized_state_dict().items():
            quantized[f"{name}.{key}"] = t.detach().cpu().clone()
        lora[f"{name}.lora_A"] = m.lora_A.detach().cpu().clone()
        lora[f"{name}.lora_B"] = m.lora_B.detach().cpu().clone()
        if m.bias is not None:
            lora[f"{name}.bias"] = m.bias.detach().cpu().clone()
    if quantized:
        save_file(quantized, os.path.join(save_path, "quantized_weights.safetensors"))
    if lora:
        save_file(lora, os.path.join(save_path, "lora_weights.safetensors"))
    return save_path


def _json(path: str) -> dict:
    try:
        with open(path) as f:
            return json.load(f)
    except (OSError, json.JSONDecodeError):
        return {}


def _index_suffixes(weights_path: str) -> set:
    keys = _json(os.path.join(weights_path, SAFE_WEIGHTS_INDEX_NAME)).get("weight_map", {})
    return {k.rsplit(".", 1)[-1] for k in keys}


def detect_prequantized_nvfp4(weights_path: Optional[str]) -> bool:
    """A local checkpoint directory in modelopt NVFP4 form: says so in `hf_quant_config.json` or in
    `config.json`'s quantization_config, or its index lists `weight_scale` tensors
    (checkpoint_handlers/buffers.py:147-203)."""
    if not weights_path or not os.path.isdir(weights_path):
        return False
    hq = _json(os.path.join(weights_path, "hf_quant_config.json"))
    if (hq.get("quantization", {}).get("quant_algo") or hq.get("quant_algo")) == "NVFP4":
        return True
    if _json(os.path.join(weights_path, "config.json")).get("quantization_config", {}).get("quant_algo") == "NVFP4":
        return True
    return "weight_scale" in _index_suffixes(weights_path)


def detect_prequantized_block_fp8(weights_path: Optional[str]) -> bool:
    """A local checkpoint directory in block-fp8 form: `quant_method == "fp8"` with 128 x 128 blocks in
    `config.json`, or an index with `weight_scale_inv` and no `weight_scale` tensors
    (checkpoint_handlers/buffers.py:206-250)."""
    if not weights_path or not os.path.isdir(weights_path):
        return False
    qc = _json(os.path.join(weights_path, "config.json")).get("quantization_config", {})
    if qc.get("quant_method") == "fp8" and qc.get("weight_block_size") == [128, 128]:
        return True
    suffixes = _index_suffixes(weights_path)
    return "weight_scale_inv" in suffixes and "weight_scale" not in suffixes
