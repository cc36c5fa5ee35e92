"""Streaming ("inline") loading of pre-quantized checkpoints into the packed module state.

A checkpoint reader that walks a safetensors file key by key offers every (key, tensor) pair to these
buffers.  A buffer claims the keys that belong to a QLoRA module, holds them until the module's last
piece has arrived and then turns them into the module's packed state -- so a quantized weight is never
expanded to bf16 on the way in.

* ``QLoRAWeightBuffer(model)`` serves the dense modules.  Completed modules come back as
  ``(state-dict name, tensor)`` pairs for the reader's own parameter / buffer dispatch
  (``xorl.models.checkpoint_handlers.buffers._QLoRAWeightBufferBase``, buffers.py:617-776; packing rules
  ``NvFP4WeightBuffer._pack`` :827-865 and ``BlockFP8WeightBuffer._pack`` :878-901).
* ``QLoRAExpertBuffer(model, ep_rank, ep_size, num_experts)`` serves the expert banks.  A projection's bank
  is written into its module once every expert of the checkpoint has been seen
  (``_QLoRAExpertBufferBase``, buffers.py:925-1200).

The arithmetic of both lives in the modules (``_pack_prequantized`` / ``_install_prequantized_bank``) and
is shared with the deferred, module-at-a-time loader of ``xorl_amd.qlora.utils``.
"""

from __future__ import annotations

import math
import re
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn
from torch import Tensor

from .. import quantize as Q
from .linear import QLoRALinear
from .moe_experts import BlockFP8QLoRAMoeExperts, QLoRAMoeExperts

_SUFFIXES = {
    "nvfp4": ("weight", "weight_scale", "weight_scale_2"),
    "block_fp8": ("weight", "weight_scale_inv"),
}
_EXPERT_KEY = re.compile(r"^model\.layers\.(\d+)\.mlp\.experts\.(\d+)\.(gate|up|down)_proj\.(.+)$")
_LAYER = re.compile(r"layers\.(\d+)")

Pairs = List[Tuple[str, Tensor]]


def parse_expert_full_key(key: str) -> Optional[Tuple[int, int, str, str]]:
    """``model.layers.L.mlp.experts.E.{gate,up,down}_proj.<suffix>`` -> (L, E, proj, suffix), else None
    (buffers.py:103-112)."""
    m = _EXPERT_KEY.match(key)
    return (int(m.group(1)), int(m.group(2)), m.group(3), m.group(4)) if m else None


def _split_key(key: str) -> Tuple[str, str]:
    head, _, tail = key.rpartition(".")
    return head, tail


# ---------------------------------------------------------------------------------------------- dense
class _Pending:
    """Pieces of one dense module: one {suffix: tensor} mapping per source projection."""

    def __init__(self, module: QLoRALinear, n_sources: int, n_suffixes: int):
        self.module = module
        self.pieces: List[Dict[str, Tensor]] = [dict() for _ in range(n_sources)]
        self.missing = n_sources * n_suffixes
        self.state: Optional[dict] = None          # set once packed


class InlineLinearBuffer:
    """Collects the checkpoint tensors of the pre-quantized dense QLoRA modules of `model` whose checkpoint is in
    this buffer's format."""

    source_format = "nvfp4"

    def __init__(self, model: nn.Module):
        self._suffixes = _SUFFIXES[self.source_format]
        self._route: Dict[str, Tuple[str, int]] = {}          # checkpoint prefix -> (module fqn, source index)
        self._pending: Dict[str, _Pending] = {}
        for fqn, mod in model.named_modules():
            if not isinstance(mod, QLoRALinear) or not mod._is_prequantized:
                continue
            if (mod._source_quant_format or mod.quant_format) != self.source_format:
                continue                                   # that module's checkpoint is in another format
            prefixes = mod._prequant_sources()
            for i, prefix in enumerate(prefixes):
                self._route[prefix] = (fqn, i)
            self._pending[fqn] = _Pending(mod, len(prefixes), len(self._suffixes))

    def is_qlora_key(self, key: str) -> bool:
        prefix, suffix = _split_key(key)
        return prefix in self._route and suffix in self._suffixes

    def try_consume(self, key: str, tensor: Tensor) -> Optional[Pairs]:
        """None: not a key of a QLoRA module (the reader handles it).  []: taken, the module is still incomplete.
        Otherwise the module's packed state as (name, tensor) pairs."""
        if not self.is_qlora_key(key):
            return None
        prefix, suffix = _split_key(key)
        fqn, src = self._route[prefix]
        pend = self._pending[fqn]
        if suffix not in pend.pieces[src]:
            pend.missing -= 1
        pend.pieces[src][suffix] = tensor
        if pend.missing > 0:
            return []
        mod = pend.module
        source = _linear_class(self.source_format)
        # the packing rule is the SOURCE format's, whatever format the module itself stores
        state = source._pack_prequantized(mod, pend.pieces)
        if mod.quant_format != self.source_format:
            state = _convert_state(mod, self.source_format, state)
        pend.state = {"scale_dtypes": state["scale_dtypes"], "ema_amax": state.get("ema_amax")}
        pend.pieces = [dict() for _ in pend.pieces]
        out: Pairs = [(f"{fqn}.packed_weight_f32",
                       state["packed"].contiguous().view(torch.float32).reshape(mod.packed_weight_f32.shape))]
        for name in state["scale_dtypes"]:
            out.append((f"{fqn}.{name}", QLoRALinear._to_uint8(state[name])))
        return out

    def set_inline_metadata(self) -> None:
        """After the reader has dispatched every pair: record what the byte buffers hold.  Modules whose target
        format is block_fp8 stay marked as not inline-loaded, so the deferred loader fills them again from disk
        (buffers.py:726-731 does the same, to survive a mixed-precision cast of the fp32-viewed bytes)."""
        for pend in self._pending.values():
            if pend.state is None:
                continue
            mod = pend.module
            mod._scale_dtypes = dict(pend.state["scale_dtypes"])
            ema = pend.state["ema_amax"]
            mod._ema_amax = None if ema is None else ema.to(mod.packed_weight_f32.device)
            mod._aqn_step_cache = None
            mod._inline_loaded = mod.quant_format != "block_fp8"


class NvFP4WeightBuffer(InlineLinearBuffer):
    source_format = "nvfp4"


class BlockFP8WeightBuffer(InlineLinearBuffer):
    source_format = "block_fp8"


def _linear_class(fmt: str):
    from .linear import BlockFP8QLoRALinear, NvFP4QLoRALinear

    return {"nvfp4": NvFP4QLoRALinear, "block_fp8": BlockFP8QLoRALinear}[fmt]


def _convert_state(mod: QLoRALinear, source_format: str, state: dict) -> dict:
    """Checkpoint format != module format: decode with the source format's kernel and quantize again in the
    module's (buffers.py:752-815).  Runs on the GPU; the result comes back on the CPU like any packed state."""
    N, K = mod.out_features, mod.in_features
    dev = torch.device("cuda")
    packed = state["packed"].to(dev)
    if source_format == "block_fp8":
        w = Q.block_fp8_dequantize_gkn(packed.view(torch.float8_e4m3fn).reshape(N, K), state["weight_block_scales"].to(dev), 128)
    else:
        w = Q.nvfp4_dequantize(packed, state["weight_block_scales"].to(dev), state["weight_global_scale"].to(dev), N * K, 16)
        w = w.reshape(N, K)
    if mod.quant_format == "block_fp8":
        fp8_w, scales = Q.block_fp8_quantize_gkn(w.float(), mod.quant_group_size)
        return {"packed": QLoRALinear._to_uint8(fp8_w).cpu(), "weight_block_scales": scales.cpu(),
                "scale_dtypes": {"weight_block_scales": torch.float32}, "ema_amax": None}
    if mod.quant_format == "nvfp4":
        amax = w.float().abs().max().reshape(1)
        codes, bs, g = Q.nvfp4_quantize(w, mod.quant_group_size, global_amax=amax)
        return {"packed": QLoRALinear._to_uint8(codes).cpu(), "weight_block_scales": bs.float().cpu(),
                "weight_global_scale": g.float().cpu(),
                "scale_dtypes": {"weight_block_scales": torch.float32, "weight_global_scale": torch.float32},
                "ema_amax": amax.cpu()}
    raise ValueError(f"no conversion from a {source_format} checkpoint to {mod.quant_format!r} modules")


def QLoRAWeightBuffer(model: nn.Module) -> InlineLinearBuffer:
    """The buffer for the checkpoint format of `model`'s pre-quantized modules (buffers.py:904-919); a model
    without any gets a buffer that claims no key."""
    for mod in model.modules():
        if isinstance(mod, QLoRALinear) and mod._is_prequantized:
            fmt = mod._source_quant_format or mod.quant_format
            return BlockFP8WeightBuffer(model) if fmt == "block_fp8" else NvFP4WeightBuffer(model)
    return NvFP4WeightBuffer(model)


# ---------------------------------------------------------------------------------------------- experts
class InlineExpertBuffer:
    """Collects per-expert checkpoint tensors and installs a projection's bank when it is complete.

    Keys of experts outside this rank's range [expert_start, expert_end) are counted, not kept: a projection is
    complete when all `num_experts * len(suffixes)` keys of the checkpoint have passed by and every local expert
    has all of its pieces."""

    source_format = "nvfp4"

    def __init__(self, model: nn.Module, ep_rank: int, ep_size: int, num_experts: int):
        self._suffixes = _SUFFIXES[self.source_format]
        self._local = num_experts // ep_size
        self._start = ep_rank * self._local
        self._keys_per_proj = num_experts * len(self._suffixes)
        self._modules: Dict[int, QLoRAMoeExperts] = {}
        for fqn, mod in model.named_modules():
            if isinstance(mod, QLoRAMoeExperts) and not mod._weights_loaded and hasattr(mod, "_install_prequantized_bank"):
                m = _LAYER.search(fqn)
                if m:
                    self._modules[int(m.group(1))] = mod
        self._pieces: Dict[Tuple[int, str], List[Dict[str, Tensor]]] = {}
        self._seen: Dict[Tuple[int, str], int] = {}
        self._done: set = set()

    expert_start = property(lambda self: self._start)
    expert_end = property(lambda self: self._start + self._local)

    def has_modules(self) -> bool:
        return bool(self._modules)

    def _count(self, layer: int, proj: str) -> None:
        self._seen[(layer, proj)] = self._seen.get((layer, proj), 0) + 1

    def try_consume(self, key: str, tensor: Tensor) -> Optional[Pairs]:
        """None: not an expert key of a module served here.  Otherwise [] -- banks are written into the module
        directly, nothing is handed back.  Suffixes the format does not use (`input_scale`) are dropped."""
        parsed = parse_expert_full_key(key)
        if parsed is None or parsed[0] not in self._modules:
            return None
        layer, expert, proj, suffix = parsed
        if suffix not in self._suffixes:
            return []
        self._count(layer, proj)
        if self.expert_start <= expert < self.expert_end:
            slots = self._pieces.setdefault((layer, proj), [dict() for _ in range(self._local)])
            slots[expert - self._start][suffix] = tensor
        self._maybe_install(layer, proj)
        return []

    def count_skipped(self, key: str) -> Pairs:
        """A key the reader skipped without loading its tensor still counts towards completion."""
        parsed = parse_expert_full_key(key)
        if parsed is not None and parsed[0] in self._modules and parsed[3] in self._suffixes:
            self._count(parsed[0], parsed[2])
            self._maybe_install(parsed[0], parsed[2])
        return []

    def _maybe_install(self, layer: int, proj: str) -> None:
        lp = (layer, proj)
        if lp in self._done or self._seen.get(lp, 0) < self._keys_per_proj:
            return
        slots = self._pieces.get(lp)
        if slots is None or any(len(s) < len(self._suffixes) for s in slots):
            return
        mod = self._modules[layer]
        with torch.no_grad():
            mod._install_prequantized_bank(proj, self._pieces.pop(lp))
        self._done.add(lp)
        if all((layer, p) in self._done for p in ("gate", "up", "down")):
            mod._weights_loaded = True

    def get_pending(self) -> List[Tuple[int, str]]:
        """(layer, projection) pairs that received keys but are not installed."""
        return [(layer, p) for layer in self._modules for p in ("gate", "up", "down")
                if (layer, p) not in self._done and self._seen.get((layer, p), 0) > 0]

    def set_inline_metadata(self) -> None:
        """Give loaded modules whose LoRA factors are still on the meta device real ones: zeros for B, the
        kaiming-uniform initialisation per expert slice for A (buffers.py:1069-1103)."""
        for mod in self._modules.values():
            if not mod._weights_loaded:
                continue
            dev = mod._load_device()
            for name, p in list(mod.named_parameters()):
                if p.device.type != "meta":
                    continue
                real = nn.Parameter(torch.zeros(p.shape, dtype=p.dtype, device=dev), requires_grad=p.requires_grad)
                if name.endswith("_A"):
                    for i in range(real.shape[0]):
                        nn.init.kaiming_uniform_(real.data[i], a=math.sqrt(5))
                setattr(mod, name, real)


class NvFP4QLoRAExpertBuffer(InlineExpertBuffer):
    source_format = "nvfp4"


class BlockFP8QLoRAExpertBuffer(InlineExpertBuffer):
    source_format = "block_fp8"


def QLoRAExpertBuffer(model: nn.Module, ep_rank: int, ep_size: int, num_experts: int) -> Optional[InlineExpertBuffer]:
    """The expert buffer for `model`'s bank format, or None when it has no unloaded expert module
    (buffers.py:1200-1215)."""
    for mod in model.modules():
        if isinstance(mod, QLoRAMoeExperts) and not mod._weights_loaded and hasattr(mod, "_install_prequantized_bank"):
            cls = BlockFP8QLoRAExpertBuffer if isinstance(mod, BlockFP8QLoRAMoeExperts) else NvFP4QLoRAExpertBuffer
            buf = cls(model, ep_rank, ep_size, num_experts)
            return buf if buf.has_modules() else None
    return None
