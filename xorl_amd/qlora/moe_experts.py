"""QLoRA MoE experts on packed expert banks (drop-in for xorl/qlora/modules/moe_experts.py).

Keeps the reference module's constructor, buffer / parameter names and shapes
(`{gate,up,down}_packed` uint8 `[E, K(/2), N]`, `{...}_block_scales` uint8 views,
`{...}_global_scale`, `{gate,up,down}_proj_lora_{A,B}` fp32 in GKN form, the
hybrid-shared factor layout) and its helper methods.  forward() differs: the
banks are never dequantized; the grouped kernels decode weight tiles in place.
Only the local (single-GPU) path exists here: expert parallelism is out of scope.
"""

from __future__ import annotations

import math
from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn
from torch import Tensor

from .. import _C
from .. import quantize as Q
from ..functional import QuantWeight
from ..moe_functional import moe_experts_qlora_ep_compute, moe_experts_qlora_forward
from .linear import LoraModule


EXPERT_PROJECTION_ROLES = frozenset({"gate_proj", "up_proj", "down_proj"})


def compute_lora_scaling(lora_alpha: float, r: int, use_rslora: bool = False) -> float:
    return lora_alpha / math.sqrt(r) if use_rslora else lora_alpha / r


class QLoRAMoeExperts(LoraModule, nn.Module):
    """Base class; use BlockFP8QLoRAMoeExperts, NvFP4QLoRAMoeExperts or NF4QLoRAMoeExperts."""

    adapter_gradient_producer_family = "fused_managed"

    def __init__(self, num_local_experts: int, num_experts: int, intermediate_size: int, hidden_size: int,
                 r: int = 16, lora_alpha: int = 16, quant_format: str = "nvfp4", quant_group_size: int = 16,
                 act_fn: Optional[nn.Module] = None, hidden_act: Optional[str] = None, expert_offset: int = 0,
                 device: Optional[torch.device] = None, moe_implementation: str = "hip", hybrid_shared: bool = True,
                 use_rslora: bool = False, ep_dispatch: str = "alltoall", deepep_buffer_size_gb: float = 2.0,
                 deepep_num_sms: int = 20, deepep_async_combine: bool = False,
                 alltoall_combine_hidden_chunk_size: int = 0, target_modules: Optional[list] = None):
        if type(self) is QLoRAMoeExperts:
            raise TypeError("QLoRAMoeExperts is abstract. Use BlockFP8QLoRAMoeExperts or NvFP4QLoRAMoeExperts.")
        super().__init__()
        if num_local_experts != num_experts or expert_offset != 0:
            raise ValueError("this build holds all experts on one GPU (num_local_experts == num_experts, offset 0)")
        if r <= 0 or r > 64:
            raise ValueError(f"LoRA rank must be in [1, 64] for the fused kernels, got {r}")
        self.num_local_experts, self.num_experts = num_local_experts, num_experts
        self.intermediate_size, self.hidden_size = intermediate_size, hidden_size
        self.hidden_dim = hidden_size
        self.r, self.lora_alpha = r, lora_alpha
        self.active_r, self.active_lora_alpha = r, lora_alpha
        self.use_rslora = use_rslora
        self.scaling = compute_lora_scaling(lora_alpha, r, use_rslora)
        self.quant_format, self.quant_group_size = quant_format, quant_group_size
        self.act_fn = act_fn or nn.SiLU()
        if hidden_act is None:
            plain = act_fn is None or isinstance(act_fn, nn.SiLU) or type(act_fn).__name__ == "SiLUActivation"
            hidden_act = "silu" if plain else f"custom:{type(act_fn).__qualname__}"
        if hidden_act != "silu":
            raise ValueError(f"the fused expert path implements SiLU gating only, got {hidden_act!r}")
        self.hidden_act = hidden_act
        self.gated = True
        self.swiglu_limit = 0.0
        self.gate_up_bias = None
        self.down_bias = None
        self.expert_offset = expert_offset
        self.moe_implementation = moe_implementation
        self.hybrid_shared = hybrid_shared
        targets = tuple(("gate_proj", "up_proj", "down_proj") if target_modules is None else target_modules)
        if not targets or len(set(targets)) != len(targets) or set(targets) - EXPERT_PROJECTION_ROLES:
            raise ValueError("QLoRA expert target_modules must be a non-empty subset of "
                             f"{sorted(EXPERT_PROJECTION_ROLES)}; got {list(targets)!r}")
        self.target_modules = targets
        self.ep_dispatch = ep_dispatch
        self.deepep_buffer_size_gb, self.deepep_num_sms = deepep_buffer_size_gb, deepep_num_sms
        self.deepep_async_combine = deepep_async_combine
        self.alltoall_combine_hidden_chunk_size = alltoall_combine_hidden_chunk_size
        self._source_fqn: Optional[str] = None
        self._source_quant_format: Optional[str] = None
        self._weights_loaded = False
        self._ema_amax: Dict[str, Optional[Tensor]] = {"gate": None, "up": None, "down": None}

        # hybrid-shared layout: gate/up share A across experts, down shares B
        # (qlora/modules/moe_experts.py:205-238)
        shared = 1 if hybrid_shared else num_experts
        self._create_lora_params("gate_proj", shared, num_experts, r, hidden_size, intermediate_size, device)
        self._create_lora_params("up_proj", shared, num_experts, r, hidden_size, intermediate_size, device)
        self._create_lora_params("down_proj", num_experts, shared, r, intermediate_size, hidden_size, device)
        self._scale_dtypes: Dict[str, Dict[str, torch.dtype]] = {"gate": {}, "up": {}, "down": {}}
        self._skip_fsdp = True
        self._qlora_expected_skip_keys = {"gate_proj", "up_proj", "down_proj"}

    # ------------------------------------------------------------------ factory
    @classmethod
    def from_module(cls, module: nn.Module, r: int = 16, lora_alpha: int = 16, quant_format: str = "nvfp4",
                    quant_group_size: int = 16, num_local_experts: Optional[int] = None, expert_offset: int = 0,
                    hybrid_shared: bool = True, target_modules: Optional[list] = None, use_rslora: bool = False,
                    **kwargs) -> "QLoRAMoeExperts":
        """An empty packed-bank module shaped like `module`, an experts container whose weights are
        [num_experts, in, out] parameters (`gate_proj` / `up_proj` / `down_proj`, or a fused `gate_up_proj`);
        the banks are filled later by load_weights() or load_and_quantize_weights()
        (qlora/modules/moe_experts.py:354-427)."""
        gate = getattr(module, "gate_proj", None)
        if isinstance(gate, Tensor) and gate.dim() == 3:
            total, hidden, inter = gate.shape
        else:
            fused = getattr(module, "gate_up_proj", None)
            if not (isinstance(fused, Tensor) and fused.dim() == 3):
                raise TypeError(f"{type(module).__name__} holds no [num_experts, in, out] expert weights")
            gate = fused
            total, hidden, inter = fused.shape[0], fused.shape[1], fused.shape[2] // 2
        for attr, want in (("gated", True), ("gate_up_bias", None), ("down_bias", None)):
            have = getattr(module, attr, want)
            if have is not None and have != want:
                raise ValueError(f"expert adapters need gated SiLU experts without biases; "
                                 f"{type(module).__name__}.{attr} = {have!r}")
        # a gate-only SwiGLU clamp (lora/expert_adapter_contract.py:39-57: the DeepSeek-V4 program) is carried over: the routed
        # kernels clamp the gate pre-activation and mask its gradient (ops/moe/triton.py:127-141)
        limit = float(getattr(module, "swiglu_limit", 0.0) or 0.0)
        if limit < 0:
            raise ValueError(f"{type(module).__name__}.swiglu_limit = {limit!r} must not be negative")
        required = {"nvfp4": 16, "block_fp8": 128, "nf4": 64}
        if quant_format not in required:
            raise ValueError(f"Expert QLoRA formats: {sorted(required)}; got {quant_format!r}")
        if quant_group_size != required[quant_format]:
            raise ValueError(f"Expert {quant_format} QLoRA requires quant_group_size={required[quant_format]}; "
                             f"got {quant_group_size}")
        if cls is QLoRAMoeExperts:
            cls = {"block_fp8": BlockFP8QLoRAMoeExperts, "nf4": NF4QLoRAMoeExperts, "nvfp4": NvFP4QLoRAMoeExperts}[quant_format]
        new = cls(num_local_experts=total if num_local_experts is None else num_local_experts, num_experts=total,
                  intermediate_size=getattr(module, "intermediate_size", inter),
                  hidden_size=getattr(module, "hidden_dim", hidden), r=r, lora_alpha=lora_alpha,
                  act_fn=getattr(module, "act_fn", None), hidden_act=getattr(module, "hidden_act", "silu"),
                  expert_offset=expert_offset, device=gate.device, hybrid_shared=hybrid_shared,
                  target_modules=target_modules, use_rslora=use_rslora)
        new.swiglu_limit = limit
        return new

    # ------------------------------------------------------------------ LoRA params
    def _create_lora_params(self, name, A_experts, B_experts, r, in_features, out_features, device=None):
        A = torch.empty(A_experts, in_features, r, dtype=torch.float32, device=device)
        B = torch.empty(B_experts, r, out_features, dtype=torch.float32, device=device)
        if name in self.target_modules:
            setattr(self, f"{name}_lora_A", nn.Parameter(A))
            setattr(self, f"{name}_lora_B", nn.Parameter(B))
        else:   # untargeted projections carry frozen zero factors
            self.register_buffer(f"{name}_lora_A", torch.zeros_like(A), persistent=False)
            self.register_buffer(f"{name}_lora_B", torch.zeros_like(B), persistent=False)

    def reset_lora_parameters(self) -> None:
        for proj in self.target_modules:
            A, B = getattr(self, f"{proj}_lora_A"), getattr(self, f"{proj}_lora_B")
            for i in range(A.shape[0]):
                nn.init.kaiming_uniform_(A.data[i], a=math.sqrt(5))
            nn.init.zeros_(B.data)

    def set_runtime_lora_config(self, lora_rank: int, lora_alpha: int) -> None:
        if lora_rank <= 0 or lora_rank > self.r:
            raise ValueError(f"Active LoRA rank must be in [1, {self.r}], got {lora_rank}")
        self.active_r, self.active_lora_alpha = lora_rank, lora_alpha

    def _active_scaling(self) -> float:
        return compute_lora_scaling(self.active_lora_alpha, self.active_r, self.use_rslora)

    def _active_lora_views(self, proj_name: str) -> Tuple[Tensor, Tensor]:
        A = getattr(self, f"{proj_name}_lora_A")[..., : self.active_r].contiguous()
        B = getattr(self, f"{proj_name}_lora_B")[:, : self.active_r, ...].contiguous()
        return A, B

    def _compute_proj_delta(self, proj_name: str) -> Tensor:
        A, B = self._active_lora_views(proj_name)
        E = max(A.shape[0], B.shape[0])
        return torch.bmm(A.expand(E, -1, -1), B.expand(E, -1, -1)) * self._active_scaling()

    # ------------------------------------------------------------------ storage helpers
    @staticmethod
    def _to_uint8(t: Tensor) -> Tensor:
        t = t.contiguous()
        if t.dim() and t.stride(-1) != 1:      # a size-1 last dimension may keep a foreign stride
            t = t.clone(memory_format=torch.contiguous_format)
        return t if t.dtype == torch.uint8 else t.view(torch.uint8)

    def _recover_tensor(self, buf: Tensor, original_dtype: torch.dtype) -> Tensor:
        return buf if original_dtype == torch.uint8 else buf.contiguous().view(original_dtype)

    def _quantize_2d(self, w: Tensor, global_amax=None):
        raise NotImplementedError

    def _dequantize_2d(self, packed: Tensor, scales_dict: dict, K: int, N: int) -> Tensor:
        raise NotImplementedError

    def _quantize_proj(self, proj_name: str, w3d: Tensor, global_amax_per_expert: Optional[Tensor] = None) -> None:
        """Quantize [E, K, N] expert by expert and stack the buffers."""
        res = []
        for i in range(w3d.shape[0]):
            ga = global_amax_per_expert[i: i + 1] if global_amax_per_expert is not None else None
            res.append(self._quantize_2d(w3d[i], global_amax=ga))
        setattr(self, f"{proj_name}_packed", torch.stack([p for p, _ in res]))
        self._scale_dtypes[proj_name] = {}
        suffix = {"weight_block_scales": "block_scales", "weight_global_scale": "global_scale",
                  "weight_scales": "scales"}
        for key in res[0][1]:
            self._scale_dtypes[proj_name][key] = res[0][1][key][1]
            setattr(self, f"{proj_name}_{suffix[key]}", torch.stack([sd[key][0] for _, sd in res]))

    def _build_scales_dict(self, proj_name: str, expert_idx: int) -> dict:
        suffix = {"weight_block_scales": "block_scales", "weight_global_scale": "global_scale",
                  "weight_scales": "scales"}
        out = {}
        for key, dt in self._scale_dtypes[proj_name].items():
            buf = getattr(self, f"{proj_name}_{suffix[key]}", None)
            if buf is not None:
                out[key] = (buf[expert_idx], dt)
        return out

    def _proj_dims(self, proj_name: str) -> Tuple[int, int]:
        return ((self.intermediate_size, self.hidden_size) if proj_name == "down"
                else (self.hidden_size, self.intermediate_size))

    def load_weights(self, gate: Tensor, up: Tensor, down: Tensor) -> None:
        """Quantize full-precision GKN banks ([E, H, I], [E, H, I], [E, I, H]) into the packed buffers."""
        with torch.no_grad():
            for name, w in (("gate", gate), ("up", up), ("down", down)):
                self._quantize_proj(name, w.float())
        self._weights_loaded = True

    # ------------------------------------------------------------------ loading from a HF checkpoint
    _HF_PROJ = (("gate", "gate_proj"), ("up", "up_proj"), ("down", "down_proj"))

    def load_and_quantize_weights(self, weights_path: str, weight_map: Optional[dict] = None,
                                  shard_cache: Optional[dict] = None) -> None:
        """Fill the packed banks from the per-expert tensors `<_source_fqn>.<i>.<proj>.*` of a safetensors
        checkpoint (qlora/modules/moe_experts.py:514-546).  `weights_path` is a local directory (or a hub id
        resolvable by transformers' cache); `weight_map` is the index's key -> shard-file map; `shard_cache`
        lets several modules share loaded shards.  Each subclass reads its own checkpoint format."""
        if self._weights_loaded or self._source_fqn is None:
            return
        import os

        import safetensors.torch

        cache = shard_cache if shard_cache is not None else {}

        def _load_tensor(key: str) -> Tensor:
            if weight_map is not None:
                shard = weight_map.get(key)
                if shard is None:
                    raise RuntimeError(f"Key {key} not found in checkpoint index")
            else:
                shard = "model.safetensors"
            if shard not in cache:
                path = os.path.join(weights_path, shard)
                if not os.path.exists(path):
                    from transformers.utils import cached_file

                    path = cached_file(weights_path, shard)
                cache[shard] = safetensors.torch.load_file(path, device="cpu")
            tensors = cache[shard]
            if key not in tensors:
                raise RuntimeError(f"Key {key} not found in {shard}")
            return tensors[key]

        with torch.no_grad():
            self._load_experts(_load_tensor, cache)
        self._weights_loaded = True

    def _load_experts(self, _load_tensor, _shard_cache) -> None:
        raise NotImplementedError

    def _load_device(self) -> torch.device:
        """Where loaded banks go: the module's device, or the GPU for a module still on the meta device."""
        dev = self.gate_proj_lora_B.device
        if dev.type in ("meta",):
            dev = torch.device("cuda") if torch.cuda.is_available() else torch.device("cpu")
        return dev

    def _expert_range(self):
        return range(self.expert_offset, self.expert_offset + self.num_local_experts)

    def _bank(self, proj_name: str) -> QuantWeight:
        raise NotImplementedError

    @torch.compiler.disable
    def dequantize_all_experts(self, proj_name: str, K: int, N: int) -> Tensor:
        """[E, K, N] decoded bank in one launch (the reference loops over experts)."""
        raise NotImplementedError

    def dequantize_expert(self, proj_name: str, expert_idx: int, K: int, N: int) -> Tensor:
        packed = getattr(self, f"{proj_name}_packed")
        return self._dequantize_2d(packed[expert_idx], self._build_scales_dict(proj_name, expert_idx), K, N)

    @property
    def gate_proj(self) -> Tensor:
        return self.dequantize_all_experts("gate", self.hidden_size, self.intermediate_size)

    @property
    def up_proj(self) -> Tensor:
        return self.dequantize_all_experts("up", self.hidden_size, self.intermediate_size)

    @property
    def down_proj(self) -> Tensor:
        return self.dequantize_all_experts("down", self.intermediate_size, self.hidden_size)

    @property
    def gate_up_proj(self) -> Tensor:
        return torch.cat([self.gate_proj, self.up_proj], dim=2)

    # ------------------------------------------------------------------ forward
    def forward(self, hidden_states: Tensor, routing_weights: Tensor = None, selected_experts: Tensor = None,
                expert_idx: int = None) -> Tensor:
        """Routed call (hidden [T, H], routing_weights / selected_experts [T, top-k]) or, with `expert_idx`, the
        MLP of one expert on the rows passed (moe_experts.py:576-620, :738-786): `expert_idx` is a global index,
        an expert that lives on another rank returns zeros."""
        if self.moe_implementation == "eager" and expert_idx is None:
            raise ValueError("moe_implementation='eager' calls the experts one at a time: pass expert_idx")
        if expert_idx is not None:
            local = expert_idx - self.expert_offset
            if local < 0 or local >= self.num_local_experts:
                return torch.zeros_like(hidden_states[..., : self.hidden_size])
            rows = hidden_states.reshape(-1, hidden_states.shape[-1])
            cumsum = torch.zeros(self.num_local_experts, dtype=torch.int64, device=rows.device)
            cumsum[local:] = rows.shape[0]
            return self.compute_dispatched(rows, cumsum).reshape(*hidden_states.shape[:-1], self.hidden_size)
        if self.num_local_experts != self.num_experts:
            raise ValueError(
                f"the routed call needs every expert on this rank (num_local_experts={self.num_local_experts}, "
                f"num_experts={self.num_experts}); an expert-parallel caller dispatches rows and uses compute_dispatched()")
        gA, gB = self._active_lora_views("gate_proj")
        uA, uB = self._active_lora_views("up_proj")
        dA, dB = self._active_lora_views("down_proj")
        return moe_experts_qlora_forward(
            num_experts=self.num_local_experts, routing_weights=routing_weights, selected_experts=selected_experts,
            hidden_states=hidden_states, gate_proj=self._bank("gate"), up_proj=self._bank("up"),
            down_proj=self._bank("down"), gate_proj_lora_A=gA, gate_proj_lora_B=gB, up_proj_lora_A=uA,
            up_proj_lora_B=uB, down_proj_lora_A=dA, down_proj_lora_B=dB, scaling=self._active_scaling(),
            swiglu_limit=float(self.swiglu_limit or 0.0))

    def compute_dispatched(self, permute_tokens: Tensor, cumsum: Tensor, expert_scores: Tensor = None) -> Tensor:
        """The compute step of an expert-parallel forward (moe_experts.py:652-698): rows already grouped by local
        expert (`cumsum` inclusive per local expert) -> their MLP outputs in the same order; `expert_scores` [R],
        when given, multiply the output rows afterwards, as the reference does between compute and combine."""
        gA, gB = self._active_lora_views("gate_proj")
        uA, uB = self._active_lora_views("up_proj")
        dA, dB = self._active_lora_views("down_proj")
        out = moe_experts_qlora_ep_compute(permute_tokens, cumsum, self._bank("gate"), self._bank("up"),
                                           self._bank("down"), gA, gB, uA, uB, dA, dB, self._active_scaling(),
                                           float(self.swiglu_limit or 0.0))
        if expert_scores is not None:
            out = out * expert_scores.unsqueeze(1).to(out.dtype)
        return out

    def merge_weights(self, ema_decay: float = 0.1, experts_per_step: int = 16) -> None:
        """W' = Q(deq(W) + delta.to(deq dtype)), then fresh LoRA factors (moe_experts.py:987-1008, :1134-1146,
        :1249-1261).  The sum is formed in the dtype the bank decodes to, as the reference does: bf16 for nvfp4 and
        nf4 (a bf16 add of two bf16 tensors), fp32 for block_fp8.  The update is added to the decoded bank in place,
        `experts_per_step` experts at a time, so the peak is the decoded bank plus one step's update."""
        with torch.no_grad():
            for name in ("gate", "up", "down"):
                K, N = self._proj_dims(name)
                w = self.dequantize_all_experts(name, K, N)
                A, B = self._active_lora_views(f"{name}_proj")
                E = w.shape[0]
                A, B = A.expand(E, -1, -1), B.expand(E, -1, -1)
                for e0 in range(0, E, experts_per_step):
                    e1 = min(E, e0 + experts_per_step)
                    delta = torch.bmm(A[e0:e1], B[e0:e1]) * self._active_scaling()
                    w[e0:e1] += delta.to(w.dtype)
                self._requantize_proj(name, w, ema_decay)
        self.reset_lora_parameters()

    def _requantize_proj(self, name: str, merged: Tensor, ema_decay: float) -> None:
        self._quantize_proj(name, merged)

    def extra_repr(self) -> str:
        return (f"num_local_experts={self.num_local_experts}, num_experts={self.num_experts}, "
                f"expert_offset={self.expert_offset}, intermediate_size={self.intermediate_size}, "
                f"hidden_size={self.hidden_size}, r={self.active_r}, max_r={self.r}, "
                f"quant_format={self.quant_format}, moe_implementation={self.moe_implementation}, "
                f"hybrid_shared={self.hybrid_shared}, target_modules={list(self.target_modules)}")


class BlockFP8QLoRAMoeExperts(QLoRAMoeExperts):
    """e4m3 banks with fp32 128x128 block scales; buffers {gate,up,down}_{packed,block_scales}."""

    def __init__(self, num_local_experts, num_experts, intermediate_size, hidden_size, r=16, lora_alpha=16, **kw):
        kw.pop("quant_format", None)
        kw.pop("quant_group_size", None)
        super().__init__(num_local_experts, num_experts, intermediate_size, hidden_size, r=r, lora_alpha=lora_alpha,
                         quant_format="block_fp8", quant_group_size=128, **kw)
        for p in ("gate", "up", "down"):
            self.register_buffer(f"{p}_packed", None)
            self.register_buffer(f"{p}_block_scales", None)
        self.reset_lora_parameters()

    def _quantize_2d(self, w: Tensor, global_amax=None):
        fp8, scales = Q.block_fp8_quantize_gkn(w.float().contiguous(), 128)
        return self._to_uint8(fp8), {"weight_block_scales": (self._to_uint8(scales), scales.dtype)}

    def _dequantize_2d(self, packed: Tensor, scales_dict: dict, K: int, N: int) -> Tensor:
        scales = self._recover_tensor(*scales_dict["weight_block_scales"])
        return Q.block_fp8_dequantize_gkn(packed.view(torch.float8_e4m3fn).reshape(K, N), scales, 128)

    _prequant_suffixes = ("weight", "weight_scale_inv")

    def _load_experts(self, _load_tensor, _shard_cache) -> None:
        """Pre-quantized block-fp8 experts (moe_experts.py:1074-1119): one projection at a time."""
        for proj, hf in self._HF_PROJ:
            pieces = [{sfx: _load_tensor(f"{self._source_fqn}.{i}.{hf}.{sfx}") for sfx in self._prequant_suffixes}
                      for i in self._expert_range()]
            self._install_prequantized_bank(proj, pieces)
            _shard_cache.clear()

    def _install_prequantized_bank(self, proj: str, pieces) -> None:
        """`pieces[i]`: local expert i's checkpoint tensors, `weight` [N, K] e4m3 and `weight_scale_inv`
        [N/128, K/128].  Bank: bytes [E, K, N] and fp32 scales [E, K/128, N/128] -- a pure transpose of bytes and
        scales, done once per projection on the device after one bulk copy."""
        dev = self._load_device()
        bank = torch.stack([p["weight"].view(torch.uint8) for p in pieces]).to(dev).transpose(1, 2).contiguous()
        scales = torch.stack([p["weight_scale_inv"].float() for p in pieces]).to(dev).transpose(1, 2).contiguous()
        setattr(self, f"{proj}_packed", self._to_uint8(bank))
        setattr(self, f"{proj}_block_scales", self._to_uint8(scales))
        self._scale_dtypes[proj] = {"weight_block_scales": torch.float32}

    def _bank(self, proj_name: str) -> QuantWeight:
        K, N = self._proj_dims(proj_name)
        return QuantWeight("block_fp8", _C.XQ_LAYOUT_GKN, getattr(self, f"{proj_name}_packed"),
                           getattr(self, f"{proj_name}_block_scales"), torch.float32, K, N, 128,
                           num_experts=self.num_local_experts)

    def merge_weights(self, ema_decay: float = 0.1, experts_per_step: int = 16) -> None:
        """Each expert's [K, N] slice is decoded, updated and re-encoded with fresh 128x128 block scales by the dense
        fused merge pass, in place in the bank (moe_experts.py:1134-1146): an expert's slice is a flat block-fp8
        matrix of K rows, and its update A_e [K, r] @ B_e [r, N] is that pass's (lora_B @ lora_A) with the factors'
        roles exchanged.  No decoded bank is ever held.  Ranks beyond the fused pass take the generic path."""
        from ..functional import MAX_FUSED_RANK, merge_requant_fp8

        packed0 = getattr(self, "gate_packed")
        if self.active_r > MAX_FUSED_RANK or packed0 is None or not packed0.is_cuda:
            return super().merge_weights(ema_decay, experts_per_step)
        with torch.no_grad():
            s = self._active_scaling()
            for name in ("gate", "up", "down"):
                K, N = self._proj_dims(name)
                packed = getattr(self, f"{name}_packed")
                scales = getattr(self, f"{name}_block_scales")
                A, B = self._active_lora_views(f"{name}_proj")       # [E|1, K, r], [E|1, r, N]
                for e in range(self.num_local_experts):
                    qw = QuantWeight("block_fp8", _C.XQ_LAYOUT_FLAT, packed[e], scales[e], torch.float32, K, N, 128)
                    merge_requant_fp8(qw, B[e if B.shape[0] > 1 else 0], A[e if A.shape[0] > 1 else 0],
                                      self.active_r, s, packed_out=packed[e], scales_out=scales[e])
        self.reset_lora_parameters()

    @torch.compiler.disable
    def dequantize_all_experts(self, proj_name: str, K: int, N: int) -> Tensor:
        import ctypes

        w = self._bank(proj_name).c()
        out = torch.empty(self.num_local_experts, K, N, dtype=torch.float32, device=getattr(self, f"{proj_name}_packed").device)
        _C.check(_C.lib().xq_decode(ctypes.byref(w), out.data_ptr(), _C.XQ_DT_F32, _C.stream_ptr(out.device)))
        return out


class NvFP4QLoRAMoeExperts(QLoRAMoeExperts):
    """e2m1 banks, per-16 block scales along K, fp32 global scale per expert;
    buffers {gate,up,down}_{packed,block_scales,global_scale}."""

    def __init__(self, num_local_experts, num_experts, intermediate_size, hidden_size, r=16, lora_alpha=16, **kw):
        kw.pop("quant_format", None)
        kw.pop("quant_group_size", None)
        super().__init__(num_local_experts, num_experts, intermediate_size, hidden_size, r=r, lora_alpha=lora_alpha,
                         quant_format="nvfp4", quant_group_size=16, **kw)
        for p in ("gate", "up", "down"):
            self.register_buffer(f"{p}_packed", None)
            self.register_buffer(f"{p}_block_scales", None)
            self.register_buffer(f"{p}_global_scale", None)
        self.reset_lora_parameters()

    def _quantize_2d(self, w: Tensor, global_amax=None):
        packed, bs, g = Q.nvfp4_quantize_gkn(w, 16, global_amax=global_amax)
        return self._to_uint8(packed), {"weight_block_scales": (self._to_uint8(bs), bs.dtype),
                                        "weight_global_scale": (self._to_uint8(g), g.dtype)}

    def _dequantize_2d(self, packed: Tensor, scales_dict: dict, K: int, N: int) -> Tensor:
        bs = self._recover_tensor(*scales_dict["weight_block_scales"])
        g = self._recover_tensor(*scales_dict["weight_global_scale"])
        return Q.nvfp4_dequantize_gkn(packed, bs, g, K, N, 16)

    _prequant_suffixes = ("weight", "weight_scale", "weight_scale_2")

    def _load_experts(self, _load_tensor, _shard_cache) -> None:
        """nvfp4 experts from a modelopt checkpoint (`weight` [N, K/2] u8, `weight_scale` [N, K/16] e4m3,
        `weight_scale_2` fp32 scalar) or, when the first expert has no `weight_scale`, from a bf16 checkpoint
        quantized here (moe_experts.py:869-971).  Either way the global scale is folded into fp32 block scales
        (stored global = 1) and the per-expert amax seeds the EMA used by re-quantisation."""
        dev = self._load_device()
        E = self.num_local_experts
        try:
            _load_tensor(f"{self._source_fqn}.{self.expert_offset}.gate_proj.weight_scale")
            prequantized = True
        except RuntimeError:
            prequantized = False
        for proj, hf in self._HF_PROJ:
            if prequantized:
                pieces = [{sfx: _load_tensor(f"{self._source_fqn}.{i}.{hf}.{sfx}") for sfx in self._prequant_suffixes}
                          for i in self._expert_range()]
                self._install_prequantized_bank(proj, pieces)
                _shard_cache.clear()
                continue
            amax, codes, sc = [], [], []
            for i in self._expert_range():
                w = _load_tensor(f"{self._source_fqn}.{i}.{hf}.weight").to(device=dev, dtype=torch.bfloat16).t().contiguous()
                a = w.float().abs().max().reshape(1)
                amax.append(a.item())
                packed, block_scales, global_scale = Q.nvfp4_quantize_gkn(w, self.quant_group_size, global_amax=a)
                codes.append(self._to_uint8(packed))
                sc.append((block_scales.float() * global_scale.float()).contiguous())
                _shard_cache.clear()
            self._set_folded_bank(proj, torch.stack(codes), torch.stack(sc), amax)

    def _install_prequantized_bank(self, proj: str, pieces) -> None:
        """`pieces[i]`: local expert i's modelopt tensors.  Codes and block scales are transposed to K-major on the
        device after one bulk copy: byte (k2, n) of the bank holds the K pair of column n."""
        dev = self._load_device()
        gs = [p["weight_scale_2"].float().item() for p in pieces]
        g_dev = torch.tensor(gs, dtype=torch.float32, device=dev)
        bs = torch.stack([p["weight_scale"].view(torch.uint8) for p in pieces]).to(dev)
        folded = bs.view(torch.float8_e4m3fn).float() * g_dev[:, None, None]
        bank = torch.stack([p["weight"] for p in pieces]).to(dev).transpose(1, 2).contiguous()      # [E, K/2, N]
        self._set_folded_bank(proj, bank, folded.transpose(1, 2).contiguous(),                     # [E, K/16, N] fp32
                              [g * Q.FP4_E2M1_MAX * Q.FP8_E4M3_MAX for g in gs])

    def _set_folded_bank(self, proj: str, bank: Tensor, scales: Tensor, amax) -> None:
        dev = bank.device
        setattr(self, f"{proj}_packed", self._to_uint8(bank))
        setattr(self, f"{proj}_block_scales", self._to_uint8(scales))
        setattr(self, f"{proj}_global_scale",
                self._to_uint8(torch.ones(self.num_local_experts, 1, dtype=torch.float32, device=dev)))
        self._scale_dtypes[proj] = {"weight_block_scales": torch.float32, "weight_global_scale": torch.float32}
        self._ema_amax[proj] = torch.tensor(amax, dtype=torch.float32, device=dev)

    def _bank(self, proj_name: str) -> QuantWeight:
        K, N = self._proj_dims(proj_name)
        sd = self._scale_dtypes[proj_name]
        g = self._recover_tensor(getattr(self, f"{proj_name}_global_scale"), sd["weight_global_scale"])
        return QuantWeight("nvfp4", _C.XQ_LAYOUT_GKN, getattr(self, f"{proj_name}_packed"),
                           getattr(self, f"{proj_name}_block_scales"), sd["weight_block_scales"], K, N, 16,
                           global_scale=g.float().reshape(-1).contiguous(), num_experts=self.num_local_experts)

    @torch.compiler.disable
    def dequantize_all_experts(self, proj_name: str, K: int, N: int) -> Tensor:
        import ctypes

        w = self._bank(proj_name).c()
        out = torch.empty(self.num_local_experts, K, N, dtype=torch.bfloat16, device=getattr(self, f"{proj_name}_packed").device)
        _C.check(_C.lib().xq_decode(ctypes.byref(w), out.data_ptr(), _C.XQ_DT_BF16, _C.stream_ptr(out.device)))
        return out

    def _requantize_proj(self, name: str, merged: Tensor, ema_decay: float) -> None:
        fresh = merged.float().abs().amax(dim=(1, 2))
        if self._ema_amax[name] is not None:
            self._ema_amax[name].lerp_(fresh.to(self._ema_amax[name].device), ema_decay)
        else:
            self._ema_amax[name] = fresh
        self._quantize_proj(name, merged, global_amax_per_expert=self._ema_amax[name])


class NF4QLoRAMoeExperts(QLoRAMoeExperts):
    """NormalFloat4 banks, one fp32 absmax per 64 elements along K; buffers
    {gate,up,down}_{packed,scales} (qlora/modules/moe_experts.py:1149-1260)."""

    def __init__(self, num_local_experts, num_experts, intermediate_size, hidden_size, r=16, lora_alpha=16, **kw):
        kw.pop("quant_format", None)
        kw.pop("quant_group_size", None)
        super().__init__(num_local_experts, num_experts, intermediate_size, hidden_size, r=r, lora_alpha=lora_alpha,
                         quant_format="nf4", quant_group_size=64, **kw)
        for p in ("gate", "up", "down"):
            self.register_buffer(f"{p}_packed", None)
            self.register_buffer(f"{p}_scales", None)
        self.reset_lora_parameters()

    def _quantize_2d(self, w: Tensor, global_amax=None):
        packed, scales = Q.nf4_quantize_gkn(w, self.quant_group_size)
        return self._to_uint8(packed), {"weight_scales": (self._to_uint8(scales), scales.dtype)}

    def _dequantize_2d(self, packed: Tensor, scales_dict: dict, K: int, N: int) -> Tensor:
        scales = self._recover_tensor(*scales_dict["weight_scales"])
        return Q.nf4_dequantize_gkn(packed, scales, K, N, self.quant_group_size)

    def _load_experts(self, _load_tensor, _shard_cache) -> None:
        """bf16 experts `[out, in]` -> transposed to `[in, out]` and quantized to NF4 along K
        (moe_experts.py:1213-1236); there is no pre-quantized NF4 checkpoint format."""
        dev = self._load_device()
        for proj, hf in self._HF_PROJ:
            w = [_load_tensor(f"{self._source_fqn}.{i}.{hf}.weight").t().contiguous().float() for i in self._expert_range()]
            self._quantize_proj(proj, torch.stack(w).to(dev))
            _shard_cache.clear()

    def _bank(self, proj_name: str) -> QuantWeight:
        K, N = self._proj_dims(proj_name)
        return QuantWeight("nf4", _C.XQ_LAYOUT_GKN, getattr(self, f"{proj_name}_packed"),
                           getattr(self, f"{proj_name}_scales"), self._scale_dtypes[proj_name]["weight_scales"],
                           K, N, self.quant_group_size, num_experts=self.num_local_experts)

    @torch.compiler.disable
    def dequantize_all_experts(self, proj_name: str, K: int, N: int) -> Tensor:
        import ctypes

        w = self._bank(proj_name).c()
        out = torch.empty(self.num_local_experts, K, N, dtype=torch.bfloat16, device=getattr(self, f"{proj_name}_packed").device)
        _C.check(_C.lib().xq_decode(ctypes.byref(w), out.data_ptr(), _C.XQ_DT_BF16, _C.stream_ptr(out.device)))
        return out
