"""QLoRA linear modules: quantized frozen base weight + trainable LoRA, on HIP kernels.

These classes keep the constructor signatures, parameter / buffer names,
shapes, dtypes and helper methods of the reference modules so that trainer
code, checkpoint code and FSDP2 wrapping written against the reference keep
working:

  QLoRALinear              xorl/qlora/modules/linear.py:29-412
  BlockFP8QLoRALinear      xorl/qlora/modules/block_fp8_linear.py
  NvFP4QLoRALinear         xorl/qlora/modules/nvfp4_linear.py
  Int4QLoRALinear          no counterpart class in the reference (its int4 is a
                           stand-alone codec, ops/quantize/int4_quantize.py);
                           follows the same subclass pattern, buffer name
                           ``weight_scales`` as the reference's NF4 module.

What differs is forward(): instead of materialising the decoded weight and
calling F.linear plus two LoRA GEMMs, it runs one fused dequant-GEMM (the
packed bytes are decoded inside the kernel) and the backward never sees a
decoded weight either.
"""

from __future__ import annotations

import math
from typing import Dict, Iterator, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from .. import _C
from .. import quantize as Q
from ..functional import MAX_FUSED_RANK, QuantWeight, qlora_linear


class LoraModule:
    """Interface shared by LoRA-carrying modules (xorl/lora/modules/base.py:18-157)."""

    r: int
    lora_alpha: int
    scaling: float
    exact_merged_forward: bool = False

    @classmethod
    def from_module(cls, module: nn.Module, r: int, lora_alpha: int, **kwargs):
        raise NotImplementedError

    def reset_lora_parameters(self) -> None:
        raise NotImplementedError

    def get_delta_weight(self) -> Tensor:
        raise NotImplementedError(
            f"{type(self).__name__} does not implement get_delta_weight(). "
            "For MoE modules, use merge_weights() directly."
        )

    def merge_weights(self) -> None:
        raise NotImplementedError

    def get_lora_parameters(self) -> Iterator[nn.Parameter]:
        if not isinstance(self, nn.Module):
            raise TypeError("LoraModule must be mixed with nn.Module")
        for name, p in self.named_parameters():
            if "lora_" in name:
                yield p

    def get_lora_state_dict(self) -> Dict[str, Tensor]:
        if not isinstance(self, nn.Module):
            raise TypeError("LoraModule must be mixed with nn.Module")
        return {n: p.detach() for n, p in self.named_parameters() if "lora_" in n}


def _is_dtensor(t) -> bool:
    return hasattr(t, "_local_tensor") and hasattr(t, "full_tensor")


class QLoRALinear(LoraModule, nn.Module):
    """Abstract base.  Subclasses register ``packed_weight_f32`` (the packed bytes
    viewed four per fp32 so FSDP2 can shard them without a dtype cast) and the
    uint8 scale buffers, then call ``reset_lora_parameters()``."""

    adapter_gradient_producer_family = "module_managed"
    # FSDP2 must not apply a parameter-cast policy to this module: the fp32
    # parameter holds raw bytes and the LoRA masters stay fp32.
    fsdp_requires_full_precision = True

    _is_prequantized: bool = False
    _inline_loaded: bool = False
    _merge_sources: Optional[Tuple[str, ...]] = None
    _source_fqn: Optional[str] = None
    _source_quant_format: Optional[str] = None

    def __init__(self, in_features: int, out_features: int, r: int = 16, lora_alpha: int = 16,
                 quant_format: str = "nvfp4", quant_group_size: int = 16, bias: bool = False,
                 device: Optional[torch.device] = None, enable_aqn: bool = False, aqn_alpha: float = 1.0):
        if type(self) is QLoRALinear:
            raise TypeError(
                "QLoRALinear is abstract. Use NvFP4QLoRALinear, BlockFP8QLoRALinear or Int4QLoRALinear."
            )
        if r <= 0:
            raise ValueError(f"LoRA rank must be positive, got {r}")
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        self.quant_format, self.quant_group_size = quant_format, quant_group_size
        self.enable_aqn, self.aqn_alpha = enable_aqn, aqn_alpha
        self._aqn_step_cache: Optional[Tensor] = None
        self._aqn_stream = None
        self._aqn_noise_buf: Optional[Tensor] = None
        self._aqn_noise_ready = False
        self.r, self.lora_alpha = r, lora_alpha
        self.active_r, self.active_lora_alpha = r, lora_alpha
        self.scaling = lora_alpha / r
        self.lora_A = nn.Parameter(torch.empty(r, in_features, dtype=torch.float32, device=device))
        self.lora_B = nn.Parameter(torch.empty(out_features, r, dtype=torch.float32, device=device))
        if bias:
            self.bias = nn.Parameter(torch.zeros(out_features, device=device), requires_grad=False)
        else:
            self.register_parameter("bias", None)
        self.register_parameter("weight", None)   # only used by deferred (meta-init) quantization
        self._ema_amax: Optional[Tensor] = None
        self._scale_dtypes: Dict[str, torch.dtype] = {}

    # ------------------------------------------------------------------ LoRA
    def reset_lora_parameters(self) -> None:
        nn.init.kaiming_uniform_(self.lora_A, a=math.sqrt(5))
        nn.init.zeros_(self.lora_B)

    def set_runtime_lora_config(self, lora_rank: int, lora_alpha: int) -> None:
        if lora_rank <= 0 or lora_rank > self.r:
            raise ValueError(f"Active LoRA rank must be in [1, {self.r}], got {lora_rank}")
        self.active_r, self.active_lora_alpha = lora_rank, lora_alpha

    def _active_scaling(self) -> float:
        return self.active_lora_alpha / self.active_r

    @staticmethod
    def _to_regular_tensor(t: Tensor) -> Tensor:
        return t.full_tensor() if hasattr(t, "full_tensor") else t

    def get_delta_weight(self) -> Tensor:
        A = self._to_regular_tensor(self.lora_A[: self.active_r])
        B = self._to_regular_tensor(self.lora_B[:, : self.active_r])
        return (B @ A) * self._active_scaling()

    # ------------------------------------------------------------------ factories
    @classmethod
    def _class_for(cls, quant_format: str):
        table = {"block_fp8": BlockFP8QLoRALinear, "nvfp4": NvFP4QLoRALinear, "int4": Int4QLoRALinear,
                 "nf4": NF4QLoRALinear}
        if quant_format not in table:
            raise ValueError(f"unsupported quant_format {quant_format!r}; expected one of {sorted(table)}")
        return table[quant_format]

    @classmethod
    def from_module(cls, module: nn.Module, r: int = 16, lora_alpha: int = 16, **kwargs) -> "QLoRALinear":
        if cls is QLoRALinear:
            fmt = kwargs.pop("quant_format", "nvfp4")
            kwargs.pop("quant_group_size", None)
            return cls._class_for(fmt).from_module(module, r=r, lora_alpha=lora_alpha, **kwargs)
        q = cls(in_features=module.in_features, out_features=module.out_features, r=r, lora_alpha=lora_alpha,
                bias=module.bias is not None, device=module.weight.device,
                enable_aqn=kwargs.get("enable_aqn", False), aqn_alpha=kwargs.get("aqn_alpha", 1.0))
        if module.bias is not None:
            with torch.no_grad():
                q.bias.copy_(module.bias.detach())
        q._init_from_weight(module.weight.detach())
        return q

    def _init_from_weight(self, w: Tensor) -> None:
        self._quantize_and_store(w)

    @classmethod
    def from_quantized(cls, packed_weight: Tensor, weight_scales: Optional[Tensor] = None,
                       weight_block_scales: Optional[Tensor] = None, weight_global_scale: Optional[Tensor] = None,
                       in_features: int = 0, out_features: int = 0, r: int = 16, lora_alpha: int = 16,
                       quant_format: str = "nvfp4", quant_group_size: int = 16, bias: bool = False,
                       device: Optional[torch.device] = None, **kwargs) -> "QLoRALinear":
        if cls is QLoRALinear:
            cls = cls._class_for(quant_format)
        q = cls(in_features=in_features, out_features=out_features, r=r, lora_alpha=lora_alpha, bias=bias,
                device=device)
        q.packed_weight_f32 = nn.Parameter(cls._to_uint8(packed_weight).contiguous().view(torch.float32),
                                           requires_grad=False)
        q._scale_dtypes = {}
        for name, t in (("weight_scales", weight_scales), ("weight_block_scales", weight_block_scales),
                        ("weight_global_scale", weight_global_scale)):
            if t is not None:
                q._scale_dtypes[name] = t.dtype
                setattr(q, name, cls._to_uint8(t))
        q._is_prequantized = True
        return q

    # ------------------------------------------------------------------ byte storage
    @staticmethod
    def _to_uint8(t: Tensor) -> Tensor:
        """uint8 view: scales and codes are stored as bytes so that no mixed
        precision policy can cast them (the true dtype lives in _scale_dtypes)."""
        t = t.contiguous()
        if t.dim() and t.stride(-1) != 1:      # a size-1 last dimension may keep a foreign stride
            t = t.clone(memory_format=torch.contiguous_format)
        return t if t.dtype == torch.uint8 else t.view(torch.uint8)

    def _recover_tensor(self, buf: Tensor, original_dtype: torch.dtype) -> Tensor:
        return buf if original_dtype == torch.uint8 else buf.contiguous().view(original_dtype)

    def _write_packed_weight(self, uint8_data: Tensor) -> None:
        """Store packed bytes into packed_weight_f32 (plain, meta or DTensor shard)."""
        f32 = uint8_data.contiguous().view(torch.float32)
        cur = self.packed_weight_f32
        if cur is None or cur.device.type == "meta":
            if cur is not None:
                f32 = f32.reshape(cur.shape)
            self.packed_weight_f32 = nn.Parameter(f32, requires_grad=False)
            return
        if _is_dtensor(cur):
            from torch.distributed._tensor import Shard

            f32 = f32.reshape(cur.shape)
            dim = next((p.dim for p in cur.placements if isinstance(p, Shard)), None)
            local = cur._local_tensor
            if dim is None:
                local.copy_(f32)
                return
            mesh = cur.device_mesh
            chunk = f32.shape[dim] // mesh.size()
            start = mesh.get_local_rank() * chunk
            local.copy_(f32.narrow(dim, start, chunk))
            return
        if cur.numel() == f32.numel():
            cur.data.copy_(f32.reshape(cur.shape))
        else:
            self.packed_weight_f32 = nn.Parameter(f32, requires_grad=False)

    @torch.compiler.disable
    def _gather_packed_weight(self, f32: Tensor) -> Tensor:
        return f32.full_tensor()

    def _read_packed_weight_uint8(self) -> Tensor:
        """The packed bytes as a uint8 view (qlora/modules/linear.py:268-280).  Only the gather of sharded state is
        kept out of traced graphs; the plain view traces, so that a compiled module is one graph."""
        f32 = self.packed_weight_f32.data
        if _is_dtensor(f32):
            f32 = self._gather_packed_weight(f32)
        elif f32.dtype != torch.float32:
            raise RuntimeError(
                f"QLoRA packed_weight_f32 has dtype {f32.dtype} (expected float32). "
                "FSDP2 mixed precision likely cast it, corrupting packed weight data. "
                "Ensure packed_weight_f32 is deregistered from FSDP param groups."
            )
        return f32.contiguous().view(torch.uint8)

    def _apply(self, fn, recurse: bool = True):
        """model.to(bf16) must not touch the packed bytes or the fp32 LoRA masters."""
        probe = fn(torch.empty(0, dtype=torch.float32, device=self.lora_A.device))
        names = [n for n in ("lora_A", "lora_B", "packed_weight_f32") if self._parameters.get(n) is not None]
        held = {n: self._parameters.pop(n) for n in names}
        try:
            out = super()._apply(fn, recurse=recurse)
        finally:
            for n, p in held.items():
                if p.is_meta:
                    p = nn.Parameter(torch.empty_like(p, dtype=torch.float32, device=probe.device),
                                     requires_grad=p.requires_grad)
                else:
                    with torch.no_grad():
                        p.data = p.data.to(device=probe.device, dtype=torch.float32)
                        if p.grad is not None:
                            p.grad.data = p.grad.data.to(device=probe.device, dtype=torch.float32)
                self._parameters[n] = p
        return out

    # ------------------------------------------------------------------ checkpoint loading
    def load_prequantized_weights(self, weight_map: dict, shard_cache: dict, weights_path: str) -> None:
        import os

        import safetensors.torch

        def _load(key: str) -> Tensor:
            shard = weight_map.get(key)
            if shard is None:
                raise RuntimeError(f"Key {key} not found in checkpoint index")
            if shard not in shard_cache:
                path = os.path.join(weights_path, shard)
                if not os.path.exists(path):
                    from transformers.utils import cached_file

                    path = cached_file(weights_path, shard)
                shard_cache[shard] = safetensors.torch.load_file(path, device="cpu")
            return shard_cache[shard][key]

        self._load_prequantized(_load)

    # suffixes of the checkpoint tensors one source projection contributes (empty: no pre-quantized format)
    _prequant_suffixes: Tuple[str, ...] = ()

    def _prequant_sources(self) -> Tuple[str, ...]:
        """Checkpoint prefixes this module is assembled from: its own, or one per merged projection."""
        if self._merge_sources is not None:
            return tuple(f"{self._source_fqn}.{p}" for p in self._merge_sources)
        return (self._source_fqn,)

    def _load_prequantized(self, _load_tensor) -> None:
        """Fetch this module's checkpoint tensors through `_load_tensor(key)` and install them."""
        if not self._prequant_suffixes:
            raise NotImplementedError
        pieces = [{sfx: _load_tensor(f"{q}.{sfx}") for sfx in self._prequant_suffixes} for q in self._prequant_sources()]
        self._install_prequantized(self._pack_prequantized(pieces))

    def _pack_prequantized(self, pieces) -> dict:
        """`pieces`: one {suffix: tensor} mapping per source projection, in row order.  Returns the module state
        they make: "packed" (uint8 rows), one entry per scale buffer (true dtype), "scale_dtypes", "ema_amax"."""
        raise NotImplementedError

    def _install_prequantized(self, state: dict) -> None:
        dev = self.lora_A.device if self.lora_A.device.type != "meta" else torch.device("cuda")
        self._write_packed_weight(state["packed"].to(dev))
        self._scale_dtypes = dict(state["scale_dtypes"])
        for name in self._scale_dtypes:
            setattr(self, name, self._to_uint8(state[name]).to(dev))
        ema = state.get("ema_amax")
        self._ema_amax = None if ema is None else ema.to(dev)
        self._aqn_step_cache = None

    def quantize_weight(self) -> None:
        """Deferred quantization: turn the (FSDP-loaded) `weight` into packed form."""
        if self.weight is None:
            return
        w = self.weight.data
        if _is_dtensor(w):
            w = w.full_tensor()
        self._quantize_and_store(w)
        self.weight = None

    def _quantize_and_store(self, w: Tensor, global_amax: Optional[Tensor] = None) -> None:
        raise NotImplementedError

    def _quant_weight(self) -> QuantWeight:
        """Describe the packed state for the kernels (no copies)."""
        raise NotImplementedError

    @torch.compiler.disable
    def _dequantize_weight(self) -> Tensor:
        raise NotImplementedError

    @torch.compiler.disable
    def _compute_aqn_step(self) -> Tensor:
        raise NotImplementedError

    def merge_weights(self, ema_decay: float = 0.1) -> None:
        """W' = Q(deq(W) + dW); re-initialise A, zero B (block_fp8_linear.py:111-119)."""
        with torch.no_grad():
            w = self._dequantize_weight()
            merged = w + self.get_delta_weight().to(w.dtype)
            self._requantize_merged(merged, ema_decay)
            nn.init.kaiming_uniform_(self.lora_A, a=math.sqrt(5))
            self.lora_B.zero_()

    def merged_weight(self, dtype: torch.dtype = torch.bfloat16) -> Tensor:
        """deq(W).to(bf16) + get_delta_weight().to(bf16): the tensor the weight-sync path publishes
        (server/weight_sync/handler.py:2119-2131), produced by one fused kernel."""
        from ..functional import merge_dense

        with torch.no_grad():
            if self.active_r > MAX_FUSED_RANK:      # beyond the fused kernel's rank: decode kernel + the update as written there
                w = self._dequantize_weight().to(torch.bfloat16) + self.get_delta_weight().to(torch.bfloat16)
                return w.to(dtype)
            return merge_dense(self._quant_weight(), self._to_regular_tensor(self.lora_A),
                               self._to_regular_tensor(self.lora_B), self.active_r, self._active_scaling(), dtype)

    def _requantize_merged(self, merged: Tensor, ema_decay: float) -> None:
        self._quantize_and_store(merged)

    # ------------------------------------------------------------------ AQN (optional, off by default)
    @torch.compiler.disable
    def _aqn_start_noise(self, device: torch.device, dtype: torch.dtype) -> None:
        shape = (self.out_features, self.in_features)
        if self._aqn_stream is None:
            self._aqn_stream = torch.cuda.Stream(device=device)
        buf = self._aqn_noise_buf
        if buf is None or buf.shape != shape or buf.dtype != dtype or buf.device != device:
            self._aqn_noise_buf = torch.empty(*shape, device=device, dtype=dtype)
        self._aqn_stream.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(self._aqn_stream):
            self._aqn_noise_buf.normal_()
        self._aqn_noise_ready = True

    @torch.compiler.disable
    def _aqn_apply_noise(self, w: Tensor) -> Tensor:
        torch.cuda.current_stream(w.device).wait_stream(self._aqn_stream)
        if self._aqn_step_cache is None:
            self._aqn_step_cache = self._compute_aqn_step()
        step = self._aqn_step_cache.to(dtype=w.dtype, device=w.device)
        self._aqn_noise_ready = False
        return torch.addcmul(w, self._aqn_noise_buf, step, value=self.aqn_alpha)

    def _forward_with_noise(self, x: Tensor) -> Tensor:
        """AQN perturbs the decoded weight, so this training-time regulariser needs
        the weight materialised (qlora/modules/linear.py:369-385 as written)."""
        if not self._aqn_noise_ready:
            self._aqn_start_noise(x.device, x.dtype)
        w = self._aqn_apply_noise(self._dequantize_weight().to(x.dtype))
        base = F.linear(x, w, self.bias)
        A, B = self.lora_A[: self.active_r], self.lora_B[:, : self.active_r]
        lo = F.linear(F.linear(x.to(A.dtype), A), B) * self._active_scaling()
        return base + lo.to(base.dtype)

    # ------------------------------------------------------------------ forward
    def forward(self, x: Tensor) -> Tensor:
        if self.enable_aqn and self.training:
            return self._forward_with_noise(x)
        return qlora_linear(x, self._forward_quant_weight(), self.lora_A, self.lora_B, self.active_r,
                            self._active_scaling(), self.bias)

    def _forward_quant_weight(self) -> QuantWeight:
        """`_quant_weight()` memoised on the addresses of the packed state: the description (and its C
        descriptor) is rebuilt only when a buffer has been replaced.  Sharded state is gathered every call."""
        p = self.packed_weight_f32
        if torch.compiler.is_compiling() or _is_dtensor(p.data):     # addresses are not traceable
            return self._quant_weight()
        key = (p.data_ptr(), p.dtype) + tuple(
            t.data_ptr() for t in (getattr(self, "weight_scales", None), getattr(self, "weight_block_scales", None),
                                   getattr(self, "weight_global_scale", None)) if t is not None)
        key += tuple(self._scale_dtypes.values())
        cached = self.__dict__.get("_qw_cache")
        if cached is None or cached[0] != key:
            cached = (key, self._quant_weight())
            self.__dict__["_qw_cache"] = cached
        return cached[1]

    # ------------------------------------------------------------------ checkpoint helpers
    def get_quantized_state_dict(self) -> Dict[str, Tensor]:
        state = {"packed_weight_f32": self.packed_weight_f32}
        for name in ("weight_scales", "weight_block_scales", "weight_global_scale"):
            t = getattr(self, name, None)
            if t is not None:
                state[name] = t
        return state

    def extra_repr(self) -> str:
        s = (f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, "
             f"r={self.r}, lora_alpha={self.lora_alpha}, quant_format={self.quant_format}, "
             f"quant_group_size={self.quant_group_size}")
        return s + (f", aqn=True(alpha={self.aqn_alpha})" if self.enable_aqn else "")


# =============================================================================
class BlockFP8QLoRALinear(QLoRALinear):
    """e4m3 bytes + fp32 scale per 128x128 block (block_fp8_linear.py:14-144)."""

    def __init__(self, in_features: int, out_features: int, r: int = 16, lora_alpha: int = 16, bias: bool = False,
                 device: Optional[torch.device] = None, enable_aqn: bool = False, aqn_alpha: float = 1.0):
        super().__init__(in_features, out_features, r=r, lora_alpha=lora_alpha, quant_format="block_fp8",
                         quant_group_size=128, bias=bias, device=device, enable_aqn=enable_aqn, aqn_alpha=aqn_alpha)
        if in_features % 4:
            raise ValueError(f"block_fp8 needs in_features % 4 == 0, got {in_features}")
        self.packed_weight_f32 = nn.Parameter(
            torch.empty(out_features, in_features // 4, dtype=torch.float32, device=device), requires_grad=False)
        self.register_buffer("weight_block_scales", torch.empty(
            math.ceil(out_features / 128), math.ceil(in_features / 128) * 4, dtype=torch.uint8, device=device))
        self._scale_dtypes = {"weight_block_scales": torch.float32}
        self.reset_lora_parameters()

    def _quantize_and_store(self, w: Tensor, global_amax: Optional[Tensor] = None) -> None:
        fp8_w, scales = Q.block_fp8_quantize_gkn(w.float().contiguous(), self.quant_group_size)
        self._write_packed_weight(self._to_uint8(fp8_w))
        self._scale_dtypes = {"weight_block_scales": scales.dtype}
        self.weight_block_scales = self._to_uint8(scales)
        self._aqn_step_cache = None

    def _quant_weight(self) -> QuantWeight:
        return QuantWeight("block_fp8", _C.XQ_LAYOUT_FLAT, self._read_packed_weight_uint8(),
                           self.weight_block_scales, torch.float32, self.out_features, self.in_features, 128)

    def merge_weights(self, ema_decay: float = 0.1) -> None:
        """Decode, add the LoRA update and re-encode with fresh block scales in one fused pass over the
        bytes (block_fp8_linear.py:111-119); falls back to the generic path for sharded (DTensor) state."""
        from ..functional import merge_requant_fp8

        if _is_dtensor(self.packed_weight_f32) or _is_dtensor(self.lora_A) or self.active_r > MAX_FUSED_RANK:
            return super().merge_weights(ema_decay)
        with torch.no_grad():
            packed, scales = merge_requant_fp8(self._quant_weight(), self.lora_A, self.lora_B, self.active_r,
                                               self._active_scaling())
            self._write_packed_weight(packed.reshape(-1))
            self._scale_dtypes = {"weight_block_scales": torch.float32}
            self.weight_block_scales = self._to_uint8(scales)
            self._aqn_step_cache = None
            nn.init.kaiming_uniform_(self.lora_A, a=math.sqrt(5))
            self.lora_B.zero_()

    @torch.compiler.disable
    def _dequantize_weight(self) -> Tensor:
        """fp32 [out, in], as block_fp8_dequantize_gkn returns it (callers cast to bf16)."""
        fp8 = self._read_packed_weight_uint8().view(torch.float8_e4m3fn).reshape(self.out_features, self.in_features)
        scales = self._recover_tensor(self.weight_block_scales, self._scale_dtypes["weight_block_scales"])
        return Q.block_fp8_dequantize_gkn(fp8, scales, self.quant_group_size)

    @torch.compiler.disable
    def _compute_aqn_step(self) -> Tensor:
        """0.125 * block scale: the e4m3 ulp at unit magnitude (block_fp8_linear.py:102-109)."""
        s = self._recover_tensor(self.weight_block_scales, self._scale_dtypes["weight_block_scales"]).float()
        step = s.repeat_interleave(128, 0).repeat_interleave(128, 1)[: self.out_features, : self.in_features]
        return (0.125 * step).contiguous()

    _prequant_suffixes = ("weight", "weight_scale_inv")

    def _pack_prequantized(self, pieces) -> dict:
        """HF fp8 checkpoints: `{m}.weight` (e4m3 [N, K]) + `{m}.weight_scale_inv` (fp32 [N/128, K/128]); merged
        projections are row-wise concatenations of bytes and of scale rows (checkpoint_handlers/buffers.py:878-901)."""
        return {
            "packed": torch.cat([self._to_uint8(p["weight"]) for p in pieces], 0),
            "weight_block_scales": torch.cat([p["weight_scale_inv"].float() for p in pieces], 0),
            "scale_dtypes": {"weight_block_scales": torch.float32},
            "ema_amax": None,
        }


# =============================================================================
class NvFP4QLoRALinear(QLoRALinear):
    """e2m1 codes, per-16 e4m3 block scales, fp32 global scale (nvfp4_linear.py:14-175)."""

    def __init__(self, in_features: int, out_features: int, r: int = 16, lora_alpha: int = 16, bias: bool = False,
                 device: Optional[torch.device] = None, enable_aqn: bool = False, aqn_alpha: float = 1.0):
        super().__init__(in_features, out_features, r=r, lora_alpha=lora_alpha, quant_format="nvfp4",
                         quant_group_size=16, bias=bias, device=device, enable_aqn=enable_aqn, aqn_alpha=aqn_alpha)
        if in_features % 16:
            raise ValueError(f"nvfp4 needs in_features % 16 == 0, got {in_features}")
        self.packed_weight_f32 = nn.Parameter(
            torch.empty(out_features, in_features // 8, dtype=torch.float32, device=device), requires_grad=False)
        self.register_buffer("weight_block_scales", torch.empty(
            out_features, (in_features // 16) * 4, dtype=torch.uint8, device=device))
        self.register_buffer("weight_global_scale", torch.empty(4, dtype=torch.uint8, device=device))
        self._scale_dtypes = {"weight_block_scales": torch.float32, "weight_global_scale": torch.float32}
        self.reset_lora_parameters()

    def _init_from_weight(self, w: Tensor) -> None:
        self._ema_amax = w.float().abs().max().reshape(1).to(w.device)
        self._quantize_and_store(w, global_amax=self._ema_amax)

    def _quantize_and_store(self, w: Tensor, global_amax: Optional[Tensor] = None) -> None:
        packed, block_scales, global_scale = Q.nvfp4_quantize(w, self.quant_group_size, global_amax=global_amax)
        self._write_packed_weight(self._to_uint8(packed))
        self._scale_dtypes = {"weight_block_scales": block_scales.dtype, "weight_global_scale": global_scale.dtype}
        self.weight_block_scales = self._to_uint8(block_scales)
        self.weight_global_scale = self._to_uint8(global_scale)
        self._aqn_step_cache = None

    def _scales(self) -> Tuple[Tensor, torch.dtype, Tensor]:
        sdt = self._scale_dtypes["weight_block_scales"]
        g = self._recover_tensor(self.weight_global_scale, self._scale_dtypes["weight_global_scale"]).float()
        return self.weight_block_scales, sdt, g

    def _quant_weight(self) -> QuantWeight:
        s, sdt, g = self._scales()
        return QuantWeight("nvfp4", _C.XQ_LAYOUT_FLAT, self._read_packed_weight_uint8(), s, sdt,
                           self.out_features, self.in_features, 16, global_scale=g)

    @torch.compiler.disable
    def _dequantize_weight(self) -> Tensor:
        s, sdt, g = self._scales()
        n = self.out_features * self.in_features
        w = Q.nvfp4_dequantize(self._read_packed_weight_uint8(), self._recover_tensor(s, sdt), g, n, 16)
        return w.reshape(self.out_features, self.in_features)

    @torch.compiler.disable
    def _compute_aqn_step(self) -> Tensor:
        """0.5 * block scale * global scale: the smallest e2m1 step (nvfp4_linear.py:115-124)."""
        s, sdt, g = self._scales()
        eff = self._recover_tensor(s, sdt).float() * g
        return (0.5 * eff.reshape(self.out_features, -1).repeat_interleave(16, 1)).contiguous()

    def merge_weights(self, ema_decay: float = 0.1) -> None:
        """Decode, add the LoRA update, blend the fresh tensor amax into the running one and re-encode with it, in
        two fused passes over the packed bytes (nvfp4_linear.py:126-139); sharded (DTensor) state and ranks beyond
        the fused kernels' take the generic path."""
        from ..functional import merge_amax, merge_requant_nvfp4

        if (_is_dtensor(self.packed_weight_f32) or _is_dtensor(self.lora_A) or self.active_r > MAX_FUSED_RANK
                or not self.packed_weight_f32.is_cuda):
            return super().merge_weights(ema_decay)
        with torch.no_grad():
            qw = self._quant_weight()
            fresh = merge_amax(qw, self.lora_A, self.lora_B, self.active_r, self._active_scaling())
            if self._ema_amax is not None:
                self._ema_amax.lerp_(fresh.to(self._ema_amax.device), ema_decay)
            else:
                self._ema_amax = fresh
            codes, bscales, gscale = merge_requant_nvfp4(qw, self.lora_A, self.lora_B, self.active_r,
                                                         self._active_scaling(), self._ema_amax)
            self._write_packed_weight(codes)
            self._scale_dtypes = {"weight_block_scales": bscales.dtype, "weight_global_scale": gscale.dtype}
            self.weight_block_scales = self._to_uint8(bscales)
            self.weight_global_scale = self._to_uint8(gscale)
            self._aqn_step_cache = None
            nn.init.kaiming_uniform_(self.lora_A, a=math.sqrt(5))
            self.lora_B.zero_()

    def _requantize_merged(self, merged: Tensor, ema_decay: float) -> None:
        fresh = merged.float().abs().max().reshape(1)
        if self._ema_amax is not None:
            self._ema_amax.lerp_(fresh.to(self._ema_amax.device), ema_decay)
        else:
            self._ema_amax = fresh
        self._quantize_and_store(merged, global_amax=self._ema_amax)

    _prequant_suffixes = ("weight", "weight_scale", "weight_scale_2")

    def _pack_prequantized(self, pieces) -> dict:
        """modelopt nvfp4 checkpoints: `.weight` (codes [N, K/2]), `.weight_scale` (e4m3 [N, K/16]), `.weight_scale_2`
        (fp32 scalar).  Each source's global scale is folded into fp32 block scales and the stored global is 1.0, so
        that merged projections with different globals share one module; the largest source amax
        (global * 6 * 448) seeds the EMA used by re-quantisation (checkpoint_handlers/buffers.py:827-865)."""
        scales, amax = [], []
        for p in pieces:
            g = p["weight_scale_2"].float()
            scales.append(p["weight_scale"].float() * g)
            amax.append(g.item() * 6.0 * 448.0)
        return {
            "packed": torch.cat([self._to_uint8(p["weight"]) for p in pieces], 0),
            "weight_block_scales": torch.cat(scales, 0),
            "weight_global_scale": torch.tensor([1.0], dtype=torch.float32),
            "scale_dtypes": {"weight_block_scales": torch.float32, "weight_global_scale": torch.float32},
            "ema_amax": torch.tensor([max(amax)], dtype=torch.float32),
        }


# =============================================================================
class Int4QLoRALinear(QLoRALinear):
    """Group-scaled int4: w = (nib - 8) * scale, one scale per `quant_group_size`
    consecutive input features; scales bf16 (symmetric absmax/7 rule) or fp32
    (the reference codec's amax*2/15 rule)."""

    def __init__(self, in_features: int, out_features: int, r: int = 16, lora_alpha: int = 16, bias: bool = False,
                 device: Optional[torch.device] = None, enable_aqn: bool = False, aqn_alpha: float = 1.0,
                 quant_group_size: int = 128, symmetric: bool = True):
        super().__init__(in_features, out_features, r=r, lora_alpha=lora_alpha, quant_format="int4",
                         quant_group_size=quant_group_size, bias=bias, device=device, enable_aqn=enable_aqn,
                         aqn_alpha=aqn_alpha)
        if in_features % quant_group_size or in_features % 8:
            raise ValueError(f"int4 needs in_features divisible by 8 and by the group size {quant_group_size}")
        self.symmetric = symmetric
        self.packed_weight_f32 = nn.Parameter(
            torch.empty(out_features, in_features // 8, dtype=torch.float32, device=device), requires_grad=False)
        sdt = torch.bfloat16 if symmetric else torch.float32
        nbytes = (in_features // quant_group_size) * (2 if symmetric else 4)
        self.register_buffer("weight_scales", torch.empty(out_features, nbytes, dtype=torch.uint8, device=device))
        self._scale_dtypes = {"weight_scales": sdt}
        self.reset_lora_parameters()

    @classmethod
    def from_module(cls, module: nn.Module, r: int = 16, lora_alpha: int = 16, **kwargs) -> "Int4QLoRALinear":
        q = cls(in_features=module.in_features, out_features=module.out_features, r=r, lora_alpha=lora_alpha,
                bias=module.bias is not None, device=module.weight.device,
                quant_group_size=kwargs.get("quant_group_size", 128), symmetric=kwargs.get("symmetric", True),
                enable_aqn=kwargs.get("enable_aqn", False), aqn_alpha=kwargs.get("aqn_alpha", 1.0))
        if module.bias is not None:
            with torch.no_grad():
                q.bias.copy_(module.bias.detach())
        q._quantize_and_store(module.weight.detach())
        return q

    def _quantize_and_store(self, w: Tensor, global_amax: Optional[Tensor] = None) -> None:
        fn = Q.int4_quantize_sym if self.symmetric else Q.int4_quantize
        packed, scales = fn(w.float(), self.quant_group_size)
        self._write_packed_weight(self._to_uint8(packed))
        self._scale_dtypes = {"weight_scales": scales.dtype}
        self.weight_scales = self._to_uint8(scales)
        self._aqn_step_cache = None

    def merge_weights(self, ema_decay: float = 0.1) -> None:
        """Decode, add the LoRA update and re-encode with fresh group scales (this module's own rule, symmetric or the
        reference codec's) in one fused pass over the bytes; sharded (DTensor) state, group sizes other than 128 and
        ranks beyond the fused kernels' take the generic path."""
        from ..functional import merge_requant_int4

        sdt = torch.bfloat16 if self.symmetric else torch.float32
        if (_is_dtensor(self.packed_weight_f32) or _is_dtensor(self.lora_A) or self.active_r > MAX_FUSED_RANK
                or not self.packed_weight_f32.is_cuda or self.quant_group_size != 128 or self.in_features % 128
                or self._scale_dtypes.get("weight_scales") != sdt):
            return super().merge_weights(ema_decay)
        with torch.no_grad():
            codes, scales = merge_requant_int4(self._quant_weight(), self.lora_A, self.lora_B, self.active_r,
                                               self._active_scaling(), self.symmetric)
            self._write_packed_weight(codes.reshape(-1))
            self.weight_scales = self._to_uint8(scales)
            self._aqn_step_cache = None
            nn.init.kaiming_uniform_(self.lora_A, a=math.sqrt(5))
            self.lora_B.zero_()

    def _quant_weight(self) -> QuantWeight:
        return QuantWeight("int4", _C.XQ_LAYOUT_FLAT, self._read_packed_weight_uint8(), self.weight_scales,
                           self._scale_dtypes["weight_scales"], self.out_features, self.in_features,
                           self.quant_group_size)

    @torch.compiler.disable
    def _dequantize_weight(self) -> Tensor:
        s = self._recover_tensor(self.weight_scales, self._scale_dtypes["weight_scales"])
        return Q.int4_dequantize(self._read_packed_weight_uint8(), s, self.out_features, self.in_features,
                                 self.quant_group_size)

    @torch.compiler.disable
    def _compute_aqn_step(self) -> Tensor:
        s = self._recover_tensor(self.weight_scales, self._scale_dtypes["weight_scales"]).float()
        return (0.5 * s.repeat_interleave(self.quant_group_size, 1)).contiguous()


# =============================================================================
class NF4QLoRALinear(QLoRALinear):
    """NormalFloat4: w = level[nib] * absmax, one fp32 absmax per 64 consecutive
    elements of the row-major weight (qlora/modules/nf4_linear.py:15-136).  State:
    `packed_weight_f32 [N, K/8]`, `weight_scales` u8 view of fp32 `[N, K/64]`."""

    def __init__(self, in_features: int, out_features: int, r: int = 16, lora_alpha: int = 16, bias: bool = False,
                 device: Optional[torch.device] = None, enable_aqn: bool = False, aqn_alpha: float = 1.0):
        super().__init__(in_features, out_features, r=r, lora_alpha=lora_alpha, quant_format="nf4",
                         quant_group_size=64, bias=bias, device=device, enable_aqn=enable_aqn, aqn_alpha=aqn_alpha)
        if in_features % self.quant_group_size:
            raise ValueError(f"nf4 needs in_features divisible by the group size {self.quant_group_size}")
        self.packed_weight_f32 = nn.Parameter(
            torch.empty(out_features, in_features // 8, dtype=torch.float32, device=device), requires_grad=False)
        self.register_buffer("weight_scales", torch.empty(out_features, (in_features // self.quant_group_size) * 4,
                                                          dtype=torch.uint8, device=device))
        self._scale_dtypes = {"weight_scales": torch.float32}
        self.reset_lora_parameters()

    @classmethod
    def from_module(cls, module: nn.Module, r: int = 16, lora_alpha: int = 16, enable_aqn: bool = False,
                    aqn_alpha: float = 1.0, **kwargs) -> "NF4QLoRALinear":
        """Quantize a bf16 nn.Linear; on the meta device keep `weight` for a later
        `quantize_weight()` (nf4_linear.py:64-96)."""
        q = cls(in_features=module.in_features, out_features=module.out_features, r=r, lora_alpha=lora_alpha,
                bias=module.bias is not None, device=module.weight.device, enable_aqn=enable_aqn,
                aqn_alpha=aqn_alpha)
        if module.weight.device.type == "meta":
            q.weight = nn.Parameter(module.weight.detach(), requires_grad=False)
            return q
        if module.bias is not None:
            with torch.no_grad():
                q.bias.copy_(module.bias.detach())
        q._quantize_and_store(module.weight.detach())
        return q

    def _quantize_and_store(self, w: Tensor, global_amax: Optional[Tensor] = None) -> None:
        packed, scales = Q.nf4_quantize(w.reshape(self.out_features, self.in_features), self.quant_group_size)
        self._write_packed_weight(self._to_uint8(packed))
        self._scale_dtypes = {"weight_scales": scales.dtype}
        self.weight_scales = self._to_uint8(scales.reshape(self.out_features, -1))
        self._aqn_step_cache = None

    def merge_weights(self, ema_decay: float = 0.1) -> None:
        """Decode, add the LoRA update and re-encode with fresh group scales in one fused pass over the bytes;
        sharded (DTensor) state, other group sizes and ranks beyond the fused kernels' take the generic path."""
        from ..functional import merge_requant_nf4

        if (_is_dtensor(self.packed_weight_f32) or _is_dtensor(self.lora_A) or self.active_r > MAX_FUSED_RANK
                or not self.packed_weight_f32.is_cuda or self.quant_group_size != 64 or self.in_features % 64
                or self._scale_dtypes.get("weight_scales") != torch.float32):
            return super().merge_weights(ema_decay)
        with torch.no_grad():
            codes, scales = merge_requant_nf4(self._quant_weight(), self.lora_A, self.lora_B, self.active_r,
                                              self._active_scaling())
            self._write_packed_weight(codes)
            self.weight_scales = self._to_uint8(scales.reshape(self.out_features, -1))
            self._aqn_step_cache = None
            nn.init.kaiming_uniform_(self.lora_A, a=math.sqrt(5))
            self.lora_B.zero_()

    def _quant_weight(self) -> QuantWeight:
        return QuantWeight("nf4", _C.XQ_LAYOUT_FLAT, self._read_packed_weight_uint8(), self.weight_scales,
                           self._scale_dtypes["weight_scales"], self.out_features, self.in_features,
                           self.quant_group_size)

    @torch.compiler.disable
    def _dequantize_weight(self) -> Tensor:
        s = self._recover_tensor(self.weight_scales, self._scale_dtypes["weight_scales"])
        n = self.out_features * self.in_features
        return Q.nf4_dequantize(self._read_packed_weight_uint8(), s, n, self.quant_group_size).reshape(
            self.out_features, self.in_features)

    @torch.compiler.disable
    def _compute_aqn_step(self) -> Tensor:
        """Half the narrowest gap between levels times the group's absmax (nf4_linear.py:113-120)."""
        s = self._recover_tensor(self.weight_scales, self._scale_dtypes["weight_scales"]).float()
        s = s.reshape(self.out_features, self.in_features // self.quant_group_size)
        return (0.5 * Q.NF4_MIN_STEP * s.repeat_interleave(self.quant_group_size, 1)).contiguous()

    def _load_prequantized(self, _load_tensor) -> None:
        raise NotImplementedError("NF4 has no pre-quantized checkpoint format; use from_module() on bf16 weights")


# =============================================================================
def qlora_mlp_forward(gate_proj: "QLoRALinear", up_proj: "QLoRALinear", down_proj: "QLoRALinear", x: Tensor) -> Tensor:
    """`down_proj(silu(gate_proj(x)) * up_proj(x))` -- the body of the reference's Qwen3MLP.forward
    (models/transformers/qwen3/modeling_qwen3.py:60-81) on three QLoRA linears -- as one fused forward and one fused
    backward of the library when the three modules allow it: same active LoRA rank (<= 64) and scaling, plain
    (unsharded) state, no quantization noise.  Otherwise the three modules and the SwiGLU kernel are called one by
    one; both ways give the same rounding points."""
    from ..functional import qlora_mlp, qlora_mlp_infer, silu_and_mul

    mods = (gate_proj, up_proj, down_proj)
    if not all(isinstance(m, QLoRALinear) for m in mods):
        return down_proj(silu_and_mul(gate_proj(x), up_proj(x)))
    r, s = gate_proj.active_r, gate_proj._active_scaling()
    fusable = (all(m.active_r == r and m._active_scaling() == s for m in mods) and r <= MAX_FUSED_RANK
               # (the fused backward forms no gradient for a gate / up bias: a trainable one takes the module path)
               and not any(m.bias is not None and m.bias.requires_grad for m in (gate_proj, up_proj))
               and not any(m.enable_aqn and m.training for m in mods)
               and not any(_is_dtensor(m.packed_weight_f32.data) or _is_dtensor(m.lora_A) for m in mods)
               and gate_proj.out_features == up_proj.out_features == down_proj.in_features
               and gate_proj.in_features == up_proj.in_features == down_proj.out_features
               and gate_proj.in_features % 64 == 0 and gate_proj.out_features % 64 == 0
               and x.dtype == torch.bfloat16 and x.is_cuda)
    if not fusable:
        return down_proj(silu_and_mul(gate_proj(x), up_proj(x)))
    needs_grad = torch.is_grad_enabled() and (x.requires_grad or any(
        p is not None and p.requires_grad for m in mods for p in (m.lora_A, m.lora_B, m.bias)))
    if not needs_grad and not torch.compiler.is_compiling():
        # inference / rollout: one library call that keeps nothing for a backward (weight-streaming kernels at decode sizes)
        return qlora_mlp_infer(x, gate_proj._forward_quant_weight(), up_proj._forward_quant_weight(), down_proj._forward_quant_weight(),
                               gate_proj.lora_A, gate_proj.lora_B, up_proj.lora_A, up_proj.lora_B, down_proj.lora_A, down_proj.lora_B,
                               r, s, gate_proj.bias, up_proj.bias, down_proj.bias)
    return qlora_mlp(x, gate_proj._forward_quant_weight(), up_proj._forward_quant_weight(), down_proj._forward_quant_weight(),
                     gate_proj.lora_A, gate_proj.lora_B, up_proj.lora_A, up_proj.lora_B, down_proj.lora_A, down_proj.lora_B,
                     r, s, gate_proj.bias, up_proj.bias, down_proj.bias)


def qlora_gate_up_silu(gate_up_proj: "QLoRALinear", x: Tensor) -> Tensor:
    """`fused_silu_and_mul(gate_up_proj(x))` -- the first half of the reference's Qwen3MLP.forward with its default fused
    module (models/transformers/qwen3/modeling_qwen3.py:62-70).  Without autograd this is one library call, at decode
    sizes one kernel launch that writes h directly (xq_linear_fwd_swiglu); otherwise the module call and the SwiGLU
    kernel.  The same bits either way."""
    from ..functional import qlora_linear_swiglu, silu_and_mul

    m = gate_up_proj
    needs_grad = torch.is_grad_enabled() and (x.requires_grad or any(
        p is not None and p.requires_grad for p in (m.lora_A, m.lora_B, m.bias)))
    one_call = (isinstance(m, QLoRALinear) and not needs_grad and not torch.compiler.is_compiling() and m.active_r <= MAX_FUSED_RANK
                and m.out_features % 2 == 0 and not (m.enable_aqn and m.training)
                and not (_is_dtensor(m.packed_weight_f32.data) or _is_dtensor(m.lora_A))
                and x.dtype == torch.bfloat16 and x.is_cuda)
    if not one_call:
        gate, up = m(x).chunk(2, dim=-1)
        return silu_and_mul(gate, up)
    return qlora_linear_swiglu(x, m._forward_quant_weight(), m.lora_A, m.lora_B, m.active_r, m._active_scaling(), m.bias)


def qlora_linears_forward(modules, x: Tensor) -> list:
    """`[m(x) for m in modules]` for QLoRA linears that share their input -- the separate q_proj / k_proj / v_proj calls
    of the reference's attention block (models/layers/attention/multi_head_attention.py:93-95) and the gate_proj /
    up_proj calls of its unfused MLP (models/transformers/qwen3/modeling_qwen3.py:75-76).  Without autograd (decode,
    rollout) up to four modules go to the library as ONE call, which at decode sizes is one kernel launch
    (xq_linear_fwd_multi); in every other case the modules are called one by one.  The results are the same bits."""
    from ..functional import qlora_linear_multi
    from .._C import XQ_LINEAR_MULTI_MAX

    mods = list(modules)
    needs_grad = torch.is_grad_enabled() and (x.requires_grad or any(
        p.requires_grad for m in mods for p in (m.lora_A, m.lora_B, m.bias) if p is not None))
    one_call = (1 < len(mods) <= XQ_LINEAR_MULTI_MAX and not needs_grad and not torch.compiler.is_compiling()
                and all(isinstance(m, QLoRALinear) for m in mods)
                and all(m.active_r <= MAX_FUSED_RANK and m.in_features == mods[0].in_features for m in mods)
                and len({m.lora_A.dtype for m in mods}) == 1
                and not any(m.enable_aqn and m.training for m in mods)
                and not any(_is_dtensor(m.packed_weight_f32.data) or _is_dtensor(m.lora_A) for m in mods)
                and x.dtype == torch.bfloat16 and x.is_cuda)
    if not one_call:
        return [m(x) for m in mods]
    return qlora_linear_multi(x, [(m._forward_quant_weight(), m.lora_A, m.lora_B, m.active_r, m._active_scaling(), m.bias)
                                  for m in mods])


def deregister_qlora_weights_from_fsdp(model: nn.Module, param_names: tuple = ("weight",)) -> int:
    """Drop QLoRALinear parameters from FSDP2 parameter groups so no mixed
    precision cast ever touches the packed bytes; they stay sharded DTensors
    and forward gathers them in fp32 (qlora/utils.py:490-542)."""
    wanted = set(param_names)
    ours = {id(m) for m in model.modules() if isinstance(m, QLoRALinear)}
    removed = 0
    for m in model.modules():
        get_state = getattr(m, "_get_fsdp_state", None)
        if get_state is None:
            continue
        try:
            group = get_state()._fsdp_param_group
        except Exception:
            continue
        if group is None:
            continue
        drop = [fp for fp in group.fsdp_params
                if hasattr(fp, "_module_info") and fp._module_info.param_name in wanted
                and id(fp._module_info.module) in ours]
        for fp in drop:
            group.fsdp_params.remove(fp)
            removed += 1
    return removed
