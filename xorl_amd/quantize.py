"""Codec functions with the names and signatures of ``xorl.ops.quantize``.

Dequantizers launch the HIP decode kernels (``xq_decode``); they are bit-exact
with the reference's Triton decoders.  Quantizers run once at load / merge
time, are plain torch ops (IEEE fp32) on whatever device the tensor lives on,
and restate the reference quantizers' arithmetic:

  int4_quantize[_gkn]        ops/quantize/int4_quantize.py:97-110, int4_gkn_quantize.py:137-173
  int4_quantize_sym          the symmetric absmax/7 bf16-scale rule (not in the reference)
  nvfp4_quantize[_gkn]       ops/quantize/nvfp4_quantize.py:114-154, nvfp4_gkn_quantize.py:176-235
  block_fp8_quantize_gkn     ops/quantize/block_fp8_gkn_quantize.py:73-121
  nf4_quantize[_gkn], nf4_dequantize[_gkn]   ops/quantize/nf4_quantize.py, nf4_gkn_quantize.py, nf4_codec.py
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _C


FP4_E2M1_MAX = 6.0
FP8_E4M3_MAX = 448.0


# ---------------------------------------------------------------------------
# decode (HIP)
# ---------------------------------------------------------------------------
def _decode(w: _C.XqWeight, out: Tensor, out_dtype: int) -> Tensor:
    import ctypes

    _C.check(_C.lib().xq_decode(ctypes.byref(w), out.data_ptr(), out_dtype, _C.stream_ptr(out.device)))
    return out


def int4_dequantize(packed: Tensor, scales: Tensor, M: int, K: int, group_size: int = -1,
                    out_dtype: torch.dtype = torch.bfloat16) -> Tensor:
    """[M, K/2] u8 + [M, K/gs] scales (fp32 or bf16) -> [M, K] bf16."""
    gs = K if group_size == -1 else group_size
    w = _C.make_weight("int4", _C.XQ_LAYOUT_FLAT, packed, scales, scales.dtype, M, K, gs)
    out = _decode(w, torch.empty(M, K, dtype=torch.bfloat16, device=packed.device), _C.XQ_DT_BF16)
    return out if out_dtype == torch.bfloat16 else out.to(out_dtype)


def int4_dequantize_gkn(packed: Tensor, scales: Tensor, K: int, N: int, group_size: int = -1,
                        out_dtype: torch.dtype = torch.bfloat16) -> Tensor:
    """[K/2, N] u8 + [K/gs, N] scales -> [K, N] bf16 (groups and nibble pairs along K)."""
    gs = K if group_size == -1 else group_size
    w = _C.make_weight("int4", _C.XQ_LAYOUT_GKN, packed, scales, scales.dtype, K, N, gs)
    out = _decode(w, torch.empty(K, N, dtype=torch.bfloat16, device=packed.device), _C.XQ_DT_BF16)
    return out if out_dtype == torch.bfloat16 else out.to(out_dtype)


def nf4_dequantize(packed: Tensor, scales: Tensor, num_elements: int, group_size: int = 64) -> Tensor:
    """Flat decode of `num_elements` NF4 values -> 1-D bf16 (ops/quantize/nf4_quantize.py:154-185)."""
    assert num_elements % group_size == 0
    sc = scales if scales.dtype in (torch.float32, torch.bfloat16) else scales.float()
    w = _C.make_weight("nf4", _C.XQ_LAYOUT_FLAT, packed.reshape(-1), sc.reshape(-1), sc.dtype, 1, num_elements, group_size)
    return _decode(w, torch.empty(num_elements, dtype=torch.bfloat16, device=packed.device), _C.XQ_DT_BF16)


def nf4_dequantize_gkn(packed: Tensor, scales: Tensor, K: int, N: int, group_size: int = 64) -> Tensor:
    """[K/2, N] u8 + [K/gs, N] scales -> [K, N] bf16 (ops/quantize/nf4_gkn_quantize.py:182-)."""
    sc = scales if scales.dtype in (torch.float32, torch.bfloat16) else scales.float()
    w = _C.make_weight("nf4", _C.XQ_LAYOUT_GKN, packed, sc, sc.dtype, K, N, group_size)
    return _decode(w, torch.empty(K, N, dtype=torch.bfloat16, device=packed.device), _C.XQ_DT_BF16)


def nvfp4_dequantize(packed: Tensor, block_scales: Tensor, global_scale: Tensor, num_elements: int,
                     block_size: int = 16) -> Tensor:
    """Flat decode of `num_elements` values -> 1-D bf16 (caller reshapes)."""
    assert num_elements % block_size == 0
    gs = global_scale.reshape(1) if global_scale.numel() == 1 else global_scale
    w = _C.make_weight("nvfp4", _C.XQ_LAYOUT_FLAT, packed, block_scales, block_scales.dtype,
                       1, num_elements, block_size, global_scale=gs.float())
    return _decode(w, torch.empty(num_elements, dtype=torch.bfloat16, device=packed.device), _C.XQ_DT_BF16)


def nvfp4_dequantize_gkn(packed: Tensor, block_scales: Tensor, global_scale: Tensor, K: int, N: int,
                         block_size: int = 16) -> Tensor:
    gs = global_scale.reshape(1) if global_scale.numel() == 1 else global_scale
    w = _C.make_weight("nvfp4", _C.XQ_LAYOUT_GKN, packed, block_scales, block_scales.dtype,
                       K, N, block_size, global_scale=gs.float())
    return _decode(w, torch.empty(K, N, dtype=torch.bfloat16, device=packed.device), _C.XQ_DT_BF16)


def block_fp8_dequantize_gkn(x: Tensor, s: Tensor, block_size: int = 128,
                             out_dtype: Optional[torch.dtype] = None) -> Tensor:
    """e4m3 [R, C] * fp32 scale [ceil(R/128), ceil(C/128)].  Like the reference
    the result is fp32 (the default dtype) unless out_dtype=torch.bfloat16,
    which fuses the `.to(bf16)` every caller applies."""
    assert x.dim() == 2 and s.dim() == 2 and x.is_contiguous() and s.is_contiguous()
    R, Cc = x.shape
    dt = out_dtype or torch.float32
    w = _C.make_weight("block_fp8", _C.XQ_LAYOUT_FLAT, x, s, torch.float32, R, Cc, block_size)
    out = torch.empty(R, Cc, dtype=dt, device=x.device)
    return _decode(w, out, _C.XQ_DT_F32 if dt == torch.float32 else _C.XQ_DT_BF16)


# ---------------------------------------------------------------------------
# quantizers (torch, load-time)
# ---------------------------------------------------------------------------
def _pack_nibbles_last(q: Tensor) -> Tensor:
    """[..., 2n] codes -> [..., n] bytes, even element in the low nibble."""
    q = q.to(torch.uint8)
    return q[..., 0::2] | (q[..., 1::2] << 4)


def _pack_nibbles_first(q: Tensor) -> Tensor:
    """[2k, N] codes -> [k, N] bytes, even K-row in the low nibble."""
    q = q.to(torch.uint8)
    return q[0::2] | (q[1::2] << 4)


# NF4 levels and the midpoints between neighbours (ops/quantize/nf4_codec.py:18-35, :42-64)
NF4_TABLE = (-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
             -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
             0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
             0.7229568362236023, 1.0)
NF4_MIN_STEP = 0.07958029955625534
_NF4_MIDPOINTS = (-0.8480964004993439, -0.6106329262256622, -0.4599952697753906, -0.3396794348955154,
                  -0.2346074059605598, -0.1379117332398891, -0.0455250181257725, 0.0397901497781277,
                  0.1202552504837513, 0.2035212516784668, 0.2920137718319893, 0.3893125355243683,
                  0.5016634166240692, 0.6427869200706482, 0.8614784181118012)


def _const(like: Tensor, v: float) -> Tensor:
    """`v` as a 0-dim fp32 tensor on `like`'s device.  Quotients are taken between tensors so that they are one
    IEEE division on every device: torch turns a Python-scalar divisor into a multiplication by its rounded
    reciprocal on the GPU, and a Python-scalar numerator into reciprocal-then-multiply everywhere (two roundings)."""
    return torch.tensor(v, dtype=torch.float32, device=like.device)


def _nf4_encode(norm: Tensor) -> Tensor:
    """code = number of midpoints strictly below the value (nf4_codec.py:42-64)."""
    mid = torch.tensor(_NF4_MIDPOINTS, dtype=torch.float32, device=norm.device)
    return (norm.unsqueeze(-1) > mid).sum(-1).to(torch.uint8)


def nf4_quantize(x: Tensor, group_size: int = 64) -> Tuple[Tensor, Tensor]:
    """[M, K] -> flat (M*K/2,) u8, flat (M*K/gs,) fp32 absmax scales (nf4_quantize.py:20-56, :118-151):
    scale = max(amax, 1e-12); code = encode(clamp(x * (1/scale), -1, 1)); even element in the low nibble."""
    assert x.dim() == 2
    n = x.numel()
    assert n % group_size == 0 and group_size % 2 == 0
    xf = x.float().reshape(n // group_size, group_size)
    scale = xf.abs().amax(-1).clamp_min(1e-12)
    norm = (xf * (_const(scale, 1.0) / scale).unsqueeze(-1)).clamp_(-1.0, 1.0)
    codes = _nf4_encode(norm).reshape(-1)
    return (codes[0::2] | (codes[1::2] << 4)).contiguous(), scale.contiguous()


def nf4_quantize_gkn(x: Tensor, group_size: int = 64) -> Tuple[Tensor, Tensor]:
    """[K, N] -> [K/2, N] u8, [K/gs, N] fp32 scales; groups and nibble pairs along K
    (nf4_gkn_quantize.py:22-81, :145-179)."""
    assert x.dim() == 2
    K, N = x.shape
    assert K % group_size == 0 and group_size % 2 == 0
    xf = x.float().reshape(K // group_size, group_size, N)
    scale = xf.abs().amax(1).clamp_min(1e-12)
    norm = (xf * (_const(scale, 1.0) / scale).unsqueeze(1)).clamp_(-1.0, 1.0)
    codes = _nf4_encode(norm).reshape(K, N)
    return _pack_nibbles_first(codes).contiguous(), scale.contiguous()


def int4_quantize(x: Tensor, group_size: int = -1) -> Tuple[Tensor, Tensor]:
    assert x.dim() == 2
    M, K = x.shape
    gs = K if group_size == -1 else group_size
    assert K % gs == 0 and gs % 2 == 0
    xf = x.float().reshape(M, K // gs, gs)
    scale = xf.abs().amax(-1).clamp_min(1e-12) * torch.tensor(2.0 / 15.0, dtype=torch.float32, device=x.device)
    inv = _const(scale, 1.0) / scale
    q = (xf * inv.unsqueeze(-1) + 8.5).to(torch.int32).clamp_(0, 15)
    return _pack_nibbles_last(q.reshape(M, K)), scale


def int4_quantize_gkn(x: Tensor, group_size: int = -1) -> Tuple[Tensor, Tensor]:
    assert x.dim() == 2
    K, N = x.shape
    gs = K if group_size == -1 else group_size
    assert K % gs == 0 and gs % 2 == 0
    xf = x.float().reshape(K // gs, gs, N)
    scale = xf.abs().amax(1).clamp_min(1e-12) * torch.tensor(2.0 / 15.0, dtype=torch.float32, device=x.device)
    inv = _const(scale, 1.0) / scale
    q = (xf * inv.unsqueeze(1) + 8.5).to(torch.int32).clamp_(0, 15)
    return _pack_nibbles_first(q.reshape(K, N)), scale


def int4_quantize_sym(x: Tensor, group_size: int = 128) -> Tuple[Tensor, Tensor]:
    """Symmetric int4: scale = bf16(absmax/7), q = clamp(rne(w/scale), -7, 7) + 8."""
    M, K = x.shape
    assert K % group_size == 0
    xf = x.float().reshape(M, K // group_size, group_size)
    scale = (xf.abs().amax(-1) / _const(xf, 7.0)).to(torch.bfloat16)
    sf = scale.float().unsqueeze(-1)
    q = torch.where(sf > 0, torch.round(xf / sf).clamp_(-7, 7), torch.zeros_like(xf)).to(torch.int32) + 8
    return _pack_nibbles_last(q.reshape(M, K)), scale


def _fp4_encode(v: Tensor) -> Tensor:
    """ops/quantize/fp4_codec.py:12-19 (ties up in magnitude)."""
    sign = (v < 0).to(torch.int32) * 8
    a = v.abs()
    lo = (a * 2.0 + 0.5).to(torch.int32).clamp_max(3)
    hi = 4 + (a >= 2.5).to(torch.int32) + (a >= 3.5).to(torch.int32) + (a >= 5.0).to(torch.int32)
    return torch.where(a >= 1.75, hi, lo) + sign


def _e4m3_satfinite(t: Tensor) -> Tensor:
    return t.clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX).to(torch.float8_e4m3fn)


def _nvfp4_scales(amax: Tensor, global_amax: Optional[Tensor]):
    gamax = amax.max().reshape(1) if global_amax is None else global_amax.float().reshape(1).to(amax.device)
    gamax = gamax.clamp_min(1e-12)
    block_scales = _e4m3_satfinite(amax / gamax * FP8_E4M3_MAX)
    global_scale = gamax * torch.tensor(1.0 / FP4_E2M1_MAX, dtype=torch.float32, device=amax.device) / _const(amax, FP8_E4M3_MAX)
    return block_scales, global_scale


def nvfp4_quantize(x: Tensor, block_size: int = 16, global_amax: Optional[Tensor] = None):
    """-> packed u8 [n/2] (flat), e4m3 block scales [n/block], global scale fp32 [1]."""
    assert x.dim() == 2
    n = x.numel()
    assert n % block_size == 0 and block_size % 2 == 0
    xf = x.float().reshape(-1, block_size)
    amax = xf.abs().amax(-1).clamp_min(1e-12)
    scaled = (xf * (_const(amax, 6.0) / amax).unsqueeze(-1)).clamp_(-6.0, 6.0)
    packed = _pack_nibbles_last(_fp4_encode(scaled).reshape(-1))
    block_scales, global_scale = _nvfp4_scales(amax, global_amax)
    return packed, block_scales, global_scale


def nvfp4_quantize_gkn(x: Tensor, block_size: int = 16, global_amax: Optional[Tensor] = None):
    """[K, N] -> packed [K/2, N], e4m3 block scales [K/block, N], global [1]."""
    assert x.dim() == 2
    K, N = x.shape
    assert K % block_size == 0 and block_size % 2 == 0
    xf = x.float().reshape(K // block_size, block_size, N)
    amax = xf.abs().amax(1).clamp_min(1e-12)
    scaled = (xf * (_const(amax, 6.0) / amax).unsqueeze(1)).clamp_(-6.0, 6.0)
    packed = _pack_nibbles_first(_fp4_encode(scaled).reshape(K, N))
    block_scales, global_scale = _nvfp4_scales(amax.reshape(-1), global_amax)
    return packed, block_scales.reshape(K // block_size, N), global_scale


def block_fp8_quantize_gkn(x: Tensor, block_size: int = 128, amax_scale: float = 1.0):
    """[R, C] -> e4m3 [R, C], fp32 scales [ceil(R/bs), ceil(C/bs)] (edge tiles partial)."""
    assert x.is_contiguous() and x.dim() == 2
    if amax_scale <= 0.0:
        raise ValueError(f"amax_scale must be positive, got {amax_scale}")
    R, Cc = x.shape
    bs = block_size
    pr, pc = (-R) % bs, (-Cc) % bs
    xf = x.float()
    if pr or pc:
        xf = torch.nn.functional.pad(xf, (0, pc, 0, pr))
    nr, nc = xf.shape[0] // bs, xf.shape[1] // bs
    blocks = xf.reshape(nr, bs, nc, bs)
    s = (blocks.abs().amax(dim=(1, 3)) * amax_scale / _const(xf, FP8_E4M3_MAX)).clamp_min(1e-12)
    y = (blocks / s[:, None, :, None]).clamp_(-FP8_E4M3_MAX, FP8_E4M3_MAX).to(torch.float8_e4m3fn)
    y = y.reshape(nr * bs, nc * bs)[:R, :Cc].contiguous()
    return y, s
