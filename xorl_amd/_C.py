"""ctypes binding of libxq_hip.so (the C ABI declared in include/xq.h).

There is no CPU fallback: if the library is missing, or a tensor is not on a
HIP device, the call raises.
"""

from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch


_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libxq_hip.so")

XQ_FMT_INT4, XQ_FMT_NVFP4, XQ_FMT_FP8, XQ_FMT_NF4 = 0, 1, 2, 3
XQ_LAYOUT_FLAT, XQ_LAYOUT_GKN = 0, 1
XQ_SCALE_F32, XQ_SCALE_BF16, XQ_SCALE_E4M3 = 0, 1, 2
XQ_DT_BF16, XQ_DT_F32 = 0, 1

FORMATS = {"int4": XQ_FMT_INT4, "nvfp4": XQ_FMT_NVFP4, "block_fp8": XQ_FMT_FP8, "nf4": XQ_FMT_NF4}


class XqWeight(ctypes.Structure):
    _fields_ = [
        ("format", ctypes.c_int32),
        ("layout", ctypes.c_int32),
        ("scale_dtype", ctypes.c_int32),
        ("group", ctypes.c_int32),
        ("rows", ctypes.c_int64),
        ("cols", ctypes.c_int64),
        ("num_experts", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("packed", ctypes.c_void_p),
        ("scales", ctypes.c_void_p),
        ("global_scale", ctypes.c_void_p),
    ]


class XqLinearJob(ctypes.Structure):
    """xq_linear_job of include/xq.h: one of the forwards of xq_linear_fwd_multi."""
    _fields_ = [("w", ctypes.POINTER(XqWeight)), ("lora_A", ctypes.c_void_p), ("lora_B", ctypes.c_void_p), ("r", ctypes.c_int32),
                ("scaling", ctypes.c_float), ("bias_bf16", ctypes.c_void_p), ("y", ctypes.c_void_p), ("ldy", ctypes.c_int64)]


XQ_LINEAR_MULTI_MAX = 4


class XqGroupedLora(ctypes.Structure):
    _fields_ = [("A", ctypes.c_void_p * 3), ("B", ctypes.c_void_p * 3), ("A_experts", ctypes.c_int32 * 3),
                ("B_experts", ctypes.c_int32 * 3), ("dtype", ctypes.c_int32), ("r", ctypes.c_int32),
                ("scaling", ctypes.c_float), ("swiglu_limit", ctypes.c_float)]


class XqGroupedSaved(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in ("xs", "gate_up", "h", "w_row", "su_gate", "su_up", "su_down",
                                               "scatter_index", "offsets", "tile_offsets", "counts", "x_tokens")] + [
                                                   ("ld_x_tokens", ctypes.c_int64)]


class XqGroupedGrads(ctypes.Structure):
    _fields_ = [("dA", ctypes.c_void_p * 3), ("dB", ctypes.c_void_p * 3)]


class XqMlpLora(ctypes.Structure):
    _fields_ = [("A", ctypes.c_void_p * 3), ("B", ctypes.c_void_p * 3), ("bias", ctypes.c_void_p * 3),
                ("dtype", ctypes.c_int32), ("r", ctypes.c_int32), ("scaling", ctypes.c_float), ("reserved", ctypes.c_int32)]


class XqMlpSaved(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in ("gate_up", "h", "su_gate_up", "su_down")] + [
        ("gate_up_fused", ctypes.c_int32), ("reserved", ctypes.c_int32)]


class XqMlpGrads(ctypes.Structure):
    _fields_ = [("dA", ctypes.c_void_p * 3), ("dB", ctypes.c_void_p * 3)]


class XqError(ValueError):
    """Argument error reported by the library before any launch."""


_lib: Optional[ctypes.CDLL] = None

_P, _I64, _I32, _F = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_float
_W = ctypes.POINTER(XqWeight)

_INT = ctypes.c_int
_SIGNATURES = {
    "xq_profile_enable": (_INT, [_INT]),
    "xq_profile_collect": (_INT, [_P, _P, _P]),
    "xq_decode": (_INT, [_W, _P, _INT, _P]),
    "xq_linear_workspace_bytes": (_I64, [_I64, _I64, _I64, _INT]),
    # w, x, ldx, M, A, B, lora_dtype, r, scaling, bias, y, ldy, su_out, ws, ws_bytes, stream
    "xq_linear_fwd": (_INT, [_W, _P, _I64, _I64, _P, _P, _INT, _INT, _F, _P, _P, _I64, _P, _P, _I64, _P]),
    "xq_linear_fwd_swiglu_workspace_bytes": (_I64, [_I64, _I64, _I64, _INT]),
    # w, x, ldx, M, A, B, lora_dtype, r, scaling, bias, h, ldh, ws, ws_bytes, stream
    "xq_linear_fwd_swiglu": (_INT, [_W, _P, _I64, _I64, _P, _P, _INT, _INT, _F, _P, _P, _I64, _P, _I64, _P]),
    # jobs, n_jobs, M
    "xq_linear_fwd_multi_workspace_bytes": (_I64, [_P, _INT, _I64]),
    # jobs, n_jobs, x, ldx, M, lora_dtype, ws, ws_bytes, stream
    "xq_linear_fwd_multi": (_INT, [_P, _INT, _P, _I64, _I64, _INT, _P, _I64, _P]),
    "xq_static_scratch_bytes": (_I64, []),
    # w, x, ldx, M, A, B, lora_dtype, r, scaling, bias, y, ldy, stream
    "xq_linear_fwd_static": (_INT, [_W, _P, _I64, _I64, _P, _P, _INT, _INT, _F, _P, _P, _I64, _P]),
    # w, x, ldx, dy, lddy, M, A, B, lora_dtype, r, scaling, su, dx, lddx, dA, dB, ws, ws_bytes, stream
    "xq_linear_bwd": (_INT, [_W, _P, _I64, _P, _I64, _I64, _P, _P, _INT, _INT, _F, _P, _P, _I64, _P, _P, _P, _I64,
                             _P]),
    # w, A, B, lora_dtype, r, scaling, out, out_dtype, stream
    "xq_merge_workspace_bytes": (_I64, [_I64, _I64, _INT]),
    "xq_merge_dense": (_INT, [_W, _P, _P, _INT, _INT, _F, _P, _INT, _P, _I64, _P]),
    # w, A, B, lora_dtype, r, scaling, packed_out, scales_out, stream
    "xq_merge_requant_fp8": (_INT, [_W, _P, _P, _INT, _INT, _F, _P, _P, _P, _I64, _P]),
    # w, A, B, lora_dtype, r, scaling, amax_out, workspace, workspace_bytes, stream
    "xq_merge_amax": (_INT, [_W, _P, _P, _INT, _INT, _F, _P, _P, _I64, _P]),
    # w, A, B, lora_dtype, r, scaling, global_amax, codes_out, block_scales_out, global_scale_out, workspace, bytes, stream
    "xq_merge_requant_nvfp4": (_INT, [_W, _P, _P, _INT, _INT, _F, _P, _P, _P, _P, _P, _I64, _P]),
    # w, A, B, lora_dtype, r, scaling, codes_out, scales_out, workspace, workspace_bytes, stream
    "xq_merge_requant_nf4": (_INT, [_W, _P, _P, _INT, _INT, _F, _P, _P, _P, _I64, _P]),
    # w, A, B, lora_dtype, r, scaling, symmetric, codes_out, scales_out, workspace, workspace_bytes, stream
    "xq_merge_requant_int4": (_INT, [_W, _P, _P, _INT, _INT, _F, _INT, _P, _P, _P, _I64, _P]),
    # gate, up, ld_in, row_w, h, ld_h, rows, cols, stream
    "xq_silu_mul_fwd": (_INT, [_P, _P, _I64, _P, _P, _I64, _I64, _I64, _P]),
    # gate, up, ld_in, dh, ld_dh, row_w, dgate, dup, ld_out, d_row_w, rows, cols, stream
    "xq_silu_mul_bwd": (_INT, [_P, _P, _I64, _P, _I64, _P, _P, _P, _I64, _P, _I64, _I64, _P]),
    # data, bytes, out, stream
    "xq_read_probe": (_INT, [_P, _I64, _P, _P]),
    "xq_set_tile_policy": (_INT, [_INT]),
    "xq_set_persistent_tiles": (_INT, [_INT]),
    "xq_set_fp8_direct_tiles": (_INT, [_INT]),
    "xq_set_mlp_gate_up_fused": (_INT, [_INT]),
    "xq_get_mlp_gate_up_fused": (_INT, []),
    "xq_set_skinny_one_launch": (_INT, [_INT]),
    "xq_set_skinny_spin_limit": (_INT, [_INT]),
    "xq_set_skinny_gemv": (_INT, [_INT]),
    "xq_skinny_reset": (_INT, []),
    # gave_up, failed_slots, stream
    "xq_skinny_status": (_INT, [_P, _P, _P]),
    "xq_route_workspace_bytes": (_I64, [_I64, _I32]),
    # selected, n_routed, E, counts, offsets, scatter_index, tile_offsets, ws, ws_bytes, stream
    "xq_route_build": (_INT, [_P, _I64, _I32, _P, _P, _P, _P, _P, _I64, _P]),
    "xq_moe_scatter": (_INT, [_P, _I64, _P, _I64, _I32, _I64, _P, _I64, _P]),
    "xq_moe_gather": (_INT, [_P, _P, _I64, _P, _I64, _I32, _I64, _P, _I64, _P]),
    "xq_moe_scatter_scalar": (_INT, [_P, _INT, _P, _I64, _P, _P]),
    "xq_moe_gather_scalar": (_INT, [_P, _P, _I64, _P, _INT, _P]),
    # w, transpose_w, a, lda, n_rows, offsets, tile_offsets, su, lora_right, r_pad, y, ldy, stream
    "xq_grouped_gemm": (_INT, [_W, _INT, _P, _I64, _I64, _P, _P, _P, _P, _INT, _P, _I64, _P]),
    # in, in_dtype, rows_in, cols_in, transpose, out, rows_out, cols_out, E, stream
    "xq_factor_prep": (_INT, [_P, _INT, _I64, _I64, _INT, _P, _I64, _I64, _I64, _P]),
    # a, lda, n_rows, offsets, tile_offsets, E, F, shared, r_pad, K, scale, t, stream
    "xq_grouped_lora_down": (_INT, [_P, _I64, _I64, _P, _P, _I32, _P, _INT, _INT, _I64, _F, _P, _P]),
    "xq_lora_wgrad_workspace_bytes": (_I64, [_I64, _I64, _INT]),
    # P, ldp, p_width, Q, r_pad, r_out, n_rows, offsets, E, transpose_out, out, ws, row_limit, stream
    "xq_grouped_lora_wgrad": (_INT, [_P, _I64, _I64, _P, _INT, _INT, _I64, _P, _I32, _INT, _P, _P, _P, _P]),
    "xq_grouped_workspace_bytes": (_I64, [_I64, _I32, _I32, _I64, _I64, _INT, _INT]),
    "xq_grouped_in_place": (_INT, [_W, _W, _W]),
    # gate, up, down, lora, hidden, ld_hidden, n_tokens, routing_w, rw_dtype, selected, topk, out, ld_out, saved, ws, ws_bytes, stream
    "xq_grouped_fwd": (_INT, [_W, _W, _W, ctypes.POINTER(XqGroupedLora), _P, _I64, _I64, _P, _INT, _P, _I32, _P, _I64,
                              ctypes.POINTER(XqGroupedSaved), _P, _I64, _P]),
    # gate, up, down, lora, dy, ld_dy, n_tokens, topk, saved, dx, ld_dx, d_routing, rw_dtype, grads, ws, ws_bytes, stream
    "xq_grouped_bwd": (_INT, [_W, _W, _W, ctypes.POINTER(XqGroupedLora), _P, _I64, _I64, _I32,
                              ctypes.POINTER(XqGroupedSaved), _P, _I64, _P, _INT, ctypes.POINTER(XqGroupedGrads), _P, _I64,
                              _P]),
    "xq_grouped_infer_supported": (_INT, [_W, _W, _W, _I64, _I32, _INT]),
    "xq_grouped_infer_workspace_bytes": (_I64, [_I64, _I32, _I32, _I64, _I64, _INT]),
    # gate, up, down, lora, hidden, ld_hidden, n_tokens, routing_w, rw_dtype, selected, topk, out, ld_out, ws, ws_bytes, stream
    "xq_grouped_fwd_infer": (_INT, [_W, _W, _W, ctypes.POINTER(XqGroupedLora), _P, _I64, _I64, _P, _INT, _P, _I32, _P, _I64,
                                    _P, _I64, _P]),
    "xq_mlp_workspace_bytes": (_I64, [_I64, _I64, _I64, _INT, _INT]),
    "xq_mlp_infer_workspace_bytes": (_I64, [_I64, _I64, _I64, _INT]),
    # gate, up, down, lora, x, ldx, M, y, ldy, ws, ws_bytes, stream
    "xq_mlp_fwd_infer": (_INT, [_W, _W, _W, ctypes.POINTER(XqMlpLora), _P, _I64, _I64, _P, _I64, _P, _I64, _P]),
    # gate, up, down, lora, x, ldx, M, y, ldy, saved, ws, ws_bytes, stream
    "xq_mlp_fwd": (_INT, [_W, _W, _W, ctypes.POINTER(XqMlpLora), _P, _I64, _I64, _P, _I64, ctypes.POINTER(XqMlpSaved), _P,
                          _I64, _P]),
    # gate, up, down, lora, x, ldx, dy, lddy, M, saved, dx, lddx, grads, ws, ws_bytes, stream
    "xq_mlp_bwd": (_INT, [_W, _W, _W, ctypes.POINTER(XqMlpLora), _P, _I64, _P, _I64, _I64, ctypes.POINTER(XqMlpSaved), _P,
                          _I64, ctypes.POINTER(XqMlpGrads), _P, _I64, _P]),
}

EXPORTS = ("xq_version", "xq_last_error") + tuple(_SIGNATURES)


def lib() -> ctypes.CDLL:
    """Load libxq_hip.so; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m xorl_amd.csrc.build` "
                "(there is no CPU or eager fallback for the QLoRA kernels)"
            )
        L = ctypes.CDLL(LIB_PATH)
        L.xq_version.restype = ctypes.c_char_p
        L.xq_last_error.restype = ctypes.c_char_p
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        msg = lib().xq_last_error().decode()
        if rc == -3:
            raise RuntimeError(msg)
        raise XqError(msg)


def require_hip(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and t.device.type != "cuda":
            raise RuntimeError(
                f"xorl_amd kernels run on a HIP device only; got a tensor on {t.device} "
                "(there is no CPU fallback)"
            )


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def stream_ptr(device: torch.device) -> int:
    """Raw handle of torch's current stream on `device` (what every kernel is launched on)."""
    idx = device.index
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if idx is None else idx)


_SCALE_DT = {torch.float32: XQ_SCALE_F32, torch.bfloat16: XQ_SCALE_BF16, torch.float8_e4m3fn: XQ_SCALE_E4M3}


def make_weight(
    fmt: str,
    layout: int,
    packed: torch.Tensor,
    scales: torch.Tensor,
    scale_dtype: torch.dtype,
    rows: int,
    cols: int,
    group: int,
    global_scale: Optional[torch.Tensor] = None,
    num_experts: int = 1,
) -> XqWeight:
    """Describe a (bank of) quantized matrices.  `packed`/`scales` may be any
    dtype view of the right bytes (uint8 buffers, fp32-packed parameters);
    `scale_dtype` is the true element type of the scales."""
    require_hip(packed, scales, global_scale)
    if not packed.is_contiguous() or not scales.is_contiguous():
        raise XqError("packed weights and scales must be contiguous")
    w = XqWeight()
    w.format = FORMATS[fmt]
    w.layout = layout
    w.scale_dtype = _SCALE_DT[scale_dtype]
    w.group = group
    w.rows, w.cols = rows, cols
    w.num_experts = num_experts
    w.packed = packed.data_ptr()
    w.scales = scales.data_ptr()
    w.global_scale = None if global_scale is None else global_scale.data_ptr()
    nbytes = rows * cols if fmt == "block_fp8" else rows * cols // 2
    if packed.numel() * packed.element_size() != nbytes * num_experts:
        raise XqError(
            f"packed buffer holds {packed.numel() * packed.element_size()} bytes, "
            f"expected {nbytes * num_experts} for {num_experts} x [{rows}, {cols}] {fmt}"
        )
    # the kernels index the scales by shape alone: a buffer of another size or element type than `scale_dtype`
    # says (a state_dict load into differently typed storage, say) would be read out of bounds
    esz = {XQ_SCALE_F32: 4, XQ_SCALE_BF16: 2, XQ_SCALE_E4M3: 1}[w.scale_dtype]
    if fmt == "block_fp8":
        if scale_dtype != torch.float32:
            raise XqError(f"block_fp8 scales are fp32, got {scale_dtype}")
        sbytes = -(-rows // 128) * -(-cols // 128) * 4
    else:
        if group <= 0 or (rows * cols) % group:
            raise XqError(f"group {group} does not divide [{rows}, {cols}]")
        sbytes = rows * cols // group * esz
    have = scales.numel() * scales.element_size()
    if have != sbytes * num_experts:
        raise XqError(f"scale buffer holds {have} bytes, expected {sbytes * num_experts} for {num_experts} x "
                      f"[{rows}, {cols}] {fmt} with {scale_dtype} scales (group {group})")
    if fmt == "nvfp4":
        if global_scale is None or global_scale.dtype != torch.float32 or global_scale.numel() < num_experts \
                or not global_scale.is_contiguous():
            raise XqError(f"nvfp4 needs a contiguous fp32 global_scale with {num_experts} element(s)")
    return w
