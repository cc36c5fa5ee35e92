"""PyTorch-ROCm custom ops and autograd functions over the C ABI.

Ops are registered for the HIP ("cuda") dispatch key only: calling them with
CPU tensors raises from the dispatcher -- there is no CPU or eager fallback.
Outputs and workspaces are allocated here with torch (device memory is
plumbing); the kernels allocate nothing.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
from torch import Tensor

from . import _C


_CODE_TO_DT = {0: torch.float32, 1: torch.bfloat16, 2: torch.float8_e4m3fn}
_DT_TO_CODE = {v: k for k, v in _CODE_TO_DT.items()}


@dataclass
class QuantWeight:
    """Host-side description of a (bank of) quantized matrices.

    packed / scales are tensors holding the right BYTES (uint8 buffers or the
    bytes-in-fp32 parameter the modules keep for FSDP2); scale_dtype is the
    true element type of the scales.  rows x cols is the decoded shape:
    [out, in] for dense (FLAT), [in, out] per expert for banks (GKN)."""

    fmt: str
    layout: int
    packed: Tensor
    scales: Tensor
    scale_dtype: torch.dtype
    rows: int
    cols: int
    group: int
    global_scale: Optional[Tensor] = None
    num_experts: int = 1
    _cw: Optional[_C.XqWeight] = None

    def c(self) -> _C.XqWeight:
        """The C descriptor (built once per QuantWeight: it holds raw pointers into the tensors above)."""
        if self._cw is None:
            self._cw = _C.make_weight(self.fmt, self.layout, self.packed, self.scales, self.scale_dtype, self.rows,
                                      self.cols, self.group, self.global_scale, self.num_experts)
        return self._cw


def _r_pad(r: int) -> int:
    return 0 if r <= 0 else ((r + 15) // 16) * 16


def _lora_dt(t: Optional[Tensor]) -> int:
    if t is None or t.dtype == torch.float32:
        return _C.XQ_DT_F32
    if t.dtype == torch.bfloat16:
        return _C.XQ_DT_BF16
    raise _C.XqError(f"LoRA factors must be fp32 or bf16, got {t.dtype}")


def _as_2d(x: Tensor) -> Tensor:
    x2 = x.reshape(-1, x.shape[-1])
    if torch.compiler.is_compiling():      # addresses are not traceable: a traced call always takes a packed copy
        return x2.contiguous()
    if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) % 8 != 0) or x2.data_ptr() % 16 != 0:
        x2 = x2.contiguous()
    return x2


def _ld(x2: Tensor) -> int:
    return x2.stride(0) if x2.shape[0] > 1 else x2.shape[1]


# ---------------------------------------------------------------------------
# dense: custom ops
# ---------------------------------------------------------------------------
_WS_BYTES: dict = {}
_EMPTY: dict = {}


def _workspace_bytes(M: int, N: int, K: int, r: int) -> int:
    key = (M, N, K, r)
    v = _WS_BYTES.get(key)
    if v is None:
        v = _WS_BYTES[key] = _C.lib().xq_linear_workspace_bytes(M, N, K, r)
    return v


# ---- failure reports of the one-launch decode kernel (M <= 16 with a LoRA term).  Its blocks pass the low-rank
# intermediate to each other through device memory with bounded waits; a wait that gives up writes NaN and counts itself
# in device memory, where xq_skinny_status() finds it.  Reading the count waits for the stream, so it is done where the
# host waits anyway: by the caller (`skinny_status()` next to its own synchronisation) and, as a backstop, here after
# every SKINNY_CHECK_EVERY forward-only calls of at most 16 rows.
SKINNY_CHECK_EVERY = 1024
_skinny_calls = 0


def skinny_status(device=None, raise_on_failure: bool = True) -> Tuple[int, int]:
    """(blocks whose wait gave up, slots marked failed) reported by the one-launch decode forwards on `device` since the
    last call; waits for the current stream.  Anything non-zero means forwards since the last call may hold NaN: the
    library has then already cleared the marks (later forwards are exact again) and this raises ``RuntimeError`` unless
    told not to."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    gave_up, failed = ctypes.c_int(0), ctypes.c_int(0)
    with torch.cuda.device(dev):
        _C.check(_C.lib().xq_skinny_status(ctypes.byref(gave_up), ctypes.byref(failed), _C.stream_ptr(dev)))
    if raise_on_failure and (gave_up.value or failed.value):
        raise RuntimeError(f"xorl_amd: {gave_up.value} block(s) of one-launch decode forwards gave up waiting and wrote NaN "
                           f"({failed.value} exchange slot(s) were marked failed) since the last check; the marks are cleared, "
                           "repeat the affected forwards")
    return gave_up.value, failed.value


def _note_decode_forward(dev, M: int) -> None:
    global _skinny_calls
    if M > 16:
        return
    _skinny_calls += 1
    if _skinny_calls >= SKINNY_CHECK_EVERY and not torch.cuda.is_current_stream_capturing():
        _skinny_calls = 0
        skinny_status(dev)


def _linear_fwd_impl(x: Tensor, packed: Tensor, scales: Tensor, global_scale: Optional[Tensor],
                     lora_A: Optional[Tensor], lora_B: Optional[Tensor], bias: Optional[Tensor],
                     fmt: str, scale_dt: torch.dtype, group: int, N: int, K: int, r: int,
                     scaling: float, want_su: bool, cw: Optional[_C.XqWeight] = None) -> Tuple[Tensor, Tensor]:
    if x.dtype != torch.bfloat16:
        raise _C.XqError(f"activations must be bf16, got {x.dtype}")
    x2 = _as_2d(x)
    M = x2.shape[0]
    if x2.shape[1] != K:
        raise _C.XqError(f"input width {x2.shape[1]} != in_features {K}")
    w = cw if cw is not None else _C.make_weight(fmt, _C.XQ_LAYOUT_FLAT, packed, scales, scale_dt, N, K, group, global_scale)
    dev = x.device
    y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    rp = _r_pad(r)
    if want_su:
        su = torch.empty(M, rp, dtype=torch.bfloat16, device=dev)
    else:
        su = _EMPTY.get(dev)
        if su is None:
            su = _EMPTY[dev] = torch.empty(0, dtype=torch.bfloat16, device=dev)
    ws_bytes = _workspace_bytes(M, N, K, r)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    A = lora_A.contiguous() if lora_A is not None else None
    B = lora_B.contiguous() if lora_B is not None else None
    b = bias.to(torch.bfloat16).contiguous() if bias is not None else None
    _C.check(_C.lib().xq_linear_fwd(ctypes.byref(w), x2.data_ptr(), _ld(x2), M, _C.ptr(A), _C.ptr(B), _lora_dt(A), r,
                                    scaling, _C.ptr(b), y.data_ptr(), N, su.data_ptr() if (rp and want_su) else None,
                                    ws.data_ptr(), ws_bytes, _C.stream_ptr(dev)))
    if not want_su:
        _note_decode_forward(dev, M)
    return y.reshape(*x.shape[:-1], N), su


@torch.library.custom_op("xq::linear_fwd", mutates_args=(), device_types="cuda")
def _linear_fwd_op(x: Tensor, packed: Tensor, scales: Tensor, global_scale: Optional[Tensor],
                   lora_A: Optional[Tensor], lora_B: Optional[Tensor], bias: Optional[Tensor],
                   fmt: str, scale_code: int, group: int, N: int, K: int, r: int,
                   scaling: float, want_su: bool) -> Tuple[Tensor, Tensor]:
    return _linear_fwd_impl(x, packed, scales, global_scale, lora_A, lora_B, bias, fmt, _CODE_TO_DT[scale_code],
                            group, N, K, r, scaling, want_su)


@_linear_fwd_op.register_fake
def _(x, packed, scales, global_scale, lora_A, lora_B, bias, fmt, scale_code, group, N, K, r, scaling, want_su):
    M = x.numel() // max(x.shape[-1], 1)
    return x.new_empty(*x.shape[:-1], N), x.new_empty(M if want_su else 0, _r_pad(r))


def _linear_bwd_impl(dy: Tensor, x: Tensor, su: Tensor, packed: Tensor, scales: Tensor,
                     global_scale: Optional[Tensor], lora_A: Optional[Tensor], lora_B: Optional[Tensor],
                     fmt: str, scale_dt: torch.dtype, group: int, N: int, K: int, r: int, scaling: float,
                     need_dx: bool, need_dA: bool, need_dB: bool,
                     cw: Optional[_C.XqWeight] = None) -> Tuple[Tensor, Tensor, Tensor]:
    dy2 = _as_2d(dy.to(torch.bfloat16))
    x2 = _as_2d(x)
    M = dy2.shape[0]
    w = cw if cw is not None else _C.make_weight(fmt, _C.XQ_LAYOUT_FLAT, packed, scales, scale_dt, N, K, group, global_scale)
    dev = dy.device
    dx = torch.empty(M, K, dtype=torch.bfloat16, device=dev) if need_dx else torch.empty(0, dtype=torch.bfloat16, device=dev)
    dA = torch.empty(r, K, dtype=torch.float32, device=dev) if need_dA else torch.empty(0, device=dev)
    dB = torch.empty(N, r, dtype=torch.float32, device=dev) if need_dB else torch.empty(0, device=dev)
    L = _C.lib()
    ws_bytes = _workspace_bytes(M, N, K, r)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    A = lora_A.contiguous() if lora_A is not None else None
    B = lora_B.contiguous() if lora_B is not None else None
    _C.check(L.xq_linear_bwd(ctypes.byref(w), x2.data_ptr(), _ld(x2), dy2.data_ptr(), _ld(dy2), M, _C.ptr(A),
                             _C.ptr(B), _lora_dt(A), r, scaling, su.data_ptr() if su.numel() else None,
                             dx.data_ptr() if need_dx else None, K, dA.data_ptr() if need_dA else None,
                             dB.data_ptr() if need_dB else None, ws.data_ptr(), ws_bytes, _C.stream_ptr(dev)))
    if need_dx:
        dx = dx.reshape(x.shape)
    return dx, dA, dB


@torch.library.custom_op("xq::linear_bwd", mutates_args=(), device_types="cuda")
def _linear_bwd_op(dy: Tensor, x: Tensor, su: Tensor, packed: Tensor, scales: Tensor,
                   global_scale: Optional[Tensor], lora_A: Optional[Tensor], lora_B: Optional[Tensor],
                   fmt: str, scale_code: int, group: int, N: int, K: int, r: int, scaling: float,
                   need_dx: bool, need_dA: bool, need_dB: bool) -> Tuple[Tensor, Tensor, Tensor]:
    return _linear_bwd_impl(dy, x, su, packed, scales, global_scale, lora_A, lora_B, fmt, _CODE_TO_DT[scale_code],
                            group, N, K, r, scaling, need_dx, need_dA, need_dB)


@_linear_bwd_op.register_fake
def _(dy, x, su, packed, scales, global_scale, lora_A, lora_B, fmt, scale_code, group, N, K, r, scaling,
      need_dx, need_dA, need_dB):
    return (x.new_empty(x.shape) if need_dx else x.new_empty(0),
            x.new_empty(r, K, dtype=torch.float32) if need_dA else x.new_empty(0, dtype=torch.float32),
            x.new_empty(N, r, dtype=torch.float32) if need_dB else x.new_empty(0, dtype=torch.float32))


class QLoRALinearFunction(torch.autograd.Function):
    """y = x . deq(W)^T + bias + s * (x . A^T) . B^T with the packed weight decoded inside the GEMM.

    Backward returns (dx, dA, dB); the frozen packed weight gets no gradient
    (qlora/modules/block_fp8_linear.py:48-51).  Nothing but x and the small
    [M, r] LoRA intermediate is saved -- no decoded weight."""

    @staticmethod
    def forward(ctx, x, lora_A, lora_B, bias, qw: QuantWeight, r: int, scaling: float, want_su: bool = True):
        A = lora_A[:r] if lora_A is not None else None
        B = lora_B[:, :r] if lora_B is not None else None
        if torch.compiler.is_compiling():
            y, su = _linear_fwd_op(x, qw.packed, qw.scales, qw.global_scale, A, B, bias, qw.fmt,
                                   _DT_TO_CODE[qw.scale_dtype], qw.group, qw.rows, qw.cols, r, float(scaling), want_su)
        else:       # eager: straight to the library (the custom-op layer costs tens of microseconds of host time per call)
            y, su = _linear_fwd_impl(x, qw.packed, qw.scales, qw.global_scale, A, B, bias, qw.fmt, qw.scale_dtype,
                                     qw.group, qw.rows, qw.cols, r, float(scaling), want_su, qw.c())
        ctx.qw, ctx.r, ctx.scaling = qw, r, float(scaling)
        ctx.save_for_backward(x, su, lora_A, lora_B)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, su, lora_A, lora_B = ctx.saved_tensors
        qw, r = ctx.qw, ctx.r
        need_dx, need_dA, need_dB = ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.needs_input_grad[2]
        A = lora_A[:r] if lora_A is not None else None
        B = lora_B[:, :r] if lora_B is not None else None
        if torch.compiler.is_compiling():
            dx, dA, dB = _linear_bwd_op(dy, x, su, qw.packed, qw.scales, qw.global_scale, A, B, qw.fmt,
                                        _DT_TO_CODE[qw.scale_dtype], qw.group, qw.rows, qw.cols, r, ctx.scaling,
                                        need_dx, need_dA, need_dB)
        else:
            dx, dA, dB = _linear_bwd_impl(dy, x, su, qw.packed, qw.scales, qw.global_scale, A, B, qw.fmt,
                                          qw.scale_dtype, qw.group, qw.rows, qw.cols, r, ctx.scaling,
                                          need_dx, need_dA, need_dB, qw.c())
        gA = gB = None
        if need_dA:
            gA = dA if lora_A.shape[0] == r else torch.cat([dA, dA.new_zeros(lora_A.shape[0] - r, dA.shape[1])], 0)
            gA = gA.to(lora_A.dtype)
        if need_dB:
            gB = dB if lora_B.shape[1] == r else torch.cat([dB, dB.new_zeros(dB.shape[0], lora_B.shape[1] - r)], 1)
            gB = gB.to(lora_B.dtype)
        gbias = None
        if ctx.needs_input_grad[3]:
            gbias = dy.reshape(-1, dy.shape[-1]).sum(0)
        return (dx if need_dx else None), gA, gB, gbias, None, None, None, None


MAX_FUSED_RANK = 64     # ranks the fused kernels carry as one extra K-step


def qlora_linear(x: Tensor, qw: QuantWeight, lora_A: Optional[Tensor], lora_B: Optional[Tensor], r: int,
                 scaling: float, bias: Optional[Tensor] = None) -> Tensor:
    if r > MAX_FUSED_RANK and lora_A is not None:
        # The first 64 ranks ride in the fused kernel; the others are two plain library GEMMs on the bf16-rounded
        # factors (fp32 accumulation), added in bf16 the way the reference adds its whole LoRA branch
        # (qlora/modules/linear.py:376-385).  Autograd differentiates the tail; the factor slices are views, so
        # both parts' gradients land in the same parameters.
        y = qlora_linear(x, qw, lora_A[:MAX_FUSED_RANK], lora_B[:, :MAX_FUSED_RANK], MAX_FUSED_RANK, scaling, bias)
        A_t, B_t = lora_A[MAX_FUSED_RANK:r].to(x.dtype), lora_B[:, MAX_FUSED_RANK:r].to(x.dtype)
        su = (torch.nn.functional.linear(x, A_t).float() * scaling).to(x.dtype)
        return y + torch.nn.functional.linear(su, B_t)
    # Without a backward (inference / rollout) nothing needs the saved LoRA intermediate, which
    # also lets small batches take the weight-streaming kernel.
    training = torch.is_grad_enabled() and any(
        t is not None and t.requires_grad for t in (x, lora_A, lora_B, bias))
    if not training and not torch.compiler.is_compiling():
        # decode-regime calls are launch-bound: go straight to the library, skipping the autograd and
        # custom-op dispatch layers (tens of microseconds of host time per call)
        A = lora_A.detach()[:r] if lora_A is not None else None
        B = lora_B.detach()[:, :r] if lora_B is not None else None
        return _linear_fwd_impl(x.detach(), qw.packed, qw.scales, qw.global_scale, A, B,
                                None if bias is None else bias.detach(), qw.fmt, qw.scale_dtype, qw.group,
                                qw.rows, qw.cols, r, float(scaling), False, qw.c())[0]
    if qw.rows % 64 != 0:
        # the backward pass contracts over the output features; say so now rather than in the middle of backward()
        raise _C.XqError(f"qlora_linear: training needs out_features % 64 == 0 (the input-gradient product contracts "
                         f"over them), got {qw.rows}; forward-only calls need out_features % 16 == 0")
    return QLoRALinearFunction.apply(x, lora_A, lora_B, bias, qw, r, scaling, training)


def qlora_linear_swiglu(x: Tensor, qw: QuantWeight, lora_A: Optional[Tensor], lora_B: Optional[Tensor], r: int, scaling: float,
                        bias: Optional[Tensor] = None) -> Tensor:
    """Forward-only: ``silu_and_mul(*qlora_linear(x, qw, ...).chunk(2, dim=-1))`` for a weight that holds gate | up stacked
    ([2 I, K]: the reference's default ``gate_up_proj`` module, qlora/utils.py:33-37, followed by ``fused_silu_and_mul``,
    models/transformers/qwen3/modeling_qwen3.py:62-70) as one library call (xq_linear_fwd_swiglu); at decode sizes one
    kernel launch that writes h [.., I] directly.  Bit-identical to the two calls.  No autograd."""
    if x.dtype != torch.bfloat16:
        raise _C.XqError(f"activations must be bf16, got {x.dtype}")
    if r > MAX_FUSED_RANK:
        raise _C.XqError(f"qlora_linear_swiglu: rank {r} exceeds {MAX_FUSED_RANK}")
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (x, lora_A, lora_B, bias)):
        raise _C.XqError("qlora_linear_swiglu is forward-only: call it under torch.no_grad()")
    if qw.rows % 2:
        raise _C.XqError(f"qlora_linear_swiglu: the weight must hold gate | up, got {qw.rows} rows")
    _C.require_hip(x)
    x2 = _as_2d(x)
    M, K = x2.shape
    if qw.cols != K:
        raise _C.XqError(f"input width {K} != in_features {qw.cols}")
    I = qw.rows // 2
    dev = x.device
    A = lora_A.detach()[:r].contiguous() if (lora_A is not None and r) else None
    B = lora_B.detach()[:, :r].contiguous() if (lora_B is not None and r) else None
    b = bias.detach().to(torch.bfloat16).contiguous() if bias is not None else None
    L = _C.lib()
    ws_bytes = L.xq_linear_fwd_swiglu_workspace_bytes(M, qw.rows, K, r)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    h = torch.empty(M, I, dtype=torch.bfloat16, device=dev)
    cw = qw.c()
    _C.check(L.xq_linear_fwd_swiglu(ctypes.byref(cw), x2.data_ptr(), _ld(x2), M, _C.ptr(A), _C.ptr(B), _lora_dt(A), r if A is not None else 0,
                                    float(scaling), _C.ptr(b), h.data_ptr(), I, ws.data_ptr(), ws_bytes, _C.stream_ptr(dev)))
    _note_decode_forward(dev, M)
    return h.reshape(*x.shape[:-1], I)


def qlora_linear_multi(x: Tensor, jobs) -> list:
    """Forward-only: several QLoRA linears on one input, ``[qlora_linear(x, *job) for job in jobs]`` as one library call
    (xq_linear_fwd_multi): the separate q_proj / k_proj / v_proj or gate_proj / up_proj calls of a model that keeps
    them unfused (reference: models/layers/attention/multi_head_attention.py:93-95, modeling_qwen3.py:75-76).

    ``jobs``: up to 4 tuples ``(qw, lora_A, lora_B, r, scaling, bias)`` with the arguments of :func:`qlora_linear`
    (r <= 64, factors of one dtype).  At decode sizes (at most 16 rows of x) weights of one format run as ONE launch;
    results are bit-identical to the separate calls either way.  No autograd: call it under ``torch.no_grad()``."""
    if not 1 <= len(jobs) <= _C.XQ_LINEAR_MULTI_MAX:
        raise _C.XqError(f"qlora_linear_multi takes 1..{_C.XQ_LINEAR_MULTI_MAX} forwards, got {len(jobs)}")
    if x.dtype != torch.bfloat16:
        raise _C.XqError(f"activations must be bf16, got {x.dtype}")
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for j in jobs for t in (x, j[1], j[2], j[5])):
        raise _C.XqError("qlora_linear_multi is forward-only: call it under torch.no_grad()")
    x2 = _as_2d(x)
    M, K = x2.shape
    dev = x.device
    arr = (_C.XqLinearJob * len(jobs))()
    keep, ys, lora_dt = [], [], None
    for i, (qw, lora_A, lora_B, r, scaling, bias) in enumerate(jobs):
        if qw.cols != K:
            raise _C.XqError(f"input width {K} != in_features {qw.cols} of forward {i}")
        if r > MAX_FUSED_RANK:
            raise _C.XqError(f"qlora_linear_multi: rank {r} of forward {i} exceeds {MAX_FUSED_RANK}")
        A = lora_A.detach()[:r].contiguous() if (lora_A is not None and r) else None
        B = lora_B.detach()[:, :r].contiguous() if (lora_B is not None and r) else None
        if A is not None:
            if lora_dt is None:
                lora_dt = _lora_dt(A)
            elif lora_dt != _lora_dt(A):
                raise _C.XqError("qlora_linear_multi: the forwards' LoRA factors must share one dtype")
        b = bias.detach().to(torch.bfloat16).contiguous() if bias is not None else None
        y = torch.empty(M, qw.rows, dtype=torch.bfloat16, device=dev)
        cw = qw.c()
        keep += [A, B, b, cw]
        arr[i].w = ctypes.pointer(cw)
        arr[i].lora_A, arr[i].lora_B, arr[i].r, arr[i].scaling = _C.ptr(A), _C.ptr(B), (r if A is not None else 0), float(scaling)
        arr[i].bias_bf16, arr[i].y, arr[i].ldy = _C.ptr(b), y.data_ptr(), qw.rows
        ys.append(y)
    L = _C.lib()
    ws_bytes = L.xq_linear_fwd_multi_workspace_bytes(arr, len(jobs), M)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    _C.check(L.xq_linear_fwd_multi(arr, len(jobs), x2.data_ptr(), _ld(x2), M, lora_dt if lora_dt is not None else _C.XQ_DT_F32,
                                   ws.data_ptr(), ws_bytes, _C.stream_ptr(dev)))
    _note_decode_forward(dev, M)
    return [y.reshape(*x.shape[:-1], y.shape[1]) for y in ys]


# ---------------------------------------------------------------------------
# dense SwiGLU MLP of three QLoRA linears (xq_mlp_fwd / xq_mlp_bwd)
# ---------------------------------------------------------------------------
_MLP_WS: dict = {}


def _mlp_lora_struct(factors, biases, r: int, scaling: float) -> _C.XqMlpLora:
    L = _C.XqMlpLora()
    for p in range(3):
        A, B = factors[2 * p], factors[2 * p + 1]
        L.A[p], L.B[p] = _C.ptr(A), _C.ptr(B)
        L.bias[p] = _C.ptr(biases[p])
    L.dtype = _lora_dt(factors[0])
    L.r, L.scaling = r, scaling
    return L


def _mlp_saved_struct(saved, gu: int) -> _C.XqMlpSaved:
    S = _C.XqMlpSaved()
    S.gate_up, S.h, S.su_gate_up, S.su_down = (t.data_ptr() for t in saved)
    S.gate_up_fused = gu
    return S


def _mlp_gate_up_mode(qg: QuantWeight, qu: QuantWeight) -> int:
    """How a forward on these weights runs gate and up right now: 1 = one launch with the SwiGLU in its epilogue, 0 = two
    launches (xq_mlp_saved::gate_up_fused).  Read once per forward and handed to the forward AND its backward, so the pair
    agrees whatever xq_set_mlp_gate_up_fused() is called with in between."""
    return int(bool(_mlp_gate_up_default()) and qg.fmt == "block_fp8" and qu.fmt == "block_fp8")


@torch.compiler.assume_constant_result
def _mlp_gate_up_default() -> int:
    # (a constant of the traced graph under torch.compile: forward and backward of one trace get the same value)
    return int(_C.lib().xq_get_mlp_gate_up_fused())


def _mlp_workspace(dev, M: int, H: int, I: int, r: int, backward: bool) -> Tensor:
    key = (M, H, I, r, backward)
    n = _MLP_WS.get(key)
    if n is None:
        n = _MLP_WS[key] = _C.lib().xq_mlp_workspace_bytes(M, H, I, r, int(backward))
    return torch.empty(n, dtype=torch.uint8, device=dev)


def _mlp_fwd_impl(x2: Tensor, factors, biases, banks, r: int, scaling: float, gu: int):
    """xq_mlp_fwd.  x2 bf16 [M, H]; factors (gA, gB, uA, uB, dA, dB) active views, contiguous (None at r == 0);
    biases three bf16 vectors or None; banks (gate, up, down) QuantWeight.  -> (y [M, H], four saved tensors)."""
    qg, qu, qd = banks
    I, H = qg.rows, qg.cols
    M, dev, rp = x2.shape[0], x2.device, max(_r_pad(r), 16)
    bf = lambda *shape: torch.empty(*shape, dtype=torch.bfloat16, device=dev)
    saved = (bf(M, 2 * I), bf(M, I), bf(M, 2 * rp), bf(M, rp))
    y = bf(M, H)
    ws = _mlp_workspace(dev, M, H, I, r, False)
    lora, S = _mlp_lora_struct(factors, biases, r, scaling), _mlp_saved_struct(saved, gu)
    wg, wu, wd = qg.c(), qu.c(), qd.c()
    _C.check(_C.lib().xq_mlp_fwd(ctypes.byref(wg), ctypes.byref(wu), ctypes.byref(wd), ctypes.byref(lora), x2.data_ptr(),
                                 _ld(x2), M, y.data_ptr(), H, ctypes.byref(S), ws.data_ptr(), ws.numel(),
                                 _C.stream_ptr(dev)))
    if S.gate_up_fused != gu:
        raise RuntimeError(f"xq_mlp_fwd ran gate and up in form {S.gate_up_fused}, asked for {gu}")
    return y, saved


def _mlp_bwd_impl(dy2: Tensor, x2: Tensor, saved, factors, banks, r: int, scaling: float, need_dx: bool, gu: int):
    """xq_mlp_bwd -> (dx [M, H] or empty, six fp32 factor gradients (empty at r == 0))."""
    qg, qu, qd = banks
    I, H = qg.rows, qg.cols
    M, dev = x2.shape[0], x2.device
    dx = torch.empty(M, H, dtype=torch.bfloat16, device=dev) if need_dx else torch.empty(0, dtype=torch.bfloat16, device=dev)
    grads = [torch.empty(f.shape if f is not None else (0,), dtype=torch.float32, device=dev) for f in factors]
    G = _C.XqMlpGrads()
    for p in range(3):
        G.dA[p], G.dB[p] = (grads[2 * p].data_ptr(), grads[2 * p + 1].data_ptr()) if r else (None, None)
    ws = _mlp_workspace(dev, M, H, I, r, True)
    lora, S = _mlp_lora_struct(factors, (None, None, None), r, scaling), _mlp_saved_struct(saved, gu)
    wg, wu, wd = qg.c(), qu.c(), qd.c()
    _C.check(_C.lib().xq_mlp_bwd(ctypes.byref(wg), ctypes.byref(wu), ctypes.byref(wd), ctypes.byref(lora), x2.data_ptr(),
                                 _ld(x2), dy2.data_ptr(), _ld(dy2), M, ctypes.byref(S), dx.data_ptr() if need_dx else None,
                                 H, ctypes.byref(G), ws.data_ptr(), ws.numel(), _C.stream_ptr(dev)))
    return dx, grads


def _qw_args(qw: QuantWeight):
    return qw.packed, qw.scales, qw.global_scale, qw.fmt, _DT_TO_CODE[qw.scale_dtype], qw.group


def _qw_from(packed, scales, gs, fmt, scale_code, group, rows, cols) -> QuantWeight:
    return QuantWeight(fmt, _C.XQ_LAYOUT_FLAT, packed, scales, _CODE_TO_DT[scale_code], rows, cols, group, global_scale=gs)


@torch.library.custom_op("xq::mlp_fwd", mutates_args=(), device_types="cuda")
def _mlp_fwd_op(x: Tensor, factors: List[Tensor], biases: List[Optional[Tensor]],
                g_packed: Tensor, g_scales: Tensor, g_gs: Optional[Tensor], g_fmt: str, g_code: int, g_group: int,
                u_packed: Tensor, u_scales: Tensor, u_gs: Optional[Tensor], u_fmt: str, u_code: int, u_group: int,
                d_packed: Tensor, d_scales: Tensor, d_gs: Optional[Tensor], d_fmt: str, d_code: int, d_group: int,
                H: int, I: int, r: int, scaling: float, gu: int) -> List[Tensor]:
    banks = (_qw_from(g_packed, g_scales, g_gs, g_fmt, g_code, g_group, I, H),
             _qw_from(u_packed, u_scales, u_gs, u_fmt, u_code, u_group, I, H),
             _qw_from(d_packed, d_scales, d_gs, d_fmt, d_code, d_group, H, I))
    y, saved = _mlp_fwd_impl(x, tuple(factors) if r else (None,) * 6, tuple(biases), banks, r, scaling, gu)
    return [y, *saved]


@_mlp_fwd_op.register_fake
def _(x, factors, biases, g_packed, g_scales, g_gs, g_fmt, g_code, g_group, u_packed, u_scales, u_gs, u_fmt, u_code, u_group,
      d_packed, d_scales, d_gs, d_fmt, d_code, d_group, H, I, r, scaling, gu):
    M, rp = x.shape[0], max(_r_pad(r), 16)
    return [x.new_empty(M, H), x.new_empty(M, 2 * I), x.new_empty(M, I), x.new_empty(M, 2 * rp), x.new_empty(M, rp)]


@torch.library.custom_op("xq::mlp_bwd", mutates_args=(), device_types="cuda")
def _mlp_bwd_op(dy: Tensor, x: Tensor, saved: List[Tensor], factors: List[Tensor],
                g_packed: Tensor, g_scales: Tensor, g_gs: Optional[Tensor], g_fmt: str, g_code: int, g_group: int,
                u_packed: Tensor, u_scales: Tensor, u_gs: Optional[Tensor], u_fmt: str, u_code: int, u_group: int,
                d_packed: Tensor, d_scales: Tensor, d_gs: Optional[Tensor], d_fmt: str, d_code: int, d_group: int,
                H: int, I: int, r: int, scaling: float, need_dx: bool, gu: int) -> List[Tensor]:
    banks = (_qw_from(g_packed, g_scales, g_gs, g_fmt, g_code, g_group, I, H),
             _qw_from(u_packed, u_scales, u_gs, u_fmt, u_code, u_group, I, H),
             _qw_from(d_packed, d_scales, d_gs, d_fmt, d_code, d_group, H, I))
    dx, grads = _mlp_bwd_impl(dy, x, tuple(saved), tuple(factors) if r else (None,) * 6, banks, r, scaling, need_dx, gu)
    return [dx, *grads]


@_mlp_bwd_op.register_fake
def _(dy, x, saved, factors, g_packed, g_scales, g_gs, g_fmt, g_code, g_group, u_packed, u_scales, u_gs, u_fmt, u_code,
      u_group, d_packed, d_scales, d_gs, d_fmt, d_code, d_group, H, I, r, scaling, need_dx, gu):
    out = [x.new_empty(x.shape if need_dx else (0,))]
    if r:
        out += [x.new_empty(f.shape, dtype=torch.float32) for f in factors]
    else:
        out += [x.new_empty(0, dtype=torch.float32) for _ in range(6)]
    return out


class QLoRAMLPFunction(torch.autograd.Function):
    """y = down(silu(gate(x)) * up(x)) over three QLoRA linears with packed weights (xq_mlp_fwd / xq_mlp_bwd).
    Gradients: x and the six factors (full parameter shapes: ranks beyond the active one get zeros)."""

    @staticmethod
    def forward(ctx, x, gA, gB, uA, uB, dA, dB, bias_g, bias_u, bias_d, qg: QuantWeight, qu: QuantWeight, qd: QuantWeight,
                r: int, scaling: float):
        _C.require_hip(x)
        if x.dtype != torch.bfloat16:
            raise _C.XqError(f"activations must be bf16, got {x.dtype}")
        I, H = qg.rows, qg.cols
        x2 = _as_2d(x)
        if x2.shape[1] != H:
            raise _C.XqError(f"input width {x2.shape[1]} != in_features {H}")
        params = (gA, gB, uA, uB, dA, dB)
        if r:
            factors = tuple((p[:r] if i % 2 == 0 else p[:, :r]).contiguous() for i, p in enumerate(params))
        else:
            factors = (None,) * 6
        biases = tuple(None if b is None else b.to(torch.bfloat16).contiguous() for b in (bias_g, bias_u, bias_d))
        s = float(scaling)
        gu = _mlp_gate_up_mode(qg, qu)
        if torch.compiler.is_compiling():
            res = _mlp_fwd_op(x2, list(factors) if r else [], list(biases), *_qw_args(qg), *_qw_args(qu), *_qw_args(qd), H, I, r, s, gu)
            y, saved = res[0], tuple(res[1:])
        else:
            y, saved = _mlp_fwd_impl(x2, factors, biases, (qg, qu, qd), r, s, gu)
        ctx.banks, ctx.r, ctx.s, ctx.shape, ctx.gu = (qg, qu, qd), r, s, x.shape, gu
        ctx.param_shapes = tuple(None if p is None else p.shape for p in params)
        ctx.param_dtypes = tuple(None if p is None else p.dtype for p in params)
        ctx.n_factors = 6 if r else 0
        ctx.bias_d_dtype = x.dtype if bias_d is None else bias_d.dtype
        ctx.save_for_backward(x2, *saved, *(factors if r else ()))
        return y.reshape(*x.shape[:-1], H)

    @staticmethod
    def backward(ctx, dy):
        x2, saved = ctx.saved_tensors[0], ctx.saved_tensors[1:5]
        factors = tuple(ctx.saved_tensors[5:]) if ctx.n_factors else (None,) * 6
        qg, qu, qd = ctx.banks
        I, H, r = qg.rows, qg.cols, ctx.r
        dy2 = _as_2d(dy.to(torch.bfloat16))
        need_dx = ctx.needs_input_grad[0]
        if torch.compiler.is_compiling():
            res = _mlp_bwd_op(dy2, x2, list(saved), list(factors) if r else [], *_qw_args(qg), *_qw_args(qu), *_qw_args(qd),
                              H, I, r, ctx.s, need_dx, ctx.gu)
            dx, grads = res[0], res[1:]
        else:
            dx, grads = _mlp_bwd_impl(dy2, x2, saved, factors, ctx.banks, r, ctx.s, need_dx, ctx.gu)
        out = []
        for i, (g, shape, dt) in enumerate(zip(grads, ctx.param_shapes, ctx.param_dtypes)):
            if shape is None or not r or not ctx.needs_input_grad[1 + i]:
                out.append(None)
                continue
            if tuple(g.shape) != tuple(shape):        # ranks beyond the active one: zero gradient
                full = g.new_zeros(shape)
                if i % 2 == 0:
                    full[:r] = g
                else:
                    full[:, :r] = g
                g = full
            out.append(g.to(dt))
        gb = [None, None, None]
        if ctx.needs_input_grad[9]:        # the down projection's bias sees dy itself
            gb[2] = dy2.float().sum(0).to(ctx.bias_d_dtype)
        if ctx.needs_input_grad[7] or ctx.needs_input_grad[8]:
            raise NotImplementedError("trainable gate / up biases are not part of the fused MLP path (frozen in QLoRA)")
        return (dx.reshape(ctx.shape) if need_dx else None, *out, *gb, None, None, None, None, None)


_MLP_INFER_WS: dict = {}


def qlora_mlp_infer(x: Tensor, qw_gate: QuantWeight, qw_up: QuantWeight, qw_down: QuantWeight, gate_A: Optional[Tensor],
                    gate_B: Optional[Tensor], up_A: Optional[Tensor], up_B: Optional[Tensor], down_A: Optional[Tensor],
                    down_B: Optional[Tensor], r: int, scaling: float, bias_gate: Optional[Tensor] = None,
                    bias_up: Optional[Tensor] = None, bias_down: Optional[Tensor] = None) -> Tensor:
    """:func:`qlora_mlp` without autograd, as one library call (xq_mlp_fwd_infer): at decode sizes gate and up share one
    launch of the weight-streaming kernel and nothing is kept for a backward.  Same rounding points as the modules."""
    if r > MAX_FUSED_RANK:
        raise _C.XqError(f"the fused MLP takes LoRA ranks up to {MAX_FUSED_RANK}, got {r}")
    if x.dtype != torch.bfloat16:
        raise _C.XqError(f"activations must be bf16, got {x.dtype}")
    _C.require_hip(x)
    x2 = _as_2d(x)
    M, H = x2.shape
    I = qw_gate.rows
    if qw_gate.cols != H:
        raise _C.XqError(f"input width {H} != in_features {qw_gate.cols}")
    factors = [None if t is None or r == 0 else t.detach()[:r].contiguous() for t in (gate_A, None, up_A, None, down_A, None)]
    for i, t in ((1, gate_B), (3, up_B), (5, down_B)):
        factors[i] = None if t is None or r == 0 else t.detach()[:, :r].contiguous()
    biases = [None if b is None else b.detach().to(torch.bfloat16).contiguous() for b in (bias_gate, bias_up, bias_down)]
    L = _mlp_lora_struct(factors, biases, r if factors[0] is not None else 0, float(scaling))
    key = (M, H, I, r)
    n = _MLP_INFER_WS.get(key)
    if n is None:
        n = _MLP_INFER_WS[key] = _C.lib().xq_mlp_infer_workspace_bytes(M, H, I, r)
    dev = x.device
    ws = torch.empty(n, dtype=torch.uint8, device=dev)
    y = torch.empty(M, H, dtype=torch.bfloat16, device=dev)
    cg, cu, cd = qw_gate.c(), qw_up.c(), qw_down.c()
    _C.check(_C.lib().xq_mlp_fwd_infer(ctypes.byref(cg), ctypes.byref(cu), ctypes.byref(cd), ctypes.byref(L), x2.data_ptr(), _ld(x2), M,
                                       y.data_ptr(), H, ws.data_ptr(), n, _C.stream_ptr(dev)))
    _note_decode_forward(dev, M)
    return y.reshape(*x.shape[:-1], H)


def qlora_mlp(x: Tensor, qw_gate: QuantWeight, qw_up: QuantWeight, qw_down: QuantWeight, gate_A: Optional[Tensor],
              gate_B: Optional[Tensor], up_A: Optional[Tensor], up_B: Optional[Tensor], down_A: Optional[Tensor],
              down_B: Optional[Tensor], r: int, scaling: float, bias_gate: Optional[Tensor] = None,
              bias_up: Optional[Tensor] = None, bias_down: Optional[Tensor] = None) -> Tensor:
    """down(silu(gate(x)) * up(x)) of three QLoRA linears that share LoRA rank and scaling, in two library calls
    (forward, backward) instead of seven.  Same rounding points as the separate modules."""
    if r > MAX_FUSED_RANK:
        raise _C.XqError(f"the fused MLP takes LoRA ranks up to {MAX_FUSED_RANK}, got {r}")
    return QLoRAMLPFunction.apply(x, gate_A, gate_B, up_A, up_B, down_A, down_B, bias_gate, bias_up, bias_down, qw_gate,
                                  qw_up, qw_down, r, scaling)


# ---------------------------------------------------------------------------
# SwiGLU
# ---------------------------------------------------------------------------
def _silu_fwd_impl(g2: Tensor, u2: Tensor) -> Tensor:
    rows, cols = g2.shape
    h = torch.empty(rows, cols, dtype=torch.bfloat16, device=g2.device)
    _C.check(_C.lib().xq_silu_mul_fwd(g2.data_ptr(), u2.data_ptr(), _ld(g2), None, h.data_ptr(), cols, rows, cols,
                                      _C.stream_ptr(g2.device)))
    return h


def _silu_bwd_impl(g2: Tensor, u2: Tensor, d2: Tensor) -> Tuple[Tensor, Tensor]:
    rows, cols = g2.shape
    dg = torch.empty(rows, cols, dtype=torch.bfloat16, device=g2.device)
    du = torch.empty(rows, cols, dtype=torch.bfloat16, device=g2.device)
    _C.check(_C.lib().xq_silu_mul_bwd(g2.data_ptr(), u2.data_ptr(), _ld(g2), d2.data_ptr(), _ld(d2), None,
                                      dg.data_ptr(), du.data_ptr(), cols, None, rows, cols, _C.stream_ptr(g2.device)))
    return dg, du


@torch.library.custom_op("xq::silu_mul_fwd", mutates_args=(), device_types="cuda")
def _silu_fwd_op(gate: Tensor, up: Tensor) -> Tensor:
    return _silu_fwd_impl(gate, up)


@_silu_fwd_op.register_fake
def _(gate, up):
    return gate.new_empty(gate.shape)


@torch.library.custom_op("xq::silu_mul_bwd", mutates_args=(), device_types="cuda")
def _silu_bwd_op(gate: Tensor, up: Tensor, dh: Tensor) -> Tuple[Tensor, Tensor]:
    return _silu_bwd_impl(gate, up, dh)


@_silu_bwd_op.register_fake
def _(gate, up, dh):
    return gate.new_empty(gate.shape), gate.new_empty(gate.shape)


class SiluAndMulFunction(torch.autograd.Function):
    """fused_silu_and_mul (ops/fused_silu_and_mul.py): h = bf16(silu(gate)) * up."""

    @staticmethod
    def forward(ctx, gate: Tensor, up: Tensor):
        _C.require_hip(gate, up)
        if gate.dtype != torch.bfloat16 or up.dtype != torch.bfloat16:
            raise _C.XqError(f"silu_and_mul takes bf16 tensors, got {gate.dtype} and {up.dtype}")
        g2, u2 = _as_2d(gate), _as_2d(up)
        if _ld(g2) != _ld(u2) or torch.compiler.is_compiling():
            g2, u2 = g2.contiguous(), u2.contiguous()
        h = _silu_fwd_op(g2, u2) if torch.compiler.is_compiling() else _silu_fwd_impl(g2, u2)
        ctx.save_for_backward(g2, u2)
        ctx.shape = gate.shape
        return h.reshape(gate.shape)

    @staticmethod
    def backward(ctx, dh):
        g2, u2 = ctx.saved_tensors
        d2 = _as_2d(dh.to(torch.bfloat16))
        if torch.compiler.is_compiling():
            dg, du = _silu_bwd_op(g2, u2, d2.contiguous())
        else:
            dg, du = _silu_bwd_impl(g2, u2, d2)
        return dg.reshape(ctx.shape), du.reshape(ctx.shape)


def silu_and_mul(gate: Tensor, up: Tensor) -> Tensor:
    return SiluAndMulFunction.apply(gate, up)


# ---------------------------------------------------------------------------
# merging the LoRA update into the base weight
# ---------------------------------------------------------------------------
def merge_dense(qw: QuantWeight, lora_A: Optional[Tensor], lora_B: Optional[Tensor], r: int, scaling: float,
                out_dtype: torch.dtype = torch.bfloat16) -> Tensor:
    """deq(W) + scaling * B[:, :r] @ A[:r] as bf16 (weight-sync arithmetic, server/weight_sync/handler.py:2119-2131)
    or fp32 (the sum merge_weights re-quantises, qlora/modules/block_fp8_linear.py:111-115), [N, K]; deq(W) is
    never materialised."""
    _C.require_hip(qw.packed, lora_A, lora_B)
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise _C.XqError(f"merge_dense: out_dtype must be bf16 or fp32, got {out_dtype}")
    dev = qw.packed.device
    A = lora_A[:r].contiguous() if r > 0 else None
    B = lora_B[:, :r].contiguous() if r > 0 else None
    out = torch.empty(qw.rows, qw.cols, dtype=out_dtype, device=dev)
    w = qw.c()
    ws_bytes = _C.lib().xq_merge_workspace_bytes(qw.rows, qw.cols, r)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    _C.check(_C.lib().xq_merge_dense(ctypes.byref(w), _C.ptr(A), _C.ptr(B), _lora_dt(A), r, float(scaling),
                                     out.data_ptr(), _C.XQ_DT_BF16 if out_dtype == torch.bfloat16 else _C.XQ_DT_F32,
                                     ws.data_ptr(), ws_bytes, _C.stream_ptr(dev)))
    return out


def merge_requant_fp8(qw: QuantWeight, lora_A: Optional[Tensor], lora_B: Optional[Tensor], r: int, scaling: float,
                      packed_out: Optional[Tensor] = None, scales_out: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """block_fp8 only: Q(deq(W) + scaling * B @ A) with fresh 128x128 block scales in one pass
    (merge_weights + _quantize_and_store, qlora/modules/block_fp8_linear.py:111-119).  Returns (e4m3 bytes as
    uint8 [N, K], fp32 scales [ceil(N/128), ceil(K/128)]); pass the weight's own buffers to update in place."""
    _C.require_hip(qw.packed, lora_A, lora_B)
    if qw.fmt != "block_fp8":
        raise _C.XqError(f"merge_requant_fp8: the weight must be block_fp8, got {qw.fmt}")
    dev = qw.packed.device
    A = lora_A[:r].contiguous() if r > 0 else None
    B = lora_B[:, :r].contiguous() if r > 0 else None
    if packed_out is None:
        packed_out = torch.empty(qw.rows, qw.cols, dtype=torch.uint8, device=dev)
    if scales_out is None:
        scales_out = torch.empty((qw.rows + 127) // 128, (qw.cols + 127) // 128, dtype=torch.float32, device=dev)
    w = qw.c()
    ws_bytes = _C.lib().xq_merge_workspace_bytes(qw.rows, qw.cols, r)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    _C.check(_C.lib().xq_merge_requant_fp8(ctypes.byref(w), _C.ptr(A), _C.ptr(B), _lora_dt(A), r, float(scaling),
                                           packed_out.data_ptr(), scales_out.data_ptr(), ws.data_ptr(), ws_bytes,
                                           _C.stream_ptr(dev)))
    return packed_out, scales_out


def merge_amax(qw: QuantWeight, lora_A: Optional[Tensor], lora_B: Optional[Tensor], r: int, scaling: float) -> Tensor:
    """max |bf16(bf16(deq(W)) + bf16(scaling * B @ A))| over the matrix, fp32 [1]: the fresh tensor amax an nvfp4
    module blends into its running one before it re-quantises (qlora/modules/nvfp4_linear.py:126-139), without
    materialising the merged weight."""
    _C.require_hip(qw.packed, lora_A, lora_B)
    dev = qw.packed.device
    A = lora_A[:r].contiguous() if r > 0 else None
    B = lora_B[:, :r].contiguous() if r > 0 else None
    out = torch.empty(1, dtype=torch.float32, device=dev)
    ws_bytes = _C.lib().xq_merge_workspace_bytes(qw.rows, qw.cols, r)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    w = qw.c()
    _C.check(_C.lib().xq_merge_amax(ctypes.byref(w), _C.ptr(A), _C.ptr(B), _lora_dt(A), r, float(scaling), out.data_ptr(),
                                    ws.data_ptr(), ws_bytes, _C.stream_ptr(dev)))
    return out


def merge_requant_nvfp4(qw: QuantWeight, lora_A: Optional[Tensor], lora_B: Optional[Tensor], r: int, scaling: float,
                        global_amax: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """nvfp4 only: nvfp4_quantize(deq(W) + scaling * B @ A, global_amax) in one pass over the packed bytes
    (merge_weights + _quantize_and_store, qlora/modules/nvfp4_linear.py:126-139).  Returns (codes uint8 [N*K/2],
    e4m3 block scales [N*K/16], fp32 global scale [1]) in fresh tensors."""
    _C.require_hip(qw.packed, lora_A, lora_B)
    if qw.fmt != "nvfp4":
        raise _C.XqError(f"merge_requant_nvfp4: the weight must be nvfp4, got {qw.fmt}")
    dev = qw.packed.device
    A = lora_A[:r].contiguous() if r > 0 else None
    B = lora_B[:, :r].contiguous() if r > 0 else None
    n = qw.rows * qw.cols
    codes = torch.empty(n // 2, dtype=torch.uint8, device=dev)
    bscales = torch.empty(n // 16, dtype=torch.uint8, device=dev)
    gscale = torch.empty(1, dtype=torch.float32, device=dev)
    gamax = global_amax.to(device=dev, dtype=torch.float32).reshape(1).contiguous()
    ws_bytes = _C.lib().xq_merge_workspace_bytes(qw.rows, qw.cols, r)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    w = qw.c()
    _C.check(_C.lib().xq_merge_requant_nvfp4(ctypes.byref(w), _C.ptr(A), _C.ptr(B), _lora_dt(A), r, float(scaling),
                                             gamax.data_ptr(), codes.data_ptr(), bscales.data_ptr(), gscale.data_ptr(),
                                             ws.data_ptr(), ws_bytes, _C.stream_ptr(dev)))
    return codes, bscales.view(torch.float8_e4m3fn), gscale


def merge_requant_int4(qw: QuantWeight, lora_A: Optional[Tensor], lora_B: Optional[Tensor], r: int, scaling: float,
                       symmetric: bool, codes_out: Optional[Tensor] = None,
                       scales_out: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """Flat int4 with 128-element groups only: Q(bf16(deq(W)) + bf16(scaling * B @ A)) in one pass over the packed
    bytes.  `symmetric` picks the quantizer: False = ops/quantize/int4_quantize.py:12-41 (fp32 scales), True =
    scale bf16(absmax / 7), codes rne(x / scale) + 8 (bf16 scales).  Returns (codes uint8 [N, K/2], scales [N, K/128]);
    pass the weight's own buffers to update in place."""
    _C.require_hip(qw.packed, lora_A, lora_B)
    if qw.fmt != "int4":
        raise _C.XqError(f"merge_requant_int4: the weight must be int4, got {qw.fmt}")
    dev = qw.packed.device
    A = lora_A[:r].contiguous() if r > 0 else None
    B = lora_B[:, :r].contiguous() if r > 0 else None
    if codes_out is None:
        codes_out = torch.empty(qw.rows, qw.cols // 2, dtype=torch.uint8, device=dev)
    if scales_out is None:
        scales_out = torch.empty(qw.rows, qw.cols // 128, dtype=torch.bfloat16 if symmetric else torch.float32, device=dev)
    ws_bytes = _C.lib().xq_merge_workspace_bytes(qw.rows, qw.cols, r)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    w = qw.c()
    _C.check(_C.lib().xq_merge_requant_int4(ctypes.byref(w), _C.ptr(A), _C.ptr(B), _lora_dt(A), r, float(scaling),
                                            1 if symmetric else 0, codes_out.data_ptr(), scales_out.data_ptr(),
                                            ws.data_ptr(), ws_bytes, _C.stream_ptr(dev)))
    return codes_out, scales_out


def merge_requant_nf4(qw: QuantWeight, lora_A: Optional[Tensor], lora_B: Optional[Tensor], r: int, scaling: float,
                      codes_out: Optional[Tensor] = None, scales_out: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """NF4 only: nf4_quantize(deq(W) + scaling * B @ A) in one pass over the packed bytes (merge_weights +
    _quantize_and_store of qlora/modules/nf4_linear.py).  Returns (codes uint8 [N*K/2], fp32 scales [N*K/64]); pass
    the weight's own buffers to update in place."""
    _C.require_hip(qw.packed, lora_A, lora_B)
    if qw.fmt != "nf4":
        raise _C.XqError(f"merge_requant_nf4: the weight must be nf4, got {qw.fmt}")
    dev = qw.packed.device
    A = lora_A[:r].contiguous() if r > 0 else None
    B = lora_B[:, :r].contiguous() if r > 0 else None
    n = qw.rows * qw.cols
    if codes_out is None:
        codes_out = torch.empty(n // 2, dtype=torch.uint8, device=dev)
    if scales_out is None:
        scales_out = torch.empty(n // 64, dtype=torch.float32, device=dev)
    ws_bytes = _C.lib().xq_merge_workspace_bytes(qw.rows, qw.cols, r)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    w = qw.c()
    _C.check(_C.lib().xq_merge_requant_nf4(ctypes.byref(w), _C.ptr(A), _C.ptr(B), _lora_dt(A), r, float(scaling),
                                           codes_out.data_ptr(), scales_out.data_ptr(), ws.data_ptr(), ws_bytes,
                                           _C.stream_ptr(dev)))
    return codes_out, scales_out
