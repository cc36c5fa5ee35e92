"""Grouped / routed QLoRA expert MLP on packed expert banks (HIP kernels over the C ABI).

Same program as the reference's local LoRA expert compute
(``_MoeExpertsLoRAFunction``, xorl/ops/moe/lora.py:525-1007): histogram +
stable sort by expert, scatter, gate/up projections with LoRA, SwiGLU, routing
weight applied before the down projection, down projection with LoRA, top-k
gather-sum -- but the expert banks stay packed: every grouped GEMM decodes its
weight tile inside the kernel, so no ``[E, K, N]`` bf16 bank is ever built
(the reference dequantizes every expert of every projection first,
qlora/modules/moe_experts.py:486-498).
"""

from __future__ import annotations

import ctypes
from typing import Dict, List, Optional, Tuple

import torch
from torch import Tensor

from . import _C
from .functional import _CODE_TO_DT, _DT_TO_CODE, QuantWeight, _as_2d, _r_pad


def _s(dev):
    return _C.stream_ptr(dev)


def route_build(selected_experts: Tensor, num_experts: int):
    """-> counts [E], offsets [E+1], scatter_index [T*topk], tile_offsets [2*(E+1)] (all int32, device).

    tile_offsets holds two row-tile schedules back to back: the prefix of ceil(count/128) and the
    prefix of ceil(count/256)."""
    _C.require_hip(selected_experts)
    dev = selected_experts.device
    sel = selected_experts.reshape(-1).to(torch.int32).contiguous()
    n = sel.numel()
    L = _C.lib()
    counts = torch.empty(num_experts, dtype=torch.int32, device=dev)
    offsets = torch.empty(num_experts + 1, dtype=torch.int32, device=dev)
    tile_offsets = torch.empty(2 * (num_experts + 1), dtype=torch.int32, device=dev)
    sidx = torch.empty(n, dtype=torch.int32, device=dev)
    wsb = L.xq_route_workspace_bytes(n, num_experts)
    ws = torch.empty(wsb, dtype=torch.uint8, device=dev)
    _C.check(L.xq_route_build(sel.data_ptr(), n, num_experts, counts.data_ptr(), offsets.data_ptr(), sidx.data_ptr(),
                              tile_offsets.data_ptr(), ws.data_ptr(), wsb, _s(dev)))
    return counts, offsets, sidx, tile_offsets


def moe_scatter(x: Tensor, sidx: Tensor, topk: int) -> Tensor:
    x = x.contiguous()
    n, width = sidx.numel(), x.shape[-1]
    out = torch.empty(n, width, dtype=torch.bfloat16, device=x.device)
    _C.check(_C.lib().xq_moe_scatter(x.data_ptr(), width, sidx.data_ptr(), n, topk, width, out.data_ptr(), width,
                                     _s(x.device)))
    return out


def moe_gather(rows: Tensor, rows2: Optional[Tensor], sidx: Tensor, n_tokens: int, topk: int) -> Tensor:
    width = rows.shape[-1]
    out = torch.empty(n_tokens, width, dtype=torch.bfloat16, device=rows.device)
    _C.check(_C.lib().xq_moe_gather(rows.data_ptr(), _C.ptr(rows2), width, sidx.data_ptr(), n_tokens, topk, width,
                                    out.data_ptr(), width, _s(rows.device)))
    return out


def _prep(t: Tensor, transpose: bool, rows_out: int, cols_out: int) -> Tensor:
    """[E, a, b] fp32/bf16 factor -> bf16 [E, rows_out, cols_out], optionally transposed, zero padded."""
    t = t.contiguous()
    E, a, b = t.shape
    out = torch.empty(E, rows_out, cols_out, dtype=torch.bfloat16, device=t.device)
    dt = _C.XQ_DT_F32 if t.dtype == torch.float32 else _C.XQ_DT_BF16
    if t.dtype not in (torch.float32, torch.bfloat16):
        raise _C.XqError(f"LoRA factors must be fp32 or bf16, got {t.dtype}")
    _C.check(_C.lib().xq_factor_prep(t.data_ptr(), dt, a, b, int(transpose), out.data_ptr(), rows_out, cols_out, E,
                                     _s(t.device)))
    return out


def _lora_down(a: Tensor, F: Tensor, offsets, tile_offsets, E: int, scale: float) -> Tensor:
    """t[rows of e] = bf16(scale * a . F[e]^T); F bf16 [E|1, r_pad, K]."""
    R, K = a.shape
    rp = F.shape[1]
    t = torch.empty(R, rp, dtype=torch.bfloat16, device=a.device)
    _C.check(_C.lib().xq_grouped_lora_down(a.data_ptr(), a.stride(0), R, offsets.data_ptr(), tile_offsets.data_ptr(),
                                           E, F.data_ptr(), int(F.shape[0] == 1), rp, K, scale, t.data_ptr(),
                                           _s(a.device)))
    return t


def _grouped_gemm(qw: QuantWeight, transpose_w: bool, a: Tensor, offsets, tile_offsets, su: Optional[Tensor],
                  lora_right: Optional[Tensor]) -> Tensor:
    R = a.shape[0]
    n_out = qw.rows if transpose_w else qw.cols
    y = torch.empty(R, n_out, dtype=torch.bfloat16, device=a.device)
    w = qw.c()
    rp = su.shape[1] if su is not None else 0
    _C.check(_C.lib().xq_grouped_gemm(ctypes.byref(w), int(transpose_w), a.data_ptr(), a.stride(0), R,
                                      offsets.data_ptr(), tile_offsets.data_ptr(), _C.ptr(su), _C.ptr(lora_right), rp,
                                      y.data_ptr(), n_out, _s(a.device)))
    return y


def _wgrad(P: Tensor, Q: Tensor, r: int, offsets: Optional[Tensor], E: int, transpose_out: bool,
           row_limit: Optional[Tensor] = None) -> Tensor:
    """Per expert (offsets given): out[e] = P[rows e]^T . Q[rows e] -> [E, width, r] or [E, r, width];
    offsets None: one product over all rows (below row_limit[0], a device int32, when given) -> [1, ...]
    (gradient of a factor shared by all experts)."""
    R, width = P.shape
    rp = Q.shape[1]
    L = _C.lib()
    n_out = E if offsets is not None else 1
    shape = (n_out, r, width) if transpose_out else (n_out, width, r)
    out = torch.empty(*shape, dtype=torch.float32, device=P.device)
    ws = torch.empty(L.xq_lora_wgrad_workspace_bytes(R, width, rp), dtype=torch.uint8, device=P.device)
    _C.check(L.xq_grouped_lora_wgrad(P.data_ptr(), P.stride(0), width, Q.data_ptr(), rp, r, R, _C.ptr(offsets), E,
                                     int(transpose_out), out.data_ptr(), _C.ptr(ws),
                                     _C.ptr(row_limit) if offsets is None else None, _s(P.device)))
    return out


def _expand(t: Tensor, E: int) -> Tensor:
    return t.expand(E, -1, -1).contiguous() if t.shape[0] == 1 else t


# ---------------------------------------------------------------------------
# the routed expert MLP: two library calls behind two custom ops
# ---------------------------------------------------------------------------
_PROJ = ("gate", "up", "down")
_WS: dict = {}


def _bank_args(qw: QuantWeight):
    return qw.packed, qw.scales, qw.global_scale


def _rebuild_bank(packed, scales, gs, fmt, layout, scale_dt, rows, cols, group, E) -> QuantWeight:
    return QuantWeight(fmt, layout, packed, scales, scale_dt, rows, cols, group, global_scale=gs, num_experts=E)


def _lora_struct(factors, r: int, scaling: float, swiglu_limit: float = 0.0) -> _C.XqGroupedLora:
    gA, gB, uA, uB, dA, dB = factors
    dt = gA.dtype
    if dt not in (torch.float32, torch.bfloat16) or any(f.dtype != dt for f in factors):
        raise _C.XqError(f"LoRA factors must all be fp32 or all be bf16, got {[f.dtype for f in factors]}")
    L = _C.XqGroupedLora()
    for p, (A, B) in enumerate(((gA, gB), (uA, uB), (dA, dB))):
        L.A[p], L.B[p] = A.data_ptr(), B.data_ptr()
        L.A_experts[p], L.B_experts[p] = A.shape[0], B.shape[0]
    L.dtype = _C.XQ_DT_F32 if dt == torch.float32 else _C.XQ_DT_BF16
    L.r, L.scaling, L.swiglu_limit = r, scaling, max(float(swiglu_limit), 0.0)
    return L


# Test switch: False keeps the expert-ordered copy of the routed rows (saved xs [R, H]) even where the banks can read the
# token matrix in place.
READ_ROUTED_ROWS_IN_PLACE = True


def _saved_struct(saved, x_tokens: Optional[Tensor] = None) -> _C.XqGroupedSaved:
    """saved[0] (xs) with no elements: the routed rows are read in place from the token matrix (`x_tokens` in the backward)."""
    S = _C.XqGroupedSaved()
    for name, t in zip(("xs", "gate_up", "h", "w_row", "su_gate", "su_up", "su_down", "scatter_index", "offsets",
                        "tile_offsets", "counts"), saved):
        setattr(S, name, t.data_ptr() if t.numel() else None)
    if x_tokens is not None and x_tokens.numel():
        S.x_tokens, S.ld_x_tokens = x_tokens.data_ptr(), (x_tokens.stride(0) if x_tokens.shape[0] > 1 else x_tokens.shape[1])
    return S


def _workspace(dev, T: int, topk: int, E: int, H: int, I: int, r: int, backward: bool) -> Tensor:
    key = (T, topk, E, H, I, r, backward)
    n = _WS.get(key)
    if n is None:
        n = _WS[key] = _C.lib().xq_grouped_workspace_bytes(T, topk, E, H, I, r, int(backward))
    return torch.empty(n, dtype=torch.uint8, device=dev)


def _moe_fwd_impl(hidden2: Tensor, rw: Tensor, sel: Tensor, factors, banks, r: int, scaling: float, allow_in_place: bool = True,
                  swiglu_limit: float = 0.0):
    """xq_grouped_fwd.  hidden2 bf16 [T, H]; rw [T, topk] fp32 / bf16; sel int32 [T, topk]; factors the six active
    LoRA views, contiguous; banks three QuantWeight.  -> (out [T, H], the eleven tensors the backward reads)."""
    qg, qu, qd = banks
    E, H, I = qg.num_experts, qg.rows, qg.cols
    T, topk = sel.shape
    R, rp, dev = T * topk, _r_pad(r), hidden2.device
    bf = lambda *shape: torch.empty(*shape, dtype=torch.bfloat16, device=dev)
    i32 = lambda n: torch.empty(n, dtype=torch.int32, device=dev)
    wg, wu, wd = qg.c(), qu.c(), qd.c()
    # where the banks allow it the routed rows are read in place from hidden2 (no [R, H] copy kept for the backward)
    # (not under torch.compile: the traced op has one output signature, with the copy)
    in_place = (allow_in_place and READ_ROUTED_ROWS_IN_PLACE and R > 0 and hidden2.data_ptr() % 16 == 0 and (T == 1 or hidden2.stride(0) % 8 == 0)
                and bool(_C.lib().xq_grouped_in_place(ctypes.byref(wg), ctypes.byref(wu), ctypes.byref(wd))))
    saved = (bf(0, H) if in_place else bf(R, H), bf(R, 2 * I), bf(R, I), torch.empty(R, dtype=torch.float32, device=dev), bf(R, rp),
             bf(R, rp), bf(R, rp), i32(R), i32(E + 1), i32(2 * (E + 1)), i32(E))
    out = bf(T, H)
    ws = _workspace(dev, T, topk, E, H, I, r, False)
    lora, S = _lora_struct(factors, r, scaling, swiglu_limit), _saved_struct(saved)
    _C.check(_C.lib().xq_grouped_fwd(ctypes.byref(wg), ctypes.byref(wu), ctypes.byref(wd), ctypes.byref(lora),
                                     hidden2.data_ptr(), hidden2.stride(0) if T > 1 else H, T, rw.data_ptr(),
                                     _C.XQ_DT_F32 if rw.dtype == torch.float32 else _C.XQ_DT_BF16, sel.data_ptr(), topk,
                                     out.data_ptr(), H, ctypes.byref(S), ws.data_ptr(), ws.numel(), _s(dev)))
    return out, saved


def _moe_bwd_impl(dy2: Tensor, saved, factors, banks, r: int, scaling: float, T: int, topk: int, rw_dtype: torch.dtype,
                  need_dx: bool, need_drw: bool, hidden2: Optional[Tensor] = None, swiglu_limit: float = 0.0):
    """xq_grouped_bwd -> (dx [T, H] or empty, d_routing [T, topk] or empty, six fp32 factor gradients)."""
    qg, qu, qd = banks
    E, H, I = qg.num_experts, qg.rows, qg.cols
    dev = dy2.device
    dx = torch.empty(T, H, dtype=torch.bfloat16, device=dev) if need_dx else torch.empty(0, dtype=torch.bfloat16, device=dev)
    out_dt = rw_dtype if rw_dtype in (torch.float32, torch.bfloat16) else torch.float32
    drw = torch.empty(T, topk, dtype=out_dt, device=dev) if need_drw else torch.empty(0, dtype=out_dt, device=dev)
    grads = [torch.empty(f.shape, dtype=torch.float32, device=dev) for f in factors]
    G = _C.XqGroupedGrads()
    for p in range(3):
        G.dA[p], G.dB[p] = grads[2 * p].data_ptr(), grads[2 * p + 1].data_ptr()
    ws = _workspace(dev, T, topk, E, H, I, r, True)
    lora, S = _lora_struct(factors, r, scaling, swiglu_limit), _saved_struct(saved, hidden2)
    wg, wu, wd = qg.c(), qu.c(), qd.c()
    _C.check(_C.lib().xq_grouped_bwd(ctypes.byref(wg), ctypes.byref(wu), ctypes.byref(wd), ctypes.byref(lora),
                                     dy2.data_ptr(), dy2.stride(0) if T > 1 else H, T, topk, ctypes.byref(S),
                                     dx.data_ptr() if need_dx else None, H, drw.data_ptr() if need_drw else None,
                                     _C.XQ_DT_F32 if out_dt == torch.float32 else _C.XQ_DT_BF16, ctypes.byref(G),
                                     ws.data_ptr(), ws.numel(), _s(dev)))
    return dx, drw, grads


@torch.library.custom_op("xq::moe_fwd", mutates_args=(), device_types="cuda")
def _moe_fwd_op(hidden: Tensor, rw: Tensor, sel: Tensor, gA: Tensor, gB: Tensor, uA: Tensor, uB: Tensor, dA: Tensor,
                dB: Tensor, g_packed: Tensor, g_scales: Tensor, g_gs: Optional[Tensor], u_packed: Tensor,
                u_scales: Tensor, u_gs: Optional[Tensor], d_packed: Tensor, d_scales: Tensor, d_gs: Optional[Tensor],
                fmt: str, layout: int, scale_code: int, group: int, E: int, H: int, I: int, r: int,
                scaling: float, swiglu_limit: float = 0.0) -> List[Tensor]:
    sd = _CODE_TO_DT[scale_code]
    banks = (_rebuild_bank(g_packed, g_scales, g_gs, fmt, layout, sd, H, I, group, E),
             _rebuild_bank(u_packed, u_scales, u_gs, fmt, layout, sd, H, I, group, E),
             _rebuild_bank(d_packed, d_scales, d_gs, fmt, layout, sd, I, H, group, E))
    out, saved = _moe_fwd_impl(hidden, rw, sel, (gA, gB, uA, uB, dA, dB), banks, r, scaling, allow_in_place=False,
                               swiglu_limit=swiglu_limit)
    return [out, *saved]


@_moe_fwd_op.register_fake
def _(hidden, rw, sel, gA, gB, uA, uB, dA, dB, g_packed, g_scales, g_gs, u_packed, u_scales, u_gs, d_packed, d_scales,
      d_gs, fmt, layout, scale_code, group, E, H, I, r, scaling, swiglu_limit=0.0):
    T, topk = sel.shape
    R, rp = T * topk, _r_pad(r)
    bf = lambda *shape: hidden.new_empty(*shape, dtype=torch.bfloat16)
    i32 = lambda n: hidden.new_empty(n, dtype=torch.int32)
    return [bf(T, H), bf(R, H), bf(R, 2 * I), bf(R, I), hidden.new_empty(R, dtype=torch.float32), bf(R, rp),
            bf(R, rp), bf(R, rp), i32(R), i32(E + 1), i32(2 * (E + 1)), i32(E)]


@torch.library.custom_op("xq::moe_bwd", mutates_args=(), device_types="cuda")
def _moe_bwd_op(dy: Tensor, hidden: Tensor, saved: List[Tensor], gA: Tensor, gB: Tensor, uA: Tensor, uB: Tensor, dA: Tensor, dB: Tensor,
                g_packed: Tensor, g_scales: Tensor, g_gs: Optional[Tensor], u_packed: Tensor, u_scales: Tensor,
                u_gs: Optional[Tensor], d_packed: Tensor, d_scales: Tensor, d_gs: Optional[Tensor], fmt: str,
                layout: int, scale_code: int, group: int, E: int, H: int, I: int, r: int, scaling: float, T: int,
                topk: int, rw_code: int, need_dx: bool, need_drw: bool, swiglu_limit: float = 0.0) -> List[Tensor]:
    sd = _CODE_TO_DT[scale_code]
    banks = (_rebuild_bank(g_packed, g_scales, g_gs, fmt, layout, sd, H, I, group, E),
             _rebuild_bank(u_packed, u_scales, u_gs, fmt, layout, sd, H, I, group, E),
             _rebuild_bank(d_packed, d_scales, d_gs, fmt, layout, sd, I, H, group, E))
    dx, drw, grads = _moe_bwd_impl(dy, tuple(saved), (gA, gB, uA, uB, dA, dB), banks, r, scaling, T, topk,
                                   _CODE_TO_DT[rw_code], need_dx, need_drw, hidden, swiglu_limit)
    return [dx, drw, *grads]


@_moe_bwd_op.register_fake
def _(dy, hidden, saved, gA, gB, uA, uB, dA, dB, g_packed, g_scales, g_gs, u_packed, u_scales, u_gs, d_packed, d_scales, d_gs,
      fmt, layout, scale_code, group, E, H, I, r, scaling, T, topk, rw_code, need_dx, need_drw, swiglu_limit=0.0):
    rw_dt = _CODE_TO_DT[rw_code]
    return [dy.new_empty((T, H) if need_dx else (0,), dtype=torch.bfloat16),
            dy.new_empty((T, topk) if need_drw else (0,), dtype=rw_dt),
            *[dy.new_empty(f.shape, dtype=torch.float32) for f in (gA, gB, uA, uB, dA, dB)]]


class MoeExpertsQLoRAFunction(torch.autograd.Function):
    """Routed SwiGLU expert MLP with LoRA on packed banks (xq_grouped_fwd / xq_grouped_bwd).

    inputs: hidden [T, H] bf16, routing_weights [T, topk], selected_experts
    [T, topk], three QuantWeight banks (GKN: gate/up [E, H, I], down [E, I, H]),
    six LoRA factors in GKN form (A [E|1, in, r], B [E|1, r, out]).  Returns
    [T, H] bf16.  Gradients: hidden, routing_weights and the six factors; the
    frozen banks get none.  Experts that receive no rows get exact-zero factor
    gradients."""

    @staticmethod
    def forward(ctx, hidden, routing_weights, selected_experts, gA, gB, uA, uB, dA, dB,
                qw_gate: QuantWeight, qw_up: QuantWeight, qw_down: QuantWeight, num_experts: int, scaling: float,
                swiglu_limit: float = 0.0):
        _C.require_hip(hidden, routing_weights, selected_experts)
        if hidden.dtype != torch.bfloat16:
            raise _C.XqError(f"hidden states must be bf16, got {hidden.dtype}")
        E = num_experts
        banks = (qw_gate, qw_up, qw_down)
        for qw in banks:
            if qw.num_experts != E:          # the tile schedules of the routing are laid out for E experts
                raise _C.XqError(f"routing over {E} experts but a bank holds {qw.num_experts}")
        shape = hidden.shape
        H, I = qw_gate.rows, qw_gate.cols
        hidden2 = hidden.reshape(-1, H)
        hidden2 = _as_2d(hidden2)
        T = hidden2.shape[0]
        topk = selected_experts.shape[-1]
        sel = selected_experts.reshape(T, topk).to(torch.int32).contiguous()
        rw = routing_weights.reshape(T, topk)
        if rw.dtype not in (torch.float32, torch.bfloat16):
            rw = rw.float()
        rw = rw.contiguous()
        r = gA.shape[-1]
        factors = tuple(f.contiguous() for f in (gA, gB, uA, uB, dA, dB))
        s = float(scaling)
        lim = max(float(swiglu_limit or 0.0), 0.0)
        if torch.compiler.is_compiling():
            res = _moe_fwd_op(hidden2, rw, sel, *factors, *_bank_args(qw_gate), *_bank_args(qw_up), *_bank_args(qw_down),
                              qw_gate.fmt, qw_gate.layout, _DT_TO_CODE[qw_gate.scale_dtype], qw_gate.group, E, H, I, r, s, lim)
            out, saved = res[0], tuple(res[1:])
        else:
            out, saved = _moe_fwd_impl(hidden2, rw, sel, factors, banks, r, s, swiglu_limit=lim)
        ctx.qw = banks
        ctx.swiglu_limit = lim
        ctx.meta = (E, T, topk, H, I, r, s, shape, routing_weights.dtype, routing_weights.shape)
        ctx.save_for_backward(*saved, *factors, hidden2)
        return out.reshape(shape)

    @staticmethod
    def backward(ctx, dy):
        saved, factors, hidden2 = ctx.saved_tensors[:11], ctx.saved_tensors[11:17], ctx.saved_tensors[17]
        qw_gate, qw_up, qw_down = ctx.qw
        E, T, topk, H, I, r, s, shape, rw_dtype, rw_shape = ctx.meta
        dy2 = dy.reshape(-1, H).to(torch.bfloat16)
        dy2 = _as_2d(dy2)
        need_dx, need_drw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        kernel_rw_dt = rw_dtype if rw_dtype in (torch.float32, torch.bfloat16) else torch.float32
        if torch.compiler.is_compiling():
            res = _moe_bwd_op(dy2, hidden2, list(saved), *factors, *_bank_args(qw_gate), *_bank_args(qw_up), *_bank_args(qw_down),
                              qw_gate.fmt, qw_gate.layout, _DT_TO_CODE[qw_gate.scale_dtype], qw_gate.group, E, H, I, r, s,
                              T, topk, _DT_TO_CODE[kernel_rw_dt], need_dx, need_drw, ctx.swiglu_limit)
            dx, drw, grads = res[0], res[1], res[2:]
        else:
            dx, drw, grads = _moe_bwd_impl(dy2, saved, factors, ctx.qw, r, s, T, topk, kernel_rw_dt, need_dx, need_drw, hidden2,
                                           ctx.swiglu_limit)
        dx = dx.reshape(shape) if need_dx else None
        drw = drw.reshape(rw_shape).to(rw_dtype) if need_drw else None
        gs = [g.to(f.dtype) for g, f in zip(grads, factors)]
        return (dx, drw, None, *gs, None, None, None, None, None, None)


# Test switch: False sends forwards that need no gradient through xq_grouped_fwd as well.
DECODE_PATH = True


def _moe_infer(hidden: Tensor, routing_weights: Tensor, selected_experts: Tensor, factors, banks, num_experts: int,
               scaling: float, swiglu_limit: float) -> Optional[Tensor]:
    """xq_grouped_fwd_infer: the forward for a handful of tokens when nothing is differentiated (block-fp8 banks; the
    touched experts' bytes streamed once).  None where the call does not fit it."""
    qg, qu, qd = banks
    H = qg.rows
    if (hidden.dtype != torch.bfloat16 or not hidden.is_cuda or hidden.numel() == 0 or hidden.shape[-1] != H
            or any(qw.num_experts != num_experts for qw in banks)):
        return None
    shape = hidden.shape
    hidden2 = _as_2d(hidden.reshape(-1, H))
    T, topk = hidden2.shape[0], selected_experts.shape[-1]
    r = factors[0].shape[-1]
    wg, wu, wd = qg.c(), qu.c(), qd.c()
    L = _C.lib()
    if not L.xq_grouped_infer_supported(ctypes.byref(wg), ctypes.byref(wu), ctypes.byref(wd), T, topk, r):
        return None
    if hidden2.data_ptr() % 16 or (T > 1 and hidden2.stride(0) % 8):
        return None
    _C.require_hip(hidden, routing_weights, selected_experts)
    sel = selected_experts.reshape(T, topk).to(torch.int32).contiguous()
    rw = routing_weights.reshape(T, topk)
    if rw.dtype not in (torch.float32, torch.bfloat16):
        rw = rw.float()
    rw = rw.contiguous()
    factors = tuple(f.detach().contiguous() for f in factors)
    dev = hidden2.device
    lora = _lora_struct(factors, r, float(scaling), swiglu_limit)
    key = ("infer", T, topk, num_experts, H, qg.cols, r)
    n = _WS.get(key)
    if n is None:
        n = _WS[key] = L.xq_grouped_infer_workspace_bytes(T, topk, num_experts, H, qg.cols, r)
    ws = torch.empty(n, dtype=torch.uint8, device=dev)
    out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    _C.check(L.xq_grouped_fwd_infer(ctypes.byref(wg), ctypes.byref(wu), ctypes.byref(wd), ctypes.byref(lora),
                                    hidden2.data_ptr(), hidden2.stride(0) if T > 1 else H, T, rw.data_ptr(),
                                    _C.XQ_DT_F32 if rw.dtype == torch.float32 else _C.XQ_DT_BF16, sel.data_ptr(), topk,
                                    out.data_ptr(), H, ws.data_ptr(), ws.numel(), _s(dev)))
    return out.reshape(shape)


def moe_experts_qlora_forward(num_experts: int, routing_weights: Tensor, selected_experts: Tensor,
                              hidden_states: Tensor, gate_proj: QuantWeight, up_proj: QuantWeight,
                              down_proj: QuantWeight, gate_proj_lora_A: Tensor, gate_proj_lora_B: Tensor,
                              up_proj_lora_A: Tensor, up_proj_lora_B: Tensor, down_proj_lora_A: Tensor,
                              down_proj_lora_B: Tensor, scaling: float, swiglu_limit: float = 0.0) -> Tensor:
    """Entry with the argument order of the reference's MOE_EXPERT_BACKENDS_LORA callables
    (models/layers/moe/backend/__init__.py:421-445), except that the three base banks are
    packed QuantWeight descriptors instead of dequantized [E, K, N] tensors.

    A forward of a handful of tokens that nothing is differentiated through (decode, rollout) takes the
    weight-streaming form xq_grouped_fwd_infer where the banks allow it."""
    factors = (gate_proj_lora_A, gate_proj_lora_B, up_proj_lora_A, up_proj_lora_B, down_proj_lora_A, down_proj_lora_B)
    if DECODE_PATH and not torch.compiler.is_compiling() and not (
            torch.is_grad_enabled() and any(t.requires_grad for t in (hidden_states, routing_weights, *factors))):
        out = _moe_infer(hidden_states, routing_weights, selected_experts, factors, (gate_proj, up_proj, down_proj),
                         num_experts, scaling, float(swiglu_limit or 0.0))
        if out is not None:
            return out
    return MoeExpertsQLoRAFunction.apply(hidden_states, routing_weights, selected_experts, gate_proj_lora_A,
                                         gate_proj_lora_B, up_proj_lora_A, up_proj_lora_B, down_proj_lora_A,
                                         down_proj_lora_B, gate_proj, up_proj, down_proj, num_experts, scaling,
                                         float(swiglu_limit or 0.0))


def moe_experts_qlora_ep_compute(permute_tokens: Tensor, cumsum: Tensor, gate_proj: QuantWeight, up_proj: QuantWeight,
                                 down_proj: QuantWeight, gate_proj_lora_A: Tensor, gate_proj_lora_B: Tensor,
                                 up_proj_lora_A: Tensor, up_proj_lora_B: Tensor, down_proj_lora_A: Tensor,
                                 down_proj_lora_B: Tensor, scaling: float, swiglu_limit: float = 0.0) -> Tensor:
    """The expert MLP on rows that are already in expert order: `permute_tokens` [R, H] holds expert 0's rows, then
    expert 1's, ...; `cumsum` [E] is the inclusive running count.  Returns [R, H] in the same order, with no routing
    score applied (the caller multiplies afterwards).  Argument order of the reference's EP_EXPERT_COMPUTE_LORA
    callables (models/layers/moe/backend/__init__.py:377-408; stated per expert in backend/eager.py:187-242), the
    three banks as packed QuantWeight descriptors.

    The rows run through the routed program as a top-1 problem with unit weights: the stable sort by expert is
    then the identity and the weight multiplication exact."""
    E = gate_proj.num_experts
    R = permute_tokens.shape[0]
    if cumsum.numel() < E:
        raise _C.XqError(f"cumsum has {cumsum.numel()} entries for {E} experts")
    factors = (gate_proj_lora_A, gate_proj_lora_B, up_proj_lora_A, up_proj_lora_B, down_proj_lora_A, down_proj_lora_B)
    if R == 0:
        # no rows on this rank: an empty output that still reaches every factor, so their gradients are zeros
        anchor = sum(f.sum() for f in factors) * 0.0
        return permute_tokens.new_zeros((0, down_proj.cols)) + anchor.to(permute_tokens.dtype)
    dev = permute_tokens.device
    ends = cumsum[:E].to(device=dev, dtype=torch.int64)
    expert_of_row = torch.searchsorted(ends, torch.arange(R, device=dev), right=True)
    if int(ends[-1]) != R:
        raise _C.XqError(f"cumsum ends at {int(ends[-1])} but {R} rows were passed")
    ones = torch.ones(R, 1, dtype=torch.float32, device=dev)
    if DECODE_PATH and not torch.compiler.is_compiling() and not (
            torch.is_grad_enabled() and any(t.requires_grad for t in (permute_tokens, *factors))):
        # a handful of rows with nothing to differentiate: the weight-streaming forward (top-1, unit weights)
        out = _moe_infer(permute_tokens, ones, expert_of_row.to(torch.int32).unsqueeze(1), factors, (gate_proj, up_proj, down_proj),
                         E, scaling, float(swiglu_limit or 0.0))
        if out is not None:
            return out
    return MoeExpertsQLoRAFunction.apply(permute_tokens, ones, expert_of_row.to(torch.int32).unsqueeze(1), *factors,
                                         gate_proj, up_proj, down_proj, E, scaling, float(swiglu_limit or 0.0))


# registry entries a maintainer adds beside "triton" / "native" / "quack"
MOE_EXPERT_BACKENDS_QLORA_PACKED: Dict[str, object] = {"hip": moe_experts_qlora_forward}
EP_EXPERT_COMPUTE_QLORA_PACKED: Dict[str, object] = {"hip": moe_experts_qlora_ep_compute}
