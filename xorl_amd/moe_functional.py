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
from typing import Dict, Optional, Tuple

import torch
from torch import Tensor

from . import _C
from .functional import QuantWeight, _r_pad


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


class MoeExpertsQLoRAFunction(torch.autograd.Function):
    """Routed SwiGLU expert MLP with LoRA on packed banks.

    inputs: hidden [T, H] bf16, routing_weights [T, topk], selected_experts
    [T, topk], three QuantWeight banks (GKN: gate/up [E, H, I], down [E, I, H]),
    six LoRA factors in GKN form (A [E|1, in, r], B [E|1, r, out]).  Returns
    [T, H] bf16.  Gradients: hidden, routing_weights and the six factors; the
    frozen banks get none.  Experts that receive no rows get exact-zero factor
    gradients."""

    @staticmethod
    def forward(ctx, hidden, routing_weights, selected_experts, gA, gB, uA, uB, dA, dB,
                qw_gate: QuantWeight, qw_up: QuantWeight, qw_down: QuantWeight, num_experts: int, scaling: float):
        _C.require_hip(hidden, routing_weights, selected_experts)
        if hidden.dtype != torch.bfloat16:
            raise _C.XqError(f"hidden states must be bf16, got {hidden.dtype}")
        E = num_experts
        for qw in (qw_gate, qw_up, qw_down):
            if qw.num_experts != E:          # the tile schedules route_build emits are laid out for E experts
                raise _C.XqError(f"routing over {E} experts but a bank holds {qw.num_experts}")
        shape = hidden.shape
        H = shape[-1]
        hidden2 = hidden.reshape(-1, H)
        T = hidden2.shape[0]
        topk = selected_experts.shape[-1]
        dev = hidden.device
        r = gA.shape[-1]
        rp = _r_pad(r)
        I = qw_gate.cols
        s = float(scaling)

        counts, offsets, sidx, tile_offsets = route_build(selected_experts, E)
        xs = moe_scatter(hidden2, sidx, topk)                                     # [R, H] expert order
        # bf16 operand layouts of the factors
        F_gA = _prep(gA, True, rp, H)                                             # [E|1, rp, H]
        F_uA = _prep(uA, True, rp, H)
        Lr_gB = _prep(_expand(gB, E), True, I, rp)                                # [E, I, rp]
        Lr_uB = _prep(_expand(uB, E), True, I, rp)
        F_dA = _prep(dA, True, rp, I)                                             # [E|1, rp, I]
        Lr_dB = _prep(_expand(dB, E), True, H, rp)                                # [E, H, rp]

        # (one pass over xs with both panels side by side takes as long as these two: the product is bound by its
        # fp32 multiply-adds, not by reading the rows)
        su_g = _lora_down(xs, F_gA, offsets, tile_offsets, E, s)
        su_u = _lora_down(xs, F_uA, offsets, tile_offsets, E, s)
        gate_out = _grouped_gemm(qw_gate, False, xs, offsets, tile_offsets, su_g, Lr_gB)    # [R, I]
        up_out = _grouped_gemm(qw_up, False, xs, offsets, tile_offsets, su_u, Lr_uB)
        L = _C.lib()
        R = xs.shape[0]
        rw = routing_weights.reshape(-1).contiguous()
        if rw.dtype not in (torch.float32, torch.bfloat16):
            rw = rw.float()
        w_row = torch.empty(R, dtype=torch.float32, device=dev)
        _C.check(L.xq_moe_scatter_scalar(rw.data_ptr(), _C.XQ_DT_F32 if rw.dtype == torch.float32 else _C.XQ_DT_BF16,
                                         sidx.data_ptr(), R, w_row.data_ptr(), _s(dev)))
        h = torch.empty(R, I, dtype=torch.bfloat16, device=dev)
        _C.check(L.xq_silu_mul_fwd(gate_out.data_ptr(), up_out.data_ptr(), I, w_row.data_ptr(), h.data_ptr(), I, R, I,
                                   _s(dev)))
        su_d = _lora_down(h, F_dA, offsets, tile_offsets, E, s)
        down_out = _grouped_gemm(qw_down, False, h, offsets, tile_offsets, su_d, Lr_dB)     # [R, H]
        out = moe_gather(down_out, None, sidx, T, topk)

        ctx.qw = (qw_gate, qw_up, qw_down)
        ctx.meta = (E, T, topk, H, I, r, rp, s, shape, routing_weights.dtype, routing_weights.shape)
        ctx.save_for_backward(xs, gate_out, up_out, h, w_row, su_g, su_u, su_d, sidx, offsets, tile_offsets,
                              gA, gB, uA, uB, dA, dB)
        return out.reshape(shape)

    @staticmethod
    def backward(ctx, dy):
        (xs, gate_out, up_out, h, w_row, su_g, su_u, su_d, sidx, offsets, tile_offsets,
         gA, gB, uA, uB, dA, dB) = ctx.saved_tensors
        qw_gate, qw_up, qw_down = ctx.qw
        E, T, topk, H, I, r, rp, s, shape, rw_dtype, rw_shape = ctx.meta
        dev = dy.device
        L = _C.lib()
        R = xs.shape[0]
        g_down = moe_scatter(dy.reshape(-1, H).to(torch.bfloat16), sidx, topk)               # [R, H]

        # ---- down projection: y = h.W + s*(h.A).B
        F_dB = _prep(dB, False, rp, H)                                                       # [E|1, rp, H]
        v_d = _lora_down(g_down, F_dB, offsets, tile_offsets, E, s)                          # s * g . B^T
        Lr_dA = _prep(_expand(dA, E), False, I, rp)                                          # [E, I, rp]
        dh = _grouped_gemm(qw_down, True, g_down, offsets, tile_offsets, v_d, Lr_dA)         # [R, I]
        shared_dB = dB.shape[0] == 1
        n_valid = offsets[E:]            # rows that belong to an expert (all of them unless an id was out of range)
        grad_dB = _wgrad(g_down, su_d, r, None if shared_dB else offsets, E, True, n_valid)  # [E|1, r, H]
        grad_dA = _wgrad(h, v_d, r, None if dA.shape[0] == 1 else offsets, E, False, n_valid)   # [E|1, I, r]

        # ---- SwiGLU + routing weight
        dgate = torch.empty(R, I, dtype=torch.bfloat16, device=dev)
        dup = torch.empty(R, I, dtype=torch.bfloat16, device=dev)
        d_w_row = torch.empty(R, dtype=torch.float32, device=dev)
        _C.check(L.xq_silu_mul_bwd(gate_out.data_ptr(), up_out.data_ptr(), I, dh.data_ptr(), I, w_row.data_ptr(),
                                   dgate.data_ptr(), dup.data_ptr(), I, d_w_row.data_ptr(), R, I, _s(dev)))
        d_rw = None
        if ctx.needs_input_grad[1]:
            out_dt = rw_dtype if rw_dtype in (torch.float32, torch.bfloat16) else torch.float32
            d_rw = torch.empty(R, dtype=out_dt, device=dev)
            _C.check(L.xq_moe_gather_scalar(d_w_row.data_ptr(), sidx.data_ptr(), R, d_rw.data_ptr(),
                                            _C.XQ_DT_F32 if out_dt == torch.float32 else _C.XQ_DT_BF16, _s(dev)))
            d_rw = d_rw.reshape(rw_shape).to(rw_dtype)

        # ---- up / gate projections: y = x.W + s*(x.A).B
        def proj_bwd(g_out, qw, A, B, su):
            F_B = _prep(B, False, rp, I)                                                     # [E|1, rp, I]
            v = _lora_down(g_out, F_B, offsets, tile_offsets, E, s)
            Lr_A = _prep(_expand(A, E), False, H, rp)                                        # [E, H, rp]
            dx = _grouped_gemm(qw, True, g_out, offsets, tile_offsets, v, Lr_A)              # [R, H]
            gB_ = _wgrad(g_out, su, r, None if B.shape[0] == 1 else offsets, E, True, n_valid)   # [E|1, r, I]
            return dx, v, gB_

        dx_u, v_u, grad_uB = proj_bwd(dup, qw_up, uA, uB, su_u)
        dx_g, v_g, grad_gB = proj_bwd(dgate, qw_gate, gA, gB, su_g)
        # gradients of the two A factors, [E|1, H, r] = x^T . v: both contract the same rows of x, so they share
        # one pass over them (v_g | v_u side by side) when the panels fit
        if gA.shape[0] == uA.shape[0] and 2 * rp <= 32:
            both = _wgrad(xs, torch.cat([v_g, v_u], dim=1), rp + r, None if gA.shape[0] == 1 else offsets, E, False, n_valid)
            grad_gA, grad_uA = both[..., :r], both[..., rp:rp + r]
        else:
            grad_gA = _wgrad(xs, v_g, r, None if gA.shape[0] == 1 else offsets, E, False, n_valid)
            grad_uA = _wgrad(xs, v_u, r, None if uA.shape[0] == 1 else offsets, E, False, n_valid)
        dx = moe_gather(dx_g, dx_u, sidx, T, topk).reshape(shape) if ctx.needs_input_grad[0] else None

        cast = lambda g, p: g.to(p.dtype)
        return (dx, d_rw, None, cast(grad_gA, gA), cast(grad_gB, gB), cast(grad_uA, uA), cast(grad_uB, uB),
                cast(grad_dA, dA), cast(grad_dB, dB), None, None, None, None, None)


def moe_experts_qlora_forward(num_experts: int, routing_weights: Tensor, selected_experts: Tensor,
                              hidden_states: Tensor, gate_proj: QuantWeight, up_proj: QuantWeight,
                              down_proj: QuantWeight, gate_proj_lora_A: Tensor, gate_proj_lora_B: Tensor,
                              up_proj_lora_A: Tensor, up_proj_lora_B: Tensor, down_proj_lora_A: Tensor,
                              down_proj_lora_B: Tensor, scaling: float, swiglu_limit: float = 0.0) -> Tensor:
    """Entry with the argument order of the reference's MOE_EXPERT_BACKENDS_LORA callables
    (models/layers/moe/backend/__init__.py:421-445), except that the three base banks are
    packed QuantWeight descriptors instead of dequantized [E, K, N] tensors."""
    if swiglu_limit:
        raise NotImplementedError("swiglu_limit clamping is not part of the packed-bank expert path")
    return MoeExpertsQLoRAFunction.apply(hidden_states, routing_weights, selected_experts, gate_proj_lora_A,
                                         gate_proj_lora_B, up_proj_lora_A, up_proj_lora_B, down_proj_lora_A,
                                         down_proj_lora_B, gate_proj, up_proj, down_proj, num_experts, scaling)


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
    if swiglu_limit:
        raise NotImplementedError("swiglu_limit clamping is not part of the packed-bank expert path")
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
    return MoeExpertsQLoRAFunction.apply(permute_tokens, ones, expert_of_row.to(torch.int32).unsqueeze(1), *factors,
                                         gate_proj, up_proj, down_proj, E, scaling)


# registry entries a maintainer adds beside "triton" / "native" / "quack"
MOE_EXPERT_BACKENDS_QLORA_PACKED: Dict[str, object] = {"hip": moe_experts_qlora_forward}
EP_EXPERT_COMPUTE_QLORA_PACKED: Dict[str, object] = {"hip": moe_experts_qlora_ep_compute}
