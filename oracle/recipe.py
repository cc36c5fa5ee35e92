"""TEST INFRASTRUCTURE ONLY: the reference's forward/backward recipe in torch CPU ops.

The reference has no CPU implementation of its decoders (they are Triton
kernels), so "the reference's CPU path" is its *recipe* -- the op sequence of
``QLoRALinear.forward`` and of the grouped LoRA MLP -- executed with torch CPU
ops on an already decoded weight.  Two flavours of each program:

* ``*_recipe``: the reference's dtypes and rounding points (bf16 GEMM output,
  fp32 LoRA branch, bf16 add).  This is what bench.py times as cpu_baseline.
* ``*_exact``: the same mathematics in float64 with no intermediate rounding,
  the "fp32-accumulated path" the tolerance tests compare kernels against
  (float64 so the yardstick's own error is negligible).

Reference statements followed (paths relative to the xorl checkout):
  dense fwd    qlora/modules/linear.py:369-385
  dense bwd    autograd of the above; stated explicitly by _surrogate_vjp,
               models/transformers/glm5/exact_qlora.py:255-317
  SwiGLU       ops/fused_silu_and_mul.py:22-60 (bf16(silu_fp32(g)) * up)
  grouped fwd  ops/moe/lora.py:525-713, bwd :715-1007; per-expert statement
               models/layers/moe/backend/eager.py:187-242
  routing      stable argsort by expert id, ops/group_gemm/kernel/moe.py:26-40
"""

from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------
# dense
# --------------------------------------------------------------------------
def linear_forward_recipe(x, w_deq, lora_A, lora_B, scaling: float, bias=None):
    """qlora/modules/linear.py:369-385, op for op.

    x bf16 [..., K]; w_deq the decoder's output (bf16, or fp32 for block_fp8);
    lora_A [r, K], lora_B [N, r] (fp32 parameters in the reference).
    """
    w = w_deq.to(x.dtype)
    result = F.linear(x, w, bias)
    x_lora = x.to(lora_A.dtype)
    lora_out = F.linear(F.linear(x_lora, lora_A), lora_B) * scaling
    return result + lora_out.to(result.dtype)


def linear_fwd_bwd_recipe(x, w_deq, lora_A, lora_B, scaling, dy):
    """Forward + autograd backward of the recipe. Returns y, dx, dA, dB."""
    x = x.detach().clone().requires_grad_(True)
    A = lora_A.detach().clone().requires_grad_(True)
    B = lora_B.detach().clone().requires_grad_(True)
    y = linear_forward_recipe(x, w_deq, A, B, scaling)
    y.backward(dy)
    return y.detach(), x.grad, A.grad, B.grad


def linear_fwd_bwd_exact(x, w_deq, lora_A, lora_B, scaling, dy=None, bias=None):
    """float64, no intermediate rounding.  The weight is first rounded to bf16
    exactly as the recipe does (that rounding is part of the decode contract,
    not of the GEMM).  Returns dict with y and, when dy is given, dx/dA/dB."""
    X = x.double().reshape(-1, x.shape[-1])
    W = w_deq.to(torch.bfloat16).double()
    A, B = lora_A.double(), lora_B.double()
    u = X @ A.t()
    y = X @ W.t() + scaling * (u @ B.t())
    if bias is not None:
        y = y + bias.double()
    out = {"y": y.reshape(*x.shape[:-1], -1)}
    if dy is not None:
        G = dy.double().reshape(-1, dy.shape[-1])
        v = scaling * (G @ B)
        out["dx"] = (G @ W + v @ A).reshape(x.shape)
        out["dA"] = v.t() @ X
        out["dB"] = scaling * (G.t() @ u)
    return out


def silu_and_mul_recipe(gate, up):
    """ops/fused_silu_and_mul.py:22-60: SiLU in fp32, rounded to the input
    dtype, then multiplied in that dtype (two roundings)."""
    g = gate.float()
    act = (g * torch.sigmoid(g)).to(gate.dtype)
    return act * up


def mlp_fwd_bwd_exact(x, w_gate, w_up, w_down, loras, scaling, dy=None, dtype=torch.float64):
    """SwiGLU MLP of three QLoRA linears without intermediate rounding (Qwen3MLP.forward,
    models/transformers/qwen3/modeling_qwen3.py:60-81: down(act(gate(x)) * up(x))).  ``loras`` maps
    'gate'/'up'/'down' to (A [r,K], B [N,r]).  Returns y and grads by autograd.

    dtype=float64 is the yardstick; dtype=float32 is the same program with fp32 accumulation (its own
    error, ~1e-6 relative, is far below the 1e-2 tolerance) for sizes float64 cannot finish in seconds."""
    need = dy is not None
    X = x.to(dtype).detach().clone().requires_grad_(need)
    P = {}
    for k, (A, B) in loras.items():
        P[k] = (A.to(dtype).detach().clone().requires_grad_(need), B.to(dtype).detach().clone().requires_grad_(need))

    def lin(inp, w, key):
        A, B = P[key]
        return inp @ w.to(torch.bfloat16).to(dtype).t() + scaling * ((inp @ A.t()) @ B.t())

    g = lin(X, w_gate, "gate")
    u = lin(X, w_up, "up")
    h = F.silu(g) * u
    y = lin(h, w_down, "down")
    out = {"y": y.detach(), "gate": g.detach(), "up": u.detach(), "h": h.detach()}
    if need:
        y.backward(dy.to(dtype))
        out["dx"] = X.grad
        for k, (A, B) in P.items():
            out[f"dA_{k}"], out[f"dB_{k}"] = A.grad, B.grad
    return out


# --------------------------------------------------------------------------
# grouped / routed
# --------------------------------------------------------------------------
def route_build(selected_experts: torch.Tensor, num_experts: int):
    """Histogram + stable permutation, ops/moe/lora.py:580-582.

    Returns (splits [E], scatter_index [T, topk]) where scatter_index[t, j] is
    the row of routed copy (t, j) in expert order."""
    flat = selected_experts.reshape(-1).long()
    splits = torch.bincount(flat, minlength=num_experts)
    scatter_index = flat.argsort(stable=True).argsort().int().view(selected_experts.shape)
    return splits, scatter_index


def _expand(t: torch.Tensor, E: int) -> torch.Tensor:
    return t.expand(E, -1, -1) if t.shape[0] == 1 else t


def moe_fwd_bwd(
    hidden: torch.Tensor,                  # [T, H]
    routing_weights: torch.Tensor,         # [T, topk]
    selected_experts: torch.Tensor,        # [T, topk] int
    w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,   # decoded GKN banks [E,H,I],[E,H,I],[E,I,H]
    lora: Dict[str, Tuple[torch.Tensor, torch.Tensor]],  # 'gate'/'up'/'down' -> (A [E|1,K,r], B [E|1,r,N])
    scaling: float,
    dy: Optional[torch.Tensor] = None,
    dtype: torch.dtype = torch.float64,
    swiglu_limit: float = 0.0,
):
    """The grouped LoRA MLP of ops/moe/lora.py:525-713 as a per-expert loop
    (the form of eager_ep_compute_lora, backend/eager.py:187-242), with the
    routing weight applied BEFORE the down projection (:644-647) and the
    top-k copies summed at the end (moe_gather).  Gradients by autograd.

    dtype=float64: the exact yardstick.  dtype=bfloat16: the reference's
    rounding points (bf16 between grouped GEMMs, factors cast to bf16)."""
    E = w_gate.shape[0]
    T, H = hidden.shape
    need = dy is not None
    X = hidden.to(dtype).detach().clone().requires_grad_(need)
    RW = routing_weights.to(dtype).detach().clone().requires_grad_(need)
    P = {}
    for k, (A, B) in lora.items():
        P[k] = (A.detach().clone().requires_grad_(need), B.detach().clone().requires_grad_(need))
    Wg = w_gate.to(torch.bfloat16).to(dtype)
    Wu = w_up.to(torch.bfloat16).to(dtype)
    Wd = w_down.to(torch.bfloat16).to(dtype)

    out = torch.zeros(T, H, dtype=torch.float64 if dtype == torch.float64 else torch.float32)
    sel = selected_experts.long()
    for e in range(E):
        tok, slot = (sel == e).nonzero(as_tuple=True)
        if tok.numel() == 0:
            continue
        xe = X[tok]
        def proj(inp, W, key):
            A, B = P[key]
            Ae = _expand(A, E)[e].to(dtype)
            Be = _expand(B, E)[e].to(dtype)
            return inp @ W[e] + ((inp @ Ae) @ Be) * scaling
        g = proj(xe, Wg, "gate")
        u = proj(xe, Wu, "up")
        if swiglu_limit > 0:
            # ops/moe/triton.py:127-141: the gate pre-activation clamped before the SiLU (lora.py:638), the gate gradient
            # zero where the unclamped value lies outside [-limit, limit] (lora.py:917-919) -- which is what autograd gives
            # for clamp, the bounds themselves passing the gradient
            g = g.clamp(-swiglu_limit, swiglu_limit)
        h = F.silu(g) * u
        h = h * RW[tok, slot].unsqueeze(1)
        d = proj(h, Wd, "down")
        out = out.index_add(0, tok, d.to(out.dtype))
    y = out.to(dtype)
    res = {"y": y.detach()}
    if need:
        y.backward(dy.to(dtype))
        res["dx"] = X.grad
        res["d_routing"] = RW.grad
        for k, (A, B) in P.items():
            res[f"dA_{k}"] = A.grad if A.grad is not None else torch.zeros_like(A)
            res[f"dB_{k}"] = B.grad if B.grad is not None else torch.zeros_like(B)
    return res


# --------------------------------------------------------------------------
# error measure used by every tolerance test
# --------------------------------------------------------------------------
def max_rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """max |got - ref| / max |ref|  (tensor-normalised: elementwise relative
    error is undefined at the zeros every GEMM output has)."""
    ref = ref.double()
    denom = ref.abs().max().item()
    if denom == 0.0:
        return float((got.double() - ref).abs().max().item())
    return float((got.double() - ref).abs().max().item() / denom)


def row_rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """max over rows of  max |got_row - ref_row| / max |ref_row|  (rows = the last dimension's vectors).

    Stricter than max_rel_err: a systematic error confined to rows of small magnitude (which the
    tensor-wide maximum hides) shows up here.  Rows whose reference is all zero must be exactly zero."""
    ref = ref.double().reshape(-1, ref.shape[-1]) if ref.dim() > 1 else ref.double().reshape(1, -1)
    got = got.double().reshape(ref.shape)
    err = (got - ref).abs().amax(dim=1)
    den = ref.abs().amax(dim=1)
    zero = den == 0
    if bool((err[zero] != 0).any()):
        return float("inf")
    if bool(zero.all()):
        return 0.0
    return float((err[~zero] / den[~zero]).max().item())


# ---------------------------------------------------------------------------
# merging the LoRA update into the base weight
# ---------------------------------------------------------------------------
def merge_delta_exact(lora_A: torch.Tensor, lora_B: torch.Tensor, scaling: float) -> torch.Tensor:
    """get_delta_weight (qlora/modules/linear.py:397-400): (B @ A) * scaling, here with the product in
    float64 and one rounding to fp32 at the end (the reference's fp32 matmul has an unspecified
    summation order; any order is within a few fp32 ulps of this)."""
    return ((lora_B.double() @ lora_A.double()) * scaling).float()


def merge_publish_recipe(w_deq: torch.Tensor, lora_A, lora_B, scaling: float) -> torch.Tensor:
    """server/weight_sync/handler.py:2119-2131: `deq.to(bf16) + delta.to(bf16)` (a bf16 add)."""
    return w_deq.to(torch.bfloat16) + merge_delta_exact(lora_A, lora_B, scaling).to(torch.bfloat16)


def merge_fp32_recipe(w_deq_f32: torch.Tensor, lora_A, lora_B, scaling: float) -> torch.Tensor:
    """block_fp8 merge_weights before re-quantisation (block_fp8_linear.py:111-115): fp32 deq + fp32 delta."""
    return w_deq_f32.float() + merge_delta_exact(lora_A, lora_B, scaling)
