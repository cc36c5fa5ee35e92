"""GPU parity of the fused dense SwiGLU MLP (xq_mlp_fwd / xq_mlp_bwd through qlora_mlp_forward) against the float64
program of the oracle and against the three modules called one by one (same rounding points: the base products
are the same kernels' sums, so the two ways agree to bf16 rounding of reordered fp32 sums)."""

import pytest
import torch

from oracle import recipe as R
from tests.util_cases import close, gen, make_dense_module

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _mods(fmt, H, I, r, dev, bias=False, seed=0):
    mods, w_ref = {}, {}
    for i, (k, (N, K)) in enumerate({"gate": (I, H), "up": (I, H), "down": (H, I)}.items()):
        mods[k], w_ref[k] = make_dense_module(fmt, N, K, r, 2 * r, seed=seed + 10 * i, device=dev, bias=bias)
    return mods, w_ref


def _grads(mods):
    return {f"d{f}_{k}": getattr(m, f"lora_{f}").grad.clone() for k, m in mods.items() for f in ("A", "B")}


def _zero(mods):
    for m in mods.values():
        m.lora_A.grad = m.lora_B.grad = None


@pytest.mark.parametrize("tile_policy", [0, 1, 2], indirect=True)
@pytest.mark.parametrize("fmt,M,H,I,r", [
    ("block_fp8", 300, 256, 512, 16),      # fused gate/up/SwiGLU launch, fused dgrad (T = 128 tiles under policy 0)
    ("block_fp8", 1100, 512, 1024, 32),    # 2 rp = 64: both intermediates from one 64-row panel
    ("block_fp8", 130, 128, 192, 8),       # intermediate size not a multiple of 128: dgrads launch by launch
    ("block_fp8", 64, 256, 512, 40),       # 2 rp > 64: separate low-rank passes and dgrads
    ("nvfp4", 260, 256, 512, 16),          # 4-bit formats: the same program launch by launch
    ("int4", 200, 256, 384, 16),
    ("nf4", 200, 256, 384, 16),
])
def test_fused_mlp_vs_oracle_and_modules(hip_device, tile_policy, fmt, M, H, I, r):
    from xorl_amd.functional import silu_and_mul
    from xorl_amd.qlora import qlora_mlp_forward

    mods, w_ref = _mods(fmt, H, I, r, hip_device, seed=M)
    x = gen((M, H), 1.0, 71, torch.bfloat16)
    dy = gen((M, H), 1.0, 72, torch.bfloat16)
    loras = {k: (m.lora_A.detach().cpu(), m.lora_B.detach().cpu()) for k, m in mods.items()}
    ex = R.mlp_fwd_bwd_exact(x, w_ref["gate"], w_ref["up"], w_ref["down"], loras, mods["gate"].scaling, dy)

    xd = x.to(hip_device).requires_grad_(True)
    y = qlora_mlp_forward(mods["gate"], mods["up"], mods["down"], xd)
    y.backward(dy.to(hip_device))
    fused = {"y": y.detach().clone(), "dx": xd.grad.clone(), **_grads(mods)}
    close(fused["y"].cpu(), ex["y"], TOL)
    close(fused["dx"].cpu(), ex["dx"], TOL)
    for k in ("gate", "up", "down"):
        close(fused[f"dA_{k}"].cpu(), ex[f"dA_{k}"], TOL)
        close(fused[f"dB_{k}"].cpu(), ex[f"dB_{k}"], TOL)

    _zero(mods)
    xs = x.to(hip_device).requires_grad_(True)
    ys = mods["down"](silu_and_mul(mods["gate"](xs), mods["up"](xs)))
    ys.backward(dy.to(hip_device))
    sep = {"y": ys.detach(), "dx": xs.grad, **_grads(mods)}
    for name in fused:
        assert R.max_rel_err(fused[name].float().cpu(), sep[name].double().cpu()) <= 2 ** -7, name     # a bf16 step of the largest entry: dX is one rounded sum here, the sum of two rounded products there
    # a forward without grad (inference) gives the training forward's bits
    with torch.no_grad():
        assert torch.equal(qlora_mlp_forward(mods["gate"], mods["up"], mods["down"], x.to(hip_device)), fused["y"])


@pytest.mark.parametrize("tile_policy", [0, 2], indirect=True)
@pytest.mark.parametrize("M,H,I,r,bias", [(300, 256, 512, 16, False), (1100, 512, 1024, 32, True), (2100, 512, 1536, 16, False)])
def test_gate_up_as_one_launch_or_two(hip_device, tile_policy, M, H, I, r, bias):
    """Block-fp8 gate and up as ONE launch with the SwiGLU in its epilogue, or as two launches followed by the pass that
    writes h and forms the down projection's low-rank intermediate (the default): same bits everywhere, and the
    one-launch form against the oracle."""
    from xorl_amd import _C
    from xorl_amd.qlora import qlora_mlp_forward

    mods, w_ref = _mods("block_fp8", H, I, r, hip_device, bias=bias, seed=M + 1)
    x = gen((M, H), 1.0, 81, torch.bfloat16)
    dy = gen((M, H), 1.0, 82, torch.bfloat16)
    got = {}
    try:
        # (the one-launch form lives in the tile kernel that all formats share: the bit-for-bit comparison keeps the two plain
        # launches on that kernel too; with the block-fp8 kernel of its own for them the sums run in another order)
        _C.check(_C.lib().xq_set_fp8_direct_tiles(0))
        for fused in (1, 0):
            _C.check(_C.lib().xq_set_mlp_gate_up_fused(fused))
            _zero(mods)
            xd = x.to(hip_device).requires_grad_(True)
            y = qlora_mlp_forward(mods["gate"], mods["up"], mods["down"], xd)
            y.backward(dy.to(hip_device))
            got[fused] = {"y": y.detach().clone(), "dx": xd.grad.clone(), **_grads(mods)}
        _C.check(_C.lib().xq_set_fp8_direct_tiles(1))
        _C.check(_C.lib().xq_set_mlp_gate_up_fused(0))
        _zero(mods)
        xd = x.to(hip_device).requires_grad_(True)
        y = qlora_mlp_forward(mods["gate"], mods["up"], mods["down"], xd)
        y.backward(dy.to(hip_device))
        direct = {"y": y.detach().clone(), "dx": xd.grad.clone(), **_grads(mods)}
    finally:
        _C.check(_C.lib().xq_set_mlp_gate_up_fused(0))
        _C.check(_C.lib().xq_set_fp8_direct_tiles(1))
    for name in got[0]:
        assert torch.equal(got[0][name], got[1][name]), name
        assert R.max_rel_err(direct[name].float().cpu(), got[0][name].double().cpu()) <= 2 ** -7, name     # same decoded operands, other summation order
    if bias:        # (the oracle's MLP program has no bias terms)
        return
    loras = {k: (m.lora_A.detach().cpu(), m.lora_B.detach().cpu()) for k, m in mods.items()}
    ex = R.mlp_fwd_bwd_exact(x, w_ref["gate"], w_ref["up"], w_ref["down"], loras, mods["gate"].scaling, dy)
    close(got[1]["y"].cpu(), ex["y"], TOL)
    close(got[1]["dx"].cpu(), ex["dx"], TOL)
    for k in ("gate", "up", "down"):
        close(got[1][f"dA_{k}"].cpu(), ex[f"dA_{k}"], TOL)
        close(got[1][f"dB_{k}"].cpu(), ex[f"dB_{k}"], TOL)


def test_fused_mlp_bias_no_lora_and_fallbacks(hip_device):
    from xorl_amd.qlora import qlora_mlp_forward

    H, I, M = 256, 512, 200
    mods, w_ref = _mods("block_fp8", H, I, 16, hip_device, bias=True, seed=3)
    x = gen((M, H), 1.0, 81, torch.bfloat16)
    dy = gen((M, H), 1.0, 82, torch.bfloat16)
    # biases on all three projections, against the float64 program
    Wg, Wu, Wd = (w_ref[k].double() for k in ("gate", "up", "down"))
    s = mods["gate"].scaling
    lin = lambda inp, W, m: inp @ W.t() + m.bias.detach().cpu().double() + s * ((inp @ m.lora_A.detach().cpu().double().t()) @ m.lora_B.detach().cpu().double().t())
    X = x.double()
    want = lin(torch.nn.functional.silu(lin(X, Wg, mods["gate"])) * lin(X, Wu, mods["up"]), Wd, mods["down"])
    with torch.no_grad():
        y = qlora_mlp_forward(mods["gate"], mods["up"], mods["down"], x.to(hip_device))
    close(y.cpu(), want, TOL)
    # frozen biases: the backward still returns dx and the factor gradients
    xd = x.to(hip_device).requires_grad_(True)
    qlora_mlp_forward(mods["gate"], mods["up"], mods["down"], xd).backward(dy.to(hip_device))
    assert xd.grad is not None and mods["down"].lora_B.grad is not None
    # different active ranks: the helper calls the modules one by one and still agrees
    mods["up"].set_runtime_lora_config(8, 16)
    with torch.no_grad():
        y2 = qlora_mlp_forward(mods["gate"], mods["up"], mods["down"], x.to(hip_device))
    assert y2.shape == y.shape and bool(torch.isfinite(y2.float()).all())
    # empty batch
    with torch.no_grad():
        y0 = qlora_mlp_forward(mods["gate"], mods["down"].__class__(H, I, device=hip_device) if False else mods["up"], mods["down"],
                               torch.zeros(0, H, dtype=torch.bfloat16, device=hip_device))
    assert y0.shape == (0, H)


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
def test_fused_mlp_under_torch_compile(hip_device, backend):
    from xorl_amd.qlora import qlora_mlp_forward

    mods, _ = _mods("block_fp8", 256, 512, 16, hip_device, seed=9)
    x = gen((300, 256), 1.0, 91, torch.bfloat16).to(hip_device)
    dy = gen((300, 256), 1.0, 92, torch.bfloat16).to(hip_device)

    def run(fn):
        _zero(mods)
        xd = x.clone().requires_grad_(True)
        y = fn(mods["gate"], mods["up"], mods["down"], xd)
        y.backward(dy)
        return [y.detach().clone(), xd.grad.clone()] + list(_grads(mods).values())

    ref = run(qlora_mlp_forward)
    torch._dynamo.reset()
    got = run(torch.compile(qlora_mlp_forward, backend=backend, fullgraph=True))
    for a, b in zip(ref, got):
        assert torch.equal(a, b)


def test_gate_up_form_travels_with_the_saved_state(hip_device):
    """The form a forward ran gate and up in (one launch or two) fixes the layout of the saved low-rank intermediates;
    it travels to the backward in xq_mlp_saved, so flipping the process-wide default between a forward and its backward
    changes nothing: every gradient equals the undisturbed step's bit for bit, in both directions of the flip."""
    from xorl_amd import _C
    from xorl_amd.qlora import qlora_mlp_forward

    M, H, I, r = 384, 512, 768, 16
    mods, _ = _mods("block_fp8", H, I, r, hip_device, bias=False, seed=77)
    x = gen((M, H), 1.0, 91, torch.bfloat16)
    dy = gen((M, H), 1.0, 92, torch.bfloat16)
    L = _C.lib()

    def step(fwd_mode, bwd_mode):
        _zero(mods)
        _C.check(L.xq_set_mlp_gate_up_fused(fwd_mode))
        xd = x.to(hip_device).requires_grad_(True)
        y = qlora_mlp_forward(mods["gate"], mods["up"], mods["down"], xd)
        _C.check(L.xq_set_mlp_gate_up_fused(bwd_mode))
        y.backward(dy.to(hip_device))
        return {"y": y.detach().clone(), "dx": xd.grad.clone(), **_grads(mods)}

    try:
        base = step(0, 0)
        for fwd_mode, bwd_mode in ((0, 1), (1, 0), (1, 1)):
            got = step(fwd_mode, bwd_mode)
            for name in base:
                assert torch.equal(got[name], base[name]), (fwd_mode, bwd_mode, name)
    finally:
        _C.check(L.xq_set_mlp_gate_up_fused(0))


def test_mlp_backward_rejects_a_saved_state_without_its_form(hip_device):
    """xq_mlp_bwd takes the form from the struct the forward filled; a struct that does not say (negative) is an argument error."""
    import ctypes
    from xorl_amd import _C
    from xorl_amd import functional as F

    M, H, I, r = 128, 256, 256, 16
    mods, _ = _mods("block_fp8", H, I, r, hip_device, bias=False, seed=5)
    banks = tuple(mods[k]._forward_quant_weight() for k in ("gate", "up", "down"))
    factors = tuple(t.detach().contiguous() for k in ("gate", "up", "down") for t in (mods[k].lora_A, mods[k].lora_B))
    x = gen((M, H), 1.0, 3, torch.bfloat16).to(hip_device)
    y, saved = F._mlp_fwd_impl(x, factors, (None, None, None), banks, r, 2.0, 0)
    with pytest.raises(ValueError, match="gate_up_fused"):
        F._mlp_bwd_impl(torch.ones_like(y), x, saved, factors, banks, r, 2.0, True, -1)
