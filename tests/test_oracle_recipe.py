"""Pins for oracle.recipe (no GPU): the dense and grouped programs."""

import torch
import torch.nn.functional as F

from oracle import recipe as R


def _glm52_fixture():
    # closed-form inputs of tests/models/test_glm52_exact_qlora.py:105-144
    A = torch.tensor([[0.1001, -0.2002, 0.3003, -0.4004, 0.5005, -0.6006, 0.7007, -0.8008]])
    B = torch.tensor([[0.1101], [-0.2202], [0.3303], [-0.4404], [0.5505], [-0.6606]])
    w = torch.arange(48, dtype=torch.float32).reshape(6, 8).sub_(17).div_(41).to(torch.bfloat16)
    x = torch.arange(32, dtype=torch.float32).reshape(2, 2, 8).sub_(9).div_(29).to(torch.bfloat16)
    g = torch.arange(24, dtype=torch.float32).reshape(2, 2, 6).sub_(7).div_(31).to(torch.bfloat16)
    return x, w, A, B, g


def test_dense_recipe_backward_matches_reference_closed_form():
    """dX = bf16 F.linear autograd through the decoded weight + fp32 LoRA chain;
    dA, dB = fp32 autograd of F.linear(F.linear(x32, A), B) -- the expectation
    the reference's own test builds (test_glm52_exact_qlora.py:124-138), here
    with the module's fp32 master factors (QLoRALinear keeps lora_A/B fp32)."""
    x, w, A, B, g = _glm52_fixture()
    y, dx, dA, dB = R.linear_fwd_bwd_recipe(x, w.float(), A, B, 1.0, g)

    bx = x.detach().clone().requires_grad_(True)
    F.linear(bx, w).backward(g)
    lx = x.detach().float().requires_grad_(True)
    rA = A.clone().requires_grad_(True)
    rB = B.clone().requires_grad_(True)
    F.linear(F.linear(lx, rA), rB).backward(g.float())
    # dense autograd: the bf16 cast of the LoRA branch sends a bf16 grad back
    expected_dx = (bx.grad.float() + lx.grad).to(torch.bfloat16)
    assert dx.dtype == torch.bfloat16
    assert R.max_rel_err(dx, expected_dx) < 2 ** -7
    assert torch.equal(dA, rA.grad)
    assert torch.equal(dB, rB.grad)
    # forward rounding points: base->bf16, lora->bf16, sum->bf16
    base = F.linear(x, w)
    lo = (F.linear(F.linear(x.float(), A), B) * 1.0).to(torch.bfloat16)
    assert torch.equal(y, base + lo)


def test_dense_exact_matches_recipe_within_bf16_and_invariants():
    torch.manual_seed(0)
    M, K, N, r, s = 24, 64, 48, 4, 2.0
    x = torch.randn(M, K).to(torch.bfloat16)
    w = (torch.randn(N, K) * 0.05).to(torch.bfloat16)
    A, B = torch.randn(r, K) * 0.05, torch.randn(N, r) * 0.05
    dy = torch.randn(M, N).to(torch.bfloat16)
    y, dx, dA, dB = R.linear_fwd_bwd_recipe(x, w, A, B, s, dy)
    ex = R.linear_fwd_bwd_exact(x, w, A, B, s, dy)
    assert R.max_rel_err(y, ex["y"]) < 1e-2
    assert R.max_rel_err(dx, ex["dx"]) < 1e-2
    assert R.max_rel_err(dA, ex["dA"]) < 1e-2
    assert R.max_rel_err(dB, ex["dB"]) < 1e-2
    # lora_B = 0  =>  y == base exactly
    y0 = R.linear_forward_recipe(x, w, A, torch.zeros_like(B), s)
    assert torch.equal(y0, F.linear(x, w))
    # a dropped scaling or a transposed factor must show
    wrong = R.linear_fwd_bwd_exact(x, w, A, B, 1.0, dy)
    assert R.max_rel_err(wrong["dB"], ex["dB"]) > 0.1


def test_dense_exact_gradients_by_finite_differences():
    torch.manual_seed(1)
    M, K, N, r, s = 3, 8, 5, 2, 1.5
    x = torch.randn(M, K).to(torch.bfloat16)
    w = torch.randn(N, K).to(torch.bfloat16)
    A, B = torch.randn(r, K), torch.randn(N, r)
    dy = torch.randn(M, N).to(torch.bfloat16)
    ex = R.linear_fwd_bwd_exact(x, w, A, B, s, dy)

    def loss(xx, AA, BB):
        return (R.linear_fwd_bwd_exact(xx, w, AA, BB, s)["y"] * dy.double()).sum()

    eps = 1e-6
    for name, t, grad in (("dA", A.double(), ex["dA"]), ("dB", B.double(), ex["dB"]), ("dx", x.double(), ex["dx"])):
        num = torch.zeros_like(t)
        for i in range(t.numel()):
            d = torch.zeros_like(t).reshape(-1)
            d[i] = eps
            d = d.reshape(t.shape)
            args = {"dA": (x.double(), t + d, B.double()), "dB": (x.double(), A.double(), t + d),
                    "dx": (t + d, A.double(), B.double())}[name]
            args_m = {"dA": (x.double(), t - d, B.double()), "dB": (x.double(), A.double(), t - d),
                      "dx": (t - d, A.double(), B.double())}[name]
            num.reshape(-1)[i] = (loss(*args) - loss(*args_m)) / (2 * eps)
        assert torch.allclose(num, grad, rtol=1e-6, atol=1e-7), name


def test_silu_and_mul_two_roundings():
    torch.manual_seed(2)
    g = (torch.randn(64, 32) * 3).to(torch.bfloat16)
    u = torch.randn(64, 32).to(torch.bfloat16)
    h = R.silu_and_mul_recipe(g, u)
    one_round = (F.silu(g.float()) * u.float()).to(torch.bfloat16)
    two_round = F.silu(g.float()).to(torch.bfloat16) * u
    assert torch.equal(h, two_round)
    assert not torch.equal(h, one_round)      # the distinction is observable


def _moe_case(E=6, T=40, H=16, I=12, r=2, topk=2, seed=3, shared=False):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T, H, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, generator=g)
    logits[:, E - 1] = -1e9                                # last expert gets no tokens
    rw, sel = torch.topk(torch.softmax(logits, -1), topk, dim=-1)
    rw = (rw / rw.sum(-1, keepdim=True)).to(torch.bfloat16)
    wg = (torch.randn(E, H, I, generator=g) * 0.2).to(torch.bfloat16)
    wu = (torch.randn(E, H, I, generator=g) * 0.2).to(torch.bfloat16)
    wd = (torch.randn(E, I, H, generator=g) * 0.2).to(torch.bfloat16)
    eA, eB = (1, E) if shared else (E, E)
    lora = {
        "gate": (torch.randn(eA, H, r, generator=g) * 0.2, torch.randn(E, r, I, generator=g) * 0.2),
        "up": (torch.randn(eA, H, r, generator=g) * 0.2, torch.randn(E, r, I, generator=g) * 0.2),
        "down": (torch.randn(E, I, r, generator=g) * 0.2, torch.randn(1 if shared else E, r, H, generator=g) * 0.2),
    }
    dy = torch.randn(T, H, generator=g).to(torch.bfloat16)
    return hidden, rw, sel, wg, wu, wd, lora, dy


def test_route_build_is_stable_sort_by_expert():
    sel = torch.tensor([[2, 0], [0, 1], [2, 1], [0, 2]])
    splits, idx = R.route_build(sel, 4)
    assert splits.tolist() == [3, 2, 3, 0]
    # rows of expert 0 first, in original (token, slot) order
    order = torch.empty(8, dtype=torch.long)
    order[idx.flatten().long()] = torch.arange(8)
    assert sel.flatten()[order].tolist() == [0, 0, 0, 1, 1, 2, 2, 2]
    assert order.tolist() == [1, 2, 6, 3, 5, 0, 4, 7]


def test_grouped_program_against_per_token_brute_force():
    hidden, rw, sel, wg, wu, wd, lora, dy = _moe_case()
    res = R.moe_fwd_bwd(hidden, rw, sel, wg, wu, wd, lora, 0.5, dy)
    # brute force: one (token, slot) at a time, routing weight BEFORE down_proj
    T, H = hidden.shape
    y = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for j in range(sel.shape[1]):
            e = int(sel[t, j])
            x = hidden[t].double()
            def p(v, W, key):
                A, B = lora[key]
                return v @ W[e].double() + ((v @ A[e].double()) @ B[e].double()) * 0.5
            h = F.silu(p(x, wg, "gate")) * p(x, wu, "up") * rw[t, j].double()
            y[t] += p(h, wd, "down")
    assert torch.allclose(res["y"], y, rtol=1e-12, atol=1e-12)
    # empty expert: structural-zero grads (group_gemm.py:346-360)
    E = wg.shape[0]
    assert (sel == E - 1).sum() == 0
    for k in ("gate", "up", "down"):
        assert torch.count_nonzero(res[f"dA_{k}"][E - 1]) == 0
        assert torch.count_nonzero(res[f"dB_{k}"][E - 1]) == 0


def test_grouped_swiglu_limit_against_the_reference_rule():
    """swiglu_limit in the oracle's grouped program against the reference's two rules written out by hand
    (ops/moe/triton.py:127-141): forward silu(clamp(gate, -L, L)) * up per (token, slot); backward the gate gradient
    silu'(clamped gate) * (dh * up), zeroed where the UNCLAMPED gate lies outside [-L, L] with the bounds themselves inside."""
    hidden, rw, sel, wg, wu, wd, lora, dy = _moe_case(seed=7)
    L = 0.6                                     # inside the spread of this case's gate values
    res = R.moe_fwd_bwd(hidden, rw, sel, wg, wu, wd, lora, 0.5, dy, swiglu_limit=L)
    plain = R.moe_fwd_bwd(hidden, rw, sel, wg, wu, wd, lora, 0.5, dy)
    T, H = hidden.shape
    y = torch.zeros(T, H, dtype=torch.float64)
    d_rw = torch.zeros(rw.shape, dtype=torch.float64)
    clamped = total = 0
    W = lambda t: t.to(torch.bfloat16).double()
    for t in range(T):
        for j in range(sel.shape[1]):
            e = int(sel[t, j])
            x = hidden[t].double()
            def p(v, Wb, key):
                A, B = lora[key]
                return v @ W(Wb)[e] + ((v @ A[e].double()) @ B[e].double()) * 0.5
            g, u = p(x, wg, "gate"), p(x, wu, "up")
            gc = torch.minimum(torch.maximum(g, torch.tensor(-L, dtype=torch.float64)), torch.tensor(L, dtype=torch.float64))
            clamped += int((g.abs() > L).sum()); total += g.numel()
            a = gc * torch.sigmoid(gc)
            h = a * u
            y[t] += p(h * rw[t, j].double(), wd, "down")
            # routing-weight gradient: dy . d(down(h * w))/dw, with down linear: = (down-projected h) . dy
            d_rw[t, j] = (p(h, wd, "down") * dy[t].double()).sum()
    assert 0.1 < clamped / total < 0.9
    assert torch.allclose(res["y"], y, rtol=1e-12, atol=1e-12)
    assert torch.allclose(res["d_routing"], d_rw, rtol=1e-10, atol=1e-12)
    assert not torch.allclose(res["y"], plain["y"])
    # the mask rule on its own: autograd through clamp = silu_backward at the clamped value times the inclusive mask
    g = torch.tensor([-2.0, -L, -L / 2, 0.0, L, 1.5 * L], dtype=torch.float64, requires_grad=True)
    F.silu(g.clamp(-L, L)).sum().backward()
    gd = g.detach()
    gc = gd.clamp(-L, L)
    sig = torch.sigmoid(gc)
    mask = ((gd >= -L) & (gd <= L)).double()
    assert torch.equal(mask, torch.tensor([0.0, 1.0, 1.0, 1.0, 1.0, 0.0], dtype=torch.float64))
    assert torch.allclose(g.grad, mask * sig * (1 + gc * (1 - sig)), rtol=1e-14, atol=0)


def test_grouped_zero_lora_equals_base_and_shared_factor_grads_sum():
    hidden, rw, sel, wg, wu, wd, lora, dy = _moe_case(seed=4)
    zero = {k: (A, torch.zeros_like(B)) for k, (A, B) in lora.items()}
    base = {k: (torch.zeros_like(A), torch.zeros_like(B)) for k, (A, B) in lora.items()}
    a = R.moe_fwd_bwd(hidden, rw, sel, wg, wu, wd, zero, 2.0)
    b = R.moe_fwd_bwd(hidden, rw, sel, wg, wu, wd, base, 2.0)
    assert torch.equal(a["y"], b["y"])          # tests/models/test_moe_experts_lora.py:439-486
    # hybrid-shared factors: grad of the shared factor == sum over experts of
    # the per-expert grads when every expert holds the same values (lora.py:976-989)
    hs, rws, sels, wg, wu, wd, lsh, dy = _moe_case(seed=5, shared=True)
    E = wg.shape[0]
    lex = {k: (A.expand(E, -1, -1).clone() if A.shape[0] == 1 else A,
               B.expand(E, -1, -1).clone() if B.shape[0] == 1 else B) for k, (A, B) in lsh.items()}
    r1 = R.moe_fwd_bwd(hs, rws, sels, wg, wu, wd, lsh, 0.5, dy)
    r2 = R.moe_fwd_bwd(hs, rws, sels, wg, wu, wd, lex, 0.5, dy)
    assert torch.allclose(r1["y"], r2["y"], rtol=1e-12, atol=1e-12)
    assert torch.allclose(r1["dA_gate"], r2["dA_gate"].sum(0, keepdim=True), rtol=1e-4, atol=1e-5)  # fp32 factor grads
    assert torch.allclose(r1["dB_down"], r2["dB_down"].sum(0, keepdim=True), rtol=1e-4, atol=1e-5)


def test_grouped_bf16_recipe_close_to_exact():
    hidden, rw, sel, wg, wu, wd, lora, dy = _moe_case(seed=6)
    ex = R.moe_fwd_bwd(hidden, rw, sel, wg, wu, wd, lora, 0.5, dy)
    lo = R.moe_fwd_bwd(hidden, rw, sel, wg, wu, wd, lora, 0.5, dy, dtype=torch.bfloat16)
    assert R.max_rel_err(lo["y"], ex["y"]) < 3e-2
    assert R.max_rel_err(lo["dx"], ex["dx"]) < 3e-2


def test_merge_recipes():
    """merge_delta_exact against a per-element brute force; the publish recipe is a bf16 add of two bf16
    tensors; zero B leaves the decoded weight; the fp32 recipe is linear in the scaling."""
    N, K, r = 24, 40, 5
    g = torch.Generator().manual_seed(5)
    A, B = torch.randn(r, K, generator=g) * 0.1, torch.randn(N, r, generator=g) * 0.1
    w = torch.randn(N, K, generator=g) * 0.02
    d = R.merge_delta_exact(A, B, 1.7)
    brute = torch.tensor([[1.7 * sum(float(B[n, j]) * float(A[j, k]) for j in range(r)) for k in range(K)] for n in range(N)])
    assert torch.allclose(d.double(), brute.double(), rtol=1e-6, atol=1e-12)
    pub = R.merge_publish_recipe(w, A, B, 1.7)
    assert pub.dtype == torch.bfloat16
    assert torch.equal(pub, (w.to(torch.bfloat16).float() + d.to(torch.bfloat16).float()).to(torch.bfloat16))
    assert torch.equal(R.merge_publish_recipe(w, A, torch.zeros_like(B), 1.7), w.to(torch.bfloat16))
    m1, m2 = R.merge_fp32_recipe(w, A, B, 1.0), R.merge_fp32_recipe(w, A, B, 2.0)
    assert torch.allclose((m2 - w).double(), 2 * (m1 - w).double(), rtol=1e-5, atol=1e-7)
