"""GPU parity: the routed expert MLP for a handful of tokens with nothing to differentiate (xq_grouped_fwd_infer: the
touched experts' block-fp8, nvfp4 or NF4 matrices streamed once, four or five launches) against the float64 per-expert oracle program and
against the training forward (xq_grouped_fwd) on the same inputs."""

import ctypes

import pytest
import torch

from oracle import recipe as R
from tests.test_gpu_moe import _make_experts, _zipf_routing
from tests.util_cases import close, gen

pytestmark = pytest.mark.gpu
TOL = 1e-2
SAME = 8e-3     # streaming form against training forward


def _lora_of(m):
    return {k: (getattr(m, f"{k}_proj_lora_A").detach().cpu(), getattr(m, f"{k}_proj_lora_B").detach().cpu())
            for k in ("gate", "up", "down")}


def _both_paths(m, x, rw, sel, device):
    """(decode form, training form) of the same forward under no_grad; asserts that the decode form took the call."""
    import xorl_amd.moe_functional as MF

    calls = []
    real = MF._moe_infer

    def spy(*a, **k):
        out = real(*a, **k)
        calls.append(out is not None)
        return out

    MF._moe_infer = spy
    try:
        with torch.no_grad():
            y = m(x.to(device), rw.to(device), sel.to(device))
    finally:
        MF._moe_infer = real
    assert calls == [True]
    MF.DECODE_PATH = False
    try:
        with torch.no_grad():
            y_train = m(x.to(device), rw.to(device), sel.to(device))
    finally:
        MF.DECODE_PATH = True
    torch.cuda.synchronize()
    return y.cpu(), y_train.cpu()


@pytest.mark.parametrize("fmt", ["block_fp8", "nvfp4", "nf4"])
@pytest.mark.parametrize("E,T,H,I,r,topk,hybrid,rw_dtype", [
    (8, 1, 256, 512, 16, 2, False, torch.bfloat16),        # one token: one row per expert, the one-row form
    (16, 1, 1024, 768, 16, 8, False, torch.float32),       # 8 experts of 16, K slices of one chunk
    (16, 3, 512, 256, 8, 4, True, torch.bfloat16),         # shared A / B factors where the module shares them
    (16, 5, 512, 256, 8, 4, True, torch.float32),          # the fewest tokens that are grouped four rows to a unit
    (16, 16, 1024, 768, 16, 8, False, torch.bfloat16),     # four-row form, experts of several units, K slices of two chunks
    (6, 64, 256, 256, 24, 2, True, torch.float32),         # r not a multiple of 16; up to dozens of rows per expert
    (40, 64, 512, 512, 64, 8, False, torch.bfloat16),      # 512 routed copies (the most), r = 64
    (8, 1, 4096, 256, 16, 2, False, torch.float32),        # one-row form, K slices of two chunks
    (40, 64, 2048, 256, 16, 8, False, torch.float32),      # four-row form, K slices of four chunks (the streaming loop proper)
    (12, 4, 2048, 768, 16, 8, False, torch.bfloat16),      # one-row form on four tokens (the most it takes), K slices of three chunks and a last one of one
])
def test_decode_forward_vs_oracle(hip_device, fmt, E, T, H, I, r, topk, hybrid, rw_dtype):
    m, banks = _make_experts(fmt, E, H, I, r, hybrid, seed=3 * E + T, device=hip_device)
    rw, sel = _zipf_routing(T, E, topk, seed=11)
    rw = rw.to(rw_dtype)
    x = gen((T, H), 1.0, 12, torch.bfloat16)
    y, y_train = _both_paths(m, x, rw, sel, hip_device)
    ex = R.moe_fwd_bwd(x, rw, sel, banks["gate"], banks["up"], banks["down"], _lora_of(m), m.scaling)
    close(y, ex["y"], TOL)
    # same rounding points as the training forward: the two differ by summation order inside the dot products only, which
    # can move a bf16 intermediate or output by an ulp (up to 2^-7 of the value)
    assert R.max_rel_err(y.float(), y_train.float()) <= SAME
    # and the call is deterministic
    y2, _ = _both_paths(m, x, rw, sel, hip_device)
    assert torch.equal(y, y2)


@pytest.mark.parametrize("fmt", ["block_fp8", "nvfp4", "nf4"])
def test_decode_forward_bf16_factors_and_swiglu_limit(hip_device, fmt):
    E, T, H, I, r, topk = 8, 4, 512, 256, 16, 2
    m, banks = _make_experts(fmt, E, H, I, r, False, seed=91, device=hip_device)
    with torch.no_grad():
        for name in ("gate_proj", "up_proj", "down_proj"):
            for f in ("A", "B"):
                p = getattr(m, f"{name}_lora_{f}")
                p.data = p.data.to(torch.bfloat16)
    rw, sel = _zipf_routing(T, E, topk, seed=92)
    x = gen((T, H), 2.0, 93, torch.bfloat16)
    lora = {k: (a.float(), b.float()) for k, (a, b) in _lora_of(m).items()}
    outs = {}
    for lim in (0.0, 0.75):
        m.swiglu_limit = lim
        y, y_train = _both_paths(m, x, rw, sel, hip_device)
        ex = R.moe_fwd_bwd(x, rw, sel, banks["gate"], banks["up"], banks["down"], lora, m.scaling, swiglu_limit=lim)
        close(y, ex["y"], TOL)
        assert R.max_rel_err(y.float(), y_train.float()) <= SAME
        outs[lim] = y
    assert not torch.equal(outs[0.0], outs[0.75])          # the clamp took part


def test_decode_forward_drops_bad_ids_and_takes_repeated_experts(hip_device):
    """Expert ids outside [0, E) drop their copy (as in the training forward); a token that names one expert twice gets
    that expert's output twice (two rows of the expert)."""
    E, T, H, I, r, topk = 8, 6, 256, 256, 8, 4
    m, banks = _make_experts("block_fp8", E, H, I, r, True, seed=55, device=hip_device)
    rw, sel = _zipf_routing(T, E, topk, seed=56)
    rw = rw.float()
    sel = sel.clone()
    sel[0, 1] = E + 5
    sel[2, 0] = -1
    sel[3, 3] = sel[3, 0]                                   # one expert twice for token 3
    x = gen((T, H), 1.0, 57, torch.bfloat16)
    y, y_train = _both_paths(m, x, rw, sel, hip_device)
    rw0 = rw.clone()
    ok = (sel >= 0) & (sel < E)
    rw0[~ok] = 0
    ex = R.moe_fwd_bwd(x, rw0, sel.clamp(0, E - 1), banks["gate"], banks["up"], banks["down"], _lora_of(m), m.scaling)
    close(y, ex["y"], TOL)
    assert R.max_rel_err(y.float(), y_train.float()) <= SAME
    # a token whose copies are all dropped gets zeros
    sel2 = sel.clone()
    sel2[5] = -3
    y3, _ = _both_paths(m, x, rw, sel2, hip_device)
    assert torch.count_nonzero(y3[5]) == 0


def test_decode_form_declines_what_it_does_not_take(hip_device):
    """Shapes outside the streaming form's limits go to the training forward from the host mirror, and the C entry
    point says so instead of running."""
    import xorl_amd.moe_functional as MF
    from xorl_amd import _C

    # hidden size not a multiple of 256; a scale group size outside the forms built; more than 512 routed copies; a forward
    # that is differentiated
    m, _ = _make_experts("block_fp8", 4, 128, 256, 8, False, seed=60, device=hip_device)
    rw, sel = _zipf_routing(2, 4, 2, seed=61)
    x = gen((2, 128), 1.0, 62, torch.bfloat16).to(hip_device)
    args = lambda mod, xx, rr, ss: (xx, rr.to(hip_device), ss.to(hip_device),
                                    tuple(getattr(mod, f"{k}_proj_lora_{f}") for k in ("gate", "up", "down") for f in ("A", "B")),
                                    (mod._bank("gate"), mod._bank("up"), mod._bank("down")), 4, mod.scaling, 0.0)
    assert MF._moe_infer(*args(m, x, rw, sel)) is None
    wg, wu, wd = (m._bank(p).c() for p in ("gate", "up", "down"))
    assert _C.lib().xq_grouped_infer_supported(ctypes.byref(wg), ctypes.byref(wu), ctypes.byref(wd), 2, 2, 8) == 0
    m4, _ = _make_experts("nf4", 4, 256, 256, 8, False, seed=63, device=hip_device)
    x4 = gen((2, 256), 1.0, 64, torch.bfloat16).to(hip_device)
    assert MF._moe_infer(*args(m4, x4, rw, sel)) is not None          # NF4 banks with fp32 scales per 64 rows are taken ...
    w4 = [m4._bank(p).c() for p in ("gate", "up", "down")]
    w4[1].group = 32                                                  # ... other group sizes are not
    assert _C.lib().xq_grouped_infer_supported(ctypes.byref(w4[0]), ctypes.byref(w4[1]), ctypes.byref(w4[2]), 2, 2, 8) == 0
    m8, _ = _make_experts("block_fp8", 4, 256, 256, 8, False, seed=65, device=hip_device)
    rw_big, sel_big = _zipf_routing(300, 4, 2, seed=66)
    x_big = gen((300, 256), 1.0, 67, torch.bfloat16).to(hip_device)
    assert MF._moe_infer(*args(m8, x_big, rw_big, sel_big)) is None
    wg, wu, wd = (m8._bank(p).c() for p in ("gate", "up", "down"))
    assert _C.lib().xq_grouped_infer_supported(ctypes.byref(wg), ctypes.byref(wu), ctypes.byref(wd), 300, 2, 8) == 0
    assert _C.lib().xq_grouped_infer_supported(ctypes.byref(wg), ctypes.byref(wu), ctypes.byref(wd), 256, 2, 8) == 1
    # with gradients wanted the module call goes through the autograd function and gives them
    xg = x4.clone().requires_grad_(True)
    y = m4(xg, rw.to(hip_device), sel.to(hip_device))
    y.sum().backward()
    assert xg.grad is not None and m4.gate_proj_lora_B.grad is not None


def test_decode_forward_in_a_hip_graph(hip_device):
    """The five launches replay from a captured graph (no memsets, no allocation inside the call beyond torch's pool)."""
    E, T, H, I, r, topk = 16, 2, 512, 256, 16, 4
    m, banks = _make_experts("block_fp8", E, H, I, r, False, seed=80, device=hip_device)
    rw, sel = _zipf_routing(T, E, topk, seed=81)
    x = gen((T, H), 1.0, 82, torch.bfloat16)
    xd, rwd, seld = x.to(hip_device), rw.to(hip_device), sel.to(hip_device)
    with torch.no_grad():
        eager = m(xd, rwd, seld).clone()
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            m(xd, rwd, seld)
        torch.cuda.current_stream().wait_stream(s)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = m(xd, rwd, seld)
        for i in range(3):
            out.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), i
        # new routing and inputs in the same buffers
        rw2, sel2 = _zipf_routing(T, E, topk, seed=83)
        x2 = gen((T, H), 1.0, 84, torch.bfloat16)
        xd.copy_(x2.to(hip_device)); rwd.copy_(rw2.to(hip_device)); seld.copy_(sel2.to(hip_device))
        graph.replay()
        torch.cuda.synchronize()
        ex = R.moe_fwd_bwd(x2, rw2, sel2, banks["gate"], banks["up"], banks["down"], _lora_of(m), m.scaling)
        close(out.cpu(), ex["y"], TOL)


def test_dispatched_rows_take_the_streaming_form(hip_device):
    """compute_dispatched (rows already grouped by expert, no routing scores) under no_grad with a handful of rows: the same
    streaming forward as a top-1 problem with unit weights; equal to the training form's result to rounding and to the
    oracle program."""
    import xorl_amd.moe_functional as MF

    E, H, I, r = 8, 512, 256, 16
    m, banks = _make_experts("block_fp8", E, H, I, r, False, seed=33, device=hip_device)
    counts = torch.tensor([3, 0, 1, 6, 0, 2, 0, 5])
    R_ = int(counts.sum())
    x = gen((R_, H), 1.0, 34, torch.bfloat16)
    cumsum = counts.cumsum(0).to(hip_device)
    calls = []
    real = MF._moe_infer

    def spy(*a, **k):
        out = real(*a, **k)
        calls.append(out is not None)
        return out

    MF._moe_infer = spy
    try:
        with torch.no_grad():
            y = m.compute_dispatched(x.to(hip_device), cumsum).cpu()
    finally:
        MF._moe_infer = real
    assert calls == [True]
    MF.DECODE_PATH = False
    try:
        with torch.no_grad():
            y_train = m.compute_dispatched(x.to(hip_device), cumsum).cpu()
    finally:
        MF.DECODE_PATH = True
    sel = torch.repeat_interleave(torch.arange(E), counts).int().unsqueeze(1)
    ex = R.moe_fwd_bwd(x, torch.ones(R_, 1), sel, banks["gate"], banks["up"], banks["down"], _lora_of(m), m.scaling)
    close(y, ex["y"], TOL)
    assert R.max_rel_err(y.float(), y_train.float()) <= SAME


def test_decode_forward_many_experts_and_widest_topk(hip_device):
    """More experts than the routing block has threads (its loops over experts take several rounds), the widest top-k the
    form takes, a rank below 16, one expert alone, and two tokens."""
    for E, T, H, I, r, topk in [(520, 5, 256, 256, 4, 16), (1, 3, 256, 256, 8, 1), (9, 2, 256, 512, 16, 8)]:
        m, banks = _make_experts("block_fp8", E, H, I, r, False, seed=E + 7, device=hip_device)
        rw, sel = _zipf_routing(T, E, topk, seed=E + 8, empty=0 if E == 1 else 1)
        x = gen((T, H), 1.0, E + 9, torch.bfloat16)
        y, y_train = _both_paths(m, x, rw, sel, hip_device)
        ex = R.moe_fwd_bwd(x, rw, sel, banks["gate"], banks["up"], banks["down"], _lora_of(m), m.scaling)
        close(y, ex["y"], TOL)
        assert R.max_rel_err(y.float(), y_train.float()) <= SAME
