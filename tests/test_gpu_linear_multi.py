"""GPU: several QLoRA linears on one input as one library call (xq_linear_fwd_multi): the separate q_proj / k_proj / v_proj
and gate_proj / up_proj calls of a model that keeps them unfused (reference: models/layers/attention/multi_head_attention.py:93-95,
models/transformers/qwen3/modeling_qwen3.py:75-76).  At decode sizes the forwards share one launch of the whole-row skinny
kernel, each with its own weight, factors, outputs and slot of library memory; the results must be the bits of the
separate calls (the arithmetic per output row does not depend on how rows are dealt to blocks), and both must match the
oracle.  Beyond arithmetic: a forward reading another forward's low-rank intermediate (distinct factors per forward, one
forward without a low-rank term), blocks finding the wrong forward at the boundaries, stale state over many calls."""

import ctypes

import pytest
import torch

from oracle import recipe as R
from tests.util_cases import close, gen, make_dense_module

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _job(m, r=None, bias=True):
    r = m.r if r is None else r
    if r == 0:
        return (m._quant_weight(), None, None, 0, 0.0, m.bias if bias else None)
    return (m._quant_weight(), m.lora_A.detach(), m.lora_B.detach(), r, m.scaling, m.bias if bias else None)


def _separate(x, jobs):
    from xorl_amd.functional import qlora_linear

    with torch.no_grad():
        return [qlora_linear(x, qw, A, B, r, s, b) for qw, A, B, r, s, b in jobs]


def _multi(x, jobs):
    from xorl_amd.functional import qlora_linear_multi

    with torch.no_grad():
        return qlora_linear_multi(x, jobs)


def _launches(fn):
    """timed regions of this library inside fn(): a skinny forward, whatever it launches, is one region"""
    from xorl_amd import _C

    L = _C.lib()
    _C.check(L.xq_profile_enable(1))
    try:
        fn()
        torch.cuda.synchronize()
        n, ms, fl = ctypes.c_int(0), ctypes.c_double(0), ctypes.c_double(0)
        _C.check(L.xq_profile_collect(ctypes.byref(n), ctypes.byref(ms), ctypes.byref(fl)))
    finally:
        _C.check(L.xq_profile_enable(0))
    return n.value


@pytest.mark.parametrize("fmt,K,Ns,rs,has_bias", [
    ("block_fp8", 4096, (4096, 1024, 1024), (16, 16, 16), False),     # q / k / v of Qwen3-8B: two row groups per block
    ("block_fp8", 4096, (12288, 12288), (16, 16), True),               # gate / up: two rounds of three row groups
    ("int4", 4096, (4096, 1024, 1024), (16, 8, 0), True),              # one forward without a low-rank term
    ("nf4", 2048, (2048, 512, 512, 2048), (8, 8, 8, 8), False),        # four forwards
    ("nvfp4", 5120, (8192, 1024, 1024), (16, 16, 16), False),          # q / k / v of Qwen3-32B: 5 steps of an 8-step kernel
    ("block_fp8", 1024, (208, 96), (4, 12), True),                     # small, ragged last blocks
])
def test_multi_vs_separate_and_oracle(hip_device, fmt, K, Ns, rs, has_bias):
    mods = [make_dense_module(fmt, N, K, max(r, 4), 2 * max(r, 4), seed=7 * i + N + K, device=hip_device, bias=has_bias)
            for i, (N, r) in enumerate(zip(Ns, rs))]
    jobs = [_job(m, r) for (m, _), r in zip(mods, rs)]
    for M in (1, 5, 8, 16, 24):
        x = gen((M, K), 1.0, 90 + M, torch.bfloat16)
        xd = x.to(hip_device)
        got = _multi(xd, jobs)
        sep = _separate(xd, jobs)
        for (m, w_ref), r, y, ys in zip(mods, rs, got, sep):
            assert y.shape == (M, m.out_features) and y.dtype == torch.bfloat16
            assert torch.equal(y, ys)
            A = m.lora_A.detach().cpu()[:r] if r else torch.zeros(1, K)
            B = m.lora_B.detach().cpu()[:, :r] if r else torch.zeros(m.out_features, 1)
            bias = None if m.bias is None else m.bias.detach().cpu()
            ex = R.linear_fwd_bwd_exact(x, w_ref, A, B, m.scaling if r else 0.0, bias=bias)
            close(y.cpu(), ex["y"], TOL)
        # a second call on new input, then the first input again: nothing of the previous call survives
        x2 = gen((M, K), 1.0, 190 + M, torch.bfloat16).to(hip_device)
        for y, ys in zip(_multi(x2, jobs), _separate(x2, jobs)):
            assert torch.equal(y, ys)
        for y, y0 in zip(_multi(xd, jobs), got):
            assert torch.equal(y, y0)


def test_decode_sizes_take_one_region(hip_device):
    mods = [make_dense_module("block_fp8", N, 4096, 16, 32, seed=N, device=hip_device)[0] for N in (4096, 1024, 1024)]
    jobs = [_job(m) for m in mods]
    x = gen((8, 4096), 1.0, 3, torch.bfloat16).to(hip_device)
    _multi(x, jobs)
    assert _launches(lambda: _multi(x, jobs)) == 1
    assert _launches(lambda: _separate(x, jobs)) == 3
    # beyond 16 rows the forwards run one after the other
    x = gen((32, 4096), 1.0, 4, torch.bfloat16).to(hip_device)
    assert _launches(lambda: _multi(x, jobs)) == 3


def test_mixed_formats_fall_back_to_separate_forwards(hip_device):
    a, wa = make_dense_module("block_fp8", 1024, 2048, 8, 16, seed=1, device=hip_device)
    b, wb = make_dense_module("int4", 512, 2048, 8, 16, seed=2, device=hip_device)
    x = gen((4, 2048), 1.0, 5, torch.bfloat16).to(hip_device)
    jobs = [_job(a), _job(b)]
    for y, ys in zip(_multi(x, jobs), _separate(x, jobs)):
        assert torch.equal(y, ys)


def test_argument_errors(hip_device):
    from xorl_amd import _C

    a, _ = make_dense_module("block_fp8", 1024, 2048, 8, 16, seed=1, device=hip_device)
    b, _ = make_dense_module("block_fp8", 1024, 1024, 8, 16, seed=2, device=hip_device)
    x = gen((4, 2048), 1.0, 5, torch.bfloat16).to(hip_device)
    with pytest.raises(_C.XqError):
        _multi(x, [_job(a), _job(b)])            # different in_features
    with pytest.raises(_C.XqError):
        _multi(x, [_job(a)] * 5)                 # more than four forwards
    with pytest.raises(_C.XqError):
        _multi(x.float(), [_job(a)])


def test_many_calls_under_hip_graph(hip_device):
    mods = [make_dense_module("block_fp8", N, 4096, 16, 32, seed=N + 1, device=hip_device)[0] for N in (4096, 1024, 1024)]
    jobs = [_job(m) for m in mods]
    x = gen((4, 4096), 1.0, 11, torch.bfloat16).to(hip_device)
    from xorl_amd import _C

    L = _C.lib()
    arr = (_C.XqLinearJob * 3)()
    keep = []
    ys = [torch.empty(4, m.out_features, dtype=torch.bfloat16, device=hip_device) for m in mods]
    for i, (qw, A, B, r, s, _) in enumerate(jobs):
        cw = qw.c()
        A, B = A.contiguous(), B.contiguous()
        keep += [cw, A, B]
        arr[i].w = ctypes.pointer(cw)
        arr[i].lora_A, arr[i].lora_B, arr[i].r, arr[i].scaling = A.data_ptr(), B.data_ptr(), r, s
        arr[i].bias_bf16, arr[i].y, arr[i].ldy = None, ys[i].data_ptr(), mods[i].out_features
    wsb = L.xq_linear_fwd_multi_workspace_bytes(arr, 3, 4)
    ws = torch.empty(wsb, dtype=torch.uint8, device=hip_device)

    def call():
        _C.check(L.xq_linear_fwd_multi(arr, 3, x.data_ptr(), 4096, 4, _C.XQ_DT_F32, ws.data_ptr(), wsb, _C.stream_ptr(hip_device)))

    call()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for it in range(4):
        x.copy_(gen((4, 4096), 1.0, 20 + it, torch.bfloat16))
        graph.replay()
        torch.cuda.synchronize()
        for y, ysep in zip(ys, _separate(x, jobs)):
            assert torch.equal(y, ysep)


def test_module_helper(hip_device):
    """qlora_linears_forward: one library call without autograd, the modules one by one with it; the same bits."""
    from xorl_amd.qlora import qlora_linears_forward

    mods = [make_dense_module("block_fp8", N, 2048, 8, 16, seed=N + 3, device=hip_device, bias=(N == 512))[0] for N in (2048, 512, 512)]
    x = gen((3, 7, 2048), 1.0, 31, torch.bfloat16).to(hip_device)
    with torch.no_grad():
        want = [m(x) for m in mods]
        assert _launches(lambda: qlora_linears_forward(mods, x)) == 3      # 21 rows: one after the other inside the one call
        assert _launches(lambda: qlora_linears_forward(mods, x[:, :2])) == 1
        got = qlora_linears_forward(mods, x[:, :2])                         # 6 rows: one launch
        for y, m in zip(got, mods):
            assert y.shape == (3, 2, m.out_features) and torch.equal(y, m(x[:, :2]))
        for y, w in zip(qlora_linears_forward(mods, x), want):
            assert torch.equal(y, w)
    xg = x.clone().requires_grad_(True)
    ys = qlora_linears_forward(mods, xg)
    for y, m, w in zip(ys, mods, want):
        assert y.requires_grad and torch.equal(y.detach(), m(xg).detach())     # the training forward of each module
        close(y.detach().float().cpu(), w.double().cpu(), TOL)
    sum(y.float().sum() for y in ys).backward()
    assert xg.grad is not None and all(m.lora_A.grad is not None for m in mods)


@pytest.mark.parametrize("fmt", ["block_fp8", "int4"])
def test_mlp_forward_without_autograd_is_the_module_calls(hip_device, fmt):
    """qlora_mlp_forward under no_grad is one library call (xq_mlp_fwd_infer); its output is, bit for bit, the three
    module calls around the SwiGLU kernel, at decode sizes (weight-streaming kernels) and above (tile kernels), and it
    matches the fp64 program."""
    from xorl_amd.functional import silu_and_mul
    from xorl_amd.qlora import qlora_mlp_forward

    H, I, r = 1024, 3072, 8
    (g, wg), (u, wu), (d, wd) = (make_dense_module(fmt, N, K, r, 16, seed=50 + i, device=hip_device)
                                 for i, (N, K) in enumerate(((I, H), (I, H), (H, I))))
    loras = {k: (m.lora_A.detach().cpu(), m.lora_B.detach().cpu()) for k, m in (("gate", g), ("up", u), ("down", d))}
    for M in (1, 8, 16, 40, 64, 300):
        x = gen((M, H), 1.0, 60 + M, torch.bfloat16)
        xd = x.to(hip_device)
        with torch.no_grad():
            got = qlora_mlp_forward(g, u, d, xd)
            want = d(silu_and_mul(g(xd), u(xd)))
        assert got.shape == (M, H) and torch.equal(got, want)
        close(got.cpu(), R.mlp_fwd_bwd_exact(x, wg, wu, wd, loras, g.scaling)["y"], 2e-2)
    # with a bias on every projection (no oracle program for it: the module calls are the reference)
    (g, _), (u, _), (d, _) = (make_dense_module(fmt, N, K, r, 16, seed=70 + i, device=hip_device, bias=True)
                              for i, (N, K) in enumerate(((I, H), (I, H), (H, I))))
    xd = gen((5, H), 1.0, 99, torch.bfloat16).to(hip_device)
    with torch.no_grad():
        assert torch.equal(qlora_mlp_forward(g, u, d, xd), d(silu_and_mul(g(xd), u(xd))))


@pytest.mark.parametrize("fmt,I,K,r,has_bias", [
    ("block_fp8", 12288, 4096, 16, False),     # Qwen3-8B gate | up: one launch (two rounds of three row groups) up to 16 rows
    ("block_fp8", 1536, 2048, 8, True),        # 4 steps of the fp8 kernel
    ("int4", 12288, 4096, 16, True),
    ("nf4", 6144, 2048, 8, False),
    ("nvfp4", 12288, 4096, 16, False),
    ("block_fp8", 1024, 1024, 4, True),        # I not a multiple of 48: the two calls inside the one
])
def test_gate_up_with_swiglu_finish(hip_device, fmt, I, K, r, has_bias):
    """xq_linear_fwd_swiglu / qlora_gate_up_silu: h = silu(gate) * up from the stacked weight, bit for bit the module call
    followed by the SwiGLU kernel, at decode sizes (one launch) and above, and against the fp64 program."""
    from xorl_amd.functional import silu_and_mul
    from xorl_amd.qlora import qlora_gate_up_silu

    m, w_ref = make_dense_module(fmt, 2 * I, K, r, 2 * r, seed=I + K, device=hip_device, bias=has_bias)
    A, B = m.lora_A.detach().cpu(), m.lora_B.detach().cpu()
    bias = None if m.bias is None else m.bias.detach().cpu()
    for M in (1, 7, 16, 24, 64):
        x = gen((M, K), 1.0, 500 + M, torch.bfloat16)
        xd = x.to(hip_device)
        with torch.no_grad():
            got = qlora_gate_up_silu(m, xd)
            gate, up = m(xd).chunk(2, dim=-1)
            want = silu_and_mul(gate, up)
        assert got.shape == (M, I) and got.dtype == torch.bfloat16
        assert torch.equal(got, want)
        y = R.linear_fwd_bwd_exact(x, w_ref, A, B, m.scaling, bias=bias)["y"]
        g64, u64 = y[:, :I], y[:, I:]
        close(got.cpu(), g64 * torch.sigmoid(g64) * u64, 2e-2)
        with torch.no_grad():
            assert torch.equal(qlora_gate_up_silu(m, xd), got)        # the same bits from a second call
    # decode sizes take one region of the library's launch counter, the two calls two
    if I % 48 == 0:
        xd = gen((4, K), 1.0, 3, torch.bfloat16).to(hip_device)
        with torch.no_grad():
            assert _launches(lambda: qlora_gate_up_silu(m, xd)) == 1
