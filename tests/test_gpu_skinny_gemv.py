"""GPU: one activation row (M = 1; block fp8, int4, nvfp4, nf4) through the dot-product kernel -- whole weight rows streamed by waves, decoded to the
reference decoder's bf16 values and multiplied without matrix cores -- against the oracle and against the MFMA kernel on
the same inputs (xq_set_skinny_gemv(0)).  Beyond arithmetic the cases aim at: blocks of one wave (rows of 1 KB), ragged
last blocks, a weight with fewer blocks than parts of the low-rank intermediate (falls back), the slot shared with the
other kernel when M alternates on one workspace, waits that give up."""

import ctypes

import pytest
import torch

from oracle import recipe as R
from tests.util_cases import close, gen, make_dense_module

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture
def kernels():
    """run(fn) -> (dot-product kernel's result, MFMA kernel's result); the switch is restored afterwards."""
    from xorl_amd import _C

    def run(fn):
        out = []
        for on in (1, 0):
            _C.check(_C.lib().xq_set_skinny_gemv(on))
            out.append(fn())
        _C.check(_C.lib().xq_set_skinny_gemv(1))
        return out

    yield run
    _C.check(_C.lib().xq_set_skinny_gemv(1))


def _forward(m, x, r):
    from xorl_amd.functional import qlora_linear

    with torch.no_grad():
        if r == 0:
            return qlora_linear(x, m._quant_weight(), None, None, 0, 0.0, m.bias)
        return qlora_linear(x, m._quant_weight(), m.lora_A.detach(), m.lora_B.detach(), r, m.scaling, m.bias)


@pytest.mark.parametrize("fmt,N,K,r,has_bias", [
    ("block_fp8", 4096, 4096, 16, False),     # q/o: 4 waves per block, one group of 4 rows per block
    ("block_fp8", 12288, 4096, 16, True),     # gate/up: two groups per block
    ("block_fp8", 24576, 4096, 16, False),    # fused gate|up: four groups per block
    ("block_fp8", 4096, 12288, 16, False),    # down: 12 waves per block, 24 parts of the intermediate
    ("block_fp8", 8208, 16384, 8, False),     # the longest row (16 waves), 32 parts, 8 and 7 groups per block
    ("block_fp8", 1040, 1024, 4, True),       # one wave per block
    ("block_fp8", 50016, 1024, 16, False),    # one wave per block, 3 and 2 groups per block
    ("block_fp8", 25008, 2048, 12, True),     # two waves per block, 3 and 2 groups per block
    ("block_fp8", 16, 1024, 16, False),       # one block, sets of one group, two parts
    ("block_fp8", 11024, 4096, 16, True),     # 11 rows per set (groups of 4, 4, 3), the last sets shorter or empty
    ("int4", 12304, 2048, 16, False),         # one wave per set, 4 rows per set and sets left without rows
    ("block_fp8", 4096, 5120, 0, True),       # no low-rank term
    ("int4", 4096, 4096, 16, False),          # 2 KB rows: two waves per set, four sets
    ("int4", 12288, 4096, 16, True),          # many short rows: stays on the MFMA kernel
    ("int4", 4096, 12288, 16, False),         # 6 waves per set, one set
    ("int4", 1024, 2048, 8, True),            # one wave per set
    ("int4", 2048, 8192, 0, False),
    ("nvfp4", 4096, 4096, 16, False),         # e2m1 codes, two e4m3 block scales per lane and row, the tensor's global scale
    ("nvfp4", 12288, 4096, 16, True),
    ("nvfp4", 4096, 12288, 8, False),
    ("nvfp4", 1040, 2048, 16, True),          # one wave per set
    ("nvfp4", 2048, 6144, 0, True),           # three waves per set, two sets
    ("nf4", 4096, 4096, 16, False),           # levels looked up in a per-wave table in LDS, fp32 scales per 64
    ("nf4", 12288, 4096, 16, True),
    ("nf4", 4096, 12288, 8, False),
    ("nf4", 1040, 2048, 0, True),             # one wave per set
])
def test_dot_product_kernel_vs_oracle_and_mfma_kernel(hip_device, kernels, fmt, N, K, r, has_bias):
    m, w_ref = make_dense_module(fmt, N, K, max(r, 1), 2 * max(r, 1), seed=N + K + r, device=hip_device, bias=has_bias)
    A = m.lora_A.detach().cpu() if r else torch.zeros(1, K)
    B = m.lora_B.detach().cpu() if r else torch.zeros(N, 1)
    bias = None if m.bias is None else m.bias.detach().cpu()
    for call in range(3):                                   # x changes between calls that share a workspace
        x = gen((1, K), 1.0, 70 + call, torch.bfloat16)
        xd = x.to(hip_device)
        dot, mfma = kernels(lambda: _forward(m, xd, r))
        ex = R.linear_fwd_bwd_exact(x, w_ref, A, B, m.scaling if r else 0.0, bias=bias)
        assert torch.isfinite(dot.float()).all()
        close(dot.cpu(), ex["y"], TOL)
        close(mfma.cpu(), ex["y"], TOL)
        # the two kernels round the same decoded weights and differ in the order of fp32 sums only
        close(dot.cpu(), mfma.float().cpu(), 4e-3)


@pytest.mark.parametrize("fmt", ["block_fp8", "int4", "nvfp4", "nf4"])
def test_one_workspace_alternating_between_the_kernels(hip_device, fmt):
    """M = 1 (dot-product kernel) and M = 8 (MFMA kernel) take turns on one workspace, hence one slot: each launch must
    see its own parts of the low-rank intermediate only.  The low-rank term dominates the output here, so that a stale or
    foreign part would show."""
    from xorl_amd import _C
    from xorl_amd.functional import _workspace_bytes

    N, K, r = 4096, 4096, 16
    m, w_ref = make_dense_module(fmt, N, K, r, 32, seed=11, device=hip_device)
    with torch.no_grad():
        m.lora_A.mul_(20.0)
        m.lora_B.mul_(20.0)
    A, B = m.lora_A.detach().contiguous(), m.lora_B.detach().contiguous()
    w = m._quant_weight().c()
    L = _C.lib()
    wsb = _workspace_bytes(8, N, K, r)
    ws = torch.empty(wsb, dtype=torch.uint8, device=hip_device)
    for i in range(24):
        M = 1 if i % 3 != 2 else 8
        x = gen((M, K), 1.0, 500 + i, torch.bfloat16)
        xd = x.to(hip_device)
        y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=hip_device)
        _C.check(L.xq_linear_fwd(ctypes.byref(w), xd.data_ptr(), K, M, A.data_ptr(), B.data_ptr(), _C.XQ_DT_F32, r,
                                 ctypes.c_float(m.scaling), None, y.data_ptr(), N, None, ws.data_ptr(), wsb, _C.stream_ptr(hip_device)))
        ex = R.linear_fwd_bwd_exact(x, w_ref, A.cpu(), B.cpu(), m.scaling)
        close(y.cpu(), ex["y"], TOL)


@pytest.mark.parametrize("N,K,group,symmetric", [(4096, 4096, 128, True), (1024, 8192, 32, True), (2048, 2048, 64, True),
                                                     (4096, 4096, 128, False), (1024, 4096, 32, False)])
def test_int4_scale_types_and_groups(hip_device, kernels, N, K, group, symmetric):
    """int4 with bf16 scales (the symmetric rule's storage) and fp32 scales (the reference codec's rule), groups of 32 to
    128: the dot-product kernel against the oracle's decode and, to rounding, against the MFMA kernel."""
    from tests.util_cases import oracle_decode_dense
    from xorl_amd.functional import qlora_linear
    from xorl_amd.qlora.linear import Int4QLoRALinear

    m = Int4QLoRALinear(K, N, r=16, lora_alpha=32, quant_group_size=group, symmetric=symmetric)
    with torch.no_grad():
        m._init_from_weight(gen((N, K), 0.02, N + K + group))
        m.lora_A.copy_(gen((16, K), 0.02, 1))
        m.lora_B.copy_(gen((N, 16), 0.02, 2))
    w_ref = oracle_decode_dense(m)
    m = m.to(hip_device)
    qw = m._quant_weight()
    assert qw.scale_dtype == (torch.bfloat16 if symmetric else torch.float32) and qw.group == group
    A, B = m.lora_A.detach(), m.lora_B.detach()
    x = gen((1, K), 1.0, 9, torch.bfloat16)
    xd = x.to(hip_device)

    def forward():
        with torch.no_grad():
            return qlora_linear(xd, qw, A, B, 16, m.scaling)

    dot, mfma = kernels(forward)
    close(dot.cpu(), mfma.float().cpu(), 4e-3)
    ex = R.linear_fwd_bwd_exact(x, w_ref, A.cpu(), B.cpu(), m.scaling)
    close(dot.cpu(), ex["y"], TOL)
    close(mfma.cpu(), ex["y"], TOL)


def test_joint_launches_on_either_kernel(hip_device, kernels):
    """q + k + v in one launch and gate | up with the SwiGLU finish, one row: the dot-product kernel's results against the
    MFMA kernel's (same decoded weights, other summation order) and against the separate calls (same bits on either)."""
    from xorl_amd.functional import qlora_linear, qlora_linear_multi, silu_and_mul
    from xorl_amd.qlora import qlora_gate_up_silu

    K = 4096
    mods = [make_dense_module("block_fp8", N, K, 16, 32, seed=N + i, device=hip_device, bias=(i == 1))[0] for i, N in enumerate((4096, 1024, 1024))]
    jobs = [(m._quant_weight(), m.lora_A.detach(), m.lora_B.detach(), 16, m.scaling, m.bias) for m in mods]
    gu, _ = make_dense_module("block_fp8", 2 * 3072, K, 16, 32, seed=77, device=hip_device)
    for call in range(2):
        x = gen((1, K), 1.0, 40 + call, torch.bfloat16).to(hip_device)

        def joint():
            with torch.no_grad():
                ys = qlora_linear_multi(x, jobs)
                sep = [qlora_linear(x, *j) for j in jobs]
                h = qlora_gate_up_silu(gu, x)
                gate, up = gu(x).chunk(2, dim=-1)
                return ys, sep, h, silu_and_mul(gate, up)

        (ys1, sep1, h1, hs1), (ys0, sep0, h0, hs0) = kernels(joint)
        for a, b, c, d in zip(ys1, sep1, ys0, sep0):
            assert torch.equal(a, b) and torch.equal(c, d)
            close(a.cpu(), c.float().cpu(), 4e-3)
        assert torch.equal(h1, hs1) and torch.equal(h0, hs0)
        close(h1.cpu(), h0.float().cpu(), 8e-3)


def test_overlapping_dot_product_forwards_on_two_streams(hip_device):
    """One-row forwards on two streams, each with its own workspace (hence its own slot), small enough to run side by side
    on the device: every result equals the one the same call gives alone."""
    from xorl_amd import _C
    from xorl_amd.functional import _workspace_bytes

    r = 16
    shapes = [("block_fp8", 1024, 4096), ("block_fp8", 2048, 2048), ("int4", 1024, 4096), ("nvfp4", 1024, 4096)]
    L = _C.lib()
    streams = [torch.cuda.Stream() for _ in shapes]
    work = []
    for i, (fmt, N, K) in enumerate(shapes):
        m, _ = make_dense_module(fmt, N, K, r, 32, seed=80 + i, device=hip_device)
        w = m._quant_weight().c()
        A, B = m.lora_A.detach().contiguous(), m.lora_B.detach().contiguous()
        wsb = _workspace_bytes(1, N, K, r)
        ws = torch.empty(wsb, dtype=torch.uint8, device=hip_device)
        xs = [gen((1, K), 1.0, 700 + 10 * i + j, torch.bfloat16).to(hip_device) for j in range(6)]
        ys = [torch.empty(1, N, dtype=torch.bfloat16, device=hip_device) for _ in xs]
        work.append((m, w, A, B, ws, wsb, xs, ys, N, K))

    def call(i, j, y, stream):
        m, w, A, B, ws, wsb, xs, _, N, K = work[i]
        _C.check(L.xq_linear_fwd(ctypes.byref(w), xs[j].data_ptr(), K, 1, A.data_ptr(), B.data_ptr(), _C.XQ_DT_F32, r,
                                 ctypes.c_float(m.scaling), None, y.data_ptr(), N, None, ws.data_ptr(), wsb, stream))

    alone = []
    for i in range(len(shapes)):
        outs = []
        for j in range(6):
            y = torch.empty_like(work[i][7][j])
            call(i, j, y, _C.stream_ptr(hip_device))
            outs.append(y)
        alone.append(outs)
    torch.cuda.synchronize()
    assert all(torch.isfinite(y.float()).all() for outs in alone for y in outs)
    for st in streams:
        st.wait_stream(torch.cuda.current_stream())
    for rep in range(20):
        for j in range(6):
            for i in range(len(shapes)):
                call(i, j, work[i][7][j], ctypes.c_void_p(streams[i].cuda_stream))
    torch.cuda.synchronize()
    for i in range(len(shapes)):
        for j in range(6):
            assert torch.equal(work[i][7][j], alone[i][j]), (i, j)


def test_dot_product_kernel_under_hip_graph(hip_device):
    """Captured once, replayed with x changing and eager calls on the same workspace in between: every replay gives the
    eager call's bits."""
    from xorl_amd import _C
    from xorl_amd.functional import _workspace_bytes

    N, K, r = 12288, 4096, 16
    m, _ = make_dense_module("block_fp8", N, K, r, 32, seed=13, device=hip_device)
    A, B = m.lora_A.detach().contiguous(), m.lora_B.detach().contiguous()
    w = m._quant_weight().c()
    L = _C.lib()
    wsb = _workspace_bytes(1, N, K, r)
    ws = torch.empty(wsb, dtype=torch.uint8, device=hip_device)
    x = torch.zeros(1, K, dtype=torch.bfloat16, device=hip_device)
    y = torch.zeros(1, N, dtype=torch.bfloat16, device=hip_device)

    def call():
        _C.check(L.xq_linear_fwd(ctypes.byref(w), x.data_ptr(), K, 1, A.data_ptr(), B.data_ptr(), _C.XQ_DT_F32, r, ctypes.c_float(m.scaling),
                                 None, y.data_ptr(), N, None, ws.data_ptr(), wsb, _C.stream_ptr(hip_device)))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for i in range(5):
        x.copy_(gen((1, K), 1.0, 800 + i, torch.bfloat16).to(hip_device))
        y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = y.clone()
        y.fill_(float("nan"))
        call()
        torch.cuda.synchronize()
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, y), i


def test_bounded_waits_in_the_dot_product_kernel(hip_device):
    """The waits cut to a single look from the host: every kernel ends; an output is right or NaN, never made from stale
    sums; a slot that was marked failed recovers through the status call."""
    from xorl_amd import _C
    from xorl_amd.functional import _workspace_bytes, skinny_status

    N, K, r = 12288, 4096, 16
    m, _ = make_dense_module("block_fp8", N, K, r, 32, seed=17, device=hip_device)
    with torch.no_grad():
        m.lora_A.mul_(20.0)
        m.lora_B.mul_(20.0)
    w = m._quant_weight().c()
    A, B = m.lora_A.detach().contiguous(), m.lora_B.detach().contiguous()
    L = _C.lib()
    wsb = _workspace_bytes(1, N, K, r)
    ws = torch.empty(wsb, dtype=torch.uint8, device=hip_device)
    y = torch.empty(1, N, dtype=torch.bfloat16, device=hip_device)

    def call(x):
        _C.check(L.xq_linear_fwd(ctypes.byref(w), x.data_ptr(), K, 1, A.data_ptr(), B.data_ptr(), _C.XQ_DT_F32, r, ctypes.c_float(m.scaling),
                                 None, y.data_ptr(), N, None, ws.data_ptr(), wsb, _C.stream_ptr(hip_device)))
        torch.cuda.synchronize()
        return y.clone()

    xs = [gen((1, K), 1.0, 600 + i, torch.bfloat16).to(hip_device) for i in range(6)]
    try:
        want = [call(x) for x in xs]
        assert all(torch.isfinite(t.float()).all() for t in want)
        assert skinny_status(hip_device) == (0, 0)
        try:
            _C.check(L.xq_set_skinny_spin_limit(1))
            for x, ref in zip(xs, want):
                got = call(x)
                bad = torch.isnan(got.float())
                assert torch.equal(got[~bad], ref[~bad])
        finally:
            _C.check(L.xq_set_skinny_spin_limit(0))
        skinny_status(hip_device, raise_on_failure=False)       # clears a failed mark, if the closing block gave up
        assert skinny_status(hip_device) == (0, 0)
        for x, ref in zip(xs, want):
            assert torch.equal(call(x), ref)
    finally:
        _C.check(L.xq_set_skinny_spin_limit(0))
        skinny_status(hip_device, raise_on_failure=False)
