"""GPU: the one-launch organisation of the skinny forward (whole weight rows per block, the low-rank intermediate formed
once per launch and passed between blocks through device memory of the library; x slices through LDS for M <= 16,
streamed for M in 17 .. 64) against the oracle and against the two-launch organisation on the same inputs.  What could go wrong here beyond arithmetic: a stale intermediate from the
previous launch (the cases change x between calls that share a workspace), slots that are not restored (many calls in a
row), ragged last blocks, short K ranges per wave, every format's scale addressing."""

import ctypes

import pytest
import torch

from oracle import recipe as R
from tests.util_cases import close, gen, make_dense_module

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture
def organisations():
    """run(fn) -> (one-launch result, two-launch result); the switch is restored afterwards."""
    from xorl_amd import _C

    def run(fn):
        out = []
        for enabled in (1, 0):
            _C.check(_C.lib().xq_set_skinny_one_launch(enabled))
            out.append(fn())
        _C.check(_C.lib().xq_set_skinny_one_launch(1))
        return out

    yield run
    _C.check(_C.lib().xq_set_skinny_one_launch(1))


def _forward(m, x, r=None, bias=True):
    from xorl_amd.functional import qlora_linear

    r = m.r if r is None else r
    with torch.no_grad():
        if r == 0:
            return qlora_linear(x, m._quant_weight(), None, None, 0, 0.0, m.bias if bias else None)
        return qlora_linear(x, m._quant_weight(), m.lora_A.detach(), m.lora_B.detach(), r, m.scaling, m.bias if bias else None)


@pytest.mark.parametrize("fmt,N,K,r,has_bias", [
    ("block_fp8", 1024, 4096, 16, False),     # kv: 64 blocks of one row group, 4 su parts
    ("block_fp8", 12288, 4096, 16, True),     # gate/up: 256 blocks of three row groups
    ("block_fp8", 4096, 12288, 16, False),    # down: 24 load steps per wave, 12 su parts (M <= 1 only: x must fit LDS)
    ("block_fp8", 12304, 2048, 8, False),     # ragged last block (769 row groups), short K
    ("block_fp8", 208, 1024, 4, True),        # two load steps per wave, 13 row groups
    ("block_fp8", 6144, 5120, 12, False),     # 10 steps of a 16-step kernel, two row groups per block
    ("int4", 4096, 4096, 16, False),
    ("int4", 12288, 4096, 16, True),
    ("int4", 1024, 1024, 16, False),          # one load step per wave
    ("nf4", 12288, 4096, 16, False),
    ("nf4", 4096, 5120, 8, True),
    ("nvfp4", 12288, 4096, 16, False),
    ("nvfp4", 1040, 2048, 16, True),
    ("block_fp8", 24576, 4096, 16, True),     # fused gate|up: 256 blocks, two rounds of three row groups each
    ("int4", 24576, 4096, 16, False),
    ("nf4", 24576, 2048, 8, True),
    ("nvfp4", 24576, 1024, 16, False),
    # scale loads that cover four load steps at a time: two and three groups of four (int4), a last group of one step
    # (nvfp4, nf4: five steps per wave), three whole groups (nvfp4)
    ("int4", 2048, 8192, 16, False),
    ("int4", 1024, 12288, 8, True),
    ("nvfp4", 2048, 5120, 16, False),
    ("nvfp4", 1024, 12288, 8, False),
    ("nf4", 1024, 8192, 16, False),
])
def test_one_launch_vs_oracle_and_two_launch(hip_device, organisations, fmt, N, K, r, has_bias):
    m, w_ref = make_dense_module(fmt, N, K, r, 2 * r, seed=N + K + r, device=hip_device, bias=has_bias)
    A, B = m.lora_A.detach().cpu(), m.lora_B.detach().cpu()
    bias = None if m.bias is None else m.bias.detach().cpu()
    for M in (1, 3, 8, 16, 17, 32, 40, 64):
        x = gen((M, K), 1.0, 40 + M, torch.bfloat16)
        xd = x.to(hip_device)
        one, two = organisations(lambda: _forward(m, xd))
        ex = R.linear_fwd_bwd_exact(x, w_ref, A, B, m.scaling, bias=bias)
        assert one.shape == (M, N) and one.dtype == torch.bfloat16
        close(one.cpu(), ex["y"], TOL)
        close(two.cpu(), ex["y"], TOL)
        close(one.cpu(), two.float().cpu(), TOL)
        # the same bits from a second call
        assert torch.equal(_forward(m, xd), one)
    # no low-rank term
    x = gen((5, K), 1.0, 77, torch.bfloat16)
    y0 = _forward(m, x.to(hip_device), r=0)
    ex0 = R.linear_fwd_bwd_exact(x, w_ref, torch.zeros(1, K), torch.zeros(N, 1), 0.0, bias=bias)
    close(y0.cpu(), ex0["y"], TOL)


def test_low_rank_term_alone_follows_x(hip_device):
    """Weight codes that decode to zero leave y = s (x A^T) B^T: the term on its own scale, for a sequence of different
    x through ONE workspace (a stale intermediate of the previous launch would show) and with the low-rank term switched
    off and on again in between."""
    from xorl_amd import _C
    from xorl_amd.functional import _workspace_bytes

    N, K, r = 4096, 4096, 16
    m, _ = make_dense_module("block_fp8", N, K, r, 32, seed=5, device=hip_device)
    qw = m._quant_weight()
    qw.packed.zero_()                           # e4m3 byte 0x00 is +0
    w = qw.c()
    A, B = m.lora_A.detach().contiguous(), m.lora_B.detach().contiguous()
    L = _C.lib()
    wsb = _workspace_bytes(64, N, K, r)
    ws = torch.empty(wsb, dtype=torch.uint8, device=hip_device)
    st = _C.stream_ptr(hip_device)
    for i, M in enumerate((1, 16, 2, 9, 1, 16, 64, 5, 33, 64)):
        x = gen((M, K), 1.0, 900 + i, torch.bfloat16).to(hip_device)
        y = torch.empty(M, N, dtype=torch.bfloat16, device=hip_device)
        with_term = i != 3
        _C.check(L.xq_linear_fwd(ctypes.byref(w), x.data_ptr(), K, M, A.data_ptr() if with_term else None,
                                 B.data_ptr() if with_term else None, _C.XQ_DT_F32, r if with_term else 0, ctypes.c_float(m.scaling),
                                 None, y.data_ptr(), N, None, ws.data_ptr(), wsb, st))
        su = x.float() @ A.to(torch.bfloat16).float().t()
        ref = (m.scaling * su) @ B.float().t() if with_term else torch.zeros(M, N, device=hip_device)
        close(y.float().cpu(), ref.cpu(), TOL)


def test_many_workspaces_and_many_calls(hip_device):
    """More workspaces than the library holds slots, each used several times.  On one stream a slot can always change
    hands (the stream runs its launches in order): every call repeats the first result bit for bit.  Across streams a slot
    is taken over only once the other stream has run dry; calls that find every slot busy elsewhere run the two-launch
    organisation instead, which agrees with the oracle to tolerance."""
    from xorl_amd import _C
    from xorl_amd.functional import _workspace_bytes

    N, K, r, M = 1024, 4096, 16, 4
    m, w_ref = make_dense_module("int4", N, K, r, 32, seed=9, device=hip_device)
    w = m._quant_weight().c()
    A, B = m.lora_A.detach().contiguous(), m.lora_B.detach().contiguous()
    L = _C.lib()
    wsb = _workspace_bytes(M, N, K, r)
    x = gen((M, K), 1.0, 31, torch.bfloat16)
    xd = x.to(hip_device)
    ex = R.linear_fwd_bwd_exact(x, w_ref, A.cpu(), B.cpu(), m.scaling)
    wss = [torch.empty(wsb, dtype=torch.uint8, device=hip_device) for _ in range(300)]

    def call(ws, st):
        y = torch.empty(M, N, dtype=torch.bfloat16, device=hip_device)
        _C.check(L.xq_linear_fwd(ctypes.byref(w), xd.data_ptr(), K, M, A.data_ptr(), B.data_ptr(), _C.XQ_DT_F32, r,
                                 ctypes.c_float(m.scaling), None, y.data_ptr(), N, None, ws.data_ptr(), wsb, st))
        return y

    try:
        _C.check(L.xq_skinny_reset())           # slots left by earlier tests are handed back
        st = _C.stream_ptr(hip_device)
        first = call(wss[0], st)
        close(first.cpu(), ex["y"], TOL)
        ys = [call(ws, st) for _ in range(3) for ws in wss]       # back to back on one stream
        torch.cuda.synchronize()
        for y in ys:
            assert torch.equal(y, first)
        # two streams in turn, nothing waited for: a call may find every candidate slot busy on the other stream
        streams = [torch.cuda.Stream(), torch.cuda.Stream()]
        ys = []
        for i, ws in enumerate(wss + wss):
            with torch.cuda.stream(streams[i & 1]):
                ys.append(call(ws, ctypes.c_void_p(streams[i & 1].cuda_stream)))
        torch.cuda.synchronize()
        for y in ys:
            if not torch.equal(y, first):
                close(y.cpu(), ex["y"], TOL)
    finally:
        torch.cuda.synchronize()
        _C.check(L.xq_skinny_reset())


def test_a_captured_forward_keeps_its_slot(hip_device):
    """A forward recorded into a HIP graph has its slot's address in the recorded launch: the slot stays with that
    workspace however many other workspaces pass through the library afterwards, and replays (with the input changing,
    and with eager forwards of other workspaces in flight on another stream) equal the eager results bit for bit."""
    from xorl_amd import _C
    from xorl_amd.functional import _workspace_bytes

    N, K, r, M = 4096, 4096, 16, 8
    m, _ = make_dense_module("block_fp8", N, K, r, 32, seed=4, device=hip_device)
    w = m._quant_weight().c()
    A, B = m.lora_A.detach().contiguous(), m.lora_B.detach().contiguous()
    L = _C.lib()
    wsb = _workspace_bytes(M, N, K, r)
    xbuf = gen((M, K), 1.0, 1, torch.bfloat16).to(hip_device)
    ws0 = torch.empty(wsb, dtype=torch.uint8, device=hip_device)
    y0 = torch.empty(M, N, dtype=torch.bfloat16, device=hip_device)

    def call(ws, y, x):
        _C.check(L.xq_linear_fwd(ctypes.byref(w), x.data_ptr(), K, M, A.data_ptr(), B.data_ptr(), _C.XQ_DT_F32, r,
                                 ctypes.c_float(m.scaling), None, y.data_ptr(), N, None, ws.data_ptr(), wsb, _C.stream_ptr(hip_device)))

    try:
        _C.check(L.xq_skinny_reset())
        call(ws0, y0, xbuf)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            call(ws0, y0, xbuf)
        torch.cuda.synchronize()
        # 300 other workspaces, each used with the device idle (so every free or idle slot is fair game)
        others = [torch.empty(wsb, dtype=torch.uint8, device=hip_device) for _ in range(300)]
        yo = torch.empty(M, N, dtype=torch.bfloat16, device=hip_device)
        xo = gen((M, K), 1.0, 2, torch.bfloat16).to(hip_device)
        for ws in others:
            call(ws, yo, xo)
            torch.cuda.synchronize()
        side = torch.cuda.Stream()
        y_side = torch.empty(M, N, dtype=torch.bfloat16, device=hip_device)
        for rep in range(4):
            xbuf.copy_(gen((M, K), 1.0, 10 + rep, torch.bfloat16).to(hip_device))
            torch.cuda.synchronize()
            with torch.cuda.stream(side):
                for ws in others[rep * 8:rep * 8 + 8]:
                    call(ws, y_side, xo)
            graph.replay()
            torch.cuda.synchronize()
            got = y0.clone()
            ws1 = torch.empty(wsb, dtype=torch.uint8, device=hip_device)
            y1 = torch.empty(M, N, dtype=torch.bfloat16, device=hip_device)
            call(ws1, y1, xbuf)
            torch.cuda.synchronize()
            assert torch.equal(got, y1), rep
    finally:
        torch.cuda.synchronize()
        _C.check(L.xq_skinny_reset())


def test_one_launch_under_hip_graph_with_changing_input(hip_device):
    """A captured forward replays against new contents of its input buffer: every replay must use the intermediate of
    ITS input (the slot is restored inside each launch), and equal the eager result bit for bit."""
    m, _ = make_dense_module("block_fp8", 4096, 4096, 16, 32, seed=3, device=hip_device)
    xbuf = gen((8, 4096), 1.0, 1, torch.bfloat16).to(hip_device)

    def step():
        with torch.no_grad():
            return m(xbuf)

    step()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step()
    for rep in range(4):
        xbuf.copy_(gen((8, 4096), 1.0, 10 + rep, torch.bfloat16).to(hip_device))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        eager = step()
        torch.cuda.synchronize()
        assert torch.equal(got, eager), rep


def test_overlapping_calls_on_two_streams(hip_device):
    """Forwards on two streams, each with its own workspace (so each with its own slot), issued so that they overlap on the
    device: small grids that leave compute units free for the other stream's kernel.  Every result equals the one the same
    call gives alone."""
    from xorl_amd import _C
    from xorl_amd.functional import _workspace_bytes

    r = 16
    shapes = [("block_fp8", 1024, 4096, 4), ("int4", 2048, 4096, 1)]
    L = _C.lib()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    work = []
    for i, (fmt, N, K, M) in enumerate(shapes):
        m, _ = make_dense_module(fmt, N, K, r, 32, seed=60 + i, device=hip_device)
        w = m._quant_weight().c()
        A, B = m.lora_A.detach().contiguous(), m.lora_B.detach().contiguous()
        wsb = _workspace_bytes(M, N, K, r)
        ws = torch.empty(wsb, dtype=torch.uint8, device=hip_device)
        xs = [gen((M, K), 1.0, 600 + 10 * i + j, torch.bfloat16).to(hip_device) for j in range(6)]
        ys = [torch.empty(M, N, dtype=torch.bfloat16, device=hip_device) for _ in xs]
        work.append((m, w, A, B, ws, wsb, xs, ys, N, K, M))

    def call(i, j, y, stream):
        m, w, A, B, ws, wsb, xs, _, N, K, M = work[i]
        _C.check(L.xq_linear_fwd(ctypes.byref(w), xs[j].data_ptr(), K, M, A.data_ptr(), B.data_ptr(), _C.XQ_DT_F32, r,
                                 ctypes.c_float(m.scaling), None, y.data_ptr(), N, None, ws.data_ptr(), wsb, stream))

    # alone, on the current stream
    alone = []
    for i in range(2):
        outs = []
        for j in range(6):
            y = torch.empty_like(work[i][7][j])
            call(i, j, y, _C.stream_ptr(hip_device))
            outs.append(y)
        alone.append(outs)
    torch.cuda.synchronize()
    # interleaved on two streams, many times over
    for st in streams:
        st.wait_stream(torch.cuda.current_stream())
    for rep in range(20):
        for j in range(6):
            for i in range(2):
                call(i, j, work[i][7][j], ctypes.c_void_p(streams[i].cuda_stream))
    torch.cuda.synchronize()
    for i in range(2):
        for j in range(6):
            assert torch.equal(work[i][7][j], alone[i][j]), (i, j)


def test_bounded_waits_give_up_and_the_slot_recovers(hip_device):
    """With the waits cut to a single look (forced from the host) every kernel still ends; a block either has all it
    waited for, and writes the right outputs, or gives up and writes NaN, never values made from stale sums -- and counts
    itself where xq_skinny_status() finds it.  Once the closing block of a launch has given up the slot is marked failed
    and every forward through it writes NaN, also after the limit is back to normal, until the status call (or a reset)
    clears the mark; then results are exact again.  Which of the two happens is a race the test does not decide: it reads
    the outcome and checks the behaviour that belongs to it."""
    from xorl_amd import _C
    from xorl_amd.functional import _workspace_bytes, skinny_status

    N, K, r = 12288, 4096, 16
    m, _ = make_dense_module("block_fp8", N, K, r, 32, seed=9, device=hip_device)
    w = m._quant_weight().c()
    A, B = m.lora_A.detach().contiguous(), m.lora_B.detach().contiguous()
    L = _C.lib()
    M = 8
    wsb = _workspace_bytes(M, N, K, r)
    ws = torch.empty(wsb, dtype=torch.uint8, device=hip_device)        # one workspace = one slot throughout
    y = torch.empty(M, N, dtype=torch.bfloat16, device=hip_device)

    def call(x, rank=r):
        _C.check(L.xq_linear_fwd(ctypes.byref(w), x.data_ptr(), K, M, A.data_ptr(), B.data_ptr(), _C.XQ_DT_F32, rank, ctypes.c_float(m.scaling),
                                 None, y.data_ptr(), N, None, ws.data_ptr(), wsb, _C.stream_ptr(hip_device)))
        torch.cuda.synchronize()
        return y.clone()

    xs = [gen((M, K), 1.0, 300 + i, torch.bfloat16).to(hip_device) for i in range(6)]
    try:
        want = [call(x) for x in xs]
        assert all(torch.isfinite(t.float()).all() for t in want)
        assert skinny_status(hip_device) == (0, 0)                          # nothing to report after exact forwards
        no_lora = call(xs[0], 0)
        n_bad = 0
        try:
            _C.check(L.xq_set_skinny_spin_limit(1))
            for x, ref in zip(xs, want):
                got = call(x)
                bad = torch.isnan(got.float())
                assert torch.equal(got[~bad], ref[~bad])                    # what is not NaN is right: nothing stale was summed
                cols = bad.any(dim=0)                                       # a block gives up as a whole: all rows of x
                assert torch.equal(bad, cols.unsqueeze(0).expand_as(bad))
                n_bad += int(bad.sum())
        finally:
            _C.check(L.xq_set_skinny_spin_limit(0))
        # with the normal limit again: a marked slot turns everything into NaN, an unmarked one is exact; a forward without a
        # low-rank term does not use the slot either way
        after = call(xs[0])
        marked = bool(torch.isnan(after.float()).all())
        if not marked:
            assert torch.equal(after, want[0])
        assert torch.equal(call(xs[0], 0), no_lora)
        gave_up, failed = skinny_status(hip_device, raise_on_failure=False)
        assert (gave_up > 0) == (n_bad > 0 or marked), (gave_up, n_bad, marked)
        assert failed == (1 if marked else 0), (failed, marked)
        if marked:
            assert gave_up >= N // 48                                       # every block of the forward through the marked slot
        # the status call has cleared what it found: exact results, nothing more to report, and the raising form is quiet
        for x, ref in zip(xs, want):
            assert torch.equal(call(x), ref)
        assert skinny_status(hip_device) == (0, 0)
        # a report makes the default form raise
        if n_bad > 0 or marked:
            try:
                _C.check(L.xq_set_skinny_spin_limit(1))
                for x in xs:
                    call(x)
            finally:
                _C.check(L.xq_set_skinny_spin_limit(0))
            gave = False
            try:
                skinny_status(hip_device)
            except RuntimeError as e:
                gave = "gave up" in str(e)
            assert gave
            assert torch.equal(call(xs[1]), want[1])
    finally:
        _C.check(L.xq_set_skinny_spin_limit(0))
        _C.check(L.xq_skinny_reset())                                       # whatever happened above, later tests start clean
