"""GPU: xq_linear_fwd_static (scratch built into the library, nothing allocated by the call) against
xq_linear_fwd with a caller workspace, through the C ABI: bit-identical outputs, on two calls in a row of which
the second is smaller (it finds the first call's leftovers in the shared scratch), and against the oracle."""

import ctypes

import pytest
import torch

from oracle import recipe as R
from tests.util_cases import close, gen, make_dense_module
from xorl_amd import _C

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _bias(m):
    return None if m.bias is None else m.bias.detach().to(torch.bfloat16).contiguous()


def _fwd_ws(m, x, r):
    """xq_linear_fwd with a torch-allocated workspace."""
    qw = m._quant_weight()
    M, K, N = x.shape[0], m.in_features, m.out_features
    w = qw.c()
    nbytes = _C.lib().xq_linear_workspace_bytes(M, N, K, r)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=x.device)
    A, B = (m.lora_A.detach(), m.lora_B.detach()) if r else (None, None)
    b = _bias(m)
    _C.check(_C.lib().xq_linear_fwd(ctypes.byref(w), x.data_ptr(), x.stride(0), M, _C.ptr(A), _C.ptr(B), _C.XQ_DT_F32, r,
                                    float(m.scaling), _C.ptr(b), y.data_ptr(), y.stride(0), None, ws.data_ptr(),
                                    nbytes, _C.stream_ptr(x.device)))
    return y


def _fwd_static(m, x, r):
    """xq_linear_fwd_static: inputs and the output only."""
    qw = m._quant_weight()
    M, N = x.shape[0], m.out_features
    w = qw.c()
    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=x.device)
    A, B = (m.lora_A.detach(), m.lora_B.detach()) if r else (None, None)
    b = _bias(m)
    args = (ctypes.byref(w), x.data_ptr(), x.stride(0), M, _C.ptr(A), _C.ptr(B), _C.XQ_DT_F32, r, float(m.scaling), _C.ptr(b),
            y.data_ptr(), y.stride(0), _C.stream_ptr(x.device))
    # a first call, so that whatever the runtime sets up once per kernel (code objects, launch attributes) is in place;
    # the measured call must then leave the DEVICE's free memory as it found it -- hipMemGetInfo sees an allocation
    # by the library itself, which torch's own counter of its caching allocator would not
    _C.check(_C.lib().xq_linear_fwd_static(*args))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(x.device)[0]
    torch_before = torch.cuda.memory_allocated()
    rc = _C.lib().xq_linear_fwd_static(*args)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(x.device)[0] == free_before
    assert torch.cuda.memory_allocated() == torch_before
    _C.check(rc)
    return y


@pytest.mark.parametrize("fmt,N,K,r,M1,M2", [
    ("block_fp8", 4096, 4096, 16, 64, 8),        # skinny path: K splits with fp32 partial tiles in the scratch
    ("int4", 1024, 4096, 16, 33, 1),
    ("nvfp4", 1024, 2048, 16, 16, 5),
    ("block_fp8", 1024, 1024, 32, 512, 200),     # tile path: LoRA panels, su and split-K partial sums in the scratch
    ("int4", 512, 1024, 0, 300, 96),             # no low-rank term
])
def test_static_scratch_forward_matches_workspace_forward(hip_device, fmt, N, K, r, M1, M2):
    m, w_ref = make_dense_module(fmt, N, K, max(r, 1), 32, seed=N + K + r, device=hip_device, bias=(fmt == "int4"))
    bias = None if m.bias is None else m.bias.detach().cpu()
    for call, M in enumerate((M1, M2)):          # the second call is smaller and reuses the same scratch
        x = gen((M, K), 1.0, 900 + M + call, torch.bfloat16)
        xd = x.to(hip_device)
        y_ws = _fwd_ws(m, xd, r)
        y_st = _fwd_static(m, xd, r)
        torch.cuda.synchronize()
        assert not torch.isnan(y_st.float()).any()
        assert torch.equal(y_st, y_ws), (fmt, M)
        A = m.lora_A.detach().cpu() if r else torch.zeros(1, K)
        B = m.lora_B.detach().cpu() if r else torch.zeros(N, 1)
        ex = R.linear_fwd_bwd_exact(x, w_ref, A, B, m.scaling if r else 0.0, bias=bias)
        close(y_st.cpu(), ex["y"], TOL)


def test_static_scratch_rejects_oversized_shapes(hip_device):
    cap = _C.lib().xq_static_scratch_bytes()
    assert cap == 32 << 20
    m, _ = make_dense_module("block_fp8", 1024, 1024, 16, 32, seed=1, device=hip_device)
    M = 1 << 20                                   # the [M, r_pad] intermediate alone exceeds the buffer
    assert _C.lib().xq_linear_workspace_bytes(M, 1024, 1024, 16) > cap
    w = m._quant_weight().c()
    x = torch.zeros(8, 1024, dtype=torch.bfloat16, device=hip_device)     # never read: the call fails on the host
    y = torch.zeros(8, 1024, dtype=torch.bfloat16, device=hip_device)
    rc = _C.lib().xq_linear_fwd_static(ctypes.byref(w), x.data_ptr(), 1024, M, m.lora_A.data_ptr(), m.lora_B.data_ptr(),
                                       _C.XQ_DT_F32, 16, 2.0, None, y.data_ptr(), 1024, _C.stream_ptr(hip_device))
    assert rc == -1
    with pytest.raises(_C.XqError, match="scratch"):
        _C.check(rc)


@pytest.mark.parametrize("fmt,N,K,r,M", [("block_fp8", 4096, 4096, 16, 8), ("int4", 1024, 4096, 16, 48), ("block_fp8", 1024, 1024, 32, 300)])
def test_static_scratch_forward_under_hip_graph(hip_device, fmt, N, K, r, M):
    """The callers this entry point is for record it into a HIP graph: captured once, replayed with the input changing
    between replays and the program's own eager work and synchronisations in between, every replay must give the eager
    call's bits (decode sizes on the one-launch and the two-launch kernels, and a tile-kernel shape)."""
    m, _ = make_dense_module(fmt, N, K, r, 32, seed=N + K + M, device=hip_device)
    w = m._quant_weight().c()
    A, B = m.lora_A.detach(), m.lora_B.detach()
    x = torch.zeros(M, K, dtype=torch.bfloat16, device=hip_device)
    y = torch.zeros(M, N, dtype=torch.bfloat16, device=hip_device)

    def call():
        _C.check(_C.lib().xq_linear_fwd_static(ctypes.byref(w), x.data_ptr(), x.stride(0), M, A.data_ptr(), B.data_ptr(),
                                               _C.XQ_DT_F32, r, float(m.scaling), None, y.data_ptr(), y.stride(0),
                                               _C.stream_ptr(hip_device)))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for i in range(4):
        x.copy_(gen((M, K), 1.0, 950 + i, torch.bfloat16).to(hip_device))
        y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = y.clone()
        y.fill_(float("nan"))
        call()                                    # the same call, eager, between the replays
        torch.cuda.synchronize()
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got, y), (fmt, M, i)
