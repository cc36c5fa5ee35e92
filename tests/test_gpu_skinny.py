"""GPU parity: the skinny-M (M <= 64) weight-streaming forward kernel vs the oracle,
and vs the generic tile kernel on the same inputs."""

import pytest
import torch

from oracle import recipe as R
from tests.util_cases import gen, make_dense_module

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.mark.parametrize("fmt", ["block_fp8", "int4", "nvfp4", "nf4"])
@pytest.mark.parametrize("M", [1, 8, 32, 64, 5, 33])
def test_skinny_forward_vs_oracle(hip_device, fmt, M):
    K, N, r = 1024, 384, 16
    m, w_ref = make_dense_module(fmt, N, K, r, 32, seed=M, device=hip_device, bias=(M == 8))
    x = gen((M, K), 1.0, 100 + M, torch.bfloat16)
    with torch.no_grad():
        y = m(x.to(hip_device))
    ex = R.linear_fwd_bwd_exact(x, w_ref, m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), m.scaling,
                                bias=None if m.bias is None else m.bias.detach().cpu())
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    assert R.max_rel_err(y.cpu(), ex["y"]) <= TOL
    # the training path (tile kernel; needs grad) gives the same answer within bf16
    y2 = m(x.to(hip_device).requires_grad_(True))
    assert R.max_rel_err(y2.detach().cpu(), ex["y"]) <= TOL


@pytest.mark.parametrize("fmt,N,K", [("block_fp8", 1024, 4096), ("int4", 1024, 4096), ("block_fp8", 4096, 12288),
                                     ("int4", 12288, 4096)])
def test_skinny_projection_shapes(hip_device, fmt, N, K):
    """Qwen3-8B projection shapes of BASELINE config 4 at M = 8 and 64 (oracle in float64 on CPU)."""
    m, w_ref = make_dense_module(fmt, N, K, 16, 32, seed=N + K, device=hip_device)
    for M in (8, 64):
        x = gen((M, K), 1.0, M, torch.bfloat16)
        with torch.no_grad():
            y = m(x.to(hip_device))
        ex = R.linear_fwd_bwd_exact(x, w_ref, m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), m.scaling)
        assert R.max_rel_err(y.cpu(), ex["y"]) <= TOL, (fmt, N, K, M)
        # repeated calls reuse the zeroed scratch correctly
        with torch.no_grad():
            y_again = m(x.to(hip_device))
        assert R.max_rel_err(y_again.cpu(), ex["y"]) <= TOL
