import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hip_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture
def tile_policy(request):
    """Selects the fused dequant-GEMM kernel for one test: 0 = by size, 1 = generic kernel, 2 / 3 = pipelined kernel with 256x256 / 128x128 tiles."""
    from xorl_amd import _C

    _C.check(_C.lib().xq_set_tile_policy(int(request.param)))
    yield int(request.param)
    _C.check(_C.lib().xq_set_tile_policy(0))


def pytest_sessionfinish(session, exitstatus):
    """Worst tolerance metrics per test (tensor-wide and per-row), for the parity table of the design notes."""
    import json

    from tests.util_cases import PARITY_WORST

    if PARITY_WORST:
        out = os.path.join(ROOT, "gpurun_out")
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "parity_worst.json"), "w") as f:
            json.dump({k: {"tensor": v[0], "row": v[1]} for k, v in sorted(PARITY_WORST.items())}, f, indent=1)
