"""GPU: the 256x256 tile kernel as a persistent program (one block per compute unit walking several tiles, the next
tile's first operands requested before the finished tile is stored) against the same kernel launched with one block per
tile.  Nothing in the arithmetic or its order depends on which block computes a tile, so every output must be equal bit
for bit -- a stale register set, a missed barrier or a wrong tile table shows up as a difference.  Shapes are chosen so
that blocks walk two or more tiles (more tiles than compute units) and the last round is ragged."""

import pytest
import torch

from tests.util_cases import gen, make_dense_module
from tests.test_gpu_moe import _make_experts, _zipf_routing

pytestmark = pytest.mark.gpu


@pytest.fixture
def both_ways():
    """run(fn) -> (persistent result, one-block-per-tile result); the switch is restored afterwards."""
    from xorl_amd import _C

    def run(fn):
        out = []
        for enabled in (1, 0):
            _C.check(_C.lib().xq_set_persistent_tiles(enabled))
            out.append(fn())
        _C.check(_C.lib().xq_set_persistent_tiles(1))
        return out

    yield run
    _C.check(_C.lib().xq_set_persistent_tiles(1))


def _same(a, b, what):
    assert len(a) == len(b)
    for i, (x, y) in enumerate(zip(a, b)):
        assert torch.equal(x, y), f"{what}[{i}]: {(x.float() - y.float()).abs().max().item()}"


@pytest.mark.parametrize("tile_policy", [2], indirect=True)      # 256x256 tiles whatever the size
@pytest.mark.parametrize("fmt,M,N,K,r,bias", [
    ("block_fp8", 4096, 12288, 1024, 32, False),     # 768 forward tiles = 3 rounds of 256 blocks
    ("block_fp8", 4096, 1024, 12288, 16, False),     # 768 dgrad tiles (two-round forward is the case above)
    ("block_fp8", 2100, 8448, 512, 16, True),        # 9 x 33 = 297 tiles: ragged rows, a second round of 41 tiles
    ("int4", 2048, 8448, 512, 16, False),            # 264 tiles
    ("nvfp4", 2304, 7680, 512, 48, True),            # 270 tiles
    ("nf4", 2048, 8448, 512, 8, False),
])
def test_dense_forward_backward_bit_equal(hip_device, tile_policy, both_ways, fmt, M, N, K, r, bias):
    m, _ = make_dense_module(fmt, N, K, r, 2 * r, seed=M + N, device=hip_device, bias=bias)
    x = gen((M, K), 1.0, 5, torch.bfloat16).to(hip_device)
    dy = gen((M, N), 1.0, 6, torch.bfloat16).to(hip_device)

    def step():
        m.lora_A.grad = m.lora_B.grad = None
        xd = x.clone().requires_grad_(True)
        y = m(xd)
        y.backward(dy)
        return y.detach(), xd.grad, m.lora_A.grad.clone(), m.lora_B.grad.clone()

    p, q = both_ways(step)
    _same(p, q, f"{fmt} dense")
    assert float(p[0].float().abs().max()) > 0 and float(p[1].float().abs().max()) > 0


def test_fused_mlp_bit_equal(hip_device, both_ways):
    """The gate|up launch with the SwiGLU epilogue (16 x 32 = 512 tiles) and the dgrad over two weights."""
    from xorl_amd.qlora import qlora_mlp_forward

    H, I, M, r = 1024, 4096, 4096, 16
    mods = {k: make_dense_module("block_fp8", n, kk, r, 32, seed=s, device=hip_device, bias=(k == "up"))[0]
            for k, n, kk, s in (("gate", I, H, 1), ("up", I, H, 2), ("down", H, I, 3))}
    x = gen((M, H), 1.0, 7, torch.bfloat16).to(hip_device)
    dy = gen((M, H), 1.0, 8, torch.bfloat16).to(hip_device)

    def step():
        for mm in mods.values():
            mm.lora_A.grad = mm.lora_B.grad = None
        xd = x.clone().requires_grad_(True)
        y = qlora_mlp_forward(mods["gate"], mods["up"], mods["down"], xd)
        y.backward(dy)
        return (y.detach(), xd.grad) + tuple(g for mm in mods.values() for g in (mm.lora_A.grad.clone(), mm.lora_B.grad.clone()))

    p, q = both_ways(step)
    _same(p, q, "fused MLP")


@pytest.mark.parametrize("tile_policy", [2], indirect=True)
@pytest.mark.parametrize("fmt,E,T,H,I,r,topk,hybrid", [
    ("block_fp8", 12, 8192, 1024, 1024, 16, 2, False),    # two-bank forward: (64 + 12) x 8 tiles; dgrad over both banks
    ("block_fp8", 9, 8192, 1024, 640, 16, 2, True),       # per-projection launches (640 is not a multiple of 256)
    ("nvfp4", 12, 8192, 1024, 1024, 16, 2, False),
    ("nf4", 7, 8192, 1280, 768, 8, 2, True),
])
def test_routed_experts_bit_equal(hip_device, tile_policy, both_ways, fmt, E, T, H, I, r, topk, hybrid):
    m, _ = _make_experts(fmt, E, H, I, r, hybrid, seed=E + T, device=hip_device)
    rw, sel = _zipf_routing(T, E, topk, seed=11)
    x = gen((T, H), 1.0, 12, torch.bfloat16).to(hip_device)
    dy = gen((T, H), 1.0, 13, torch.bfloat16).to(hip_device)
    rwd0, seld = rw.to(torch.bfloat16).to(hip_device), sel.to(hip_device)
    names = [f"{k}_proj_lora_{f}" for k in ("gate", "up", "down") for f in ("A", "B")]

    def step():
        for n in names:
            getattr(m, n).grad = None
        xd = x.clone().requires_grad_(True)
        rwd = rwd0.clone().requires_grad_(True)
        y = m(xd, rwd, seld)
        y.backward(dy)
        return (y.detach(), xd.grad, rwd.grad) + tuple(getattr(m, n).grad.clone() for n in names)

    p, q = both_ways(step)
    _same(p, q, f"{fmt} experts")
    assert float(p[0].float().abs().max()) > 0


def test_more_tiles_than_a_block_may_walk(hip_device, both_ways):
    """131072 x 16384 outputs are 32768 tiles of 256 x 256: more than 64 per block of a one-block-per-CU grid, so the
    launcher grows the grid (a block keeps a table of at most 64 tiles).  Forward only, a short contraction."""
    M, N, K, r = 131072, 16384, 64, 16
    m, _ = make_dense_module("block_fp8", N, K, r, 32, seed=9, device=hip_device)
    x = gen((M, K), 1.0, 15, torch.bfloat16).to(hip_device)

    def fwd():
        with torch.no_grad():
            y = m(x)
        # a digest instead of the 4 GiB tensor: two launches that differ anywhere differ here
        v = y.view(torch.int16).to(torch.int32)
        w = torch.arange(1, N + 1, device=hip_device, dtype=torch.int32)
        return ((v * w).sum(dim=1, dtype=torch.int64), y[::4099].clone())

    p, q = both_ways(fwd)
    _same(p, q, "many tiles")
    assert float(p[1].float().abs().max()) > 0
