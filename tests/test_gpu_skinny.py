"""GPU parity: the skinny-M (M <= 64) weight-streaming forward kernel vs the oracle,
and vs the generic tile kernel on the same inputs."""

import pytest
import torch

from oracle import recipe as R
from oracle import decode_np as NP
from tests.util_cases import close, bits_to_bf16, gen, make_dense_module

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
    close(y.cpu(), ex["y"], TOL)
    # the training path (tile kernel; needs grad) gives the same answer within bf16
    y2 = m(x.to(hip_device).requires_grad_(True))
    close(y2.detach().cpu(), ex["y"], TOL)


@pytest.mark.parametrize("fmt", ["int4", "block_fp8"])
@pytest.mark.parametrize("proj,N,K", [("q", 4096, 4096), ("kv", 1024, 4096), ("gate_up", 12288, 4096), ("down", 4096, 12288)])
def test_config4_full_grid(hip_device, fmt, proj, N, K):
    """BASELINE configs[4] in full: {int4, block_fp8} x the Qwen3-8B projection set x M in {1, 8, 32, 64}, r = 16,
    forward only, every cell against the float64 program on the oracle's decode of the module's bytes."""
    m, w_ref = make_dense_module(fmt, N, K, 16, 32, seed=N + K, device=hip_device)
    A, B = m.lora_A.detach().cpu(), m.lora_B.detach().cpu()
    for M in (1, 8, 32, 64):
        x = gen((M, K), 1.0, M, torch.bfloat16)
        with torch.no_grad():
            y = m(x.to(hip_device))
        ex = R.linear_fwd_bwd_exact(x, w_ref, A, B, m.scaling)
        assert y.shape == (M, N) and y.dtype == torch.bfloat16
        close(y.cpu(), ex["y"], TOL)
        with torch.no_grad():                     # the same bits from a second call on fresh scratch
            assert torch.equal(m(x.to(hip_device)), y)


@pytest.mark.parametrize("N,K", [(4096, 12288), (12288, 4096)])
def test_skinny_projection_shapes_nf4(hip_device, N, K):
    m, w_ref = make_dense_module("nf4", N, K, 16, 32, seed=N + K, device=hip_device)
    for M in (8, 64):
        x = gen((M, K), 1.0, M, torch.bfloat16)
        with torch.no_grad():
            y = m(x.to(hip_device))
        ex = R.linear_fwd_bwd_exact(x, w_ref, m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), m.scaling)
        close(y.cpu(), ex["y"], TOL)


@pytest.mark.parametrize("fmt,N,K,M,r,bf16_factors", [
    ("block_fp8", 21888, 1280, 3, 16, False),    # 10 chunks over 3 splits: 4 + 3 + 3 chunks per block
    ("int4", 21888, 1280, 16, 16, False),
    ("nvfp4", 208, 1024, 16, 6, False),          # ragged last row block, rank not a multiple of 4
    ("block_fp8", 384, 2048, 17, 64, True),      # four 16-rank tiles, bf16 factors
    ("int4", 1024, 4096, 32, 40, False),         # rank padded to 48
    ("nvfp4", 4096, 4096, 9, 16, True),
    ("nf4", 21888, 1280, 5, 16, False),          # uneven splits with two scales per chunk
    ("nf4", 208, 1024, 40, 24, True),
])
def test_skinny_split_plans(hip_device, fmt, N, K, M, r, bf16_factors):
    """K-split organisation: uneven splits, ragged row blocks, every rank-tile count, both factor dtypes."""
    from xorl_amd.functional import qlora_linear

    m, w_ref = make_dense_module(fmt, N, K, r, 2 * r, seed=N + K + M, device=hip_device, bias=(M == 16))
    x = gen((M, K), 1.0, 300 + M, torch.bfloat16)
    A, B = m.lora_A.detach(), m.lora_B.detach()
    if bf16_factors:
        A, B = A.to(torch.bfloat16), B.to(torch.bfloat16)
    with torch.no_grad():
        y = qlora_linear(x.to(hip_device), m._quant_weight(), A, B, r, m.scaling, m.bias)
    ex = R.linear_fwd_bwd_exact(x, w_ref, A.float().cpu(), B.float().cpu(), m.scaling,
                                bias=None if m.bias is None else m.bias.detach().cpu())
    assert y.shape == (M, N)
    close(y.cpu(), ex["y"], TOL)
    # deterministic: a second call returns the same bits
    with torch.no_grad():
        y2 = qlora_linear(x.to(hip_device), m._quant_weight(), A, B, r, m.scaling, m.bias)
    assert torch.equal(y, y2)
    # no low-rank term at all
    with torch.no_grad():
        y0 = qlora_linear(x.to(hip_device), m._quant_weight(), None, None, 0, 0.0, None)
    ex0 = R.linear_fwd_bwd_exact(x, w_ref, torch.zeros(1, K), torch.zeros(N, 1), 0.0)
    close(y0.cpu(), ex0["y"], TOL)


def test_skinny_forward_under_hip_graph(hip_device):
    """A captured decode step (several skinny forwards) replays to the eager result bit for bit, also with
    eager work and synchronisations between replays."""
    mods = [make_dense_module(fmt, N, K, 16, 32, seed=i, device=hip_device)[0]
            for i, (fmt, N, K) in enumerate((("block_fp8", 1024, 4096), ("int4", 4096, 4096), ("nvfp4", 1024, 1024)))]
    xs = [gen((M, m.in_features), 1.0, 500 + M, torch.bfloat16).to(hip_device) for M, m in zip((1, 8, 48), mods)]

    def step():
        with torch.no_grad():
            return [m(x) for m, x in zip(mods, xs)]

    eager = [y.clone() for y in step()]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for rep in range(4):
        for y in outs:
            y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for y, e in zip(outs, eager):
            assert torch.equal(y, e), rep
        again = step()                      # eager work between replays
        torch.cuda.synchronize()
        for y, e in zip(again, eager):
            assert torch.equal(y, e)


@pytest.mark.parametrize("M", [1, 24, 40])
def test_skinny_scale_storage_variants(hip_device, M):
    """Scale storages the default modules do not produce: nvfp4 with fp32 block scales and a folded global scale
    (pre-quantized checkpoints), int4 with fp32 scales and with groups shorter than a 128-element chunk."""
    from xorl_amd import quantize as Q
    from xorl_amd.qlora import Int4QLoRALinear, QLoRALinear

    N, K, r = 384, 1024, 16
    x = gen((M, K), 1.0, 700 + M, torch.bfloat16)
    w = gen((N, K), 0.02, 701)
    A, B = gen((r, K), 0.02, 702), gen((N, r), 0.02, 703)

    def check(m, w_ref):
        m = m.to(hip_device)
        with torch.no_grad():
            m.lora_A.copy_(A)
            m.lora_B.copy_(B)
            y = m(x.to(hip_device))
        ex = R.linear_fwd_bwd_exact(x, w_ref, A, B, m.scaling)
        close(y.cpu(), ex["y"], TOL)
        assert torch.equal(m._dequantize_weight().cpu().reshape(N, K), w_ref)      # same bytes, same decode

    # nvfp4: fold the global scale into fp32 block scales, as the checkpoint loaders do
    packed, bs, g = Q.nvfp4_quantize(w, 16)
    folded = (bs.float() * g.float()).reshape(N, K // 16).contiguous()
    m = QLoRALinear.from_quantized(packed.reshape(N, K // 2), weight_block_scales=folded,
                                   weight_global_scale=torch.ones(1), in_features=K, out_features=N, r=r,
                                   lora_alpha=2 * r, quant_format="nvfp4")
    check(m, bits_to_bf16(NP.nvfp4_decode_flat(packed.numpy().reshape(N, K // 2), folded.numpy(), 1.0, N, K)))

    # int4, reference codec (fp32 scales), group 128 and group 32
    for group in (128, 32):
        lin = torch.nn.Linear(K, N, bias=False)
        with torch.no_grad():
            lin.weight.copy_(w)
        m = Int4QLoRALinear.from_module(lin, r=r, lora_alpha=2 * r, quant_group_size=group, symmetric=False)
        pk = m.packed_weight_f32.detach().contiguous().view(torch.uint8).numpy()
        sc = m.weight_scales.contiguous().view(torch.float32).numpy()
        check(m, bits_to_bf16(NP.int4_decode_flat(pk, sc, N, K, group)))


@pytest.mark.parametrize("fmt", ["block_fp8", "int4", "nvfp4", "nf4"])
@pytest.mark.parametrize("M", [16, 64])
def test_skinny_decode_bit_exact(hip_device, fmt, M):
    """Rows of X that are unit vectors (and no low-rank term) make every output a single product 1 * w: the
    forward returns columns of the decoded weight, which must equal the oracle's decode bit for bit (up to the sign
    of zero: a sum of zeros is +0).  The columns cover every K split and both halves of a scale group."""
    from xorl_amd.functional import qlora_linear

    N, K = 384, 2048
    m, w_ref = make_dense_module(fmt, N, K, 8, 16, seed=31 + M, device=hip_device)
    cols = torch.tensor([(37 * i * i + 11 * i) % K for i in range(M)])
    cols[0], cols[1] = 0, K - 1
    x = torch.zeros(M, K, dtype=torch.bfloat16)
    x[torch.arange(M), cols] = 1.0
    with torch.no_grad():
        y = qlora_linear(x.to(hip_device), m._quant_weight(), None, None, 0, 0.0, None).cpu()
    want = w_ref[:, cols].t().contiguous()                       # [M, N]
    same = y.view(torch.int16) == want.view(torch.int16)
    both_zero = (y.float() == 0) & (want.float() == 0)
    assert bool((same | both_zero).all())


def test_skinny_seeded_shape_sweep(hip_device):
    """Twenty-four seeded draws of (format, N, K, M, r, bias, factor dtype) within the path's shape rules --
    N any multiple of 16 (ragged last row block), K any multiple of 128 from 1024 (every split / chunk
    combination the planner makes), M 1..64, r 1..64 -- against the float64 form."""
    import numpy as np

    from xorl_amd.functional import qlora_linear

    rng = np.random.default_rng(2024)
    fmts = ["block_fp8", "int4", "nvfp4", "nf4"]
    for case in range(24):
        fmt = fmts[case % 4]
        N = int(rng.integers(1, 40)) * 16 * int(rng.choice([1, 1, 3, 8]))
        K = int(rng.integers(8, 41)) * 128
        M = int(rng.integers(1, 65))
        r = int(rng.integers(1, 65))
        bf16_factors = bool(rng.integers(0, 2))
        m, w_ref = make_dense_module(fmt, N, K, r, 2 * r, seed=1000 + case, device=hip_device, bias=bool(case % 3 == 0))
        x = gen((M, K), 1.0, 2000 + case, torch.bfloat16)
        A, B = m.lora_A.detach(), m.lora_B.detach()
        if bf16_factors:
            A, B = A.to(torch.bfloat16), B.to(torch.bfloat16)
        with torch.no_grad():
            y = qlora_linear(x.to(hip_device), m._quant_weight(), A, B, r, m.scaling, m.bias)
        ex = R.linear_fwd_bwd_exact(x, w_ref, A.float().cpu(), B.float().cpu(), m.scaling,
                                    bias=None if m.bias is None else m.bias.detach().cpu())
        assert y.shape == (M, N), (case, fmt, N, K, M, r, bf16_factors)
        close(y.cpu(), ex["y"], TOL)
