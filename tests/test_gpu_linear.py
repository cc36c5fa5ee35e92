"""GPU parity: fused dequant-GEMM + LoRA forward/backward (through the C ABI)
vs the CPU oracle.  Tolerance: max|got-ref| / max|ref| <= 1e-2 against the
float64 restatement of the reference recipe (the "fp32-accumulated path")."""

import pytest
import torch

from oracle import recipe as R
from tests.util_cases import close, gen, make_dense_module

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _run(m, x, dy):
    x = x.clone().requires_grad_(True)
    y = m(x)
    y.backward(dy)
    return y.detach(), x.grad, m.lora_A.grad, m.lora_B.grad


@pytest.mark.parametrize("tile_policy", [0, 1, 2], indirect=True)
@pytest.mark.parametrize("fmt", ["block_fp8", "int4", "nvfp4", "nf4"])
@pytest.mark.parametrize("M,K,N,r", [(200, 256, 384, 16), (1, 128, 64, 8), (129, 384, 320, 24), (512, 1024, 512, 64), (1100, 512, 768, 32)])
def test_dense_fwd_bwd_vs_oracle(hip_device, tile_policy, fmt, M, K, N, r):
    m, w_ref = make_dense_module(fmt, N, K, r, 2 * r, seed=M + K, device=hip_device)
    x = gen((M, K), 1.0, 11, torch.bfloat16)
    dy = gen((M, N), 1.0, 12, torch.bfloat16)
    y, dx, dA, dB = _run(m, x.to(hip_device), dy.to(hip_device))
    ex = R.linear_fwd_bwd_exact(x, w_ref, m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), m.scaling, dy)
    assert y.dtype == torch.bfloat16 and dx.dtype == torch.bfloat16
    assert dA.dtype == torch.float32 and dA.shape == (r, K) and dB.shape == (N, r)
    for name, got, ref in (("y", y, ex["y"]), ("dx", dx, ex["dx"]), ("dA", dA, ex["dA"]), ("dB", dB, ex["dB"])):
        close(got.cpu(), ref, TOL)


@pytest.mark.parametrize("tile_policy", [0, 1, 2], indirect=True)
def test_config0_int4_full_size(hip_device, tile_policy):
    """BASELINE config 0: X [512,4096], W [4096,4096] int4 g128 absmax/7 bf16 scales, r=16, alpha=32."""
    M, K, N, r = 512, 4096, 4096, 16
    m, w_ref = make_dense_module("int4", N, K, r, 32, seed=0, device=hip_device)
    x = gen((M, K), 1.0, 1, torch.bfloat16)
    dy = gen((M, N), 1.0, 2, torch.bfloat16)
    y, dx, dA, dB = _run(m, x.to(hip_device), dy.to(hip_device))
    ex = R.linear_fwd_bwd_exact(x, w_ref, m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), 2.0, dy)
    for name, got, ref in (("y", y, ex["y"]), ("dx", dx, ex["dx"]), ("dA", dA, ex["dA"]), ("dB", dB, ex["dB"])):
        close(got.cpu(), ref, TOL)
    # the module's own decode is bit-exact with the oracle
    assert torch.equal(m._dequantize_weight().cpu(), w_ref)


@pytest.mark.parametrize("tile_policy", [1, 2, 3], indirect=True)
@pytest.mark.parametrize("fmt", ["block_fp8", "int4", "nvfp4", "nf4"])
def test_gemm_decode_bit_exact(hip_device, tile_policy, fmt):
    """With X = I (and lora_B = 0) every output is a single product 1 * w, so the forward returns the
    decoded weight itself and the dgrad of dY = I returns it transposed: the in-kernel decode of both
    fused kernels, in both contraction directions, must equal the oracle's decode bit for bit."""
    N = K = 512
    m, w_ref = make_dense_module(fmt, N, K, 16, 32, seed=77, device=hip_device)
    with torch.no_grad():
        m.lora_B.zero_()
    eye = torch.eye(K, dtype=torch.bfloat16, device=hip_device)
    x = eye.clone().requires_grad_(True)
    y = m(x)                                   # y[m, n] = w[n, m]
    y.backward(eye)                            # dx[m, k] = sum_n I[m, n] w[n, k] = w[m, k]
    wd = w_ref.to(hip_device)
    assert torch.equal(y.detach().view(torch.int16), wd.t().contiguous().view(torch.int16)) or \
        _equal_mod_zero_sign(y.detach(), wd.t())
    assert torch.equal(x.grad.view(torch.int16), wd.view(torch.int16)) or _equal_mod_zero_sign(x.grad, wd)


@pytest.mark.parametrize("fmt", ["block_fp8", "int4", "nvfp4", "nf4"])
def test_split_k_decode_bit_exact(hip_device, fmt):
    """N = K = M = 1024 under the default policy: 64 tiles of 128 x 128 leave most of the chip idle, so the 16
    K-steps are divided over two blocks per tile whose fp32 sums a second kernel adds.  With X = I every sum has
    one non-zero term, so forward and dgrad must still return the oracle's decode bit for bit."""
    from xorl_amd import _C

    N = K = 1024
    assert _C.lib().xq_linear_workspace_bytes(K, N, K, 0) >= 2 * K * N * 4       # the plan does split
    m, w_ref = make_dense_module(fmt, N, K, 16, 32, seed=78, device=hip_device)
    with torch.no_grad():
        m.lora_B.zero_()
    eye = torch.eye(K, dtype=torch.bfloat16, device=hip_device)
    x = eye.clone().requires_grad_(True)
    y = m(x)
    y.backward(eye)
    wd = w_ref.to(hip_device)
    assert _equal_mod_zero_sign(y.detach(), wd.t()) and _equal_mod_zero_sign(x.grad, wd)


@pytest.mark.parametrize("fmt,M,N,K,r,bias", [
    ("block_fp8", 512, 1024, 4096, 16, True),     # 32 tiles -> 8 splits forward, 2 in the dgrad (contraction 1024)
    ("int4", 192, 320, 2048, 8, False),           # ragged tiles in both directions, 4 splits
    ("nvfp4", 320, 512, 1536, 32, False),         # 24 K-steps -> 3 splits of 8
    ("nf4", 130, 256, 1088, 16, True),            # 17 K-steps -> 2 splits of 9 and 8
])
def test_split_k_fwd_bwd_vs_oracle(hip_device, fmt, M, N, K, r, bias):
    from xorl_amd import _C

    assert _C.lib().xq_linear_workspace_bytes(M, N, K, 0) >= 2 * M * N * 4
    m, w_ref = make_dense_module(fmt, N, K, r, 2 * r, seed=M + K, device=hip_device, bias=bias)
    x = gen((M, K), 1.0, 31, torch.bfloat16)
    dy = gen((M, N), 1.0, 32, torch.bfloat16)
    y, dx, dA, dB = _run(m, x.to(hip_device), dy.to(hip_device))
    ex = R.linear_fwd_bwd_exact(x, w_ref, m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), m.scaling, dy,
                                bias=m.bias.detach().cpu() if bias else None)
    for name, got, ref in (("y", y, ex["y"]), ("dx", dx, ex["dx"]), ("dA", dA, ex["dA"]), ("dB", dB, ex["dB"])):
        close(got.cpu(), ref, TOL)
    # the same call again gives the same bits (fixed summation order, no atomics)
    y2, dx2, _, _ = _run(m, x.to(hip_device), dy.to(hip_device))
    assert torch.equal(y, y2) and torch.equal(dx, dx2)
    # and the unsplit kernel agrees to rounding
    _C.check(_C.lib().xq_set_tile_policy(1))
    try:
        with torch.no_grad():
            y1 = m(x.to(hip_device))
    finally:
        _C.check(_C.lib().xq_set_tile_policy(0))
    assert R.max_rel_err(y.cpu(), y1.cpu().double()) <= 4e-3


def _equal_mod_zero_sign(a, b):
    """Bitwise equality except that a sum may return +0 where the decoded weight is -0."""
    a16, b16 = a.contiguous().view(torch.int16), b.contiguous().view(torch.int16)
    diff = a16 != b16
    return bool(((a.float() == 0) & (b.float() == 0))[diff].all())


def test_invariants(hip_device):
    m, w_ref = make_dense_module("block_fp8", 384, 256, 16, 32, seed=5, device=hip_device, bias=True)
    x = gen((3, 7, 256), 1.0, 13, torch.bfloat16).to(hip_device)        # leading dims are kept
    with torch.no_grad():
        y = m(x)
        assert y.shape == (3, 7, 384)
        b_saved = m.lora_B.clone()
        m.lora_B.zero_()
        y0 = m(x)
        m.lora_B.copy_(b_saved)
    base = R.linear_fwd_bwd_exact(x.cpu(), w_ref, m.lora_A.detach().cpu(), torch.zeros(384, 16), 2.0,
                                  bias=m.bias.detach().cpu())["y"]
    close(y0.cpu(), base, TOL)          # lora_B = 0 => base only (+ bias)
    assert not torch.equal(y, y0)
    # linearity in x of the whole op (size-independent property)
    with torch.no_grad():
        m.bias.zero_()
        a, b = m(x), m(2 * x)
    close(b.cpu().float(), 2 * a.cpu().float(), TOL)
    # active rank slice (set_runtime_lora_config)
    m.set_runtime_lora_config(8, 16)
    with torch.no_grad():
        y8 = m(x)
    ex8 = R.linear_fwd_bwd_exact(x.cpu(), w_ref, m.lora_A.detach().cpu()[:8], m.lora_B.detach().cpu()[:, :8], 2.0)["y"]
    close(y8.cpu(), ex8, TOL)
    with pytest.raises(ValueError):
        m.set_runtime_lora_config(0, 1)


def test_errors(hip_device):
    from xorl_amd.qlora import BlockFP8QLoRALinear, QLoRALinear

    with pytest.raises(TypeError):
        QLoRALinear(64, 64)
    m = BlockFP8QLoRALinear(200, 64, device=hip_device)       # K not a multiple of 64
    with pytest.raises(ValueError):
        m(torch.zeros(2, 200, dtype=torch.bfloat16, device=hip_device))
    m2 = BlockFP8QLoRALinear(128, 64, device=hip_device)
    with pytest.raises(ValueError):
        m2(torch.zeros(2, 128, dtype=torch.float32, device=hip_device))   # activations must be bf16
    m2.packed_weight_f32.data = m2.packed_weight_f32.data.to(torch.bfloat16)
    with pytest.raises(RuntimeError):
        m2(torch.zeros(2, 128, dtype=torch.bfloat16, device=hip_device))


def test_silu_and_mul(hip_device):
    from xorl_amd.functional import silu_and_mul

    g = (gen((300, 512), 2.0, 20)).to(torch.bfloat16)
    u = gen((300, 512), 1.0, 21, torch.bfloat16)
    dh = gen((300, 512), 1.0, 22, torch.bfloat16)
    gd, ud = g.to(hip_device).requires_grad_(True), u.to(hip_device).requires_grad_(True)
    h = silu_and_mul(gd, ud)
    h.backward(dh.to(hip_device))
    ref = R.silu_and_mul_recipe(g, u)
    # two-rounding recipe: identical up to 1 bf16 ulp where expf differs in the last bit
    assert R.max_rel_err(h.cpu(), ref) <= 2 ** -7
    assert (h.cpu() == ref).float().mean() > 0.99
    g64, u64 = g.double().requires_grad_(True), u.double().requires_grad_(True)
    (torch.nn.functional.silu(g64) * u64).backward(dh.double())
    close(gd.grad.cpu(), g64.grad, TOL)
    close(ud.grad.cpu(), u64.grad, TOL)


@pytest.mark.parametrize("fmt,M,K,N", [("block_fp8", 4100, 256, 4096), ("int4", 4352, 384, 5120), ("nvfp4", 4099, 256, 4352),
                                       ("block_fp8", 4352, 2048, 4096), ("nvfp4", 4200, 2048, 4096)])
def test_dense_split_launch_tail_rows(hip_device, fmt, M, K, N):
    """Shapes whose 256x256 tiling leaves a partly filled last round of the chip: the launcher runs the leading
    tile rows on large tiles and the trailing rows (here 4, 256, 3 + 256, 256 and 104 of them) as a second launch:
    of small tiles when the contraction is short, of large tiles in K splits (fp32 partial sums added by a reduce
    kernel) when it has at least 16 K-steps -- the last two cases.  Forward, dgrad and both factor gradients
    against the float64 form, with particular attention to the rows on either side of the seam."""
    r = 16
    if K >= 1024:
        from xorl_amd import _C

        tail = M - (M // 256) * 256 if M % 256 else 256
        assert _C.lib().xq_linear_workspace_bytes(M, N, K, 0) >= 2 * tail * N * 4      # the plan splits the tail
    m, w_ref = make_dense_module(fmt, N, K, r, 32, seed=M + N, device=hip_device, bias=True)
    x = gen((M, K), 1.0, 31, torch.bfloat16)
    dy = gen((M, N), 1.0, 32, torch.bfloat16)
    y, dx, dA, dB = _run(m, x.to(hip_device), dy.to(hip_device))
    ex = R.linear_fwd_bwd_exact(x, w_ref, m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), m.scaling, dy,
                                bias=m.bias.detach().cpu())
    for name, got, ref in (("y", y, ex["y"]), ("dx", dx, ex["dx"]), ("dA", dA, ex["dA"]), ("dB", dB, ex["dB"])):
        close(got.cpu(), ref, TOL)
    seam = slice((M // 256) * 256 - 300, M)
    close(y.cpu()[seam], ex["y"][seam], TOL)
    close(dx.cpu()[seam], ex["dx"][seam], TOL)


@pytest.mark.parametrize("fmt", ["block_fp8", "nvfp4"])
@pytest.mark.parametrize("M", [8, 300])
def test_row_strided_activations(hip_device, fmt, M):
    """x and dY that are column windows of wider tensors (row stride > width, 16-byte aligned) are consumed in
    place through their leading dimension: skinny forward (M = 8, no grad), tile forward and backward."""
    K, N, r = 1024, 384, 16
    m, w_ref = make_dense_module(fmt, N, K, r, 32, seed=M, device=hip_device)
    xw = gen((M, K + 64), 1.0, 41, torch.bfloat16).to(hip_device)
    dyw = gen((M, N + 128), 1.0, 42, torch.bfloat16).to(hip_device)
    x, dy = xw[:, 32:32 + K], dyw[:, 64:64 + N]
    assert not x.is_contiguous() and not dy.is_contiguous()
    A, B = m.lora_A.detach().cpu(), m.lora_B.detach().cpu()
    ex = R.linear_fwd_bwd_exact(x.cpu(), w_ref, A, B, m.scaling, dy.cpu())
    with torch.no_grad():
        close(m(x).cpu(), ex["y"], TOL)
    xg = x.detach().requires_grad_(True)
    y = m(xg)
    y.backward(dy)
    close(y.detach().cpu(), ex["y"], TOL)
    close(xg.grad.cpu(), ex["dx"], TOL)
    close(m.lora_A.grad.cpu(), ex["dA"], TOL)
    close(m.lora_B.grad.cpu(), ex["dB"], TOL)


@pytest.mark.parametrize("fmt,r", [("block_fp8", 96), ("nvfp4", 128), ("int4", 72)])
def test_ranks_above_the_fused_limit(hip_device, fmt, r):
    """Ranks above 64: the first 64 ride in the fused kernel, the rest as library GEMMs.  Forward (tile and skinny
    paths), all gradients, the published merged weight and merge_weights against the float64 forms."""
    M, K, N = 300, 512, 384
    m, w_ref = make_dense_module(fmt, N, K, r, 2 * r, seed=r, device=hip_device)
    x = gen((M, K), 1.0, 51, torch.bfloat16)
    dy = gen((M, N), 1.0, 52, torch.bfloat16)
    y, dx, dA, dB = _run(m, x.to(hip_device), dy.to(hip_device))
    A, B = m.lora_A.detach().cpu(), m.lora_B.detach().cpu()
    ex = R.linear_fwd_bwd_exact(x, w_ref, A, B, m.scaling, dy)
    assert dA.shape == (r, K) and dB.shape == (N, r)
    for name, got, ref in (("y", y, ex["y"]), ("dx", dx, ex["dx"]), ("dA", dA, ex["dA"]), ("dB", dB, ex["dB"])):
        close(got.cpu(), ref, TOL)
    # every rank contributes: the tail ranks' gradients are not zero
    assert float(dA[64:].abs().max()) > 0 and float(dB[:, 64:].abs().max()) > 0
    with torch.no_grad():
        ys = m(x[:4].to(hip_device))                                        # skinny path
    close(ys.cpu(), ex["y"][:4], TOL)
    # publish and merge
    pub = m.merged_weight().cpu()
    want = R.merge_publish_recipe(w_ref, A, B, m.scaling)
    assert R.max_rel_err(pub, want) <= 2 ** -7
    m.merge_weights()
    assert torch.count_nonzero(m.lora_B) == 0
    merged = w_ref.double() + R.merge_delta_exact(A, B, m.scaling)
    step = {"block_fp8": 2 ** -3, "nvfp4": 0.3, "int4": 0.2}[fmt]             # one quantization step of the format
    assert R.max_rel_err(m._dequantize_weight().cpu().float(), merged) <= step


@pytest.mark.parametrize("tile_policy", [0, 2], indirect=True)
def test_dense_seeded_shape_sweep(hip_device, tile_policy):
    """Sixteen seeded draws of (format, M, K, N, r, bias): K and N any multiple of 64, ragged M,
    every rank 1..64 -- forward and all three gradients against the float64 form, by size-selected tiles and with
    256x256 tiles forced."""
    import numpy as np

    rng = np.random.default_rng(7)
    fmts = ["block_fp8", "int4", "nvfp4", "nf4"]
    for case in range(16):
        fmt = fmts[case % 4]
        M = int(rng.integers(1, 700))
        K = int(rng.integers(1, 17)) * 64
        N = int(rng.integers(1, 13)) * 64           # the backward contracts over N: multiples of 64
        r = int(rng.integers(1, 65))
        if fmt == "int4" and K % 128:
            K += 64
        m, w_ref = make_dense_module(fmt, N, K, r, 2 * r, seed=3000 + case, device=hip_device, bias=bool(case % 2))
        x = gen((M, K), 1.0, 4000 + case, torch.bfloat16)
        dy = gen((M, N), 1.0, 5000 + case, torch.bfloat16)
        y, dx, dA, dB = _run(m, x.to(hip_device), dy.to(hip_device))
        ex = R.linear_fwd_bwd_exact(x, w_ref, m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), m.scaling, dy,
                                    bias=None if m.bias is None else m.bias.detach().cpu())
        for name, got, ref in (("y", y, ex["y"]), ("dx", dx, ex["dx"]), ("dA", dA, ex["dA"]), ("dB", dB, ex["dB"])):
            close(got.cpu(), ref, TOL)


def test_training_shape_rule_is_reported_at_the_forward(hip_device):
    """out_features = 48 is fine for a forward-only call; with gradients enabled the call says at once that the
    backward product needs out_features % 64 == 0."""
    m, w_ref = make_dense_module("block_fp8", 48, 128, 8, 16, seed=9, device=hip_device)
    x = gen((5, 128), 1.0, 61, torch.bfloat16).to(hip_device)
    with torch.no_grad():
        y = m(x)
    ex = R.linear_fwd_bwd_exact(x.cpu(), w_ref, m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), m.scaling)
    close(y.cpu(), ex["y"], TOL)
    with pytest.raises(ValueError, match="out_features % 64"):
        m(x.requires_grad_(True))


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
def test_module_under_torch_compile(hip_device, backend):
    """Traced by torch.compile the module reaches the library through the registered custom ops (fake tensors for
    shapes); forward and all gradients equal the eager call bit for bit."""
    from torch.library import opcheck

    from xorl_amd import functional as Fn

    m, _ = make_dense_module("block_fp8", 512, 256, 16, 32, seed=1, device=hip_device)
    x = gen((200, 256), 1.0, 3, torch.bfloat16).to(hip_device)
    dy = gen((200, 512), 1.0, 4, torch.bfloat16).to(hip_device)
    ref = _run(m, x, dy)
    ref = tuple(t.clone() for t in ref)
    m.lora_A.grad = m.lora_B.grad = None
    torch._dynamo.reset()
    got = _run(torch.compile(m, backend=backend, fullgraph=True), x, dy)
    for a, b in zip(ref, got):
        assert torch.equal(a, b)
    qw = m._forward_quant_weight()
    args = (x, qw.packed, qw.scales, qw.global_scale, m.lora_A.detach(), m.lora_B.detach(), None, qw.fmt,
            Fn._DT_TO_CODE[qw.scale_dtype], qw.group, qw.rows, qw.cols, 16, 2.0, True)
    assert set(opcheck(Fn._linear_fwd_op, args, test_utils=("test_schema", "test_faketensor")).values()) == {"SUCCESS"}


_ZERO_CODE = {"block_fp8": 0x00, "int4": 0x88, "nvfp4": 0x00, "nf4": 0x77}    # bytes whose codes all decode to 0.0


@pytest.mark.parametrize("tile_policy", [0, 1, 2], indirect=True)
@pytest.mark.parametrize("fmt", ["block_fp8", "int4", "nvfp4", "nf4"])
@pytest.mark.parametrize("M", [16, 640])
def test_lora_term_alone(hip_device, tile_policy, fmt, M):
    """Base codes that decode to zero (e4m3 byte 0x00, int4 code 8, e2m1 code 0, NF4 level 7), so that y and dx
    are the low-rank term alone and are judged on ITS scale, not the base product's: the kernels round the factors
    and the [M, r] intermediate to bf16 where the reference runs this branch in fp32
    (qlora/modules/linear.py:378-382); y, dx, dA, dB must stay within 1e-2 of the fp64 program all the same.
    M = 16 without grad takes the skinny path, M = 640 the tile kernels."""
    K, N, r = 1024, 768, 16
    m, _ = make_dense_module(fmt, N, K, r, 32, seed=M, device=hip_device)
    nbytes = N * K if fmt == "block_fp8" else N * K // 2
    with torch.no_grad():
        m._write_packed_weight(torch.full((nbytes,), _ZERO_CODE[fmt], dtype=torch.uint8, device=hip_device))
    assert torch.count_nonzero(m._dequantize_weight()) == 0
    w0 = torch.zeros(N, K, dtype=torch.bfloat16)
    x = gen((M, K), 1.0, 61, torch.bfloat16)
    dy = gen((M, N), 1.0, 62, torch.bfloat16)
    A, B = m.lora_A.detach().cpu(), m.lora_B.detach().cpu()
    ex = R.linear_fwd_bwd_exact(x, w0, A, B, m.scaling, dy)
    assert float(ex["y"].abs().max()) > 0
    with torch.no_grad():
        close(m(x.to(hip_device)).cpu(), ex["y"], TOL)
    y, dx, dA, dB = _run(m, x.to(hip_device), dy.to(hip_device))
    for got, ref in ((y, ex["y"]), (dx, ex["dx"]), (dA, ex["dA"]), (dB, ex["dB"])):
        close(got.cpu(), ref, TOL)


@pytest.mark.parametrize("fmt", ["block_fp8", "nvfp4", "nf4", "int4"])
def test_aqn_forward(hip_device, fmt):
    """Adaptive quantization noise (qlora/modules/linear.py:337-363): in training the decoded weight is perturbed by
    aqn_alpha * N(0, 1) * step, step = 0.125 * block scale (block_fp8_linear.py:102-109), 0.5 * block scale * global
    scale (nvfp4_linear.py:115-124), 0.5 * NF4_MIN_STEP * group absmax (nf4_linear.py:113-120).  With alpha = 0 the
    noisy forward is the plain recipe and must agree with the fused kernels; with alpha > 0 the perturbation of the
    weight, recovered through X = I, has the stated per-element standard deviation; eval mode never adds noise."""
    from xorl_amd import quantize as Q

    N = K = 512
    r = 16
    m, w_ref = make_dense_module(fmt, N, K, r, 32, seed=91, device=hip_device)
    x = gen((96, K), 1.0, 92, torch.bfloat16).to(hip_device)
    m.eval()
    with torch.no_grad():
        y_fused = m(x)
    m.enable_aqn, m.aqn_alpha = True, 0.0
    with torch.no_grad():
        assert torch.equal(m(x), y_fused)                    # eval: the fused path whatever enable_aqn says
    m.train()
    ex = R.linear_fwd_bwd_exact(x.cpu(), w_ref, m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), m.scaling)
    with torch.no_grad():
        y0 = m(x)
    close(y0.cpu(), ex["y"], TOL)                            # alpha = 0: same function as the fused kernels
    assert R.max_rel_err(y0.cpu(), y_fused.cpu().double()) <= TOL

    # the step tensor against the oracle's decode of the scales
    step = m._compute_aqn_step().cpu()
    assert step.shape == (N, K) and step.dtype == torch.float32
    if fmt == "block_fp8":
        s = m.weight_block_scales.cpu().contiguous().view(torch.float32).reshape(N // 128, K // 128)
        want = 0.125 * s.repeat_interleave(128, 0).repeat_interleave(128, 1)
    elif fmt == "nvfp4":
        bs = m.weight_block_scales.cpu().contiguous().view(torch.float8_e4m3fn).float().reshape(N, K // 16)
        gs = m.weight_global_scale.cpu().contiguous().view(torch.float32)
        want = 0.5 * (bs * gs).repeat_interleave(16, 1)
    elif fmt == "nf4":
        s = m.weight_scales.cpu().contiguous().view(torch.float32).reshape(N, K // 64)
        want = 0.5 * Q.NF4_MIN_STEP * s.repeat_interleave(64, 1)
    else:
        s = m.weight_scales.cpu().contiguous().view(m._scale_dtypes["weight_scales"]).float().reshape(N, K // 128)
        want = 0.5 * s.repeat_interleave(128, 1)
    assert torch.equal(step, want)

    # alpha > 0: y(I) - y0(I) = (alpha * noise * step)^T up to the bf16 rounding of the perturbed weight, which a
    # large alpha makes negligible against the perturbation (a step is a fraction of the weight's own bf16 ulp)
    alpha = 64.0
    eye = torch.eye(K, dtype=torch.bfloat16, device=hip_device)
    with torch.no_grad():
        m.lora_B.zero_()
        m.aqn_alpha = 0.0
        base = m(eye).float()
        m.aqn_alpha = alpha
        pert = (m(eye).float() - base).t().cpu()             # [N, K] perturbation of w
        pert2 = (m(eye).float() - base).t().cpu()            # a fresh draw every forward
    z = pert / (alpha * step)
    assert abs(float(z.mean())) < 0.02 and abs(float(z.std()) - 1.0) < 0.05, (float(z.mean()), float(z.std()))
    assert not torch.equal(pert, pert2)
    # gradients flow to the factors and to x through the noisy weight
    m.aqn_alpha = 1.0
    with torch.no_grad():
        m.lora_B.copy_(gen((N, r), 0.02, 93).to(hip_device))
    xg = x.clone().requires_grad_(True)
    m(xg).sum().backward()
    assert xg.grad is not None and m.lora_A.grad is not None and float(m.lora_B.grad.abs().max()) > 0


def test_weight_descriptor_checks_scale_storage(hip_device):
    """The kernels index scales by shape alone, so the descriptor refuses a scale buffer whose size or element type
    does not match what it says, and an nvfp4 weight without a proper fp32 global scale."""
    from xorl_amd import _C

    N, K = 256, 512
    packed8 = torch.zeros(N, K, dtype=torch.uint8, device=hip_device)
    packed4 = torch.zeros(N, K // 2, dtype=torch.uint8, device=hip_device)
    ok = _C.make_weight("block_fp8", _C.XQ_LAYOUT_FLAT, packed8, torch.ones(2, 4, device=hip_device), torch.float32, N, K, 128)
    assert ok.rows == N
    with pytest.raises(_C.XqError, match="scale buffer"):
        _C.make_weight("block_fp8", _C.XQ_LAYOUT_FLAT, packed8, torch.ones(2, 3, device=hip_device), torch.float32, N, K, 128)
    with pytest.raises(_C.XqError, match="scale buffer"):       # bf16 storage announced as fp32
        _C.make_weight("int4", _C.XQ_LAYOUT_FLAT, packed4, torch.ones(N, K // 128, dtype=torch.bfloat16, device=hip_device),
                       torch.float32, N, K, 128)
    e4 = torch.zeros(N * K // 16, dtype=torch.uint8, device=hip_device)
    with pytest.raises(_C.XqError, match="global_scale"):
        _C.make_weight("nvfp4", _C.XQ_LAYOUT_FLAT, packed4, e4, torch.float8_e4m3fn, N, K, 16,
                       global_scale=torch.ones(1, dtype=torch.bfloat16, device=hip_device))
    with pytest.raises(_C.XqError, match="global_scale"):
        _C.make_weight("nvfp4", _C.XQ_LAYOUT_GKN, torch.zeros(4, K // 2, N, dtype=torch.uint8, device=hip_device),
                       torch.zeros(4, K // 16, N, dtype=torch.uint8, device=hip_device), torch.float8_e4m3fn, K, N, 16,
                       global_scale=torch.ones(3, device=hip_device), num_experts=4)


def test_activation_rows_that_span_4gib(hip_device):
    """The block-fp8 kernel for large tiles addresses a lane's activation row by a 32-bit byte offset from a base all lanes
    share; a launch whose rows span 4 GiB or more (here: a column slice of a [2304, 932072] bf16 matrix) must take the kernel
    with 64-bit lane addresses instead.  Same forward as on the contiguous copy to rounding (another summation order),
    and equal to the oracle."""
    from xorl_amd.functional import qlora_linear

    M, K, N, r = 2304, 512, 4096, 16
    ld = ((1 << 32) // (2 * M) + 8) // 8 * 8
    assert M * ld * 2 >= 1 << 32
    m, w_ref = make_dense_module("block_fp8", N, K, r, 2 * r, seed=77, device=hip_device)
    x = gen((M, K), 1.0, 78, torch.bfloat16)
    parent = torch.zeros(M, ld, dtype=torch.bfloat16, device=hip_device)
    parent[:, :K] = x.to(hip_device)
    view = parent[:, :K]
    assert view.stride(0) == ld and (view[-1].data_ptr() - view.data_ptr()) >= (1 << 32) - 2 * ld
    with torch.no_grad():
        y_view = qlora_linear(view, m._quant_weight(), m.lora_A, m.lora_B, r, m.scaling)
        y_copy = qlora_linear(view.contiguous(), m._quant_weight(), m.lora_A, m.lora_B, r, m.scaling)
    torch.cuda.synchronize()
    del parent, view
    ex = R.linear_fwd_bwd_exact(x, w_ref, m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), m.scaling)
    close(y_view.cpu(), ex["y"], TOL)
    close(y_copy.cpu(), ex["y"], TOL)
    assert R.max_rel_err(y_view.cpu().float(), y_copy.cpu().float()) <= 2 ** -7
