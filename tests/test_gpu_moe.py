"""GPU parity: routing kernels (bit-exact vs the oracle's stable sort) and the grouped
routed QLoRA expert MLP (forward + backward) vs the float64 per-expert oracle program."""

import numpy as np
import pytest
import torch

from oracle import cdecode as C
from oracle import decode_np as NP
from oracle import recipe as R
from tests.util_cases import close, bits_to_bf16, gen

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _zipf_routing(T, E, topk, seed, empty=1):
    """Seeded logits: Zipf(1.1) popularity over a permutation of experts, the last `empty` never chosen."""
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(E, generator=g)
    pmf = 1.0 / torch.arange(1, E + 1, dtype=torch.float64) ** 1.1
    logits = torch.log(pmf / pmf.sum())[perm.argsort()].float()
    gumbel = -torch.log(-torch.log(torch.rand(T, E, generator=g).clamp_min(1e-9)))
    z = logits[None, :] + gumbel
    if empty:
        z[:, perm[-empty:]] = -1e9
    rw, sel = torch.topk(torch.softmax(z, -1), topk, dim=-1)
    rw = rw / rw.sum(-1, keepdim=True)
    return rw, sel.int()


@pytest.mark.parametrize("T,E,topk", [(64, 8, 2), (1000, 128, 8), (5, 4, 1), (16384, 128, 8)])
def test_route_scatter_gather_exact(hip_device, T, E, topk):
    from xorl_amd import moe_functional as MF

    rw, sel = _zipf_routing(T, E, topk, seed=T)
    splits, sidx_ref = R.route_build(sel, E)
    counts, offsets, sidx, tile_offsets = MF.route_build(sel.to(hip_device), E)
    assert torch.equal(counts.cpu().long(), splits)
    assert torch.equal(sidx.cpu().view(T, topk), sidx_ref)
    assert torch.equal(offsets.cpu().long(), torch.cat([torch.zeros(1, dtype=torch.long), splits.cumsum(0)]))
    tiles = (splits + 127) // 128
    assert torch.equal(tile_offsets.cpu().long()[: E + 1], torch.cat([torch.zeros(1, dtype=torch.long), tiles.cumsum(0)]))
    tiles2 = (counts.cpu().long() + 255) // 256
    assert torch.equal(tile_offsets.cpu().long()[E + 1 :], torch.cat([torch.zeros(1, dtype=torch.long), tiles2.cumsum(0)]))
    assert (splits == 0).any() or E <= 4
    # scatter then gather: out[t] = sum_j x[t] = topk * x[t] (exact in bf16 for power-of-two topk)
    x = gen((T, 64), 1.0, 3, torch.bfloat16).to(hip_device)
    xs = MF.moe_scatter(x, sidx, topk)
    ref = torch.empty(T * topk, 64, dtype=torch.bfloat16)
    ref[sidx_ref.flatten().long()] = x.cpu().repeat_interleave(topk, 0)
    assert torch.equal(xs.cpu(), ref)
    back = MF.moe_gather(xs, None, sidx, T, topk)
    assert torch.equal(back.cpu(), (x.cpu().float() * topk).to(torch.bfloat16))


def _make_experts(fmt, E, H, I, r, hybrid, seed, device):
    from xorl_amd.qlora import BlockFP8QLoRAMoeExperts, NF4QLoRAMoeExperts, NvFP4QLoRAMoeExperts

    cls = {"block_fp8": BlockFP8QLoRAMoeExperts, "nvfp4": NvFP4QLoRAMoeExperts, "nf4": NF4QLoRAMoeExperts}[fmt]
    m = cls(E, E, I, H, r=r, lora_alpha=2 * r, hybrid_shared=hybrid)
    m.load_weights(gen((E, H, I), 0.05, seed), gen((E, H, I), 0.05, seed + 1), gen((E, I, H), 0.05, seed + 2))
    with torch.no_grad():
        for i, name in enumerate(("gate_proj", "up_proj", "down_proj")):
            A, B = getattr(m, f"{name}_lora_A"), getattr(m, f"{name}_lora_B")
            A.copy_(gen(tuple(A.shape), 0.05, seed + 10 + i))
            B.copy_(gen(tuple(B.shape), 0.05, seed + 20 + i))
    # oracle decode of the banks (CPU)
    banks = {}
    for p in ("gate", "up", "down"):
        K, N = m._proj_dims(p)
        packed = getattr(m, f"{p}_packed").numpy()
        per = []
        for e in range(E):
            if fmt == "block_fp8":
                s = getattr(m, f"{p}_block_scales")[e].contiguous().view(torch.float32).numpy()
                per.append(bits_to_bf16(NP.fp8_decode(packed[e].reshape(K, N), s, K, N)[1]))
            elif fmt == "nf4":
                s = getattr(m, f"{p}_scales")[e].contiguous().view(torch.float32).numpy()
                per.append(bits_to_bf16(NP.nf4_decode_gkn(packed[e], s, K, N, 64)))
            else:
                sb = getattr(m, f"{p}_block_scales")[e].numpy()
                g = getattr(m, f"{p}_global_scale")[e].contiguous().view(torch.float32).item()
                per.append(bits_to_bf16(NP.nvfp4_decode_gkn(packed[e], C.e4m3_scales_to_f32(sb), g, K, N)))
        banks[p] = torch.stack(per)
    return m.to(device), banks


@pytest.mark.parametrize("tile_policy", [0, 1, 2], indirect=True)
@pytest.mark.parametrize("fmt", ["block_fp8", "nvfp4", "nf4"])
@pytest.mark.parametrize("E,T,H,I,r,topk,hybrid", [(6, 300, 128, 192, 8, 2, True), (16, 700, 256, 128, 16, 4, False),
                                                   # intermediate sizes of whole 256-column tiles: block-fp8 banks run gate
                                                   # and up as one forward launch and their dgrads as one sum
                                                   (4, 900, 256, 512, 16, 2, False), (5, 600, 128, 768, 24, 3, True)])
def test_moe_fwd_bwd_vs_oracle(hip_device, tile_policy, fmt, E, T, H, I, r, topk, hybrid):
    m, banks = _make_experts(fmt, E, H, I, r, hybrid, seed=E + T, device=hip_device)
    # the module's own bank decode is bit-exact with the oracle
    for p in ("gate", "up", "down"):
        K, N = m._proj_dims(p)
        assert torch.equal(m.dequantize_all_experts(p, K, N).to(torch.bfloat16).cpu(), banks[p]), p
    rw, sel = _zipf_routing(T, E, topk, seed=7)
    rw = rw.to(torch.bfloat16)
    x = gen((T, H), 1.0, 8, torch.bfloat16)
    dy = gen((T, H), 1.0, 9, torch.bfloat16)
    xd = x.to(hip_device).requires_grad_(True)
    rwd = rw.to(hip_device).requires_grad_(True)
    y = m(xd, rwd, sel.to(hip_device))
    y.backward(dy.to(hip_device))
    lora = {k: (getattr(m, f"{k}_proj_lora_A").detach().cpu(), getattr(m, f"{k}_proj_lora_B").detach().cpu())
            for k in ("gate", "up", "down")}
    ex = R.moe_fwd_bwd(x, rw, sel, banks["gate"], banks["up"], banks["down"], lora, m.scaling, dy)
    close(y.cpu(), ex["y"], TOL)
    close(xd.grad.cpu(), ex["dx"], TOL)
    # routing-weight grads pass through bf16 intermediates (ops/moe/lora.py:855-861): 2e-2
    close(rwd.grad.cpu(), ex["d_routing"], 2e-2, rows="none")
    for k in ("gate", "up", "down"):
        gA, gB = getattr(m, f"{k}_proj_lora_A").grad.cpu(), getattr(m, f"{k}_proj_lora_B").grad.cpu()
        assert gA.shape == lora[k][0].shape and gB.shape == lora[k][1].shape
        close(gA, ex[f"dA_{k}"], TOL, rows="first")
        close(gB, ex[f"dB_{k}"], TOL, rows="first")
    # experts without rows: exact-zero factor gradients (structural zeros)
    empty = (torch.bincount(sel.flatten().long(), minlength=E) == 0).nonzero().flatten()
    assert empty.numel() >= 1
    for k in ("gate", "up", "down"):
        for t in (getattr(m, f"{k}_proj_lora_A").grad, getattr(m, f"{k}_proj_lora_B").grad):
            if t.shape[0] == E:
                assert torch.count_nonzero(t[empty.to(t.device)]) == 0


@pytest.mark.parametrize("E,T,H,I,r,topk,hybrid", [(6, 300, 128, 192, 8, 2, True), (4, 900, 256, 512, 16, 2, False)])
def test_moe_swiglu_limit_vs_oracle(hip_device, E, T, H, I, r, topk, hybrid):
    """The gate-only SwiGLU clamp (ops/moe/triton.py:127-141, ops/moe/lora.py:638,863,917-919): the gate pre-activation
    clamped to [-limit, limit] before the SiLU, its gradient zero outside.  The mask is a discontinuity, so the data are
    built to make it the same on both sides: inputs in {-1, 0, 1}, gate weights multiples of 1/8 with every 128 x 128 block
    reaching 1.75 (block scale 2^-8: the e4m3 codes hold them exactly), a zero gate B factor -- the gate pre-activations are
    then exact multiples of 1/8 in the kernels and in the float64 program alike, and the limit sits between two of them."""
    from xorl_amd.qlora import BlockFP8QLoRAMoeExperts

    limit = 4.0625
    g = torch.Generator().manual_seed(E * 1000 + T)
    ints = lambda *shape, lo, hi: torch.randint(lo, hi + 1, shape, generator=g).float()
    wg = ints(E, H, I, lo=-14, hi=14) / 8.0
    wg[:, ::128, ::128] = 1.75                      # every scale block holds the value that makes its scale 2^-8
    m = BlockFP8QLoRAMoeExperts(E, E, I, H, r=r, lora_alpha=2 * r, hybrid_shared=hybrid)
    m.load_weights(wg, gen((E, H, I), 0.05, 5), gen((E, I, H), 0.05, 6))
    m.swiglu_limit = limit
    with torch.no_grad():
        for i, name in enumerate(("gate_proj", "up_proj", "down_proj")):
            A, B = getattr(m, f"{name}_lora_A"), getattr(m, f"{name}_lora_B")
            A.copy_(gen(tuple(A.shape), 0.05, 30 + i))
            B.copy_(gen(tuple(B.shape), 0.05, 40 + i) if name != "gate_proj" else torch.zeros_like(B))
    m = m.to(hip_device)
    banks = {p: m.dequantize_all_experts(p, *m._proj_dims(p)).to(torch.bfloat16).cpu() for p in ("gate", "up", "down")}
    assert torch.equal(banks["gate"].float(), wg)                    # the gate bank came through the codes exactly
    rw, sel = _zipf_routing(T, E, topk, seed=7)
    rw = rw.to(torch.bfloat16)
    x = ints(T, H, lo=-1, hi=1).to(torch.bfloat16)
    dy = gen((T, H), 1.0, 9, torch.bfloat16)
    # the construction does what it is for: a good share of the gate values on each side of the limit, none on it
    gates = torch.cat([x.double()[(sel == e).any(1)] @ wg[e].double() for e in range(E)])
    share = (gates.abs() > limit).double().mean().item()
    assert 0.05 < share < 0.95 and (gates.abs() - limit).abs().min() >= 0.0625
    lora = {k: (getattr(m, f"{k}_proj_lora_A").detach().cpu(), getattr(m, f"{k}_proj_lora_B").detach().cpu())
            for k in ("gate", "up", "down")}
    got = {}
    for lim in (limit, 0.0):
        m.swiglu_limit = lim
        for p in m.parameters():
            p.grad = None
        xd = x.to(hip_device).requires_grad_(True)
        rwd = rw.to(hip_device).requires_grad_(True)
        y = m(xd, rwd, sel.to(hip_device))
        y.backward(dy.to(hip_device))
        got[lim] = y.detach().cpu()
        ex = R.moe_fwd_bwd(x, rw, sel, banks["gate"], banks["up"], banks["down"], lora, m.scaling, dy, swiglu_limit=lim)
        close(y.cpu(), ex["y"], TOL)
        close(xd.grad.cpu(), ex["dx"], TOL)
        close(rwd.grad.cpu(), ex["d_routing"], 2e-2, rows="none")
        for k in ("gate", "up", "down"):
            gA, gB = getattr(m, f"{k}_proj_lora_A").grad.cpu(), getattr(m, f"{k}_proj_lora_B").grad.cpu()
            close(gA, ex[f"dA_{k}"], TOL, rows="first")
            close(gB, ex[f"dB_{k}"], TOL, rows="first")
    assert not torch.equal(got[limit], got[0.0])                     # the clamp changes the result


def test_moe_zero_lora_equals_base(hip_device):
    m, banks = _make_experts("block_fp8", 8, 128, 128, 8, True, seed=40, device=hip_device)
    rw, sel = _zipf_routing(200, 8, 2, seed=41)
    x = gen((200, 128), 1.0, 42, torch.bfloat16)
    with torch.no_grad():
        for k in ("gate", "up", "down"):
            getattr(m, f"{k}_proj_lora_B").zero_()
        y = m(x.to(hip_device), rw.to(torch.bfloat16).to(hip_device), sel.to(hip_device))
    zero = {k: (getattr(m, f"{k}_proj_lora_A").detach().cpu(), getattr(m, f"{k}_proj_lora_B").detach().cpu())
            for k in ("gate", "up", "down")}
    ex = R.moe_fwd_bwd(x, rw.to(torch.bfloat16), sel, banks["gate"], banks["up"], banks["down"], zero, m.scaling)
    close(y.cpu(), ex["y"], TOL)


def test_prequantized_checkpoint_load_on_device_matches_direct_quantisation(hip_device):
    """HF-layout block-fp8 experts ([out, in] bytes + [out/128, in/128] scales) loaded through `_load_experts` on
    the GPU give the same banks as quantizing the transposed weights directly, and the module then runs."""
    from xorl_amd import quantize as Q
    from xorl_amd.qlora import BlockFP8QLoRAMoeExperts

    E, H, I, r = 4, 256, 384, 8
    hf = {(e, p): gen((H, I) if p == "down_proj" else (I, H), 0.05, 900 + 7 * e + i)
          for e in range(E) for i, p in enumerate(("gate_proj", "up_proj", "down_proj"))}
    data = {}
    for (e, p), w in hf.items():
        b, s = Q.block_fp8_quantize_gkn(w.float().contiguous(), 128)      # per-128x128-block rule: layout agnostic
        data[f"experts.{e}.{p}.weight"] = b
        data[f"experts.{e}.{p}.weight_scale_inv"] = s
    m = BlockFP8QLoRAMoeExperts(E, E, I, H, r=r, lora_alpha=2 * r).to(hip_device)
    m._source_fqn = "experts"
    m._load_experts(lambda k: data[k], {})
    d = BlockFP8QLoRAMoeExperts(E, E, I, H, r=r, lora_alpha=2 * r)
    d.load_weights(torch.stack([hf[(e, "gate_proj")].t() for e in range(E)]),
                   torch.stack([hf[(e, "up_proj")].t() for e in range(E)]),
                   torch.stack([hf[(e, "down_proj")].t() for e in range(E)]))
    for p in ("gate", "up", "down"):
        assert getattr(m, f"{p}_packed").device.type == "cuda"
        assert torch.equal(getattr(m, f"{p}_packed").cpu(), getattr(d, f"{p}_packed")), p
        assert torch.equal(getattr(m, f"{p}_block_scales").cpu(), getattr(d, f"{p}_block_scales")), p
    rw, sel = _zipf_routing(64, E, 2, seed=3, empty=0)
    x = gen((64, H), 1.0, 4, torch.bfloat16).to(hip_device)
    with torch.no_grad():
        y = m(x, rw.to(torch.bfloat16).to(hip_device), sel.to(hip_device))
        y2 = d.to(hip_device)(x, rw.to(torch.bfloat16).to(hip_device), sel.to(hip_device))
    assert torch.equal(y, y2)


@pytest.mark.parametrize("src,dst", [("block_fp8", "nvfp4"), ("nvfp4", "block_fp8")])
def test_inline_buffer_converts_between_checkpoint_and_module_format(hip_device, src, dst):
    """A checkpoint in one format streamed into modules of the other: the buffer decodes with the source format's
    kernel and re-quantizes; the pairs it hands back equal the CPU quantizer run on the oracle's decode."""
    from xorl_amd import quantize as Q
    from xorl_amd.qlora import BlockFP8QLoRALinear, NvFP4QLoRALinear
    from xorl_amd.qlora.inline_buffers import QLoRAWeightBuffer

    N, K = 256, 384
    w = gen((N, K), 0.05, 77)
    tensors = {}
    if src == "block_fp8":
        b, s = Q.block_fp8_quantize_gkn(w, 128)
        tensors = {"m.proj.weight": b, "m.proj.weight_scale_inv": s}
        deq = torch.from_numpy(NP.fp8_decode(b.view(torch.uint8).numpy(), s.numpy(), N, K)[0])     # fp32, as decoded
    else:
        codes, bs, g = Q.nvfp4_quantize(w, 16)
        tensors = {"m.proj.weight": codes.reshape(N, K // 2), "m.proj.weight_scale": bs.reshape(N, K // 16),
                   "m.proj.weight_scale_2": g.reshape(())}
        folded = (bs.reshape(N, K // 16).float() * g.float()).numpy()           # what the buffer folds before decoding
        deq = bits_to_bf16(NP.nvfp4_decode_flat(codes.reshape(N, K // 2).numpy(), folded, 1.0, N, K))

    class Holder(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.proj = (NvFP4QLoRALinear if dst == "nvfp4" else BlockFP8QLoRALinear)(K, N, r=4, lora_alpha=4)
            self.proj._is_prequantized, self.proj._source_fqn, self.proj._source_quant_format = True, "m.proj", src

    model = Holder()
    buf = QLoRAWeightBuffer(model)
    assert buf.source_format == src
    pairs = None
    for k, t in tensors.items():
        pairs = buf.try_consume(k, t)
    got = dict(pairs)
    if dst == "nvfp4":
        codes, bs, g = Q.nvfp4_quantize(deq, 16, global_amax=deq.float().abs().max().reshape(1))
        assert torch.equal(got["proj.packed_weight_f32"].contiguous().view(torch.uint8).flatten(), codes.flatten())
        assert torch.equal(got["proj.weight_block_scales"].contiguous().view(torch.float32).flatten(), bs.float().flatten())
        assert torch.equal(got["proj.weight_global_scale"].contiguous().view(torch.float32), g.float().reshape(-1))
    else:
        b, s = Q.block_fp8_quantize_gkn(deq.float(), 128)
        assert torch.equal(got["proj.packed_weight_f32"].contiguous().view(torch.uint8).flatten(), b.view(torch.uint8).flatten())
        assert torch.equal(got["proj.weight_block_scales"].contiguous().view(torch.float32).flatten(), s.flatten())
    assert got["proj.packed_weight_f32"].shape == model.proj.packed_weight_f32.shape


@pytest.mark.parametrize("tile_policy", [1, 2, 3], indirect=True)
@pytest.mark.parametrize("fmt", ["block_fp8", "nvfp4", "nf4"])
def test_grouped_gemm_decode_bit_exact(hip_device, tile_policy, fmt):
    """Every expert gets the rows of an identity matrix, so the grouped forward product (contraction along the
    bank's rows) returns the expert's decoded [K, N] matrix and the dgrad product (contraction along its columns)
    returns the transpose: the in-kernel decode of each grouped kernel, in both directions, must equal the oracle's
    bank decode bit for bit (up to the sign of zero)."""
    from xorl_amd import moe_functional as MF

    E, H, I = 3, 256, 384
    m, banks = _make_experts(fmt, E, H, I, 8, False, seed=60, device=hip_device)
    for proj, (K, N) in (("gate", (H, I)), ("down", (I, H))):
        qw = m._bank(proj)
        ref = banks[proj].to(hip_device)                                   # [E, K, N] bf16
        for transpose_w, rows in ((False, K), (True, N)):
            sel = torch.arange(E, dtype=torch.int32).repeat_interleave(rows).reshape(-1, 1).to(hip_device)
            counts, offsets, sidx, tile_offsets = MF.route_build(sel, E)
            assert torch.equal(sidx.cpu().flatten(), torch.arange(E * rows, dtype=torch.int32))   # already in expert order
            a = torch.eye(rows, dtype=torch.bfloat16, device=hip_device).repeat(E, 1)
            y = MF._grouped_gemm(qw, transpose_w, a, offsets, tile_offsets, None, None)
            want = (ref.transpose(1, 2) if transpose_w else ref).reshape(E * rows, -1).contiguous()
            same = y.view(torch.int16) == want.view(torch.int16)
            both_zero = (y.float() == 0) & (want.float() == 0)
            assert bool((same | both_zero).all()), (proj, transpose_w)


@pytest.mark.parametrize("tile_policy", [1, 2, 3], indirect=True)
@pytest.mark.parametrize("scale_dtype,group", [(torch.float32, 128), (torch.bfloat16, 32), (torch.float32, 16)])
def test_grouped_gemm_int4_gkn_bank_bit_exact(hip_device, tile_policy, scale_dtype, group):
    """int4 banks have no module of their own; through the C ABI they take the same grouped kernels (and, with bf16
    scales, the one scale storage the modules do not produce).  Identity rows again: both products must return the
    oracle's bank decode bit for bit."""
    from xorl_amd import _C, moe_functional as MF
    from xorl_amd import quantize as Q
    from xorl_amd.functional import QuantWeight

    E, K, N = 3, 256, 320
    packed, scales, ref = [], [], []
    for e in range(E):
        p, s = Q.int4_quantize_gkn(gen((K, N), 0.05, 80 + e), group)
        s = s.to(scale_dtype)
        packed.append(p)
        scales.append(s)
        ref.append(bits_to_bf16(NP.int4_decode_gkn(p.numpy(), s.float().numpy(), K, N, group)))
    qw = QuantWeight("int4", _C.XQ_LAYOUT_GKN, torch.stack(packed).to(hip_device), torch.stack(scales).to(hip_device),
                     scale_dtype, K, N, group, num_experts=E)
    ref = torch.stack(ref).to(hip_device)
    for transpose_w, rows in ((False, K), (True, N)):
        sel = torch.arange(E, dtype=torch.int32).repeat_interleave(rows).reshape(-1, 1).to(hip_device)
        counts, offsets, sidx, tile_offsets = MF.route_build(sel, E)
        a = torch.eye(rows, dtype=torch.bfloat16, device=hip_device).repeat(E, 1)
        y = MF._grouped_gemm(qw, transpose_w, a, offsets, tile_offsets, None, None)
        want = (ref.transpose(1, 2) if transpose_w else ref).reshape(E * rows, -1).contiguous()
        same = y.view(torch.int16) == want.view(torch.int16)
        both_zero = (y.float() == 0) & (want.float() == 0)
        assert bool((same | both_zero).all()), transpose_w


def test_nvfp4_bank_with_folded_fp32_scales_matches_e4m3_storage(hip_device):
    """A modelopt checkpoint loads as fp32 block scales with the global scale folded in (stored global = 1); the
    same codes with e4m3 block scales and a separate global decode to the same values, so both storages must give
    identical outputs and gradients through the grouped kernels."""
    E, H, I, r = 4, 256, 384, 8
    m1, _ = _make_experts("nvfp4", E, H, I, r, False, seed=90, device=hip_device)
    m2, _ = _make_experts("nvfp4", E, H, I, r, False, seed=90, device=hip_device)
    for p in ("gate", "up", "down"):
        bs = getattr(m1, f"{p}_block_scales").view(torch.float8_e4m3fn).float()             # [E, K/16, N]
        g = getattr(m1, f"{p}_global_scale").contiguous().view(torch.float32).reshape(E, 1, 1)
        setattr(m2, f"{p}_block_scales", m2._to_uint8((bs * g).contiguous()))
        setattr(m2, f"{p}_global_scale", m2._to_uint8(torch.ones(E, 1, dtype=torch.float32, device=hip_device)))
        m2._scale_dtypes[p] = {"weight_block_scales": torch.float32, "weight_global_scale": torch.float32}
    rw, sel = _zipf_routing(500, E, 2, seed=5, empty=0)
    x = gen((500, H), 1.0, 6, torch.bfloat16).to(hip_device)
    dy = gen((500, H), 1.0, 7, torch.bfloat16).to(hip_device)
    outs = []
    for m in (m1, m2):
        xd = x.clone().requires_grad_(True)
        y = m(xd, rw.to(torch.bfloat16).to(hip_device), sel.to(hip_device))
        y.backward(dy)
        outs.append((y.detach(), xd.grad, m.gate_proj_lora_A.grad.clone(), m.down_proj_lora_B.grad.clone()))
    for a, b in zip(*outs):
        assert torch.equal(a, b)


def test_empty_batches(hip_device):
    """No tokens at all: the dense module and the expert module return empty outputs, and a backward pass leaves
    exact-zero factor gradients (the reference's zero-size guards, ops/moe/lora.py:566-570)."""
    m, _ = _make_experts("block_fp8", 4, 128, 128, 8, True, seed=70, device=hip_device)
    x = torch.zeros(0, 128, dtype=torch.bfloat16, device=hip_device, requires_grad=True)
    rw = torch.zeros(0, 2, dtype=torch.bfloat16, device=hip_device)
    sel = torch.zeros(0, 2, dtype=torch.int32, device=hip_device)
    y = m(x, rw, sel)
    assert y.shape == (0, 128)
    y.sum().backward()
    for k in ("gate", "up", "down"):
        for f in ("A", "B"):
            g = getattr(m, f"{k}_proj_lora_{f}").grad
            assert g is not None and torch.count_nonzero(g) == 0
    from tests.util_cases import make_dense_module

    d, _ = make_dense_module("nvfp4", 128, 256, 8, 16, seed=71, device=hip_device)
    xd = torch.zeros(0, 256, dtype=torch.bfloat16, device=hip_device, requires_grad=True)
    yd = d(xd)
    assert yd.shape == (0, 128)
    yd.sum().backward()
    assert torch.count_nonzero(d.lora_A.grad) == 0 and torch.count_nonzero(d.lora_B.grad) == 0


def test_moe_seeded_shape_sweep(hip_device):
    """Nine seeded draws of (format, E, T, H, I, r, top-k, shared / per-expert factors): forward and every
    gradient against the float64 per-expert program."""
    rng = np.random.default_rng(11)
    fmts = ["block_fp8", "nvfp4", "nf4"]
    for case in range(9):
        fmt = fmts[case % 3]
        E = int(rng.integers(2, 21))
        T = int(rng.integers(1, 500))
        H = int(rng.integers(1, 5)) * 128 if fmt == "block_fp8" else int(rng.integers(1, 7)) * 64
        I = int(rng.integers(1, 5)) * 128 if fmt == "block_fp8" else int(rng.integers(1, 7)) * 64
        r = int(rng.integers(1, 65))
        topk = int(rng.integers(1, min(E, 8) + 1))
        hybrid = bool(rng.integers(0, 2))
        m, banks = _make_experts(fmt, E, H, I, r, hybrid, seed=200 + case, device=hip_device)
        rw, sel = _zipf_routing(T, E, topk, seed=300 + case, empty=1 if E > topk else 0)
        rw = rw.to(torch.bfloat16)
        x = gen((T, H), 1.0, 400 + case, torch.bfloat16)
        dy = gen((T, H), 1.0, 500 + case, torch.bfloat16)
        xd = x.to(hip_device).requires_grad_(True)
        rwd = rw.to(hip_device).requires_grad_(True)
        y = m(xd, rwd, sel.to(hip_device))
        y.backward(dy.to(hip_device))
        lora = {k: (getattr(m, f"{k}_proj_lora_A").detach().cpu(), getattr(m, f"{k}_proj_lora_B").detach().cpu())
                for k in ("gate", "up", "down")}
        ex = R.moe_fwd_bwd(x, rw, sel, banks["gate"], banks["up"], banks["down"], lora, m.scaling, dy)
        tag = (case, fmt, E, T, H, I, r, topk, hybrid)
        close(y.cpu(), ex["y"], TOL)
        close(xd.grad.cpu(), ex["dx"], TOL)
        close(rwd.grad.cpu(), ex["d_routing"], 2e-2, rows="none")
        # factor gradients pass through bf16 intermediates in the reference too (ops/moe/lora.py:557-564): where
        # the float64 distance exceeds the tolerance, it must not exceed what the reference's own rounding points
        # (the oracle's bf16 mode) leave
        rec = None
        for k in ("gate", "up", "down"):
            for f in ("A", "B"):
                err = R.max_rel_err(getattr(m, f"{k}_proj_lora_{f}").grad.cpu(), ex[f"d{f}_{k}"])
                if err > TOL:
                    if rec is None:
                        rec = R.moe_fwd_bwd(x, rw, sel, banks["gate"], banks["up"], banks["down"], lora, m.scaling, dy,
                                            dtype=torch.bfloat16)
                    assert err <= 1.5 * R.max_rel_err(rec[f"d{f}_{k}"].float(), ex[f"d{f}_{k}"]), tag + (k, f, err)


@pytest.mark.parametrize("fmt,hybrid", [("block_fp8", False), ("nvfp4", True)])
def test_dispatched_rows_compute_and_single_expert_calls(hip_device, fmt, hybrid):
    """The compute step of an expert-parallel forward (rows already grouped by expert + inclusive cumsum, no routing
    weight) and the per-expert call of the eager implementation, against the float64 per-expert program."""
    from xorl_amd.moe_functional import EP_EXPERT_COMPUTE_QLORA_PACKED

    E, H, I, r = 6, 128, 192, 8
    m, banks = _make_experts(fmt, E, H, I, r, hybrid, seed=61, device=hip_device)
    counts = torch.tensor([37, 0, 130, 1, 0, 64])
    R_ = int(counts.sum())
    cumsum = counts.cumsum(0)
    expert = torch.repeat_interleave(torch.arange(E), counts).int()
    x = gen((R_, H), 1.0, 62, torch.bfloat16)
    dy = gen((R_, H), 1.0, 63, torch.bfloat16)
    lora = {k: (getattr(m, f"{k}_proj_lora_A").detach().cpu(), getattr(m, f"{k}_proj_lora_B").detach().cpu())
            for k in ("gate", "up", "down")}
    ex = R.moe_fwd_bwd(x, torch.ones(R_, 1), expert.unsqueeze(1), banks["gate"], banks["up"], banks["down"], lora,
                       m.scaling, dy)

    xd = x.to(hip_device).requires_grad_(True)
    y = m.compute_dispatched(xd, cumsum.to(hip_device))
    y.backward(dy.to(hip_device))
    assert y.shape == (R_, H)
    close(y.cpu(), ex["y"], TOL)
    close(xd.grad.cpu(), ex["dx"], TOL)
    for k in ("gate", "up", "down"):
        close(getattr(m, f"{k}_proj_lora_A").grad.cpu(), ex[f"dA_{k}"], TOL, rows="first")
        close(getattr(m, f"{k}_proj_lora_B").grad.cpu(), ex[f"dB_{k}"], TOL, rows="first")
    # the registry callable is the same program; scores multiply afterwards
    gA, gB = m._active_lora_views("gate_proj")
    uA, uB = m._active_lora_views("up_proj")
    dA, dB = m._active_lora_views("down_proj")
    with torch.no_grad():
        y2 = EP_EXPERT_COMPUTE_QLORA_PACKED["hip"](x.to(hip_device), cumsum.to(hip_device), m._bank("gate"), m._bank("up"),
                                                   m._bank("down"), gA, gB, uA, uB, dA, dB, m._active_scaling())
        assert torch.equal(y2, y.detach())
        scores = torch.rand(R_, device=hip_device)
        y3 = m.compute_dispatched(x.to(hip_device), cumsum.to(hip_device), expert_scores=scores)
        assert torch.equal(y3, y.detach() * scores.unsqueeze(1).to(torch.bfloat16))
        # one expert at a time: the same rows give the same values as inside the grouped call
        lo = int(cumsum[1])
        y_e2 = m(x[lo:lo + 130].to(hip_device), expert_idx=2)
        close(y_e2.cpu(), ex["y"][lo:lo + 130], TOL)
        assert torch.count_nonzero(m(x[:4].to(hip_device), expert_idx=E + 3)) == 0       # lives on another rank
        # a rank that received no rows
        empty = m.compute_dispatched(x[:0].to(hip_device), torch.zeros(E, dtype=torch.int64, device=hip_device))
        assert empty.shape == (0, H)
    with pytest.raises(ValueError):
        m.compute_dispatched(x.to(hip_device), (cumsum - 1).clamp_min(0).to(hip_device))   # cumsum must end at the row count
    m.moe_implementation = "eager"
    with pytest.raises(ValueError, match="expert_idx"):
        m(x.to(hip_device), torch.ones(R_, 1, device=hip_device), expert.unsqueeze(1).to(hip_device))


@pytest.mark.parametrize("hybrid", [True, False])
def test_out_of_range_expert_ids_drop_their_copies(hip_device, hybrid):
    """Expert ids outside [0, E) (the reference asserts on them on the device, group_gemm/kernel/moe.py) must not
    turn into row numbers: such a routed copy is not counted, gets scatter_index -1 and is skipped by every row
    mover, so the result is that of the same routing with the copy's weight set to zero -- forward, dX, the
    routing-weight gradients (zero for the dropped copies) and all six factor gradients, shared or per expert.
    Every kernel exits normally."""
    from xorl_amd.moe_functional import route_build

    E, T, H, I, r, topk = 8, 300, 128, 128, 8, 2
    m, banks = _make_experts("block_fp8", E, H, I, r, hybrid, seed=70, device=hip_device)
    rw, sel = _zipf_routing(T, E, topk, seed=71)
    rw = rw.to(torch.bfloat16)
    bad = sel.clone()
    g = torch.Generator().manual_seed(72)
    drop = torch.rand(T, topk, generator=g) < 0.15
    bad[drop] = torch.where(torch.rand(int(drop.sum()), generator=g) < 0.5, torch.tensor(E + 3), torch.tensor(-2)).int()
    n_bad = int(drop.sum())
    assert 20 < n_bad < T

    counts, offsets, sidx, _ = route_build(bad.to(hip_device), E)
    assert int(offsets[E]) == T * topk - n_bad and int(counts.sum()) == T * topk - n_bad
    sidx = sidx.cpu().view(T, topk)
    assert bool((sidx[drop] == -1).all()) and bool((sidx[~drop] >= 0).all())
    # the valid copies keep the positions of the stable sort over the valid entries alone
    _, want = R.route_build(sel[~drop].unsqueeze(1), E)
    assert torch.equal(sidx[~drop], want.flatten())

    x = gen((T, H), 1.0, 73, torch.bfloat16)
    dy = gen((T, H), 1.0, 74, torch.bfloat16)
    xd = x.to(hip_device).requires_grad_(True)
    rwd = rw.to(hip_device).requires_grad_(True)
    y = m(xd, rwd, bad.to(hip_device))
    y.backward(dy.to(hip_device))
    torch.cuda.synchronize()
    lora = {k: (getattr(m, f"{k}_proj_lora_A").detach().cpu(), getattr(m, f"{k}_proj_lora_B").detach().cpu())
            for k in ("gate", "up", "down")}
    rw0 = rw.clone()
    rw0[drop] = 0                                   # the same routing with the dropped copies weighted zero
    ex = R.moe_fwd_bwd(x, rw0, sel, banks["gate"], banks["up"], banks["down"], lora, m.scaling, dy)
    close(y.cpu(), ex["y"], TOL)
    close(xd.grad.cpu(), ex["dx"], TOL)
    drw = rwd.grad.cpu()
    assert torch.count_nonzero(drw[drop]) == 0
    close(drw[~drop], ex["d_routing"][~drop], 2e-2, rows="none")
    rec = None
    for k in ("gate", "up", "down"):
        for f in ("A", "B"):
            got = getattr(m, f"{k}_proj_lora_{f}").grad.cpu()
            assert bool(torch.isfinite(got).all())
            err = R.max_rel_err(got, ex[f"d{f}_{k}"])
            if err > TOL:        # bf16 intermediates, as in the reference: not beyond what its own rounding points leave
                if rec is None:
                    rec = R.moe_fwd_bwd(x, rw0, sel, banks["gate"], banks["up"], banks["down"], lora, m.scaling, dy,
                                        dtype=torch.bfloat16)
                assert err <= 1.5 * R.max_rel_err(rec[f"d{f}_{k}"].float(), ex[f"d{f}_{k}"]), (k, f, err)


def test_routed_call_needs_all_experts_local(hip_device):
    """The routed program's tile schedules are laid out for the bank's expert count: a module cannot be built with
    fewer local experts than experts, and the function refuses a routing over another count than the banks hold."""
    from xorl_amd.moe_functional import moe_experts_qlora_forward
    from xorl_amd.qlora import BlockFP8QLoRAMoeExperts

    with pytest.raises(ValueError):
        BlockFP8QLoRAMoeExperts(4, 8, 128, 128, r=8, lora_alpha=16)
    m, _ = _make_experts("block_fp8", 4, 128, 128, 8, True, seed=5, device=hip_device)
    x = torch.zeros(4, 128, dtype=torch.bfloat16, device=hip_device)
    f = [getattr(m, f"{k}_proj_lora_{ab}").detach() for k in ("gate", "up", "down") for ab in ("A", "B")]
    with pytest.raises(ValueError, match="bank holds"):
        moe_experts_qlora_forward(8, torch.ones(4, 1, device=hip_device),
                                  torch.zeros(4, 1, dtype=torch.int32, device=hip_device), x, m._bank("gate"),
                                  m._bank("up"), m._bank("down"), *f, scaling=1.0)


@pytest.mark.parametrize("fmt,hybrid", [("block_fp8", True), ("nvfp4", False), ("nvfp4", True), ("nf4", True)])
def test_expert_merge_weights_matches_reference_arithmetic(hip_device, fmt, hybrid):
    """QLoRAMoeExperts.merge_weights (moe_experts.py:987-1008, :1134-1146, :1249-1261): the merged bank is
    deq(W) + delta.to(deq dtype) -- a bf16 add for nvfp4 / nf4 (their decoders return bf16), an fp32 add for
    block_fp8 --, nvfp4 blends each expert's fresh amax into the running one (lerp by ema_decay) and re-quantises
    against it.  The module's new packed bytes, scales, global scales and running amax must equal, byte for byte,
    the oracle's quantizer applied to that sum built from the oracle's decode; merging twice exercises the blend.
    block_fp8 banks go through the dense fused merge pass expert by expert, which forms the update itself: there the
    quantizer is checked bit for bit on the pass's own fp32 sums and to neighbouring codes on the oracle's."""
    from xorl_amd import _C
    from xorl_amd import functional as Fn

    E, H, I, r = 4, 128, 256, 8
    m, banks = _make_experts(fmt, E, H, I, r, hybrid, seed=80, device=hip_device)
    dt = torch.float32 if fmt == "block_fp8" else torch.bfloat16

    def oracle_decode(p):
        """The bank as the reference's dequantize_all_experts returns it (fp32 for block_fp8, else bf16)."""
        K, N = m._proj_dims(p)
        packed = getattr(m, f"{p}_packed").cpu().numpy()
        out = []
        for e in range(E):
            if fmt == "block_fp8":
                s = getattr(m, f"{p}_block_scales")[e].cpu().contiguous().view(torch.float32).numpy()
                out.append(torch.from_numpy(NP.fp8_decode(packed[e].reshape(K, N), s, K, N)[0]))
            elif fmt == "nf4":
                s = getattr(m, f"{p}_scales")[e].cpu().contiguous().view(torch.float32).numpy()
                out.append(bits_to_bf16(NP.nf4_decode_gkn(packed[e], s, K, N, 64)))
            else:
                sd = m._scale_dtypes[p]["weight_block_scales"]
                sb = getattr(m, f"{p}_block_scales")[e].cpu().contiguous()
                sc = C.e4m3_scales_to_f32(sb.numpy()) if sd == torch.float8_e4m3fn else sb.view(torch.float32).numpy()
                g = getattr(m, f"{p}_global_scale")[e].cpu().contiguous().view(torch.float32).item()
                out.append(bits_to_bf16(NP.nvfp4_decode_gkn(packed[e], sc, g, K, N)))
        return torch.stack(out)

    for round_ in range(2):
        with torch.no_grad():
            for i, name in enumerate(("gate_proj", "up_proj", "down_proj")):
                A, B = getattr(m, f"{name}_lora_A"), getattr(m, f"{name}_lora_B")
                A.copy_(gen(tuple(A.shape), 0.2, 300 + 10 * round_ + i).to(hip_device))
                B.copy_(gen(tuple(B.shape), 0.2, 400 + 10 * round_ + i).to(hip_device))
        want = {}
        for p in ("gate", "up", "down"):
            K, N = m._proj_dims(p)
            w = oracle_decode(p)
            assert w.dtype == dt and torch.equal(m.dequantize_all_experts(p, K, N).cpu(), w)
            delta = m._compute_proj_delta(f"{p}_proj").detach().cpu()  # fp32 [E, K, N], the module's own torch product
            merged = w + delta.to(w.dtype)
            assert float((merged.float() - w.float()).abs().max()) > 0
            ema = None
            if fmt == "nvfp4":
                fresh = merged.float().abs().amax(dim=(1, 2))
                prev = m._ema_amax[p]
                ema = fresh if prev is None else prev.detach().cpu().clone().lerp_(fresh, 0.1)
            per = []
            for e in range(E):
                x = merged[e].float().numpy()
                if fmt == "block_fp8":
                    # the fused pass forms the update itself (split-bf16 MFMA products, fp32 sums): its own fp32 sums, read
                    # through the publish mode of the same kernel, are within 3e-5 of the oracle's (the update dominates the sum
                    # here, and a split-bf16 product drops the lo x lo terms: 2^-16 relative), and the bank must hold
                    # the oracle quantizer applied to them bit for bit
                    qw = Fn.QuantWeight("block_fp8", _C.XQ_LAYOUT_FLAT, getattr(m, f"{p}_packed")[e],
                                        getattr(m, f"{p}_block_scales")[e], torch.float32, K, N, 128)
                    A, B = m._active_lora_views(f"{p}_proj")
                    own = Fn.merge_dense(qw, B[e if B.shape[0] > 1 else 0], A[e if A.shape[0] > 1 else 0], m.active_r,
                                         m._active_scaling(), torch.float32).cpu()
                    assert R.max_rel_err(own, merged[e]) <= 3e-5, (round_, p, e)
                    per.append(C.fp8_quantize(own.numpy(), 128, 1.0) + C.fp8_quantize(x, 128, 1.0))
                elif fmt == "nf4":
                    per.append(C.nf4_quantize_gkn(x, 64))
                else:
                    per.append(C.nvfp4_quantize_gkn(x, 16, global_amax=float(ema[e])))
            want[p] = (per, ema)
        m.merge_weights(ema_decay=0.1, experts_per_step=3)
        for name in ("gate_proj", "up_proj", "down_proj"):
            assert torch.count_nonzero(getattr(m, f"{name}_lora_B")) == 0
        for p in ("gate", "up", "down"):
            per, ema = want[p]
            K, N = m._proj_dims(p)
            got_packed = getattr(m, f"{p}_packed").cpu().numpy()
            for e in range(E):
                assert np.array_equal(got_packed[e].ravel(), per[e][0].ravel()), (round_, p, e, "codes")
                if fmt == "block_fp8":
                    s = getattr(m, f"{p}_block_scales")[e].cpu().contiguous().view(torch.float32).numpy()
                    assert np.array_equal(s.view(np.uint32).ravel(), per[e][1].view(np.uint32).ravel()), (round_, p, e)
                    # against the oracle's own sums: scales to 5e-5, codes equal or neighbours (a sum on a rounding edge)
                    assert np.allclose(s.ravel(), per[e][3].ravel(), rtol=5e-5, atol=0)
                    gb, wb = got_packed[e].ravel().astype(np.int32), per[e][2].ravel().astype(np.int32)
                    assert float((gb != wb).mean()) <= 5e-3
                    sg, sw = np.where(gb & 0x80, -(gb & 0x7f), gb & 0x7f), np.where(wb & 0x80, -(wb & 0x7f), wb & 0x7f)
                    assert bool(((np.abs(sg - sw) <= 1) | ((np.abs(sg) <= 1) & (np.abs(sw) <= 1))).all())
                elif fmt == "nf4":
                    s = getattr(m, f"{p}_scales")[e].cpu().contiguous().view(torch.float32).numpy()
                    assert np.array_equal(s.view(np.uint32).ravel(), per[e][1].view(np.uint32).ravel()), (round_, p, e)
                else:
                    assert m._scale_dtypes[p]["weight_block_scales"] == torch.float8_e4m3fn
                    sb = getattr(m, f"{p}_block_scales")[e].cpu().numpy()
                    assert np.array_equal(sb.ravel(), per[e][1].ravel()), (round_, p, e, "block scales")
                    g = getattr(m, f"{p}_global_scale")[e].cpu().contiguous().view(torch.float32).numpy()
                    assert g.view(np.uint32).item() == np.float32(per[e][2]).view(np.uint32).item(), (round_, p, e)
            if fmt == "nvfp4":
                assert torch.equal(m._ema_amax[p].cpu(), ema), (round_, p)


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
def test_expert_module_and_swiglu_under_torch_compile(hip_device, backend):
    """Traced by torch.compile, the expert module and SwiGLU reach the library through registered custom ops
    (xq::moe_fwd / moe_bwd, xq::silu_mul_fwd / silu_mul_bwd) with fake-tensor shape functions: outputs and every
    gradient equal the eager call bit for bit, and the ops pass torch's schema and fake-tensor checks."""
    from torch.library import opcheck

    from xorl_amd import functional as Fn
    from xorl_amd import moe_functional as MF

    E, T, H, I, r, topk = 6, 200, 128, 192, 8, 2
    m, _ = _make_experts("block_fp8", E, H, I, r, True, seed=90, device=hip_device)
    rw, sel = _zipf_routing(T, E, topk, seed=91)
    rw, sel = rw.to(torch.bfloat16).to(hip_device), sel.to(hip_device)
    x = gen((T, H), 1.0, 92, torch.bfloat16).to(hip_device)
    dy = gen((T, H), 1.0, 93, torch.bfloat16).to(hip_device)
    names = [f"{k}_proj_lora_{f}" for k in ("gate", "up", "down") for f in ("A", "B")]

    def run(mod):
        for n in names:
            getattr(m, n).grad = None
        xd, rwd = x.clone().requires_grad_(True), rw.clone().requires_grad_(True)
        y = mod(xd, rwd, sel)
        y.backward(dy)
        return [y.detach().clone(), xd.grad.clone(), rwd.grad.clone()] + [getattr(m, n).grad.clone() for n in names]

    ref = run(m)
    torch._dynamo.reset()
    got = run(torch.compile(m, backend=backend, fullgraph=True))
    for a, b in zip(ref, got):
        assert torch.equal(a, b)

    # SwiGLU
    g = gen((T, I), 2.0, 94).to(torch.bfloat16).to(hip_device)
    u = gen((T, I), 1.0, 95, torch.bfloat16).to(hip_device)
    dh = gen((T, I), 1.0, 96, torch.bfloat16).to(hip_device)

    def run_silu(fn):
        gd, ud = g.clone().requires_grad_(True), u.clone().requires_grad_(True)
        h = fn(gd, ud)
        h.backward(dh)
        return h.detach(), gd.grad, ud.grad

    ref = run_silu(Fn.silu_and_mul)
    torch._dynamo.reset()
    got = run_silu(torch.compile(Fn.silu_and_mul, backend=backend, fullgraph=True))
    for a, b in zip(ref, got):
        assert torch.equal(a, b)

    if backend == "eager":
        ok = {"SUCCESS"}
        assert set(opcheck(Fn._silu_fwd_op, (g, u), test_utils=("test_schema", "test_faketensor")).values()) == ok
        assert set(opcheck(Fn._silu_bwd_op, (g, u, dh), test_utils=("test_schema", "test_faketensor")).values()) == ok
        qg, qu, qd = m._bank("gate"), m._bank("up"), m._bank("down")
        f = [getattr(m, n).detach().contiguous() for n in names]
        args = (x, rw, sel, *f, qg.packed, qg.scales, qg.global_scale, qu.packed, qu.scales, qu.global_scale, qd.packed,
                qd.scales, qd.global_scale, qg.fmt, qg.layout, Fn._DT_TO_CODE[qg.scale_dtype], qg.group, E, H, I, r, 2.0)
        assert set(opcheck(MF._moe_fwd_op, args, test_utils=("test_schema", "test_faketensor")).values()) == ok


def test_grouped_low_rank_entry_points(hip_device):
    """xq_factor_prep, xq_grouped_lora_down and xq_grouped_lora_wgrad one at a time against plain torch arithmetic
    on the same bf16 operands (fp32 accumulation; the products are small enough for float64 to be the yardstick)."""
    from xorl_amd import moe_functional as MF

    E, K, r, rp, width = 5, 256, 12, 16, 192
    counts = torch.tensor([70, 0, 300, 1, 129])
    R_ = int(counts.sum())
    sel = torch.arange(E, dtype=torch.int32).repeat_interleave(counts).reshape(-1, 1).to(hip_device)
    _, offsets, _, tile_offsets = MF.route_build(sel, E)
    F32 = gen((E, K, r), 0.1, 1)                                            # a per-expert A factor [E, in, r]
    F = MF._prep(F32.to(hip_device), True, rp, K)                           # -> bf16 [E, rp, K], zero padded
    want = torch.zeros(E, rp, K)
    want[:, :r] = F32.transpose(1, 2).to(torch.bfloat16).float()
    assert torch.equal(F.float().cpu(), want)
    a = gen((R_, K), 1.0, 2, torch.bfloat16)
    t = MF._lora_down(a.to(hip_device), F, offsets, tile_offsets, E, 0.5).cpu()        # [R, rp] = bf16(0.5 * a . F[e]^T)
    ends = counts.cumsum(0)
    e_of = torch.searchsorted(ends, torch.arange(R_), right=True)
    ref_t = 0.5 * torch.einsum("rk,rjk->rj", a.double(), want.double()[e_of])
    close(t, ref_t, 1e-2, rows="none")
    assert torch.count_nonzero(t[:, r:]) == 0
    P = gen((R_, width), 1.0, 3, torch.bfloat16)
    g = MF._wgrad(P.to(hip_device), t.to(hip_device), r, offsets, E, False).cpu()       # [E, width, r]
    for e in range(E):
        lo, hi = int(ends[e] - counts[e]), int(ends[e])
        ref = P[lo:hi].double().t() @ t[lo:hi, :r].double()
        if hi == lo:
            assert torch.count_nonzero(g[e]) == 0
        else:
            close(g[e], ref, 1e-2, rows="none")
    g1 = MF._wgrad(P.to(hip_device), t.to(hip_device), r, None, E, True).cpu()          # one product over all rows, [1, r, width]
    close(g1[0], t[:, :r].double().t() @ P.double(), 1e-2, rows="none")


@pytest.mark.parametrize("fmt,hybrid", [("block_fp8", True), ("block_fp8", False), ("nvfp4", True), ("nf4", False)])
def test_routed_rows_read_in_place_equal_the_copy(hip_device, fmt, hybrid):
    """Where the banks run on the pipelined tile kernel the forward keeps no expert-ordered copy of the routed rows (and the
    backward none of the routed gradient rows): the launches read the token matrices through the routing.  Same values in
    the same order: outputs and every gradient are the bits of the form that writes the copies."""
    import xorl_amd.moe_functional as MF

    E, T, H, I, r, topk = 12, 1500, 256, 512, 16, 4
    m, _ = _make_experts(fmt, E, H, I, r, hybrid, seed=31, device=hip_device)
    rw, sel = _zipf_routing(T, E, topk, seed=3)
    x = gen((T, H), 1.0, 4, torch.bfloat16).to(hip_device)
    dy = gen((T, H), 1.0, 5, torch.bfloat16).to(hip_device)
    res = []
    try:
        for in_place in (True, False):
            MF.READ_ROUTED_ROWS_IN_PLACE = in_place
            xd = x.clone().requires_grad_(True)
            rwd = rw.to(hip_device).requires_grad_(True)
            for p in m.parameters():
                p.grad = None
            y = m(xd, rwd, sel.to(hip_device))
            saved_xs = y.grad_fn.saved_tensors[0] if hasattr(y.grad_fn, "saved_tensors") else None
            y.backward(dy)
            grads = [getattr(m, f"{k}_proj_lora_{ab}").grad.clone() for k in ("gate", "up", "down") for ab in "AB"]
            res.append((y.detach(), xd.grad, rwd.grad, grads, saved_xs))
    finally:
        MF.READ_ROUTED_ROWS_IN_PLACE = True
    (y0, dx0, drw0, g0, xs0), (y1, dx1, drw1, g1, xs1) = res
    assert torch.equal(y0, y1) and torch.equal(dx0, dx1) and torch.equal(drw0, drw1)
    for a, b in zip(g0, g1):
        assert torch.equal(a, b)
