"""GPU parity: merging the LoRA update into the quantized base weight (through the C ABI)
vs the CPU oracle.

publish  : bf16(bf16(deq) + bf16(delta)) -- the reference's weight-sync arithmetic.  Expected bit-exact
           except where the fp32 value of delta lies within the kernel's product error (2^-16 relative per
           factor) of a bf16 rounding boundary; the test allows one bf16 step at operand magnitude on at
           most 1e-3 of the elements.
requant  : block_fp8 decode -> add -> re-encode.  With the LoRA update switched off the kernel must
           reproduce the oracle quantizer byte for byte on the decoded weight (the e4m3 encoder, the
           division and the block absmax are then the only arithmetic); with a large update on, the kernel's fp32
           sums are within 1e-5 of the oracle's (the reference's own fp32 product has no pinned summation order), the
           oracle quantizer applied to THOSE sums gives the kernel's scales and bytes bit for bit, and against the
           oracle's own sums the scales match to 5e-5 relative and bytes differ by at most one code on at most 5e-3
           of the elements.
"""

import numpy as np
import pytest
import torch

from oracle import cdecode as C
from oracle import recipe as R
from tests.util_cases import gen, make_dense_module

pytestmark = pytest.mark.gpu


def _deq_f32(m, w_ref_bf16):
    """fp32 decode of a block_fp8 module from the oracle (fl(e4m3 * scale)); bf16 decode for the others."""
    if m.quant_format != "block_fp8":
        return w_ref_bf16.float()
    N, K = m.out_features, m.in_features
    packed = m.packed_weight_f32.detach().cpu().contiguous().view(torch.uint8).numpy().reshape(N, K)
    s = m.weight_block_scales.cpu().contiguous().view(torch.float32).numpy()
    from oracle import decode_np as NP

    return torch.from_numpy(NP.fp8_decode(packed, s, N, K)[0].copy())


@pytest.mark.parametrize("fmt", ["block_fp8", "int4", "nvfp4", "nf4"])
@pytest.mark.parametrize("N,K,r", [(384, 256, 16), (200, 320, 24), (1024, 512, 64), (128, 128, 0)])
def test_merge_publish_bf16(hip_device, fmt, N, K, r):
    if fmt != "block_fp8" and N % 16:
        N = 208
    if fmt == "int4" and K % 128:
        K = 384
    m, w_ref = make_dense_module(fmt, N, K, max(r, 8), 32, seed=N + K, device=hip_device)
    if r == 0:
        with torch.no_grad():
            m.lora_B.zero_()
    else:
        m.set_runtime_lora_config(r, 2 * r) if r != m.r else None
    got = m.merged_weight(torch.bfloat16).cpu()
    A, B = m.lora_A.detach().cpu()[: m.active_r], m.lora_B.detach().cpu()[:, : m.active_r]
    want = R.merge_publish_recipe(_deq_f32(m, w_ref), A, B, m._active_scaling())
    assert got.shape == (N, K) and got.dtype == torch.bfloat16
    mism = got.view(torch.int16) != want.view(torch.int16)
    assert float(mism.float().mean()) <= 1e-3
    # where they differ it is by one bf16 step of the update (its own rounding may flip) plus one of the result
    a = _deq_f32(m, w_ref).to(torch.bfloat16).float().abs()
    # the low-rank product carries ~2^-16 relative error per TERM, i.e. relative to sum_j |B||A|, not to a
    # sum that cancels
    terms = (B.abs().double() @ A.abs().double()).float() * abs(m._active_scaling())
    delta_bf16 = R.merge_delta_exact(A, B, m._active_scaling()).to(torch.bfloat16).float().abs()
    tol = 2.0 ** -7 * (torch.maximum(a, want.float().abs()) + delta_bf16) + 2.0 ** -14 * terms
    assert bool(((got.float() - want.float()).abs() <= tol).all())
    if r == 0:
        assert not bool(mism.any())           # no update: the decoded weight itself


@pytest.mark.parametrize("N,K", [(384, 256), (200, 320), (1024, 1024)])
def test_requant_identity_matches_oracle_quantizer(hip_device, N, K):
    """LoRA off: requant(deq(W)) must equal the oracle quantizer applied to the oracle decode, byte for byte."""
    from xorl_amd.functional import merge_requant_fp8

    m, w_ref = make_dense_module("block_fp8", N, K, 8, 16, seed=3 * N + K, device=hip_device)
    deq = _deq_f32(m, w_ref).numpy()
    want_b, want_s = C.fp8_quantize(deq, 128, 1.0)
    packed, scales = merge_requant_fp8(m._quant_weight(), None, None, 0, 1.0)
    got_b, want_b = packed.cpu().numpy(), want_b.reshape(N, K)
    # a decoded -0 plus the (+0) update is +0, as in the reference's `w + delta`: byte 0x00 where the
    # quantizer alone would keep 0x80
    neg_zero = (want_b == 0x80) & (deq == 0)
    assert np.array_equal(np.where(neg_zero, 0, want_b), got_b)
    assert np.array_equal(scales.cpu().numpy().view(np.uint32).ravel(), want_s.view(np.uint32).ravel())


@pytest.mark.parametrize("N,K,r", [(384, 256, 16), (200, 320, 32), (1024, 512, 64)])
def test_merge_requant_fp8(hip_device, N, K, r):
    from xorl_amd.functional import merge_dense, merge_requant_fp8

    m, w_ref = make_dense_module("block_fp8", N, K, r, 4 * r, seed=N - K, device=hip_device)
    with torch.no_grad():                      # a visible update: |delta| comparable to the e4m3 step
        m.lora_A.mul_(8.0)
        m.lora_B.mul_(8.0)
    A, B, s = m.lora_A.detach().cpu(), m.lora_B.detach().cpu(), m._active_scaling()
    merged = R.merge_fp32_recipe(_deq_f32(m, w_ref), A, B, s)
    # fp32 sum from the kernel: within the product error of the oracle's
    got32 = merge_dense(m._quant_weight(), m.lora_A, m.lora_B, r, s, torch.float32).cpu()
    assert R.max_rel_err(got32, merged) <= 1e-5
    want_b, want_s = C.fp8_quantize(merged.numpy(), 128, 1.0)
    packed, scales = merge_requant_fp8(m._quant_weight(), m.lora_A, m.lora_B, r, s)
    sc = scales.cpu().numpy()
    assert np.allclose(sc, want_s.reshape(sc.shape), rtol=5e-5, atol=0)
    gb, wb = packed.cpu().numpy().astype(np.int32), want_b.reshape(N, K).astype(np.int32)
    assert float((gb != wb).mean()) <= 5e-3
    sg, sw = np.where(gb & 0x80, -(gb & 0x7f), gb & 0x7f), np.where(wb & 0x80, -(wb & 0x7f), wb & 0x7f)
    assert bool(((np.abs(sg - sw) <= 1) | ((np.abs(sg) <= 1) & (np.abs(sw) <= 1))).all())   # neighbouring codes only
    # the quantiser itself, with the update on, is exact: the oracle quantizer applied to the kernel's own fp32 sums (which
    # are within 1e-5 of the oracle's, above) gives the kernel's scales and bytes bit for bit
    own_b, own_s = C.fp8_quantize(got32.numpy(), 128, 1.0)
    assert np.array_equal(sc.view(np.uint32), own_s.reshape(sc.shape).astype(np.float32).view(np.uint32))
    assert np.array_equal(gb, own_b.reshape(N, K).astype(np.int32))
    # the module method: in place, LoRA reset, and the new weight decodes to ~merged (e4m3 step: 2^-4 relative)
    m.merge_weights()
    assert torch.count_nonzero(m.lora_B) == 0
    w_new = m._dequantize_weight().cpu().float()
    assert R.max_rel_err(w_new, merged) <= 2 ** -4


@pytest.mark.parametrize("N,K,r", [(384, 256, 0), (384, 256, 16), (200, 320, 32), (1024, 512, 64)])
def test_merge_requant_nvfp4(hip_device, N, K, r):
    """Fused nvfp4 merge + re-quantise: the tensor amax pass and the encode pass against the oracle's C quantizer
    applied to the merged values the publish kernel writes (same decode, same update), byte for byte: codes, e4m3
    block scales and the global scale; then the module method (running amax, scale convention, LoRA reset)."""
    from xorl_amd.functional import merge_amax, merge_dense, merge_requant_nvfp4

    m, w_ref = make_dense_module("nvfp4", N, K, max(r, 8), 4 * max(r, 8), seed=N + 3 * K, device=hip_device)
    with torch.no_grad():
        m.lora_A.mul_(8.0)
        m.lora_B.mul_(8.0)
        if r == 0:
            m.lora_B.zero_()                      # the module below then merges a zero update as well
    s = m._active_scaling()
    qw = m._quant_weight()
    merged = merge_dense(qw, m.lora_A, m.lora_B, r, s, torch.bfloat16).cpu()          # bf16(bf16(deq) + bf16(delta))
    if r == 0:
        assert torch.equal(merged, w_ref) or bool(((merged.float() == 0) & (w_ref.float() == 0))[merged != w_ref].all())
    fresh = merge_amax(qw, m.lora_A, m.lora_B, r, s)
    assert fresh.shape == (1,) and fresh.item() == merged.float().abs().max().item()
    gamax = torch.tensor([0.9 * m._ema_amax.item() + 0.1 * fresh.item()])
    codes, bscales, gscale = merge_requant_nvfp4(qw, m.lora_A, m.lora_B, r, s, gamax.to(hip_device))
    want_codes, want_bs, want_g = C.nvfp4_quantize_flat(merged.float().numpy(), 16, global_amax=gamax.item())
    assert np.array_equal(codes.cpu().numpy(), np.asarray(want_codes).reshape(-1))
    assert np.array_equal(bscales.cpu().view(torch.uint8).numpy(), np.asarray(want_bs).reshape(-1).view(np.uint8))
    assert np.float32(gscale.item()) == np.float32(np.asarray(want_g).reshape(-1)[0])
    # the module method
    ema0 = m._ema_amax.clone()
    # (decay 1: the running amax jumps to the fresh one -- with this test's exaggerated update a slowly moving
    # amax would leave the block scales saturated, which is the recipe's behaviour, not the kernel's)
    m.merge_weights(ema_decay=1.0)
    assert torch.count_nonzero(m.lora_B) == 0 and not torch.all(m.lora_A == 0)
    want_ema = torch.lerp(ema0.cpu(), fresh.cpu(), 1.0)
    assert abs(m._ema_amax.item() - want_ema.item()) <= 1e-6 * want_ema.item()
    assert torch.equal(m._read_packed_weight_uint8().reshape(-1).cpu(), codes.cpu())
    gs_new = m._recover_tensor(m.weight_global_scale, m._scale_dtypes["weight_global_scale"]).item()
    assert abs(gs_new - m._ema_amax.item() / (6.0 * 448.0)) / gs_new < 1e-6
    w_new = m._dequantize_weight().cpu().float()
    assert (w_new - merged.float()).abs().mean() / merged.float().abs().mean() < 0.15    # e2m1 round trip


@pytest.mark.parametrize("N,K,r", [(384, 256, 0), (200, 320, 16), (1024, 512, 64)])
def test_merge_requant_nf4(hip_device, N, K, r):
    """Fused NF4 merge + re-quantise against the oracle's C quantizer applied to the merged values the publish
    kernel writes: codes and fp32 group scales byte for byte; then the module method, in place."""
    from xorl_amd.functional import merge_dense, merge_requant_nf4

    m, w_ref = make_dense_module("nf4", N, K, max(r, 8), 4 * max(r, 8), seed=2 * N + K, device=hip_device)
    with torch.no_grad():
        m.lora_A.mul_(8.0)
        m.lora_B.mul_(8.0)
        if r == 0:
            m.lora_B.zero_()
    s = m._active_scaling()
    qw = m._quant_weight()
    merged = merge_dense(qw, m.lora_A, m.lora_B, r, s, torch.bfloat16).cpu()
    codes, scales = merge_requant_nf4(qw, m.lora_A, m.lora_B, r, s)
    want_codes, want_scales = C.nf4_quantize_flat(merged.float().numpy(), 64)
    assert np.array_equal(codes.cpu().numpy(), np.asarray(want_codes).reshape(-1))
    assert np.array_equal(scales.cpu().numpy().view(np.uint32), np.asarray(want_scales).reshape(-1).view(np.uint32))
    m.merge_weights()
    assert torch.count_nonzero(m.lora_B) == 0
    assert torch.equal(m._read_packed_weight_uint8().reshape(-1).cpu(), codes.cpu())
    w_new = m._dequantize_weight().cpu().float()
    assert (w_new - merged.float()).abs().mean() / merged.float().abs().mean() < 0.10


def test_merge_errors(hip_device):
    from xorl_amd import _C
    from xorl_amd.functional import merge_requant_fp8

    m, _ = make_dense_module("int4", 256, 256, 8, 16, seed=1, device=hip_device)
    with pytest.raises(ValueError):
        merge_requant_fp8(m._quant_weight(), m.lora_A, m.lora_B, 8, 2.0)      # block_fp8 only
    with pytest.raises(ValueError):
        m.merged_weight(torch.float16)


@pytest.mark.parametrize("symmetric", [True, False])
@pytest.mark.parametrize("N,K,r", [(384, 256, 0), (200, 384, 16), (1024, 512, 64)])
def test_merge_requant_int4(hip_device, N, K, r, symmetric):
    """Fused int4 merge + re-quantise (128-element groups) against the oracle's C quantizers applied to the merged
    values the publish kernel writes -- the reference codec's rule (ops/quantize/int4_quantize.py:12-41, fp32 scales)
    and the symmetric absmax/7 rule (bf16 scales): codes and scales byte for byte; then the module method."""
    from xorl_amd.functional import merge_dense, merge_requant_int4
    from xorl_amd.qlora import Int4QLoRALinear

    rr = max(r, 8)
    lin = torch.nn.Linear(K, N, bias=False)
    with torch.no_grad():
        lin.weight.copy_(gen((N, K), 0.02, 5 * N + K))
        lin.weight[3].zero_()                          # a group of zeros: scale 0 (symmetric) or the 1e-12 floor
    m = Int4QLoRALinear.from_module(lin, r=rr, lora_alpha=4 * rr, symmetric=symmetric).to(hip_device)
    with torch.no_grad():
        m.lora_A.copy_(gen((rr, K), 0.16, 5 * N + K + 1).to(hip_device))
        m.lora_B.copy_(gen((N, rr), 0.16, 5 * N + K + 2).to(hip_device))
        m.lora_B[3].zero_()
        if r == 0:
            m.lora_B.zero_()
    s = m._active_scaling()
    qw = m._quant_weight()
    merged = merge_dense(qw, m.lora_A, m.lora_B, r, s, torch.bfloat16).cpu()
    assert r == 0 or float((merged.float() - m._dequantize_weight().cpu().float()).abs().max()) > 0
    assert torch.count_nonzero(merged[3]) == 0
    codes, scales = merge_requant_int4(qw, m.lora_A, m.lora_B, r, s, symmetric)
    if symmetric:
        want_codes, want_scales = C.int4_quantize_sym_flat(merged.float().numpy(), 128)
        assert scales.dtype == torch.bfloat16
        got_scales = scales.cpu().view(torch.int16).numpy().view(np.uint16)
    else:
        want_codes, want_scales = C.int4_quantize_flat(merged.float().numpy(), 128)
        assert scales.dtype == torch.float32
        got_scales, want_scales = scales.cpu().numpy().view(np.uint32), np.asarray(want_scales).view(np.uint32)
    assert np.array_equal(got_scales.reshape(-1), np.asarray(want_scales).reshape(-1))
    assert np.array_equal(codes.cpu().numpy().reshape(-1), np.asarray(want_codes).reshape(-1))
    m.merge_weights()
    assert torch.count_nonzero(m.lora_B) == 0
    assert torch.equal(m._read_packed_weight_uint8().reshape(-1).cpu(), codes.cpu().reshape(-1))
    assert m._scale_dtypes["weight_scales"] == scales.dtype
    w_new = m._dequantize_weight().cpu().float()
    assert (w_new - merged.float()).abs().mean() / merged.float().abs().mean() < 0.16   # 15 or 16 levels per group: mean error ~ absmax / 28
