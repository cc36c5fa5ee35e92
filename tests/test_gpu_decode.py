"""GPU parity: xq_decode (through the C ABI) vs the CPU oracle, bit for bit."""

import numpy as np
import pytest
import torch

from oracle import cdecode as C
from oracle import decode_np as NP

pytestmark = pytest.mark.gpu


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _codes(rng, shape):
    return rng.integers(0, 256, shape, dtype=np.uint8)


@pytest.mark.parametrize("rows,cols,group,sdt", [
    (64, 256, 128, "f32"), (64, 256, 128, "bf16"), (8, 96, 32, "f32"), (5, 30, 6, "f32"),
    (4096, 4096, 128, "bf16"),
])
def test_int4_flat(hip_device, rows, cols, group, sdt):
    from xorl_amd import quantize as Q

    rng = np.random.default_rng(rows + cols)
    packed = _codes(rng, (rows, cols // 2))
    scales = rng.normal(0, 0.02, (rows, cols // group)).astype(np.float32)
    st = torch.from_numpy(scales)
    if sdt == "bf16":
        st = st.to(torch.bfloat16)
        scales = st.float().numpy()
    got = Q.int4_dequantize(torch.from_numpy(packed).to(hip_device), st.to(hip_device), rows, cols, group)
    ref = NP.int4_decode_flat(packed, scales, rows, cols, group)
    assert np.array_equal(_bits(got), ref)
    if rows * cols <= 1 << 16:
        assert np.array_equal(ref, C.int4_decode_flat(packed, scales, rows, cols, group))


@pytest.mark.parametrize("K,N,group", [(256, 64, 128), (64, 48, 32), (6, 5, 2), (2048, 768, 128)])
def test_int4_gkn(hip_device, K, N, group):
    from xorl_amd import quantize as Q

    rng = np.random.default_rng(K + N)
    packed = _codes(rng, (K // 2, N))
    scales = rng.normal(0, 0.02, (K // group, N)).astype(np.float32)
    got = Q.int4_dequantize_gkn(torch.from_numpy(packed).to(hip_device), torch.from_numpy(scales).to(hip_device), K, N, group)
    assert np.array_equal(_bits(got), NP.int4_decode_gkn(packed, scales, K, N, group))


@pytest.mark.parametrize("rows,cols,group,sdt", [
    (64, 256, 64, "f32"), (64, 256, 64, "bf16"), (8, 96, 32, "f32"), (5, 30, 6, "f32"), (4096, 4096, 64, "f32"),
])
def test_nf4_flat(hip_device, rows, cols, group, sdt):
    from xorl_amd import quantize as Q

    rng = np.random.default_rng(rows + cols + 1)
    packed = _codes(rng, (rows, cols // 2))
    scales = np.abs(rng.normal(0, 0.05, (rows, cols // group))).astype(np.float32)
    st = torch.from_numpy(scales)
    if sdt == "bf16":
        st = st.to(torch.bfloat16)
        scales = st.float().numpy()
    got = Q.nf4_dequantize(torch.from_numpy(packed).to(hip_device), st.to(hip_device), rows * cols, group)
    ref = NP.nf4_decode_flat(packed, scales, rows, cols, group)
    assert np.array_equal(_bits(got).reshape(rows, cols), ref)
    if rows * cols <= 1 << 16:
        assert np.array_equal(ref, C.nf4_decode_flat(packed, scales, rows, cols, group))


@pytest.mark.parametrize("K,N,group", [(256, 64, 64), (64, 48, 32), (6, 5, 2), (2048, 768, 64)])
def test_nf4_gkn(hip_device, K, N, group):
    from xorl_amd import quantize as Q

    rng = np.random.default_rng(K + N + 1)
    packed = _codes(rng, (K // 2, N))
    scales = np.abs(rng.normal(0, 0.05, (K // group, N))).astype(np.float32)
    got = Q.nf4_dequantize_gkn(torch.from_numpy(packed).to(hip_device), torch.from_numpy(scales).to(hip_device), K, N, group)
    assert np.array_equal(_bits(got), NP.nf4_decode_gkn(packed, scales, K, N, group))


def test_quantizers_on_device_match_oracle(hip_device):
    """The package's torch quantizers run on the GPU (bank loading, re-quantisation, format conversion do that) emit
    the oracle's bytes: every quotient in them is a tensor-by-tensor IEEE division, not the reciprocal
    multiplication torch substitutes for Python-scalar operands."""
    from xorl_amd import quantize as Q

    g = torch.Generator().manual_seed(9)
    w = torch.randn(256, 512, generator=g) * 0.02
    wd = w.to(hip_device)
    p, s = Q.nf4_quantize(wd, 64)
    pc, sc = C.nf4_quantize_flat(w.numpy(), 64)
    assert np.array_equal(p.cpu().numpy(), pc.reshape(-1)) and np.array_equal(s.cpu().numpy(), sc.reshape(-1))
    p, s = Q.int4_quantize(wd, 128)
    pc, sc = C.int4_quantize_flat(w.numpy(), 128)
    assert np.array_equal(p.cpu().numpy(), pc) and np.array_equal(s.cpu().numpy(), sc)
    p, s = Q.int4_quantize_sym(wd, 128)
    pc, sc = C.int4_quantize_sym_flat(w.numpy(), 128)
    assert np.array_equal(p.cpu().numpy(), pc)
    assert np.array_equal(s.cpu().view(torch.int16).numpy().view(np.uint16), sc)
    p, bs, gs = Q.nvfp4_quantize(wd)
    pc, bsc, gc = C.nvfp4_quantize_flat(w.numpy())
    assert np.array_equal(p.cpu().numpy().reshape(pc.shape), pc)
    assert np.array_equal(bs.cpu().view(torch.uint8).numpy().reshape(bsc.shape), bsc) and gs.item() == gc
    p, bs, gs = Q.nvfp4_quantize_gkn(wd.t().contiguous())
    pc, bsc, gc = C.nvfp4_quantize_gkn(w.t().contiguous().numpy())
    assert np.array_equal(p.cpu().numpy(), pc) and np.array_equal(bs.cpu().view(torch.uint8).numpy(), bsc) and gs.item() == gc
    for shape in ((256, 512), (200, 300)):
        x = w[: shape[0], : shape[1]].contiguous()
        y, s = Q.block_fp8_quantize_gkn(x.to(hip_device))
        yc, sc = C.fp8_quantize(x.numpy())
        assert np.array_equal(y.cpu().view(torch.uint8).numpy(), yc) and np.array_equal(s.cpu().numpy(), sc)


@pytest.mark.parametrize("rows,cols,e4m3", [(64, 256, True), (64, 256, False), (3, 48, True), (8192, 5120, True)])
def test_nvfp4_flat(hip_device, rows, cols, e4m3):
    from xorl_amd import quantize as Q

    rng = np.random.default_rng(rows)
    packed = _codes(rng, (rows, cols // 2))
    packed[0, :8] = [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]          # every code
    g = np.float32(0.0042)
    if e4m3:
        sb = rng.integers(0, 0x7F, (rows, cols // 16), dtype=np.uint8)
        sb[0, :] = np.arange(cols // 16) % 0x7F                                 # subnormal + normal scale codes
        st = torch.from_numpy(sb).view(torch.float8_e4m3fn)
        sf = C.e4m3_scales_to_f32(sb)
    else:
        sf = rng.uniform(1e-3, 2.0, (rows, cols // 16)).astype(np.float32)
        st = torch.from_numpy(sf)
    got = Q.nvfp4_dequantize(torch.from_numpy(packed).to(hip_device), st.to(hip_device),
                             torch.tensor([g], device=hip_device), rows * cols)
    ref = NP.nvfp4_decode_flat(packed, sf, g, rows, cols)
    assert np.array_equal(_bits(got).reshape(rows, cols), ref)


@pytest.mark.parametrize("K,N", [(256, 64), (32, 40), (2048, 768)])
def test_nvfp4_gkn(hip_device, K, N):
    from xorl_amd import quantize as Q

    rng = np.random.default_rng(K)
    packed = _codes(rng, (K // 2, N))
    sb = rng.integers(0, 0x7F, (K // 16, N), dtype=np.uint8)
    g = np.float32(0.0117)
    got = Q.nvfp4_dequantize_gkn(torch.from_numpy(packed).to(hip_device),
                                 torch.from_numpy(sb).view(torch.float8_e4m3fn).to(hip_device),
                                 torch.tensor([g], device=hip_device), K, N)
    assert np.array_equal(_bits(got), NP.nvfp4_decode_gkn(packed, C.e4m3_scales_to_f32(sb), g, K, N))


@pytest.mark.parametrize("R,Cc", [(256, 384), (384, 256), (200, 576), (1, 130), (12288, 4096), (4096, 12288)])
def test_block_fp8(hip_device, R, Cc):
    from xorl_amd import quantize as Q

    rng = np.random.default_rng(R + Cc)
    wb = _codes(rng, (R, Cc))
    wb[(wb & 0x7F) == 0x7F] = 0x3C
    if R * Cc >= 256:
        wb.reshape(-1)[:256] = np.where((np.arange(256) & 0x7F) == 0x7F, 0x3C, np.arange(256))   # every byte code
    s = rng.uniform(1e-4, 2e-2, (-(-R // 128), -(-Cc // 128))).astype(np.float32)
    x = torch.from_numpy(wb).view(torch.float8_e4m3fn).to(hip_device)
    st = torch.from_numpy(s).to(hip_device)
    p_ref, b_ref = NP.fp8_decode(wb, s, R, Cc)
    got32 = Q.block_fp8_dequantize_gkn(x, st)
    assert got32.dtype == torch.float32
    assert np.array_equal(got32.cpu().numpy().view(np.uint32), p_ref.view(np.uint32))
    got16 = Q.block_fp8_dequantize_gkn(x, st, out_dtype=torch.bfloat16)
    assert np.array_equal(_bits(got16), b_ref)


def test_closed_form_fp8_fixture(hip_device):
    """tests/ops/test_block_fp8_frozen_dgrad.py:44-55 of the reference."""
    from xorl_amd import quantize as Q

    IN, OUT = 256, 384
    v = torch.arange(OUT * IN, dtype=torch.float32)
    w8 = (((v * 3 + 1) % 29) - 14).reshape(OUT, IN).div(16.0).to(torch.float8_e4m3fn)
    s = (torch.arange(6, dtype=torch.float32).reshape(3, 2) + 1.0) / 7.0
    got = Q.block_fp8_dequantize_gkn(w8.to(hip_device), s.to(hip_device))
    exact = ((((v * 3 + 1) % 29) - 14).reshape(OUT, IN) / 16.0) * s.repeat_interleave(128, 0).repeat_interleave(128, 1)
    assert torch.equal(got.cpu(), exact)


def test_errors_and_empty(hip_device):
    from xorl_amd import _C, quantize as Q

    with pytest.raises(ValueError):
        Q.int4_dequantize(torch.zeros(4, 8, dtype=torch.uint8, device=hip_device),
                          torch.zeros(4, 3, device=hip_device), 4, 16, 5)          # 16 % 5 != 0
    with pytest.raises(RuntimeError):
        Q.int4_dequantize(torch.zeros(4, 8, dtype=torch.uint8), torch.zeros(4, 1), 4, 16, 16)   # CPU tensors
    out = Q.block_fp8_dequantize_gkn(torch.empty(0, 128, dtype=torch.float8_e4m3fn, device=hip_device),
                                     torch.empty(0, 1, device=hip_device))
    assert out.shape == (0, 128)
