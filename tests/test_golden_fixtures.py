"""The committed fixtures under tests/golden/ (written by tests/golden/make_fixtures.py).

CPU: the C oracle and its numpy twin must reproduce the stored bit patterns (so neither can
drift unnoticed).  GPU: the HIP decode must reproduce them bit for bit through the C ABI, and
the closed-form block-fp8 case (inputs re-derived from the formulas of the reference's
tests/ops/test_block_fp8_frozen_dgrad.py:44-60) must give Y and dX within max rel err <= 1e-2.
"""

import os

import numpy as np
import pytest
import torch

from oracle import cdecode as C
from oracle import decode_np as NP
from oracle.recipe import max_rel_err

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = 1e-2   # max |got - ref| / max |ref|


def _load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _same_bits_nan_aware(got: np.ndarray, exp: np.ndarray) -> bool:
    """Bit equality, except that any NaN matches any NaN.  The two e4m3 NaN bytes (0x7f, 0xff)
    never come out of a quantizer; which NaN bit pattern a decode gives for them is a property
    of the converting instruction (torch's CPU cast gives 0x7ff00000, this oracle 0x7fc00000 with
    the byte's sign, gfx950's v_cvt_pk_f32_fp8 0xffc00000 for both) and nothing in the reference
    fixes it."""
    if got.dtype == np.uint32:
        gn, en = (got & 0x7FFFFFFF) > 0x7F800000, (exp & 0x7FFFFFFF) > 0x7F800000
    else:
        gn, en = (got & 0x7FFF) > 0x7F80, (exp & 0x7FFF) > 0x7F80
    return bool(np.array_equal(gn, en) and np.array_equal(got[~gn], exp[~en]))


# ------------------------------------------------------------------ CPU: oracle vs fixtures
def test_oracle_int4_fixture():
    f = _load("decode_int4.npz")
    R, Cc = f["packed"].shape[0], f["packed"].shape[1] * 2
    for g in (32, 128):
        for impl in (C, NP):
            assert np.array_equal(impl.int4_decode_flat(f["packed"], f[f"scales_g{g}"], R, Cc, g), f[f"flat_g{g}"])
    K, N = f["packed_gkn"].shape[0] * 2, f["packed_gkn"].shape[1]
    for impl in (C, NP):
        assert np.array_equal(impl.int4_decode_gkn(f["packed_gkn"], f["scales_gkn"], K, N, 128), f["gkn"])


def test_oracle_nf4_fixture():
    f = _load("decode_nf4.npz")
    R, Cc = f["packed"].shape[0], f["packed"].shape[1] * 2
    for g in (32, 64):
        for impl in (C, NP):
            assert np.array_equal(impl.nf4_decode_flat(f["packed"], f[f"scales_g{g}"], R, Cc, g), f[f"flat_g{g}"])
    # with scale 1.0 the first sixteen elements are the bf16 roundings of the level table
    assert np.array_equal(f["flat_g64"][0, :16], NP.bf16_rne_bits(NP.NF4))
    K, N = f["packed_gkn"].shape[0] * 2, f["packed_gkn"].shape[1]
    for impl in (C, NP):
        assert np.array_equal(impl.nf4_decode_gkn(f["packed_gkn"], f["scales_gkn"], K, N, 64), f["gkn"])


def test_oracle_nvfp4_fixture():
    f = _load("decode_nvfp4.npz")
    R, Cc = f["packed"].shape[0], f["packed"].shape[1] * 2
    g = f["global_scale"][0]
    s = C.e4m3_scales_to_f32(f["scale_bytes"])
    # block-scale bytes decode like torch's e4m3fn (library routine)
    assert np.array_equal(s, torch.from_numpy(f["scale_bytes"].copy()).view(torch.float8_e4m3fn).float().numpy())
    for impl in (C, NP):
        assert np.array_equal(impl.nvfp4_decode_flat(f["packed"], s, g, R, Cc), f["flat"])
        assert np.array_equal(impl.nvfp4_decode_flat(f["packed"], f["scales_f32_folded"], np.float32(1.0), R, Cc),
                              f["flat_folded"])
    K, N = f["packed_gkn"].shape[0] * 2, f["packed_gkn"].shape[1]
    sg = C.e4m3_scales_to_f32(f["scale_bytes_gkn"])
    for impl in (C, NP):
        assert np.array_equal(impl.nvfp4_decode_gkn(f["packed_gkn"], sg, g, K, N), f["gkn"])


def test_oracle_fp8_fixture():
    f = _load("decode_fp8.npz")
    R, Cc = f["bytes"].shape
    for impl in (C, NP):
        p, b = impl.fp8_decode(f["bytes"], f["scales"], R, Cc)
        assert np.array_equal(p.view(np.uint32), f["f32_bits"]) and np.array_equal(b, f["bf16_bits"])


def test_oracle_fp8_closed_form_fixture():
    f = _load("fp8_closed_form.npz")
    OUT, IN = f["bytes"].shape
    # the bytes are what torch's e4m3fn cast makes of the formula
    v = torch.arange(OUT * IN, dtype=torch.float32)
    w8 = (((v * 3 + 1) % 29) - 14).reshape(OUT, IN).div(16.0).to(torch.float8_e4m3fn)
    assert np.array_equal(w8.view(torch.uint8).numpy(), f["bytes"])
    s = (torch.arange(6, dtype=torch.float32).reshape(3, 2) + 1.0) / 7.0
    assert np.array_equal(s.numpy(), f["scales"])
    for impl in (C, NP):
        assert np.array_equal(impl.fp8_decode(f["bytes"], f["scales"], OUT, IN)[1], f["bf16_bits"])
    w = NP.bf16_bits_to_f32(f["bf16_bits"]).astype(np.float64)
    assert np.array_equal(f["x"].astype(np.float64) @ w.T, f["y_f64"])
    assert np.array_equal(f["dy"].astype(np.float64) @ w, f["dx_f64"])


# ------------------------------------------------------------------ GPU: HIP path vs fixtures
@pytest.mark.gpu
def test_hip_decode_fixtures(hip_device):
    from xorl_amd import quantize as Q

    dev = hip_device
    f = _load("decode_int4.npz")
    R, Cc = f["packed"].shape[0], f["packed"].shape[1] * 2
    for g in (32, 128):
        got = Q.int4_dequantize(torch.from_numpy(f["packed"]).to(dev), torch.from_numpy(f[f"scales_g{g}"]).to(dev), R, Cc, g)
        assert np.array_equal(_bits(got), f[f"flat_g{g}"])
        got = Q.int4_dequantize(torch.from_numpy(f["packed"]).to(dev),
                                torch.from_numpy(f[f"scales_g{g}"]).to(torch.bfloat16).to(dev), R, Cc, g)
        assert np.array_equal(_bits(got), f[f"flat_g{g}"])          # the stored scales are bf16-representable
    K, N = f["packed_gkn"].shape[0] * 2, f["packed_gkn"].shape[1]
    got = Q.int4_dequantize_gkn(torch.from_numpy(f["packed_gkn"]).to(dev), torch.from_numpy(f["scales_gkn"]).to(dev), K, N, 128)
    assert np.array_equal(_bits(got), f["gkn"])

    f = _load("decode_nf4.npz")
    R, Cc = f["packed"].shape[0], f["packed"].shape[1] * 2
    for g in (32, 64):
        got = Q.nf4_dequantize(torch.from_numpy(f["packed"]).to(dev), torch.from_numpy(f[f"scales_g{g}"]).to(dev), R * Cc, g)
        assert np.array_equal(_bits(got).reshape(R, Cc), f[f"flat_g{g}"])
    K, N = f["packed_gkn"].shape[0] * 2, f["packed_gkn"].shape[1]
    got = Q.nf4_dequantize_gkn(torch.from_numpy(f["packed_gkn"]).to(dev), torch.from_numpy(f["scales_gkn"]).to(dev), K, N, 64)
    assert np.array_equal(_bits(got), f["gkn"])

    f = _load("decode_nvfp4.npz")
    R, Cc = f["packed"].shape[0], f["packed"].shape[1] * 2
    gs = torch.from_numpy(f["global_scale"]).to(dev)
    sb = torch.from_numpy(f["scale_bytes"].copy()).view(torch.float8_e4m3fn).to(dev)
    got = Q.nvfp4_dequantize(torch.from_numpy(f["packed"]).to(dev), sb, gs, R * Cc)
    assert np.array_equal(_bits(got).reshape(R, Cc), f["flat"])
    got = Q.nvfp4_dequantize(torch.from_numpy(f["packed"]).to(dev), torch.from_numpy(f["scales_f32_folded"]).to(dev),
                             torch.ones(1, device=dev), R * Cc)
    assert np.array_equal(_bits(got).reshape(R, Cc), f["flat_folded"])
    K, N = f["packed_gkn"].shape[0] * 2, f["packed_gkn"].shape[1]
    sgb = torch.from_numpy(f["scale_bytes_gkn"].copy()).view(torch.float8_e4m3fn).to(dev)
    got = Q.nvfp4_dequantize_gkn(torch.from_numpy(f["packed_gkn"]).to(dev), sgb, gs, K, N)
    assert np.array_equal(_bits(got), f["gkn"])

    f = _load("decode_fp8.npz")
    wb = torch.from_numpy(f["bytes"].copy()).view(torch.float8_e4m3fn).to(dev)
    st = torch.from_numpy(f["scales"]).to(dev)
    got32 = Q.block_fp8_dequantize_gkn(wb, st, 128)                          # fp32, as the reference returns
    assert _same_bits_nan_aware(got32.cpu().view(torch.int32).numpy().view(np.uint32), f["f32_bits"])
    got16 = Q.block_fp8_dequantize_gkn(wb, st, 128, out_dtype=torch.bfloat16)
    assert _same_bits_nan_aware(_bits(got16), f["bf16_bits"])


@pytest.mark.gpu
def test_hip_fp8_closed_form_linear(hip_device):
    from xorl_amd.qlora import QLoRALinear

    f = _load("fp8_closed_form.npz")
    OUT, IN = f["bytes"].shape
    m = QLoRALinear.from_quantized(
        torch.from_numpy(f["bytes"].copy()), weight_block_scales=torch.from_numpy(f["scales"].copy()),
        in_features=IN, out_features=OUT, r=16, lora_alpha=16, quant_format="block_fp8").to(hip_device)
    assert np.array_equal(_bits(m._dequantize_weight().to(torch.bfloat16)), f["bf16_bits"])
    with torch.no_grad():
        m.lora_B.zero_()                                                     # y == base exactly in form
    x = torch.from_numpy(f["x"]).to(torch.bfloat16).to(hip_device).requires_grad_(True)   # n/8: exact in bf16
    dy = torch.from_numpy(f["dy"]).to(torch.bfloat16).to(hip_device)
    y = m(x)
    y.backward(dy)
    assert max_rel_err(y.float().cpu().double(), torch.from_numpy(f["y_f64"])) <= TOL
    assert max_rel_err(x.grad.float().cpu().double(), torch.from_numpy(f["dx_f64"])) <= TOL
    # stronger than the stated bar: each output is the bf16 rounding of an fp32-accumulated sum
    yr = torch.from_numpy(f["y_f64"]).to(torch.bfloat16)
    assert (y.cpu().float() - yr.float()).abs().max() <= 2 * torch.finfo(torch.bfloat16).eps * yr.float().abs().max()
