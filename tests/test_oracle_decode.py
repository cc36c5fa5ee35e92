"""Pins for the CPU oracle's codecs (no GPU).

Each check is chosen so that a plausible slip (wrong nibble order, wrong bias,
dropped global scale, transposed scale grid, truncation instead of RNE) fails.
Library routines used as independent authorities: torch.float8_e4m3fn and
torch.bfloat16 casts on CPU.
"""

import numpy as np
import pytest
import torch

from oracle import cdecode as C
from oracle import decode_np as NP


def _bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def test_e4m3_table_matches_torch_all_256():
    b = torch.arange(256, dtype=torch.uint8)
    ref = b.view(torch.float8_e4m3fn).float().numpy()
    for tab in (C.e4m3_table(), NP.E4M3):
        assert np.array_equal(np.isnan(tab), np.isnan(ref))
        m = ~np.isnan(ref)
        assert np.array_equal(tab[m].view(np.uint32), ref[m].view(np.uint32))
    assert C.e4m3_table()[0x7E] == 448.0  # FP8_E4M3_MAX, fp4_codec.py:8


def test_e4m3_encode_matches_torch_on_finite_range():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.normal(0, 50, 20000), rng.normal(0, 1, 20000), rng.normal(0, 0.01, 20000),
        NP.E4M3[~np.isnan(NP.E4M3)],                       # exact values
        (NP.E4M3[1:0x7E] + NP.E4M3[2:0x7F]) / 2,           # all positive ties
    ]).astype(np.float32)
    x = x[np.abs(x) <= 448.0]
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    L = C.lib()
    got = np.array([L.xqo_f32_to_e4m3(float(v)) for v in x], dtype=np.uint8)
    assert np.array_equal(got, ref)
    # saturation (satfinite) beyond the finite range
    assert L.xqo_f32_to_e4m3(1e9) == 0x7E and L.xqo_f32_to_e4m3(-500.0) == 0xFE


def test_e2m1_table():
    # {0,.5,1,1.5,2,3,4,6}, sign = bit 3, code 8 = -0.0 (fp4_codec.py:22-30)
    t = C.e2m1_table()
    assert np.array_equal(t[:8], np.array([0, .5, 1, 1.5, 2, 3, 4, 6], dtype=np.float32))
    assert np.array_equal(t[8:], -t[:8])
    assert np.signbit(t[8]) and t[8] == 0.0
    assert np.array_equal(t.view(np.uint32), NP.E2M1.view(np.uint32))


def test_e2m1_encode_thresholds_ties_up():
    L = C.lib()
    # a<.25->0, <.75->.5, <1.25->1, <1.75->1.5, <2.5->2, <3.5->3, <5->4, else 6
    edges = [(0.2499, 0), (0.25, 1), (0.7499, 1), (0.75, 2), (1.2499, 2), (1.25, 3),
             (1.7499, 3), (1.75, 4), (2.4999, 4), (2.5, 5), (3.4999, 5), (3.5, 6),
             (4.9999, 6), (5.0, 7), (6.0, 7)]
    for v, code in edges:
        assert L.xqo_f32_to_e2m1(v) == code, v
        assert L.xqo_f32_to_e2m1(-v) == code + 8, v
    assert L.xqo_f32_to_e2m1(0.0) == 0


def test_bf16_rne_matches_torch():
    rng = np.random.default_rng(1)
    x = rng.normal(0, 1, 50000).astype(np.float32)
    # exact ties: bf16 value + half ulp
    base = (rng.integers(0, 2 ** 15, 2000).astype(np.uint32) << 16) | 0x8000
    x = np.concatenate([x, base.view(np.float32), np.array([0.0, -0.0, 1e-40, 3.4e38], np.float32)])
    x = x[np.isfinite(x)]
    ref = _bf16_bits(torch.from_numpy(x))
    assert np.array_equal(NP.bf16_rne_bits(x), ref)
    assert np.array_equal(C.bf16_rne(x[:5000]), ref[:5000])


@pytest.mark.parametrize("group", [32, 128])
def test_int4_flat_decode_enumeration(group):
    # every nibble code against a sweep of scales, independent torch restatement
    rng = np.random.default_rng(2)
    rows, cols = 16, 256
    packed = rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8)
    packed[0, :8] = [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]   # element i == code i
    scales = (rng.normal(0, 0.02, (rows, cols // group)).astype(np.float32))
    scales_bf16 = torch.from_numpy(scales).to(torch.bfloat16).float().numpy()
    for sc in (scales, scales_bf16):
        got_c = C.int4_decode_flat(packed, sc, rows, cols, group)
        got_np = NP.int4_decode_flat(packed, sc, rows, cols, group)
        # torch restatement: low nibble = even element (int4_quantize.py:62-63)
        p = torch.from_numpy(packed).int()
        nib = torch.stack([p & 0xF, p >> 4], dim=-1).reshape(rows, cols).float()
        w = ((nib - 8.0) * torch.from_numpy(sc).repeat_interleave(group, dim=1)).to(torch.bfloat16)
        assert np.array_equal(got_c, _bf16_bits(w))
        assert np.array_equal(got_np, got_c)
    # element order: first 16 elements of row 0 decode codes 0..15 in order
    vals = NP.bf16_bits_to_f32(got_c[0, :16]) / sc[0, 0]
    assert np.allclose(vals, np.arange(16) - 8, rtol=1e-2)


def test_int4_gkn_is_transposed_flat():
    # GKN packs K-row pairs per column; decoding W^T laid out GKN must equal
    # the transpose of decoding W laid out flat (same codes, same scales).
    rng = np.random.default_rng(3)
    N, K, group = 24, 128, 32
    codes = rng.integers(0, 16, (N, K), dtype=np.uint8)
    scales = rng.normal(0, 0.05, (N, K // group)).astype(np.float32)
    flat_packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
    ct = codes.T.copy()                                   # [K, N]
    gkn_packed = (ct[0::2] | (ct[1::2] << 4)).astype(np.uint8)
    a = C.int4_decode_flat(flat_packed, scales, N, K, group)
    b = C.int4_decode_gkn(gkn_packed, scales.T.copy(), K, N, group)
    assert np.array_equal(a.T, b)
    assert np.array_equal(NP.int4_decode_gkn(gkn_packed, scales.T.copy(), K, N, group), b)


def test_int4_reference_quantizer_closed_form():
    # scale = max(amax,1e-12)*(2/15); q = clamp(trunc(x/scale + 8.5), 0, 15)
    x = np.zeros((1, 32), dtype=np.float32)
    x[0, :8] = [-7.2, -5.9, -3.4, -0.2, 0.2, 2.6, 6.4, 7.5]
    packed, scales = C.int4_quantize_flat(x, 32)
    assert scales[0, 0] == np.float32(7.5) * np.float32(2.0 / 15.0)
    codes = np.stack([packed[0] & 0xF, packed[0] >> 4], -1).reshape(-1)
    # scale ~= 1: q = trunc(x + 8.5), 16 clamps to 15, zeros land on code 8
    assert list(codes[:8]) == [1, 2, 5, 8, 8, 11, 14, 15]
    assert set(codes[8:]) == {8}
    # round trip error bounded by half a step
    w = NP.bf16_bits_to_f32(C.int4_decode_flat(packed, scales, 1, 32, 32))
    assert np.max(np.abs(w - x)) <= scales[0, 0] * 0.51 + 1e-2
    # GKN twin gives the transposed codes
    pk, sk = C.int4_quantize_gkn(x.T.copy(), 32)
    ck = np.stack([pk & 0xF, pk >> 4], 1).reshape(32)
    assert np.array_equal(ck, codes) and sk[0, 0] == scales[0, 0]


def test_int4_sym_quantizer_rule():
    rng = np.random.default_rng(4)
    x = rng.normal(0, 0.02, (8, 256)).astype(np.float32)
    packed, sb = C.int4_quantize_sym_flat(x, 128)
    s = NP.bf16_bits_to_f32(sb)
    amax = np.abs(x.reshape(8, 2, 128)).max(-1)
    assert np.array_equal(sb, _bf16_bits(torch.from_numpy(amax / np.float32(7.0))))
    codes = np.stack([packed & 0xF, packed >> 4], -1).reshape(8, 256).astype(np.int32) - 8
    assert codes.min() >= -7 and codes.max() <= 7
    ref = np.clip(np.rint(x / np.repeat(s, 128, 1)), -7, 7)
    assert np.array_equal(codes, ref.astype(np.int32))


def test_nf4_level_table_is_the_normal_quantile_map():
    # The levels are published as a construction, not only as numbers: eight
    # standard-normal quantiles on the positive side, seven on the negative,
    # zero, normalised by the largest (offset 0.9677083, Dettmers et al. 2023).
    from scipy.stats import norm

    off = 0.9677083
    pos = norm.ppf(np.linspace(off, 0.5, 9)[:-1])
    neg = -norm.ppf(np.linspace(off, 0.5, 8)[:-1])
    want = np.sort(np.concatenate([pos, [0.0], neg]))
    want /= want.max()
    t = C.nf4_table()
    assert t.dtype == np.float32 and np.array_equal(t.view(np.uint32), NP.NF4.view(np.uint32))
    assert np.max(np.abs(t - want)) < 5e-7
    assert np.all(np.diff(t) > 0) and t[0] == -1.0 and t[7] == 0.0 and t[15] == 1.0
    # asymmetric by construction: 7 negative and 8 positive non-zero levels
    assert (t < 0).sum() == 7 and (t > 0).sum() == 8


def test_nf4_encoder_is_nearest_level():
    # Decision points are the means of neighbouring levels, so the encoder is
    # nearest-level; check against a brute-force argmin away from the cuts and
    # the strict ">" at them (nf4_codec.py:42-64).
    t = C.nf4_table().astype(np.float64)
    v = np.linspace(-1, 1, 4001).astype(np.float32)
    got = C.nf4_encode(v)
    d = np.abs(v.astype(np.float64)[:, None] - t[None, :])
    near = d.argmin(1)
    srt = np.sort(d, 1)
    clear = (srt[:, 1] - srt[:, 0]) > 1e-6
    assert np.array_equal(got[clear], near[clear].astype(np.uint8))
    cuts = ((t[1:] + t[:-1]) / 2).astype(np.float32)
    assert np.array_equal(C.nf4_encode(cuts), np.arange(15, dtype=np.uint8))               # not above the cut
    assert np.array_equal(C.nf4_encode(np.nextafter(cuts, np.float32(2))), np.arange(1, 16, dtype=np.uint8))
    assert np.array_equal(C.nf4_encode(t.astype(np.float32)), np.arange(16, dtype=np.uint8))


def test_nf4_decode_flat_and_gkn():
    rng = np.random.default_rng(11)
    rows, cols, group = 16, 256, 64
    packed = rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8)
    packed[0, :8] = [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]   # element i == code i
    scales = np.abs(rng.normal(0, 0.05, (rows, cols // group))).astype(np.float32)
    scales[0, 0] = 1.0
    got_c = C.nf4_decode_flat(packed, scales, rows, cols, group)
    assert np.array_equal(got_c, NP.nf4_decode_flat(packed, scales, rows, cols, group))
    # torch restatement: LUT gather, low nibble = even element (nf4_quantize.py:89-103)
    p = torch.from_numpy(packed).long()
    nib = torch.stack([p & 0xF, p >> 4], dim=-1).reshape(rows, cols)
    w = (torch.from_numpy(C.nf4_table())[nib] * torch.from_numpy(scales).repeat_interleave(group, dim=1)).to(torch.bfloat16)
    assert np.array_equal(got_c, _bf16_bits(w))
    assert np.array_equal(got_c[0, :16], _bf16_bits(torch.from_numpy(C.nf4_table())))
    # GKN of the transposed codes decodes to the transpose
    codes = nib.numpy().astype(np.uint8)
    ct = codes.T.copy()
    gkn_packed = (ct[0::2] | (ct[1::2] << 4)).astype(np.uint8)
    b = C.nf4_decode_gkn(gkn_packed, scales.T.copy(), cols, rows, group)
    assert np.array_equal(got_c.T, b)
    assert np.array_equal(NP.nf4_decode_gkn(gkn_packed, scales.T.copy(), cols, rows, group), b)


def test_nf4_quantizer_rule_and_roundtrip():
    # scale = absmax (so +-absmax land exactly on codes 15 / 0), zeros on code 7,
    # an all-zero group keeps the 1e-12 floor; round-trip error under the
    # 0.10 the reference's own round-trip test allows.
    rng = np.random.default_rng(12)
    x = rng.normal(0, 0.02, (8, 256)).astype(np.float32)
    x[0, :64] = 0.0
    x[1, 0], x[1, 1], x[1, 2] = 0.5, -0.5, 0.0
    packed, scales = C.nf4_quantize_flat(x, 64)
    assert np.array_equal(scales, np.maximum(np.abs(x.reshape(8, 4, 64)).max(-1), np.float32(1e-12)))
    codes = np.stack([packed & 0xF, packed >> 4], -1).reshape(8, 256)
    assert set(codes[0, :64]) == {7} and scales[0, 0] == np.float32(1e-12)
    assert list(codes[1, :3]) == [15, 0, 7] and scales[1, 0] == np.float32(0.5)
    w = NP.bf16_bits_to_f32(C.nf4_decode_flat(packed, scales, 8, 256, 64))
    assert np.abs(w - x)[2:].mean() / np.abs(x)[2:].mean() < 0.10  # the metric of tests/qlora/test_qlora.py:151-152
    # every element sits on the level nearest to x/scale
    norm = x / np.repeat(scales, 64, 1)
    t = C.nf4_table()
    assert np.all(np.abs(t[codes] - norm) <= np.abs(t[None, None, :] - norm[..., None]).min(-1) + 1e-6)
    # GKN twin: transposed input -> transposed codes, same scales
    pk, sk = C.nf4_quantize_gkn(x.T.copy(), 64)
    ck = np.stack([pk & 0xF, pk >> 4], 1).reshape(256, 8)
    assert np.array_equal(ck, codes.T) and np.array_equal(sk, scales.T)


def test_nvfp4_decode_flat_and_gkn():
    rng = np.random.default_rng(5)
    N, K = 16, 128
    codes = rng.integers(0, 16, (N, K), dtype=np.uint8)
    codes[0, :16] = np.arange(16)
    sc_bytes = rng.integers(0, 0x7F, (N, K // 16), dtype=np.uint8)      # finite e4m3
    g = np.float32(0.00371)
    sc = torch.from_numpy(sc_bytes).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(C.e4m3_scales_to_f32(sc_bytes), sc)
    packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
    got = C.nvfp4_decode_flat(packed, sc, g, N, K)
    # torch restatement: sc = fl(block*global); w = bf16(fl(e2m1*sc))  (nvfp4_quantize.py:81,93-96)
    tab = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6])
    eff = (torch.from_numpy(sc) * torch.tensor(g)).repeat_interleave(16, dim=1)
    ref = (tab[torch.from_numpy(codes).long()] * eff).to(torch.bfloat16)
    assert np.array_equal(got, _bf16_bits(ref))
    assert np.array_equal(NP.nvfp4_decode_flat(packed, sc, g, N, K), got)
    # dropping the global scale must change the answer
    assert not np.array_equal(C.nvfp4_decode_flat(packed, sc, 1.0, N, K), got)
    # prequantized form: fp32 scales with global folded in and global = 1 (nvfp4_linear.py:158-164)
    folded = (sc * g).astype(np.float32)
    assert np.array_equal(C.nvfp4_decode_flat(packed, folded, 1.0, N, K), got)
    # GKN = transpose of bytes and scales (tests/qlora/test_moe_load_experts.py:15-26)
    ct = codes.T.copy()
    gk = (ct[0::2] | (ct[1::2] << 4)).astype(np.uint8)
    b = C.nvfp4_decode_gkn(gk, sc.T.copy(), g, K, N)
    assert np.array_equal(b, got.T)
    assert np.array_equal(NP.nvfp4_decode_gkn(gk, sc.T.copy(), g, K, N), b)


def test_nvfp4_quantizer_scale_convention_and_roundtrip():
    # global*6*448 == amax; block scales use the full fp8 range
    # (tests/qlora/test_qlora.py:191-230); round trip atol=rtol=0.05 (:137-154)
    torch.manual_seed(0)
    w = torch.randn(64, 256) * 0.02
    packed, sb, g = C.nvfp4_quantize_flat(w.numpy())
    amax = w.abs().max().item()
    assert abs(g * 6 * 448 - amax) / amax < 1e-6
    sc = C.e4m3_scales_to_f32(sb)
    assert sc.max() == 448.0
    deq = NP.bf16_bits_to_f32(C.nvfp4_decode_flat(packed, sc, g, 64, 256))
    torch.testing.assert_close(torch.from_numpy(deq), w, atol=0.05, rtol=0.05)
    rel = np.abs(deq - w.numpy()).mean() / np.abs(w.numpy()).mean()
    assert rel < 0.15
    # GKN twin on the transpose gives transposed codes and scales
    pk, sk, gk = C.nvfp4_quantize_gkn(w.t().contiguous().numpy())
    assert gk == g and np.array_equal(sk, sb.T)
    deq_k = NP.bf16_bits_to_f32(C.nvfp4_decode_gkn(pk, C.e4m3_scales_to_f32(sk), gk, 256, 64))
    assert np.array_equal(deq_k, deq.T)


def _ref_dequant_block_fp8_2d(weight, scale, block):
    # restatement held by the reference's tests:
    # tests/server/weight_sync/test_fp8_quantization.py:19-28
    e = scale.float().repeat_interleave(block, dim=0).repeat_interleave(block, dim=1)
    return weight.float() * e[: weight.shape[0], : weight.shape[1]]


@pytest.mark.parametrize("shape", [(256, 384), (384, 256), (200, 576), (128, 128), (1, 130)])
def test_fp8_decode_against_reference_held_restatement(shape):
    rng = np.random.default_rng(6)
    R, Cc = shape
    wb = rng.integers(0, 256, (R, Cc), dtype=np.uint8)
    wb[(wb & 0x7F) == 0x7F] = 0x3C                        # no NaN codes
    s = rng.uniform(1e-4, 2e-2, (-(-R // 128), -(-Cc // 128))).astype(np.float32)
    p, b16 = C.fp8_decode(wb, s, R, Cc)
    ref = _ref_dequant_block_fp8_2d(torch.from_numpy(wb).view(torch.float8_e4m3fn), torch.from_numpy(s), 128)
    assert np.array_equal(p.view(np.uint32), ref.numpy().view(np.uint32))
    assert np.array_equal(b16, _bf16_bits(ref))
    p2, b2 = NP.fp8_decode(wb, s, R, Cc)
    assert np.array_equal(p2.view(np.uint32), p.view(np.uint32)) and np.array_equal(b2, b16)
    # a scale grid indexed the other way round (block (k, n) in place of (n, k)) must change the result: decoding the
    # transposed matrix with the transposed grid gives the transpose, with the untransposed grid (same element count,
    # read in the wrong order) it does not
    if s.shape[0] != s.shape[1]:
        wt = np.ascontiguousarray(wb.T)
        pt, _ = C.fp8_decode(wt, np.ascontiguousarray(s.T), Cc, R)
        assert np.array_equal(pt.view(np.uint32), np.ascontiguousarray(p.T).view(np.uint32))
        if min(s.shape) > 1:      # (a grid of one row or column reads the same in either order)
            wrong, _ = C.fp8_decode(wt, s.reshape(s.shape[1], s.shape[0]), Cc, R)
            assert not np.array_equal(wrong.view(np.uint32), pt.view(np.uint32))


def test_fp8_closed_form_fixture():
    # tests/ops/test_block_fp8_frozen_dgrad.py:44-55: weight (((i*3+1)%29)-14)/16 -> e4m3,
    # scales (k+1)/7 on a [3,2] grid, IN=256, OUT=384
    IN, OUT = 256, 384
    v = torch.arange(OUT * IN, dtype=torch.float32)
    w8 = (((v * 3 + 1) % 29) - 14).reshape(OUT, IN).div(16.0).to(torch.float8_e4m3fn)
    s = (torch.arange(6, dtype=torch.float32).reshape(3, 2) + 1.0) / 7.0
    p, b16 = C.fp8_decode(w8.view(torch.uint8).numpy(), s.numpy(), OUT, IN)
    # all values k/16 are exact in e4m3, so the decode is (k/16)*scale in fp32
    exact = ((((v * 3 + 1) % 29) - 14).reshape(OUT, IN) / 16.0) * s.repeat_interleave(128, 0).repeat_interleave(128, 1)
    assert np.array_equal(p, exact.numpy())
    assert np.array_equal(b16, _bf16_bits(exact))


def test_fp8_quantizer_matches_reference_held_restatement():
    # _slime_blockwise_fp8_reference, tests/server/weight_sync/test_fp8_quantization.py:31-51
    torch.manual_seed(1)
    for shape in [(256, 384), (200, 300)]:
        w = torch.randn(*shape) * 0.02
        q, s = C.fp8_quantize(w.numpy())
        R, Cc = shape
        pr, pc = (-R) % 128, (-Cc) % 128
        padded = torch.zeros(R + pr, Cc + pc)
        padded[:R, :Cc] = w
        nr, nc = padded.shape[0] // 128, padded.shape[1] // 128
        blocks = padded.reshape(nr, 128, nc, 128).permute(0, 2, 1, 3)
        scale = blocks.abs().reshape(nr, nc, -1).max(-1).values.clamp(min=1e-12) / 448.0
        qb = (blocks / scale[..., None, None]).clamp(-448, 448).to(torch.float8_e4m3fn)
        qref = qb.permute(0, 2, 1, 3).reshape(padded.shape)[:R, :Cc].contiguous()
        assert np.array_equal(s, scale.numpy())
        assert np.array_equal(q, qref.view(torch.uint8).numpy())
        # round trip rel err < 0.03 (tests/qlora/test_qlora.py:358-361)
        p, _ = C.fp8_decode(q, s, R, Cc)
        assert np.abs(p - w.numpy()).mean() / np.abs(w.numpy()).mean() < 0.03
