#!/usr/bin/env python3
"""Writes the small golden fixtures in this folder (run from the repo root:
`python tests/golden/make_fixtures.py`).

The reference holds no stored tensors for the decode path, so the vectors here
are (a) seeded raw bytes + scales with the expected decoded bf16 bit patterns,
produced by the C oracle and cross-checked against its independent numpy twin
at generation time, and (b) the closed-form block-fp8 case that the reference's
own test builds from `arange` formulas
(/root/reference/tests/ops/test_block_fp8_frozen_dgrad.py:44-60), re-derived
here from the formulas, with the expected forward/dgrad from float64 matmuls of
the exactly known decoded weight.

Every array is plain numeric data in `.npz` files (loadable with
numpy.load(allow_pickle=False)).
"""

from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import cdecode as C      # noqa: E402
from oracle import decode_np as NP   # noqa: E402

ROWS, COLS = 64, 256


def _same(a, b):
    return np.array_equal(np.asarray(a).view(np.uint16), np.asarray(b).view(np.uint16))


def decode_int4(rng):
    out = {}
    packed = rng.integers(0, 256, size=(ROWS, COLS // 2), dtype=np.uint8)
    for group in (32, 128):
        # bf16-representable scales of both signs and wide magnitude (the module stores bf16 scales)
        s = (rng.standard_normal((ROWS, COLS // group)) * np.exp2(rng.integers(-12, 4, size=(ROWS, COLS // group))))
        s = NP.bf16_bits_to_f32(NP.bf16_rne_bits(s.astype(np.float32)))
        flat = C.int4_decode_flat(packed, s, ROWS, COLS, group)
        assert _same(flat, NP.int4_decode_flat(packed, s, ROWS, COLS, group))
        out[f"scales_g{group}"] = s
        out[f"flat_g{group}"] = flat
    # GKN: bytes [K/2, N] pair rows; scales [K/group, N]
    K, N = COLS, ROWS
    pg = rng.integers(0, 256, size=(K // 2, N), dtype=np.uint8)
    sg = NP.bf16_bits_to_f32(NP.bf16_rne_bits((rng.standard_normal((K // 128, N)) * 0.01).astype(np.float32)))
    gkn = C.int4_decode_gkn(pg, sg, K, N, 128)
    assert _same(gkn, NP.int4_decode_gkn(pg, sg, K, N, 128))
    out.update(packed=packed, packed_gkn=pg, scales_gkn=sg, gkn=gkn)
    return out


def decode_nf4(rng):
    out = {}
    packed = rng.integers(0, 256, size=(ROWS, COLS // 2), dtype=np.uint8)
    packed[0, :8] = [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]      # element i == code i
    for group in (32, 64):
        # absmax scales are positive; a wide range of magnitudes and the 1e-12 floor
        s = np.abs(rng.standard_normal((ROWS, COLS // group))) * np.exp2(rng.integers(-14, 4, size=(ROWS, COLS // group)))
        s = s.astype(np.float32)
        s[0, 0], s[1, 0] = 1.0, 1e-12
        flat = C.nf4_decode_flat(packed, s, ROWS, COLS, group)
        assert _same(flat, NP.nf4_decode_flat(packed, s, ROWS, COLS, group))
        out[f"scales_g{group}"] = s
        out[f"flat_g{group}"] = flat
    K, N = COLS, ROWS
    pg = rng.integers(0, 256, size=(K // 2, N), dtype=np.uint8)
    sg = (np.abs(rng.standard_normal((K // 64, N))) * 0.05).astype(np.float32)
    gkn = C.nf4_decode_gkn(pg, sg, K, N, 64)
    assert _same(gkn, NP.nf4_decode_gkn(pg, sg, K, N, 64))
    out.update(packed=packed, packed_gkn=pg, scales_gkn=sg, gkn=gkn)
    return out


def decode_nvfp4(rng):
    packed = rng.integers(0, 256, size=(ROWS, COLS // 2), dtype=np.uint8)
    # every finite e4m3 byte appears as a block scale (0x7f / 0xff are NaN and excluded)
    sb = rng.integers(0, 256, size=(ROWS, COLS // 16), dtype=np.uint8)
    sb[(sb & 0x7F) == 0x7F] = 0x38
    sb.reshape(-1)[:256] = np.where((np.arange(256) & 0x7F) == 0x7F, 0x38, np.arange(256)).astype(np.uint8)
    s = C.e4m3_scales_to_f32(sb).reshape(ROWS, COLS // 16)
    g = np.float32(0.000173)
    flat = C.nvfp4_decode_flat(packed, s, g, ROWS, COLS)
    assert _same(flat, NP.nvfp4_decode_flat(packed, s, float(g), ROWS, COLS))
    K, N = COLS, ROWS
    pg = rng.integers(0, 256, size=(K // 2, N), dtype=np.uint8)
    sgb = rng.integers(0, 0x7F, size=(K // 16, N), dtype=np.uint8)
    sg = C.e4m3_scales_to_f32(sgb).reshape(K // 16, N)
    gkn = C.nvfp4_decode_gkn(pg, sg, g, K, N)
    assert _same(gkn, NP.nvfp4_decode_gkn(pg, sg, float(g), K, N))
    # fp32 block scales with the global folded in (prequantized checkpoints), global = 1
    s32 = (s * g).astype(np.float32)
    flat32 = C.nvfp4_decode_flat(packed, s32, np.float32(1.0), ROWS, COLS)
    return dict(packed=packed, scale_bytes=sb, global_scale=np.array([g], np.float32), flat=flat,
                packed_gkn=pg, scale_bytes_gkn=sgb, gkn=gkn, scales_f32_folded=s32, flat_folded=flat32)


def decode_fp8(rng):
    R, Cc = 200, 328           # ragged against the 128x128 scale grid
    wb = rng.integers(0, 256, size=(R, Cc), dtype=np.uint8)
    wb.reshape(-1)[:256] = np.arange(256, dtype=np.uint8)   # all 256 codes incl. both NaNs and -0
    s = np.abs(rng.standard_normal(((R + 127) // 128, (Cc + 127) // 128))).astype(np.float32) * 0.01 + 1e-5
    f32, b16 = C.fp8_decode(wb, s, R, Cc)
    f32n, b16n = NP.fp8_decode(wb, s, R, Cc)
    assert np.array_equal(f32.view(np.uint32), f32n.view(np.uint32)) and _same(b16, b16n)
    return dict(bytes=wb, scales=s, f32_bits=f32.view(np.uint32), bf16_bits=b16)


def fp8_closed_form():
    """IN=256, OUT=384; weight (((3i+1) mod 29) - 14)/16 (exact in e4m3), scale grid (k+1)/7 on
    [3,2]; input ((i mod 23) - 11)/8 on 8 rows; grad_output ((i mod 13) - 6)/4.  The decoded
    weight is bf16(fl(k/16 * s)); y and dx are float64 products of that weight."""
    IN, OUT, ROWS_X = 256, 384, 8
    i = np.arange(OUT * IN, dtype=np.float64)
    wv = ((((i * 3 + 1) % 29) - 14) / 16.0).reshape(OUT, IN)
    s = ((np.arange(6, dtype=np.float32).reshape(3, 2) + np.float32(1.0)) / np.float32(7.0)).astype(np.float32)
    table = C.e4m3_table()
    codes = np.zeros(wv.shape, np.uint8)
    finite = np.array([c for c in range(256) if (c & 0x7F) != 0x7F])
    # exact lookup: each value has exactly one e4m3 code (zero maps to +0)
    for c in finite:
        if c == 0x80:
            continue
        codes[wv.astype(np.float32) == table[c]] = c
    assert np.array_equal(table[codes].astype(np.float64), wv)
    f32, b16 = C.fp8_decode(codes, s, OUT, IN)
    sfull = np.repeat(np.repeat(s, 128, 0), 128, 1)
    assert np.array_equal(f32, (wv.astype(np.float32) * sfull))
    w = NP.bf16_bits_to_f32(b16).astype(np.float64)
    j = np.arange(ROWS_X * IN, dtype=np.float64)
    x = (((j % 23) - 11) / 8.0).reshape(ROWS_X, IN)
    k = np.arange(ROWS_X * OUT, dtype=np.float64)
    dy = (((k % 13) - 6) / 4.0).reshape(ROWS_X, OUT)
    return dict(bytes=codes, scales=s, bf16_bits=b16, x=x.astype(np.float32), dy=dy.astype(np.float32),
                y_f64=x @ w.T, dx_f64=dy @ w)


def main():
    C.build()
    rng = np.random.default_rng(20240607)
    np.savez_compressed(os.path.join(HERE, "decode_int4.npz"), **decode_int4(rng))
    np.savez_compressed(os.path.join(HERE, "decode_nvfp4.npz"), **decode_nvfp4(rng))
    np.savez_compressed(os.path.join(HERE, "decode_fp8.npz"), **decode_fp8(rng))
    np.savez_compressed(os.path.join(HERE, "fp8_closed_form.npz"), **fp8_closed_form())
    np.savez_compressed(os.path.join(HERE, "decode_nf4.npz"), **decode_nf4(np.random.default_rng(20240608)))
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
