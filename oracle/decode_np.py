"""TEST INFRASTRUCTURE ONLY: numpy twin of the decoders in xq_oracle.c.

Written independently of the C file (value tables and vectorised index
arithmetic instead of per-element bit construction) so that a slip in either
shows up as a mismatch.  Fast enough for full-size weights, so the GPU parity
tests use these on the big shapes.

Reference arithmetic restated (paths relative to the xorl checkout):
  int4   ops/quantize/int4_quantize.py:45-76, int4_gkn_quantize.py:79-130
  nvfp4  ops/quantize/nvfp4_quantize.py:64-98, nvfp4_gkn_quantize.py:112-169,
         fp4_codec.py:22-30
  fp8    ops/quantize/block_fp8_gkn_quantize.py:131-180
  nf4    ops/quantize/nf4_quantize.py:62-105, nf4_gkn_quantize.py:84-142,
         nf4_codec.py:18-35
"""

from __future__ import annotations

import numpy as np


# e2m1 magnitudes by 3-bit code; the same table is stated at
# ops/quantize/nvfp4_fake_quant.py:40.
E2M1_ABS = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)
E2M1 = np.concatenate([E2M1_ABS, -E2M1_ABS]).astype(np.float32)  # code 8 = -0.0


# NormalFloat4 levels as fp32 bit patterns (the fp32 roundings of the sixteen
# constants at ops/quantize/nf4_codec.py:18-35).
NF4 = np.array([0xBF800000, 0xBF3239B1, 0xBF066B30, 0xBECA32A0, 0xBE91A24D, 0xBE3D353F, 0xBDBA7871, 0x00000000,
                0x3DA2FAFF, 0x3E24CAE3, 0x3E7C04DD, 0x3EAD033A, 0x3EE1A4B8, 0x3F1007AB, 0x3F3913B3, 0x3F800000],
               dtype=np.uint32).view(np.float32)


def _e4m3_table() -> np.ndarray:
    t = np.empty(256, dtype=np.float32)
    for b in range(256):
        e, m = (b >> 3) & 15, b & 7
        if e == 15 and m == 7:
            v = np.nan
        elif e == 0:
            v = m / 8.0 * 2.0 ** -6
        else:
            v = (1.0 + m / 8.0) * 2.0 ** (e - 7)
        t[b] = -v if b & 0x80 else v
    return t


E4M3 = _e4m3_table()


def bf16_rne_bits(x: np.ndarray) -> np.ndarray:
    """fp32 array -> bf16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def _unpack_flat(packed: np.ndarray, rows: int, cols: int) -> np.ndarray:
    p = np.ascontiguousarray(packed, dtype=np.uint8).reshape(rows, cols // 2)
    out = np.empty((rows, cols), dtype=np.uint8)
    out[:, 0::2] = p & 0xF
    out[:, 1::2] = p >> 4
    return out


def _unpack_gkn(packed: np.ndarray, K: int, N: int) -> np.ndarray:
    p = np.ascontiguousarray(packed, dtype=np.uint8).reshape(K // 2, N)
    out = np.empty((K, N), dtype=np.uint8)
    out[0::2] = p & 0xF
    out[1::2] = p >> 4
    return out


def int4_decode_flat(packed, scales_f32, rows, cols, group):
    nib = _unpack_flat(packed, rows, cols).astype(np.float32)
    s = np.repeat(np.asarray(scales_f32, dtype=np.float32).reshape(rows, cols // group), group, axis=1)
    return bf16_rne_bits((nib - np.float32(8.0)) * s)


def int4_decode_gkn(packed, scales_f32, K, N, group):
    nib = _unpack_gkn(packed, K, N).astype(np.float32)
    s = np.repeat(np.asarray(scales_f32, dtype=np.float32).reshape(K // group, N), group, axis=0)
    return bf16_rne_bits((nib - np.float32(8.0)) * s)


def nf4_decode_flat(packed, scales_f32, rows, cols, group):
    v = NF4[_unpack_flat(packed, rows, cols)]
    s = np.repeat(np.asarray(scales_f32, dtype=np.float32).reshape(rows, cols // group), group, axis=1)
    return bf16_rne_bits(v * s)


def nf4_decode_gkn(packed, scales_f32, K, N, group):
    v = NF4[_unpack_gkn(packed, K, N)]
    s = np.repeat(np.asarray(scales_f32, dtype=np.float32).reshape(K // group, N), group, axis=0)
    return bf16_rne_bits(v * s)


def nvfp4_decode_flat(packed, scales_f32, global_scale, rows, cols, block=16):
    v = E2M1[_unpack_flat(packed, rows, cols)]
    sc = np.asarray(scales_f32, dtype=np.float32).reshape(rows, cols // block) * np.float32(global_scale)
    return bf16_rne_bits(v * np.repeat(sc, block, axis=1))


def nvfp4_decode_gkn(packed, scales_f32, global_scale, K, N, block=16):
    v = E2M1[_unpack_gkn(packed, K, N)]
    sc = np.asarray(scales_f32, dtype=np.float32).reshape(K // block, N) * np.float32(global_scale)
    return bf16_rne_bits(v * np.repeat(sc, block, axis=0))


def fp8_decode(w_bytes, scales, rows, cols, block=128):
    """-> (fp32 product, bf16 bits of it)."""
    v = E4M3[np.ascontiguousarray(w_bytes, dtype=np.uint8).reshape(rows, cols)]
    s = np.asarray(scales, dtype=np.float32).reshape(-(-rows // block), -(-cols // block))
    s = np.repeat(np.repeat(s, block, axis=0), block, axis=1)[:rows, :cols]
    p = (v * s).astype(np.float32)
    return p, bf16_rne_bits(p)
