"""TEST INFRASTRUCTURE ONLY: ctypes binding of oracle/xq_oracle.c.

All functions take and return numpy arrays (uint8 codes, float32 scales,
uint16 bf16 bit patterns) so results can be compared bit for bit.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np


_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libxq_oracle.so")


def build(force: bool = False) -> str:
    """Compile xq_oracle.c with gcc (seconds)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
        os.path.join(_HERE, "xq_oracle.c")
    ):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE])
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        i64, f32, p = ctypes.c_int64, ctypes.c_float, ctypes.c_void_p
        L.xqo_bf16_rne.restype = ctypes.c_uint16
        L.xqo_bf16_rne.argtypes = [f32]
        L.xqo_bf16_to_f32.restype = f32
        L.xqo_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.xqo_e4m3_to_f32.restype = f32
        L.xqo_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        L.xqo_f32_to_e4m3.restype = ctypes.c_uint8
        L.xqo_f32_to_e4m3.argtypes = [f32]
        L.xqo_e2m1_to_f32.restype = f32
        L.xqo_e2m1_to_f32.argtypes = [ctypes.c_uint8]
        L.xqo_f32_to_e2m1.restype = ctypes.c_uint8
        L.xqo_f32_to_e2m1.argtypes = [f32]
        L.xqo_int4_decode_flat.argtypes = [p, p, p, i64, i64]
        L.xqo_int4_decode_gkn.argtypes = [p, p, p, i64, i64, i64]
        L.xqo_int4_quantize_flat.argtypes = [p, p, p, i64, i64]
        L.xqo_int4_quantize_gkn.argtypes = [p, p, p, i64, i64, i64]
        L.xqo_int4_quantize_sym_flat.argtypes = [p, p, p, i64, i64]
        L.xqo_nf4_decode_flat.argtypes = [p, p, p, i64, i64]
        L.xqo_nf4_decode_gkn.argtypes = [p, p, p, i64, i64, i64]
        L.xqo_nf4_quantize_flat.argtypes = [p, p, p, i64, i64]
        L.xqo_nf4_quantize_gkn.argtypes = [p, p, p, i64, i64, i64]
        L.xqo_nf4_level.argtypes = [ctypes.c_int]
        L.xqo_nf4_level.restype = ctypes.c_float
        L.xqo_nf4_encode.argtypes = [ctypes.c_float]
        L.xqo_nf4_encode.restype = ctypes.c_uint8
        L.xqo_nvfp4_decode_flat.argtypes = [p, p, f32, p, i64, i64]
        L.xqo_nvfp4_decode_gkn.argtypes = [p, p, f32, p, i64, i64, i64]
        L.xqo_nvfp4_quantize_flat.restype = f32
        L.xqo_nvfp4_quantize_flat.argtypes = [p, p, p, p, i64, i64, f32]
        L.xqo_nvfp4_quantize_gkn.restype = f32
        L.xqo_nvfp4_quantize_gkn.argtypes = [p, p, p, p, i64, i64, i64, f32]
        L.xqo_fp8_decode.argtypes = [p, p, p, p, i64, i64, i64]
        L.xqo_fp8_quantize.argtypes = [p, p, p, i64, i64, i64, f32]
        for name in (
            "xqo_int4_decode_flat", "xqo_int4_decode_gkn", "xqo_int4_quantize_flat",
            "xqo_int4_quantize_gkn", "xqo_int4_quantize_sym_flat", "xqo_nvfp4_decode_flat",
            "xqo_nf4_decode_flat", "xqo_nf4_decode_gkn", "xqo_nf4_quantize_flat", "xqo_nf4_quantize_gkn",
            "xqo_nvfp4_decode_gkn", "xqo_fp8_decode", "xqo_fp8_quantize",
        ):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def _c(a: np.ndarray, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


# ---------------------------------------------------------------- scalars
def e4m3_table() -> np.ndarray:
    """fp32 value of each of the 256 e4m3fn bytes."""
    L = lib()
    return np.array([L.xqo_e4m3_to_f32(b) for b in range(256)], dtype=np.float32)


def e2m1_table() -> np.ndarray:
    L = lib()
    return np.array([L.xqo_e2m1_to_f32(c) for c in range(16)], dtype=np.float32)


def bf16_rne(x: np.ndarray) -> np.ndarray:
    L = lib()
    flat = _c(x, np.float32).reshape(-1)
    return np.array([L.xqo_bf16_rne(float(v)) for v in flat], dtype=np.uint16).reshape(x.shape)


def e4m3_scales_to_f32(b: np.ndarray) -> np.ndarray:
    return e4m3_table()[_c(b, np.uint8)]


# ---------------------------------------------------------------- int4
def int4_decode_flat(packed, scales_f32, rows, cols, group) -> np.ndarray:
    packed, scales = _c(packed, np.uint8), _c(scales_f32, np.float32)
    assert packed.size == rows * cols // 2 and scales.size == rows * cols // group
    out = np.empty((rows, cols), dtype=np.uint16)
    lib().xqo_int4_decode_flat(_p(packed), _p(scales), _p(out), rows * cols, group)
    return out


def int4_decode_gkn(packed, scales_f32, K, N, group) -> np.ndarray:
    packed, scales = _c(packed, np.uint8), _c(scales_f32, np.float32)
    assert packed.size == K * N // 2 and scales.size == (K // group) * N
    out = np.empty((K, N), dtype=np.uint16)
    lib().xqo_int4_decode_gkn(_p(packed), _p(scales), _p(out), K, N, group)
    return out


def int4_quantize_flat(x, group):
    x = _c(x, np.float32)
    rows, cols = x.shape
    packed = np.zeros((rows, cols // 2), dtype=np.uint8)
    scales = np.empty((rows, cols // group), dtype=np.float32)
    lib().xqo_int4_quantize_flat(_p(x), _p(packed), _p(scales), rows * cols, group)
    return packed, scales


def int4_quantize_gkn(x, group):
    x = _c(x, np.float32)
    K, N = x.shape
    packed = np.zeros((K // 2, N), dtype=np.uint8)
    scales = np.empty((K // group, N), dtype=np.float32)
    lib().xqo_int4_quantize_gkn(_p(x), _p(packed), _p(scales), K, N, group)
    return packed, scales


# ---------------------------------------------------------------- nf4
def nf4_table() -> np.ndarray:
    L = lib()
    return np.array([L.xqo_nf4_level(c) for c in range(16)], dtype=np.float32)


def nf4_encode(v: np.ndarray) -> np.ndarray:
    L = lib()
    return np.array([L.xqo_nf4_encode(float(t)) for t in np.asarray(v, dtype=np.float32).ravel()], dtype=np.uint8)


def nf4_decode_flat(packed, scales_f32, rows, cols, group) -> np.ndarray:
    packed, scales = _c(packed, np.uint8), _c(scales_f32, np.float32)
    assert packed.size == rows * cols // 2 and scales.size == rows * cols // group
    out = np.empty((rows, cols), dtype=np.uint16)
    lib().xqo_nf4_decode_flat(_p(packed), _p(scales), _p(out), rows * cols, group)
    return out


def nf4_decode_gkn(packed, scales_f32, K, N, group) -> np.ndarray:
    packed, scales = _c(packed, np.uint8), _c(scales_f32, np.float32)
    assert packed.size == K * N // 2 and scales.size == (K // group) * N
    out = np.empty((K, N), dtype=np.uint16)
    lib().xqo_nf4_decode_gkn(_p(packed), _p(scales), _p(out), K, N, group)
    return out


def nf4_quantize_flat(x, group):
    x = _c(x, np.float32)
    rows, cols = x.shape
    packed = np.zeros((rows, cols // 2), dtype=np.uint8)
    scales = np.empty((rows, cols // group), dtype=np.float32)
    lib().xqo_nf4_quantize_flat(_p(x), _p(packed), _p(scales), rows * cols, group)
    return packed, scales


def nf4_quantize_gkn(x, group):
    x = _c(x, np.float32)
    K, N = x.shape
    packed = np.zeros((K // 2, N), dtype=np.uint8)
    scales = np.empty((K // group, N), dtype=np.float32)
    lib().xqo_nf4_quantize_gkn(_p(x), _p(packed), _p(scales), K, N, group)
    return packed, scales


def int4_quantize_sym_flat(x, group):
    """scale = bf16(absmax/7) (returned as uint16 bit patterns), codes in 1..15."""
    x = _c(x, np.float32)
    rows, cols = x.shape
    packed = np.zeros((rows, cols // 2), dtype=np.uint8)
    scales = np.empty((rows, cols // group), dtype=np.uint16)
    lib().xqo_int4_quantize_sym_flat(_p(x), _p(packed), _p(scales), rows * cols, group)
    return packed, scales


# ---------------------------------------------------------------- nvfp4
def nvfp4_decode_flat(packed, scales_f32, global_scale, rows, cols, block=16) -> np.ndarray:
    packed, scales = _c(packed, np.uint8), _c(scales_f32, np.float32)
    assert packed.size == rows * cols // 2 and scales.size == rows * cols // block
    out = np.empty((rows, cols), dtype=np.uint16)
    lib().xqo_nvfp4_decode_flat(_p(packed), _p(scales), float(global_scale), _p(out), rows * cols, block)
    return out


def nvfp4_decode_gkn(packed, scales_f32, global_scale, K, N, block=16) -> np.ndarray:
    packed, scales = _c(packed, np.uint8), _c(scales_f32, np.float32)
    assert packed.size == K * N // 2 and scales.size == (K // block) * N
    out = np.empty((K, N), dtype=np.uint16)
    lib().xqo_nvfp4_decode_gkn(_p(packed), _p(scales), float(global_scale), _p(out), K, N, block)
    return out


def nvfp4_quantize_flat(x, block=16, global_amax=None):
    """-> packed u8 [rows, cols/2], e4m3 scale bytes [rows, cols/block], global fp32."""
    x = _c(x, np.float32)
    rows, cols = x.shape
    packed = np.zeros((rows, cols // 2), dtype=np.uint8)
    sc = np.empty((rows, cols // block), dtype=np.uint8)
    amax = np.empty(rows * cols // block, dtype=np.float32)
    g = lib().xqo_nvfp4_quantize_flat(
        _p(x), _p(packed), _p(sc), _p(amax), rows * cols, block, -1.0 if global_amax is None else float(global_amax)
    )
    return packed, sc, np.float32(g)


def nvfp4_quantize_gkn(x, block=16, global_amax=None):
    x = _c(x, np.float32)
    K, N = x.shape
    packed = np.zeros((K // 2, N), dtype=np.uint8)
    sc = np.empty((K // block, N), dtype=np.uint8)
    amax = np.empty((K // block) * N, dtype=np.float32)
    g = lib().xqo_nvfp4_quantize_gkn(
        _p(x), _p(packed), _p(sc), _p(amax), K, N, block, -1.0 if global_amax is None else float(global_amax)
    )
    return packed, sc, np.float32(g)


# ---------------------------------------------------------------- block fp8
def fp8_decode(w_bytes, scales, rows, cols, block=128):
    """-> (fp32 product array, bf16 bit patterns)."""
    w, s = _c(w_bytes, np.uint8), _c(scales, np.float32)
    assert w.size == rows * cols
    assert s.size == -(-rows // block) * -(-cols // block)
    o32 = np.empty((rows, cols), dtype=np.float32)
    o16 = np.empty((rows, cols), dtype=np.uint16)
    lib().xqo_fp8_decode(_p(w), _p(s), _p(o32), _p(o16), rows, cols, block)
    return o32, o16


def fp8_quantize(x, block=128, amax_scale=1.0):
    x = _c(x, np.float32)
    rows, cols = x.shape
    w = np.empty((rows, cols), dtype=np.uint8)
    s = np.empty((-(-rows // block), -(-cols // block)), dtype=np.float32)
    lib().xqo_fp8_quantize(_p(x), _p(w), _p(s), rows, cols, block, float(amax_scale))
    return w, s
