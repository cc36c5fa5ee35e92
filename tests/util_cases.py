"""Seeded synthetic QLoRA cases shared by the GPU tests, smoke() and bench.py.

Builds quantized weights with the package's torch quantizers (host logic,
checked byte-for-byte against the oracle in tests/test_quantizers_cpu.py) and
decodes them with the CPU oracle for the expected values.
"""

from __future__ import annotations

import numpy as np
import torch

import os

from oracle import cdecode as C
from oracle import decode_np as NP
from oracle import recipe as R

# worst value of each tolerance metric seen per test function: {test name: [tensor-wide, per-row]};
# tests/conftest.py writes it out at the end of a session that ran GPU tests
PARITY_WORST: dict = {}
ROW_TOL_FACTOR = 2.0


def close(got, ref, tol, row_tol=None, rows="last"):
    """Tolerance check of a kernel result against the oracle under two metrics: max|err| / max|ref| over the
    tensor (<= tol), and the same quotient row by row (<= row_tol, by default ROW_TOL_FACTOR * tol: a row's own
    maximum is a smaller yardstick than the tensor's).  rows = "last": the vectors of the last dimension (token
    rows of Y / dX, rows of a dense factor gradient); "first": one row per leading index (one expert's whole factor
    gradient: its r-element vectors are single dot products each and can lie arbitrarily near zero); "none": the
    tensor-wide metric only (routing-weight gradients: a token's top-k scalars are unrelated dot products)."""
    e = R.max_rel_err(got, ref)
    if rows == "first":
        er = R.row_rel_err(got.reshape(got.shape[0], -1), ref.reshape(ref.shape[0], -1))
    elif rows == "none":
        er = 0.0
    else:
        er = R.row_rel_err(got, ref)
    name = os.environ.get("PYTEST_CURRENT_TEST", "?").split(" ")[0].split("::")[-1].split("[")[0]
    w = PARITY_WORST.setdefault(name, [0.0, 0.0])
    w[0], w[1] = max(w[0], e), max(w[1], er)
    assert e <= tol, f"max|err|/max|ref| = {e:.3e} > {tol}"
    rt = ROW_TOL_FACTOR * tol if row_tol is None else row_tol
    assert er <= rt, f"per-row max|err|/max|ref_row| = {er:.3e} > {rt}"
    return e


def gen(shape, std, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(dtype)


def bits_to_bf16(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def make_dense_module(fmt: str, N: int, K: int, r: int, alpha: int, seed: int, device, bias=False):
    """Returns (module on `device`, decoded weight bf16 on CPU from the oracle)."""
    from xorl_amd.qlora import QLoRALinear

    lin = torch.nn.Linear(K, N, bias=bias)
    with torch.no_grad():
        lin.weight.copy_(gen((N, K), 0.02, seed))
        if bias:
            lin.bias.copy_(gen((N,), 0.1, seed + 7))
    m = QLoRALinear.from_module(lin, r=r, lora_alpha=alpha, quant_format=fmt)
    with torch.no_grad():
        m.lora_A.copy_(gen((r, K), 0.02, seed + 1))
        m.lora_B.copy_(gen((N, r), 0.02, seed + 2))
    w_ref = oracle_decode_dense(m)
    return m.to(device), w_ref


def oracle_decode_dense(m) -> torch.Tensor:
    """Decode a (CPU) module's packed state with the numpy oracle -> bf16 [N, K]."""
    N, K = m.out_features, m.in_features
    packed = m.packed_weight_f32.detach().cpu().contiguous().view(torch.uint8).numpy()
    if m.quant_format == "block_fp8":
        s = m.weight_block_scales.cpu().contiguous().view(torch.float32).numpy()
        return bits_to_bf16(NP.fp8_decode(packed.reshape(N, K), s, N, K)[1])
    if m.quant_format == "nvfp4":
        sdt = m._scale_dtypes["weight_block_scales"]
        sb = m.weight_block_scales.cpu().contiguous()
        s = C.e4m3_scales_to_f32(sb.numpy()) if sdt == torch.float8_e4m3fn else sb.view(torch.float32).numpy()
        g = m.weight_global_scale.cpu().contiguous().view(torch.float32).item()
        return bits_to_bf16(NP.nvfp4_decode_flat(packed, s.reshape(N, K // 16), g, N, K))
    if m.quant_format == "int4":
        sdt = m._scale_dtypes["weight_scales"]
        s = m.weight_scales.cpu().contiguous().view(sdt).float().numpy()
        return bits_to_bf16(NP.int4_decode_flat(packed, s, N, K, m.quant_group_size))
    if m.quant_format == "nf4":
        s = m.weight_scales.cpu().contiguous().view(torch.float32).numpy()
        return bits_to_bf16(NP.nf4_decode_flat(packed, s, N, K, m.quant_group_size))
    raise ValueError(m.quant_format)
