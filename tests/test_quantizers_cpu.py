"""Host logic: the package's torch quantizers emit the same bytes as the C oracle (no GPU)."""

import numpy as np
import torch

from oracle import cdecode as C
from xorl_amd import quantize as Q


def _w(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * 0.02


def test_int4_quantizers_match_oracle():
    w = _w((32, 256), 0)
    p, s = Q.int4_quantize(w, 128)
    pc, sc = C.int4_quantize_flat(w.numpy(), 128)
    assert np.array_equal(p.numpy(), pc) and np.array_equal(s.numpy(), sc)
    pk, sk = Q.int4_quantize_gkn(w.t().contiguous(), 128)
    pkc, skc = C.int4_quantize_gkn(w.t().contiguous().numpy(), 128)
    assert np.array_equal(pk.numpy(), pkc) and np.array_equal(sk.numpy(), skc)
    ps, ss = Q.int4_quantize_sym(w, 128)
    psc, ssc = C.int4_quantize_sym_flat(w.numpy(), 128)
    assert np.array_equal(ps.numpy(), psc)
    assert np.array_equal(ss.view(torch.int16).numpy().view(np.uint16), ssc)


def test_nf4_quantizers_match_oracle():
    w = _w((32, 256), 5)
    w[3, :64] = 0.0
    p, s = Q.nf4_quantize(w, 64)
    pc, sc = C.nf4_quantize_flat(w.numpy(), 64)
    assert np.array_equal(p.numpy(), pc.reshape(-1)) and np.array_equal(s.numpy(), sc.reshape(-1))
    pk, sk = Q.nf4_quantize_gkn(w.t().contiguous(), 64)
    pkc, skc = C.nf4_quantize_gkn(w.t().contiguous().numpy(), 64)
    assert np.array_equal(pk.numpy(), pkc) and np.array_equal(sk.numpy(), skc)
    assert np.array_equal(np.array(Q.NF4_TABLE, dtype=np.float32), C.nf4_table())
    assert Q.NF4_MIN_STEP == min(b - a for a, b in zip(Q.NF4_TABLE, Q.NF4_TABLE[1:]))


def test_nvfp4_quantizers_match_oracle():
    w = _w((32, 256), 1)
    p, bs, g = Q.nvfp4_quantize(w)
    pc, bsc, gc = C.nvfp4_quantize_flat(w.numpy())
    assert np.array_equal(p.numpy().reshape(32, 128), pc)
    assert np.array_equal(bs.view(torch.uint8).numpy().reshape(32, 16), bsc)
    assert g.item() == gc
    pk, bk, gk = Q.nvfp4_quantize_gkn(w.t().contiguous())
    pkc, bkc, gkc = C.nvfp4_quantize_gkn(w.t().contiguous().numpy())
    assert np.array_equal(pk.numpy(), pkc) and np.array_equal(bk.view(torch.uint8).numpy(), bkc) and gk.item() == gkc
    # EMA override of the global amax (nvfp4_quantize.py:139-141)
    p2, bs2, g2 = Q.nvfp4_quantize(w, global_amax=torch.tensor([0.2]))
    pc2, bsc2, gc2 = C.nvfp4_quantize_flat(w.numpy(), global_amax=0.2)
    assert np.array_equal(p2.numpy().reshape(32, 128), pc2) and g2.item() == gc2
    assert np.array_equal(bs2.view(torch.uint8).numpy().reshape(32, 16), bsc2)


def test_block_fp8_quantizer_matches_oracle():
    for shape, seed in (((256, 384), 2), ((200, 300), 3)):
        w = _w(shape, seed)
        y, s = Q.block_fp8_quantize_gkn(w)
        yc, sc = C.fp8_quantize(w.numpy())
        assert np.array_equal(y.view(torch.uint8).numpy(), yc)
        assert np.array_equal(s.numpy(), sc)


def test_nvfp4_multiplier_is_one_ieee_division():
    """The codes are taken from x * fl(6 / amax): ONE division.  `6.0 / tensor` in torch is reciprocal-then-multiply
    (two roundings, a different multiplier for about a third of all amax values), which moves an element across an
    encode threshold only once in millions of random draws -- so the cases are constructed: for blocks whose two
    multipliers differ, an element is placed where the products fall on opposite sides of a threshold."""
    rng = np.random.default_rng(3)
    amax = (rng.random(200000, dtype=np.float32) * 4 + 0.5).astype(np.float32)
    m1 = (np.float32(6.0) / amax).astype(np.float32)
    m2 = ((np.float32(1.0) / amax).astype(np.float32) * np.float32(6.0)).astype(np.float32)
    idx = np.nonzero(m1 != m2)[0]
    assert idx.size > 1000
    thresholds = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)
    blocks = []
    for i in idx[:20000]:
        t = thresholds[i % 7]
        x0 = np.float32(t / m1[i])
        for x in (x0, np.nextafter(x0, np.float32(0)), np.nextafter(x0, np.float32(8))):
            if x < amax[i] and (np.float32(x * m1[i]) >= t) != (np.float32(x * m2[i]) >= t):
                b = np.zeros(16, dtype=np.float32)
                b[0], b[1] = amax[i], x
                blocks.append(b)
                break
    assert len(blocks) >= 20, len(blocks)
    x = torch.from_numpy(np.stack(blocks))
    packed, bs, g = Q.nvfp4_quantize(x, 16)
    po, so, go = C.nvfp4_quantize_flat(x.numpy())
    assert np.array_equal(packed.numpy().reshape(po.shape), po)
