"""The torch page parsers of the host front end (flagrot_releaser_amd.kernels) against the numpy oracle, on the CPU."""
import numpy as np
import pytest
import torch

from oracle import attend as OA
from oracle import pages as PG
from oracle import quant as Q


def _pool(fmt, P, seed, Np=3, H=2):
    """random codes / scale words packed by the oracle's packer into a garbage pool"""
    rng = np.random.default_rng(seed)
    T = Np * P
    qk = Q.QK_OF_KIND[fmt]
    if qk == "sym":
        codes = rng.integers(-7, 8, (T, 2 * H, 128))
    else:
        codes = rng.integers(0, 16 if qk == "asym4" else 4, (T, 2 * H, 128))
    words = rng.integers(0, 1 << 16, (T, 2 * H, 4)).astype(np.int64)
    words &= ~0x7C00 | 0x3C00                      # keep the FP16 exponent finite
    pool = rng.integers(0, 256, (Np, H, PG.chunk_bytes(fmt, P)), dtype=np.uint8)
    slots = rng.permutation(Np * P)[:T]
    PG.pack_tokens(pool, slots, codes, words, fmt, P)
    return pool


@pytest.mark.parametrize("fmt", ["int4", "int4a", "int2a", "konly", "konlya", "konlya2"])
@pytest.mark.parametrize("P", [16, 32])
def test_torch_parser_matches_oracle(fmt, P):
    from flagrot_releaser_amd import kernels as K
    pool = _pool(fmt, P, seed=sum(map(ord, fmt)) + P)
    codes, words = PG.parse_pages(pool, fmt, P)                       # [Np, H, P, 2, 128], [Np, H, P, 2, 4]
    c, mag, sb = K.parse_pages(torch.from_numpy(pool), P, fmt)
    w = np.asarray(words).astype(np.int64)
    z = 0 if Q.QK_OF_KIND[fmt] == "sym" else np.repeat(w & (15 if Q.QK_OF_KIND[fmt] == "asym4" else 3), 32, -1)
    assert np.array_equal(c.numpy().astype(np.int64), codes.astype(np.int64) - z)
    assert np.array_equal(sb.numpy().astype(np.int64) & 0xFFFF, w & 0xFFFF)
    assert np.array_equal(mag.numpy(), Q.word_scale(w).astype(np.float32))
    Kp, Vp = OA.dequant_pages(pool, fmt, P, dtype=np.float64)           # [Np, P, H, 128]
    if fmt in ("int4", "int4a", "int2a"):
        k, v = K.dequant_v2_pages(torch.from_numpy(pool), P, dtype=torch.float32, fmt=fmt)
    else:
        k, v = K.dequant_cb_pages(torch.from_numpy(pool), P, fmt, dtype=torch.float32)
    sc = max(np.abs(Kp).max(), 1e-30)
    assert np.abs(k.numpy() - Kp).max() <= 2e-6 * sc and np.abs(v.numpy() - Vp).max() <= 2e-6 * max(np.abs(Vp).max(), 1e-30)


def test_torch_parser_head_256_and_rejects():
    from flagrot_releaser_amd import kernels as K
    a, b = _pool("int4a", 16, 5), _pool("int4a", 16, 6)
    both = np.concatenate([a, b], -1)                                   # two 128-d half chunks
    c, mag, sb = K.parse_pages(torch.from_numpy(both), 16, "int4a", Dh=256)
    ca, _, _ = K.parse_pages(torch.from_numpy(a), 16, "int4a")
    cb, _, _ = K.parse_pages(torch.from_numpy(b), 16, "int4a")
    assert torch.equal(c[..., :128], ca) and torch.equal(c[..., 128:], cb) and mag.shape[-1] == 8
    with pytest.raises(NotImplementedError):
        K.dequant_cb_pages(torch.from_numpy(a), 16, "nf4")
    h = K.hadamard(32, "cpu", torch.float64)
    assert torch.allclose(h @ h, torch.eye(32, dtype=torch.float64)) and torch.equal(h, h.T)


@pytest.mark.parametrize("f8", [False, True], ids=["f16meta", "f8meta"])
def test_kivi_torch_parser_matches_reference_vectors(f8):
    """flagrot_releaser_amd.kivi.dequant_groups (torch, here on the CPU) on the random chunk bytes of
    tests/golden/kivi_layout.npz against what the reference's parser returned for them, both bases."""
    import os

    from flagrot_releaser_amd import kivi as KV
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "kivi_layout.npz"))
    tag = "f8" if f8 else "f16"
    ch = torch.from_numpy(g[f"{tag}_chunks"])
    vf = KV.parse_chunks(ch, 128, f8)[4]
    assert np.array_equal(vf.numpy() != 0, g[f"{tag}_vf"] != 0)
    for basis in ("orig", "stored"):
        k, v = KV.dequant_groups(ch, 128, basis, f8)
        for a, ref in ((k, g[f"{tag}_k_{basis}"]), (v, g[f"{tag}_v_{basis}"])):
            assert tuple(a.shape) == ref.shape
            assert np.abs(a.numpy() - ref).max() <= 3e-6 * np.abs(ref).max(), (tag, basis)
