"""The oracle's selecting encoder against the vectors written by the reference's own codebook_ref.encode
(tests/golden/make_golden.py; CPU run of the reference => IEEE division in the asymmetric step => true_div=True)."""
import os

import numpy as np
import pytest

from oracle import quant as Q

GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.mark.parametrize("kind", ["konly", "konlya", "konlya2"])
def test_k2_encode_matches_reference_vectors(kind):
    g = np.load(os.path.join(GOLD, f"k2_encode_{kind}.npz"))
    Hkv = g["C"].shape[0]
    codes, words, info = Q.k2_encode(g["x_bits"], g["C"], kind, true_div=True)
    assert np.array_equal(codes[:, :Hkv], g["kq"])
    assert np.array_equal(codes[:, Hkv:], g["vq"])
    assert np.array_equal(Q.word_scale(words[:, :Hkv]), g["ks"])
    assert np.array_equal(Q.word_scale(words[:, Hkv:]), g["vs"])
    assert np.array_equal(info["local"], g["klocal"])
    assert np.array_equal(info["full"].astype(np.uint8) * 2, g["kmode"])     # reference mode ids: 0 base, 2 F
    assert np.array_equal(info["err_head"], g["kherr"])                       # fp32 error values, bit for bit
    assert not g["vmode"].any()
    # the vectors exercise every choice
    assert info["local"].any() and info["full"].any() and (~info["full"]).any()


@pytest.mark.parametrize("kind", ["konlya", "konlya2"])
def test_kernel_form_differs_only_in_the_step(kind):
    """true_div=False (reciprocal multiply, the kernels' form) may move a step by one ulp: stored scale words stay
    within one zero-point-preserving step and almost all codes are unchanged."""
    g = np.load(os.path.join(GOLD, f"k2_encode_{kind}.npz"))
    Hkv = g["C"].shape[0]
    a, wa, _ = Q.k2_encode(g["x_bits"], g["C"], kind, true_div=True)
    b, wb, _ = Q.k2_encode(g["x_bits"], g["C"], kind, true_div=False)
    assert (a[:, Hkv:] == b[:, Hkv:]).mean() > 0.99
    nb = 16 if kind == "konlya" else 4
    assert np.abs((wa[:, Hkv:] & 0x7FFF) - (wb[:, Hkv:] & 0x7FFF)).max() <= nb + nb - 1
