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


@pytest.mark.parametrize("kind", ["konly", "konlya"])
def test_k2_encode_head_dim_256_matches_reference_vectors(kind):
    """codebook_ref.encode at Dq = 256: eight 32-groups, whole-head H256, head error over eight column blocks"""
    g = np.load(os.path.join(GOLD, f"k2_encode_d256_{kind}.npz"))
    Hkv = g["C"].shape[0]
    assert g["x_bits"].shape[-1] == 256
    codes, words, info = Q.k2_encode(g["x_bits"], g["C"], kind, true_div=True)
    assert np.array_equal(codes[:, :Hkv], g["kq"]) and np.array_equal(codes[:, Hkv:], g["vq"])
    assert np.array_equal(Q.word_scale(words[:, :Hkv]), g["ks"]) and np.array_equal(Q.word_scale(words[:, Hkv:]), g["vs"])
    assert np.array_equal(info["local"], g["klocal"])
    assert np.array_equal(info["full"].astype(np.uint8) * 2, g["kmode"])
    assert np.array_equal(info["err_head"], g["kherr"])
    assert info["local"].any() and info["full"].any() and (~info["full"]).any()
    # flags: H32 bit of group g in K word g, H256 bit in V word 0
    kw, vw = words[:, :Hkv], words[:, Hkv:]
    assert np.array_equal((kw >> 15) & 1, info["local"].astype(np.int64))
    assert np.array_equal((vw[..., 0] >> 15) & 1, info["full"].astype(np.int64)) and not ((vw[..., 1:] >> 15) & 1).any()


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


# ------------------------------------------------------------------------------------------------ page layouts
# Vectors written by the reference's own page parsers (vllm_flagrot/kernels.py parse_pages / dequant_v2_pages /
# dequant_cb_pages) on pools of random bytes into which oracle.pages.pack_tokens packed seeded tokens.
from oracle import attend as A  # noqa: E402
from oracle import kivi as KV  # noqa: E402
from oracle import pages as PG  # noqa: E402

FMTS = ["int4", "int4a", "int2a", "konly", "konlya", "konlya2"]


@pytest.mark.parametrize("P", [16, 32])
@pytest.mark.parametrize("fmt", FMTS)
def test_page_parser_and_packer_match_reference_parsers(fmt, P):
    g = np.load(os.path.join(GOLD, f"pages_{fmt}_p{P}.npz"))
    pool = g["pool"]
    codes, words = PG.parse_pages(pool, fmt, P)                      # raw codes, raw words
    zmask = {"int4": 0, "konly": 0, "int4a": 15, "konlya": 15, "int2a": 3, "konlya2": 3}[fmt]
    # (a) the oracle's parser on arbitrary bytes (garbage pages included) == the reference's parser
    assert np.array_equal(words & 0xFFFF, g["sbits"].astype(np.int32) & 0xFFFF)
    ref_codes = g["codes"].astype(np.int64)                          # reference: zero point already subtracted
    assert np.array_equal(codes.astype(np.int64) - np.repeat(words & zmask, 32, -1), ref_codes)
    mag = Q.word_scale(words).astype(np.float32)
    ref_mag = g["mag_bits"].view(np.float32)
    assert np.array_equal(np.isnan(mag), np.isnan(ref_mag))
    assert np.array_equal(mag[~np.isnan(mag)], ref_mag[~np.isnan(mag)])
    # (b) the oracle's packer through the reference's parser: what was packed comes back at its slots
    slots, pc, pw = g["slots"], g["packed_codes"].astype(np.int64), g["packed_words"].astype(np.int64)
    Hkv = pool.shape[1]
    for t, sl in enumerate(slots):
        if sl < 0:
            continue
        pg, off = divmod(int(sl), P)
        for kv in range(2):
            rows = slice(kv * Hkv, (kv + 1) * Hkv)
            w = g["sbits"][pg, :, off, kv].astype(np.int64) & 0xFFFF
            assert np.array_equal(w, pw[t, rows] & 0xFFFF), (fmt, P, t, kv)
            assert np.array_equal(ref_codes[pg, :, off, kv], pc[t, rows] - np.repeat(pw[t, rows] & zmask, 32, -1))
    # (c) dequantised pages (the attention oracle's input) == the reference's dequantisers at the written slots
    k, v = A.dequant_pages(pool, fmt, P, dtype=np.float64)           # [Np, P, H, 128]
    rk, rv = g["k"].view(np.float32), g["v"].view(np.float32)
    for t, sl in enumerate(slots):
        if sl < 0:
            continue
        pg, off = divmod(int(sl), P)
        for a, b in ((k, rk), (v, rv)):
            ref = b[pg, off].astype(np.float64)
            assert np.abs(a[pg, off] - ref).max() <= 2e-6 * max(1.0, np.abs(ref).max()), (fmt, P, t)


def test_static_writers_match_reference_vectors():
    """kernels/ref.py kv_selrot_quant(fmt int4) / int4a_quant and formats.quant_asym_dep(bits 2) + scale_word_b on
    rotated rows (CPU run of the reference => IEEE division in the asymmetric step => true_div=True)"""
    g = np.load(os.path.join(GOLD, "static_writer.npz"))
    x, mask = g["x_bits"], g["mask"]
    y = Q.sel_fwht(Q.bf16_to_f32(x), mask, 32)
    assert np.array_equal(y.view(np.uint32), g["y_bits"])
    q, w = Q.static_encode(x, mask, "int4", true_div=True)
    assert np.array_equal(q, g["int4_q"]) and np.array_equal(w & 0xFFFF, g["int4_s_bits"])
    q, w = Q.static_encode(x, mask, "int4a", true_div=True)
    assert np.array_equal(q, g["int4a_q"]) and np.array_equal(w & 0xFFFF, g["int4a_w"])
    q, w = Q.static_encode(x, mask, "int2a", true_div=True)
    assert np.array_equal(q, g["int2a_q"]) and np.array_equal(w & 0xFFFF, g["int2a_w"])
    assert mask.any() and not mask.all()


# ------------------------------------------------------------------------------------------------ KIVI pages
@pytest.mark.parametrize("f8", [False, True])
@pytest.mark.parametrize("D", [128, 256])
def test_kivi_layout_matches_reference_parser(f8, D):
    """vllm_flagrot/kivi.py parse_chunks / _kcodes / _codes / dequant_groups on random chunk bytes, head dim 128 and 256"""
    g = np.load(os.path.join(GOLD, "kivi_layout.npz" if D == 128 else "kivi_layout_d256.npz"))
    tag = "f8" if f8 else "f16"
    ch = g[f"{tag}_chunks"]
    kc, km, vc, vm, vf = KV.parse_chunks(ch, D, f8)
    assert np.array_equal(kc, g[f"{tag}_kcodes"]) and np.array_equal(vc, g[f"{tag}_vcodes"])
    assert np.array_equal(vf != 0, g[f"{tag}_vf"] != 0)
    for m, ref in ((km, g[f"{tag}_km"]), (vm, g[f"{tag}_vm"])):
        flag, s, mn = KV.meta_values(m, f8)
        assert np.array_equal(np.where(flag, -s, s), ref[..., 0]) and np.array_equal(mn, ref[..., 1])
        assert np.array_equal(flag, np.signbit(ref[..., 0]))
    assert (g[f"{tag}_vf"] != 0).any() and not (g[f"{tag}_vf"] != 0).all()
    for basis in ("orig", "stored"):
        k, v = KV.dequant_groups(ch, D, dtype=np.float64, basis=basis, f8=f8)
        for a, ref in ((k, g[f"{tag}_k_{basis}"]), (v, g[f"{tag}_v_{basis}"])):
            assert a.shape == ref.shape
            assert np.abs(a - ref).max() <= 3e-6 * np.abs(ref).max(), (tag, basis)      # the reference is fp32 matmuls


def test_e4m3_conversion_exhaustive():
    """every finite E4M3 pattern round-trips; midpoints go to the even pattern; saturation at +-448"""
    b = np.array([i for i in range(256) if (i & 0x7F) != 0x7F], np.uint8)
    v = KV.e4m3_value(b)
    assert np.array_equal(KV.e4m3_bits(v) & 0x7F, b & 0x7F) and np.array_equal(np.signbit(v), (b >> 7).astype(bool))
    pos = KV.e4m3_value(np.arange(127, dtype=np.uint8)).astype(np.float64)
    mid = ((pos[:-1] + pos[1:]) / 2).astype(np.float32)              # exactly representable in fp32
    got = KV.e4m3_bits(mid)
    assert np.array_equal(got, np.where(np.arange(126) % 2 == 0, np.arange(126), np.arange(1, 127)).astype(np.uint8))
    assert KV.e4m3_bits(np.float32(1e6)) == 0x7E and KV.e4m3_bits(np.float32(-1e6)) == 0xFE
    assert KV.e4m3_value(np.uint8(0x7E)) == 448.0 and KV.e4m3_value(np.uint8(0x08)) == 2.0 ** -6
    assert KV.e4m3_value(np.uint8(0x01)) == 2.0 ** -9 and KV.e4m3_value(np.uint8(0x38)) == 1.0


def _rel_groups(rec, ref, x, axes):
    d = np.sqrt(((rec - ref) ** 2).sum(axes))
    n = np.maximum(np.sqrt(((ref - x) ** 2).sum(axes)), 1e-12)
    return d / n


@pytest.mark.parametrize("f8", [False, True])
def test_kivi_selection_matches_simulator(f8):
    """blockflag.qattention.dyn_quant (kivi2:32 / kivi2f8:32, rule att + F) on the generator of the reference's KIVI
    test: the oracle's choices equal the simulator's except where the oracle's own fp64 margin is small (the
    reference accepts 2 % mismatches between its kernels and this simulator, tests/test_kivi.py:139-140), and where
    the choices agree the stored reconstruction is the simulator's up to the storage rounding of (scale, min).  The
    simulator ran on a CPU: its step is the IEEE division (max - min) / 3 => true_div=True, as for the other vectors."""
    g = np.load(os.path.join(GOLD, "kivi_select.npz"))
    tag = "f8" if f8 else "f16"
    xk, qs, lz, co, qsc, S = g["xk_bits"], g["qs"], g["lz"], g["co"], float(g["qscale"]), int(g["S"])
    T, H, D = xk.shape
    NV = D // 32
    x = Q.bf16_to_f32(xk).astype(np.float64)
    ref = g[f"{tag}_k_rec"].astype(np.float64)
    loc, full = g[f"{tag}_k_local"].astype(bool), g[f"{tag}_k_full"].astype(bool)     # [ng, H, NV], [ng, H]
    ng = T // 32
    mism, worst, rels = 0, 0.0, []
    for gi in range(ng):
        valid = np.ones(32, bool)
        if gi == 0:
            valid[:S] = False
        for h in range(H):
            enc = KV.k_encode_group(xk[32 * gi:32 * gi + 32, h], valid, qs[h], lz[h], qsc, f8=f8, true_div=True)
            same = bool(enc["useF"]) == bool(full[gi, h]) and (full[gi, h] or np.array_equal(enc["useH"], loc[gi, h]))
            if not same:
                mism += 1
                m = enc["marginF"] if bool(enc["useF"]) != bool(full[gi, h]) else enc["marginH"][enc["useH"] != loc[gi, h]].min()
                worst = max(worst, float(m))
            # reconstruction under the SIMULATOR's choice (so that codes and meta are compared, not the choice)
            codes, meta = KV.k_stored(enc, useH=loc[gi, h], useF=full[gi, h], f8=f8)
            flag, s, mn = KV.meta_values(meta, f8)
            rec = codes.astype(np.float64) * s.astype(np.float64)[None] + mn.astype(np.float64)[None]
            if full[gi, h]:
                rec = rec @ Q.sylvester(D)
            else:
                rb = rec.reshape(32, NV, 32)
                rec = np.where(loc[gi, h][None, :, None], rb @ Q.sylvester(32), rb).reshape(32, D)
            rows = slice(32 * gi, 32 * gi + 32)
            r = _rel_groups(rec[valid], ref[rows, h][valid], x[rows, h][valid], (0, 1))
            rels.append(float(r))
    assert mism <= max(1, ng * H // 50) or worst < 1e-3, (mism, worst)
    assert worst < 2e-2, worst
    # fp16 storage of (scale, min) against the simulator's fp32 values: ~1e-3 of the quantisation error; f8: the
    # simulator stores E4M3 too, so only the reciprocal-multiply step (1 ulp of the scale) is left
    assert np.median(rels) < (1e-4 if f8 else 5e-3) and max(rels) < (2e-2 if f8 else 5e-2), (np.median(rels), max(rels))
    # values: per token; rel > 0.2 counts as a flipped choice (tests/test_kivi.py:172-175)
    xv = g["xv_bits"]
    enc = KV.v_encode(xv, co, f8=f8, true_div=True)
    codes, meta, vf = KV.v_stored(enc, f8=f8)
    flag, s, mn = KV.meta_values(meta, f8)
    Tv = xv.shape[0]
    rec = codes.reshape(Tv, H, NV, 32).astype(np.float64) * s.astype(np.float64)[..., None] + mn.astype(np.float64)[..., None]
    rec = np.where(flag[..., None], rec @ Q.sylvester(32), rec).reshape(Tv, H, D)
    rec = np.where((vf != 0)[..., None], rec @ Q.sylvester(D), rec)
    xvf = Q.bf16_to_f32(xv).astype(np.float64)
    r = _rel_groups(rec, g[f"{tag}_v_rec"].astype(np.float64), xvf, (2,))
    assert int((r > 0.2).sum()) <= max(1, r.size // 200), int((r > 0.2).sum())
    assert np.median(r) < (1e-4 if f8 else 5e-3), np.median(r)


@pytest.mark.parametrize("fmt", FMTS)
def test_page_dequantiser_head_dim_256_matches_reference(fmt):
    """vllm_flagrot/kernels.py dequant_v2_pages / dequant_cb_pages with Dh = 256 on random chunk bytes: two 128-d half
    chunks per (page, head), eight key groups, the whole-head H256 flag in the group-0 V scale word of half 0"""
    g = np.load(os.path.join(GOLD, "pages_d256.npz"))
    pool = g[f"{fmt}_pool"]
    K, V = A.dequant_pages(pool, fmt, 16, dtype=np.float64, Dh=256)
    for a, ref in ((K, g[f"{fmt}_k"]), (V, g[f"{fmt}_v"])):
        assert a.shape == ref.shape == (2, 16, 2, 256)
        assert np.isfinite(ref).all()
        assert np.abs(a - ref).max() <= 3e-6 * np.abs(ref).max(), fmt          # the reference multiplies in fp32
