"""GPU parity of the KIVI-style pages at head dim 256 (kv_v_write, kv_k_encode, kv_attn, kv_dequant with D = 256;
integrations/vllm_flagrot/csrc/kivi.cu k_v_write<256>, k_k_encode<256>, the 256-d attention launches :1997-2036 and
dequantisers) against oracle/kivi.py, whose 256-d layout the reference's parser pins (tests/golden/kivi_layout_d256.npz).
Same bars as the 128-d tests (tests/test_gpu_kivi.py): writers bit-equal given the stored flags, choices inside the
fp64 margin, pinned modes byte-equal on the whole pool; attention within 1e-2 max|ref| of fp64 and inside the
element-wise bar |err| <= 2e-3 + 1e-2 |ref|; dequantiser within 2e-6 max|ref| in fp32.  Both meta formats (3088- and
2560-byte chunks; eight sub-vectors, key cells of eight channels, the value whole-head flag of FP8 pages in slot 7).
"""
import math

import numpy as np
import pytest
import torch

from oracle import kivi as OK
from oracle import quant as Q
from tests.gpu_util import bits
from tests.test_gpu_kivi import (F8, _calib, _cb, _filled_cache, _group_rows, _groups, _kv, _ref_attn, _stored_key_flags,
                                 _stored_value_flags)

pytestmark = pytest.mark.gpu
D, NV = 256, 8


@F8
@pytest.mark.parametrize("seed,T,Hkv", [(0, 64, 2), (1, 333, 8), (2, 1, 1)])
def test_v_write_given_flags(dev, seed, T, Hkv, f8):
    from flagrot_releaser_amd import kivi as KV
    g = torch.Generator().manual_seed(seed)
    kv = _kv(T, Hkv, g, hd=D)
    _, _, co = _calib(Hkv, 8, g, hd=D)
    npg = (T + 15) // 16 + 2
    slots = torch.randperm(npg * 16, generator=g)[:T].long()
    if T > 10:
        slots[7] = -1
    init = torch.randint(0, 256, (npg, Hkv, _cb(f8, D)), generator=g, dtype=torch.uint8)
    pool = init.to(dev)
    KV.v_write(kv.to(dev), slots.to(dev), co.to(dev), None, pool, Hkv, D, f8=f8)
    torch.cuda.synchronize()
    got = pool.cpu().numpy()
    enc = OK.v_encode(bits(kv)[:, Hkv:], co.numpy(), f8=f8)
    sH, sF = _stored_value_flags(got, f8, D)
    useH = np.zeros((T, Hkv, NV), bool)
    useF = np.zeros((T, Hkv), bool)
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            useH[t], useF[t] = sH[s // 16, :, s % 16], sF[s // 16, :, s % 16]
    want = init.numpy().copy()
    OK.pack_values(want, slots.numpy(), *OK.v_stored(enc, useH, useF, f8=f8), f8=f8)
    assert np.array_equal(got, want), "value codes / meta differ from the oracle given the stored flags"
    live = (slots.numpy() >= 0)
    badF = (useF != enc["useF"]) & live[:, None]
    assert (enc["marginF"][badF] < 1e-3).all(), enc["marginF"][badF]
    badH = (useH != enc["useH"]) & ~useF[..., None] & ~enc["useF"][..., None] & live[:, None, None]
    assert (enc["marginH"][badH] < 1e-3).all(), enc["marginH"][badH]
    if T >= 64:      # a rate needs rows to be a rate of: with a dozen rows one tie on the zero or constant row is 10 %
        assert badF.mean() < 0.02 and badH.mean() < 0.02
    if T > 32:
        assert useH.any() and (~useH).any()


@F8
@pytest.mark.parametrize("mode", ["ident", "fix"])
def test_v_write_pinned_modes(dev, mode, f8):
    from flagrot_releaser_amd import kivi as KV
    g = torch.Generator().manual_seed(5)
    T, Hkv = 200, 4
    kv = _kv(T, Hkv, g, hd=D)
    _, _, co = _calib(Hkv, 8, g, hd=D)
    npg = 14
    slots = torch.randperm(npg * 16, generator=g)[:T].long()
    fix = torch.tensor([0b10010101, 1 << 16, 0b11111111, 0], dtype=torch.int32)
    pool = torch.zeros(npg, Hkv, _cb(f8, D), dtype=torch.uint8, device=dev)
    KV.v_write(kv.to(dev), slots.to(dev), co.to(dev), None, pool, Hkv, D, ident=mode == "ident",
               fix=fix.to(dev) if mode == "fix" else None, f8=f8)
    enc = OK.v_encode(bits(kv)[:, Hkv:], co.numpy(), ident=mode == "ident", fix=fix.numpy() if mode == "fix" else None,
                      f8=f8)
    want = np.zeros((npg, Hkv, _cb(f8, D)), np.uint8)
    OK.pack_values(want, slots.numpy(), *OK.v_stored(enc, f8=f8), f8=f8)
    assert np.array_equal(pool.cpu().numpy(), want)


@F8
def test_v_write_matrix_weight(dev, f8):
    """the value selection weighted by a full 256 x 256 matrix per head (e^T M e; kivi.cu:213-287): bytes equal to the
    oracle's given the stored flags, a different choice only inside the fp64 margin; M = diag(co) writes what the
    diagonal criterion writes (up to choices inside the margin); ident ignores M"""
    from flagrot_releaser_amd import kivi as KV
    g = torch.Generator().manual_seed(17)
    T, Hkv = 120, 3
    kv = _kv(T, Hkv, g, hd=D)
    _, _, co = _calib(Hkv, 8, g, hd=D)
    A = torch.randn(Hkv, D, D, generator=g) * 0.15
    M = (A @ A.transpose(1, 2) + torch.diag_embed(co)).contiguous()
    npg = (T + 15) // 16 + 1
    slots = torch.randperm(npg * 16, generator=g)[:T].long()
    xb = bits(kv)[:, Hkv:]
    for Mx, name in ((M, "dense"), (torch.diag_embed(co).contiguous(), "diagonal")):
        pool = torch.zeros(npg, Hkv, _cb(f8, D), dtype=torch.uint8, device=dev)
        KV.v_write(kv.to(dev), slots.to(dev), co.to(dev), Mx.to(dev), pool, Hkv, D, f8=f8)
        torch.cuda.synchronize()
        got = pool.cpu().numpy()
        enc = OK.v_encode(xb, co.numpy(), f8=f8, M=Mx.numpy())
        sH, sF = _stored_value_flags(got, f8, hd=D)
        sl = slots.numpy()
        useH, useF = sH[sl // 16, :, sl % 16], sF[sl // 16, :, sl % 16]
        want = np.zeros_like(got)
        OK.pack_values(want, sl, *OK.v_stored(enc, useH, useF, f8=f8), f8=f8)
        assert np.array_equal(got, want), name
        badF = useF != enc["useF"]
        badH = (useH != enc["useH"]) & ~useF[..., None] & ~enc["useF"][..., None]
        assert (enc["marginF"][badF] < 1e-3).all() and (enc["marginH"][badH] < 1e-3).all(), name
        assert badF.mean() < 0.02 and badH.mean() < 0.02
        if name == "diagonal":
            ref = torch.zeros_like(pool)
            KV.v_write(kv.to(dev), slots.to(dev), co.to(dev), None, ref, Hkv, D, f8=f8)
            assert (ref != pool).any(dim=-1).float().mean().item() < 0.05
        else:
            dg = OK.v_encode(xb, co.numpy(), f8=f8)
            assert (dg["useH"] != enc["useH"]).any()               # the dense matrix does change choices
    pool = torch.zeros(npg, Hkv, _cb(f8, D), dtype=torch.uint8, device=dev)
    ref = torch.zeros_like(pool)
    KV.v_write(kv.to(dev), slots.to(dev), co.to(dev), M.to(dev), pool, Hkv, D, ident=True, f8=f8)
    KV.v_write(kv.to(dev), slots.to(dev), co.to(dev), None, ref, Hkv, D, ident=True, f8=f8)
    assert torch.equal(pool, ref)


@F8
@pytest.mark.parametrize("seed,NG,Hkv,NQ", [(0, 4, 2, 64), (1, 6, 8, 37), (2, 1, 1, 8)])
def test_k_encode_given_flags(dev, seed, NG, Hkv, NQ, f8):
    from flagrot_releaser_amd import kivi as KV
    g = torch.Generator().manual_seed(seed)
    rows, rows2, sidx, dslot = _groups(NG, Hkv, g, hd=D)
    qs, lz, _ = _calib(Hkv, NQ, g, hd=D)
    qsc = 1 / math.sqrt(D)
    npg = 2 * NG + 3
    pool = torch.zeros(npg, Hkv, _cb(f8, D), dtype=torch.uint8, device=dev)
    KV.k_encode(rows.to(dev), sidx.to(dev), dslot.to(dev), qs.to(dev), lz.to(dev), qsc, pool, Hkv, D, src2=rows2.to(dev),
                f8=f8)
    torch.cuda.synchronize()
    got = pool.cpu().numpy()
    want = np.zeros_like(got)
    nbad = ntot = 0
    seenH = set()
    for n in range(NG):
        xb, valid = _group_rows(rows, rows2, sidx[n], Hkv)
        for h in range(Hkv):
            enc = OK.k_encode_group(xb[:, h], valid, qs[h].numpy(), lz[h].numpy(), qsc, f8=f8)
            uH, uF = _stored_key_flags(got, dslot[n].numpy(), h, f8, D)
            OK.pack_key_group(want, h, dslot[n].numpy(), valid, *OK.k_stored(enc, uH, uF, f8=f8), f8=f8)
            if uF != enc["useF"]:
                assert enc["marginF"] < 1e-3, (n, h, enc["marginF"])
                nbad += 1
            if not uF and not enc["useF"]:
                d = uH != enc["useH"]
                assert (enc["marginH"][d] < 1e-3).all(), (n, h, enc["marginH"][d])
                nbad += int(d.sum())
                seenH.update(uH.tolist())
            ntot += NV + 1
    assert np.array_equal(got, want), "key codes / meta differ from the oracle given the stored flags"
    assert nbad <= max(1, 0.02 * ntot)
    if NG * Hkv >= 8:
        assert seenH == {True, False}


@F8
@pytest.mark.parametrize("mode", ["ident", "fix"])
def test_k_encode_pinned_modes_keep_value_fields(dev, mode, f8):
    from flagrot_releaser_amd import kivi as KV
    g = torch.Generator().manual_seed(9)
    NG, Hkv = 5, 4
    rows, rows2, sidx, dslot = _groups(NG, Hkv, g, hd=D)
    qs, lz, co = _calib(Hkv, 16, g, hd=D)
    fix = torch.tensor([0b00110011, 1 << 16, 0b10000000, 0], dtype=torch.int32)
    npg = 2 * NG + 3
    init = torch.randint(0, 256, (npg, Hkv, _cb(f8, D)), generator=g, dtype=torch.uint8)
    pool = init.to(dev)
    KV.k_encode(rows.to(dev), sidx.to(dev), dslot.to(dev), qs.to(dev), lz.to(dev), 0.1, pool, Hkv, D, src2=rows2.to(dev),
                ident=mode == "ident", fix=fix.to(dev) if mode == "fix" else None, f8=f8)
    want = init.numpy().copy()
    for n in range(NG):
        xb, valid = _group_rows(rows, rows2, sidx[n], Hkv)
        for h in range(Hkv):
            enc = OK.k_encode_group(xb[:, h], valid, qs[h].numpy(), lz[h].numpy(), 0.1, ident=mode == "ident",
                                    fix=int(fix[h]) if mode == "fix" else None, f8=f8)
            OK.pack_key_group(want, h, dslot[n].numpy(), valid, *OK.k_stored(enc, f8=f8), f8=f8)
    assert np.array_equal(pool.cpu().numpy(), want)


CASES = [
    # lens, Hkv, G, kv_start, (nsplit, chunk), tail lengths
    ([96], 1, 1, 0, (1, 256), [0]),
    ([512, 300, 64], 2, 4, 0, (2, 256), [5, 0, 17]),
    ([1000, 32], 2, 8, 64, (4, 256), [31, 1]),
    ([40, 40], 2, 2, 64, (1, 256), [3, 0]),       # nothing left in the pages: tail only (and one empty sequence)
    ([333, 97, 1], 2, 3, 37, (2, 256), [2, 0, 9]),
    ([1500, 31], 1, 6, 5, (5, 320), [0, 128]),
    ([777], 4, 7, 255, (3, 288), [64]),
]


@F8
@pytest.mark.parametrize("case", range(len(CASES)))
def test_attn_against_fp64(dev, case, f8):
    attn_case(dev, CASES[case], 300 + case, f8, 1.0, label=f"case {case}")


def attn_case(dev, shape, seed, f8, el_bar, label=""):
    """one head-dim-256 decode-attention shape against fp64 attention over the oracle's dequantised pages: the
    reference's row bar, and el_bar times the element-wise bar"""
    from flagrot_releaser_amd import kivi as KV
    lens, Hkv, G, kv_start, (ns, chunk), tails = shape
    case = label
    g = torch.Generator().manual_seed(seed)
    B, Hq = len(lens), Hkv * G
    pool, bt, Ks, Vs = _filled_cache(dev, lens, Hkv, g, f8=f8, hd=D)
    T = 128
    R = B + 1
    ring = (torch.randn((R + 1) * T, 2 * Hkv, D, generator=g) * 1.5).bfloat16()
    tail_idx = torch.randperm(R + 1, generator=g)[:B].int()
    tail_len = torch.tensor(tails, dtype=torch.int32)
    cached = torch.tensor(lens, dtype=torch.int32)
    q = (torch.randn(B, Hq, D, generator=g) * 1.2).bfloat16()
    ws = KV.Workspace(B * Hkv * (ns + 1), G, D, dev)
    outbuf = torch.full((B, Hq * D + 64), 7.0, dtype=torch.bfloat16, device=dev)       # padded row stride
    out = outbuf[:, :Hq * D]
    scale = 1 / math.sqrt(D)
    ringf = Q.bf16_to_f32(bits(ring)).astype(np.float64).reshape(R + 1, T, 2 * Hkv, D)
    qf = Q.bf16_to_f32(bits(q)).astype(np.float64)
    worst_el = worst_mx = 0.0
    for rep in range(2):
        KV.attn(q.to(dev), pool, bt.to(dev), cached.to(dev), out, ns, chunk, ws, scale * math.log2(math.e), kv_start, G,
                ring=ring.to(dev), tail_len=tail_len.to(dev), tail_idx=tail_idx.to(dev), T=T, f8=f8)
        torch.cuda.synchronize()
        got = Q.bf16_to_f32(bits(out.contiguous())).astype(np.float64).reshape(B, Hq, D)
        for b in range(B):
            tb = ringf[int(tail_idx[b]), :tails[b]]
            ref = _ref_attn(qf[b], Ks[b], Vs[b], min(kv_start, lens[b]), lens[b], tb[:, :Hkv], tb[:, Hkv:], G, scale)
            if min(kv_start, lens[b]) >= lens[b] and tails[b] == 0:
                assert not got[b].any()
                continue
            err = np.abs(got[b] - ref)
            worst_el = max(worst_el, float((err / (2e-3 + 1e-2 * np.abs(ref))).max()))
            worst_mx = max(worst_mx, float(err.max() / (np.abs(ref).max() + 1e-30)))
    print(f"\n{case} f8={f8}: worst max |err| / max |ref| = {worst_mx:.2e} (bar 1e-2); element-wise "
          f"|err| / (2e-3 + 1e-2 |ref|) = {worst_el:.2f} (bar 1)", flush=True)
    assert worst_mx <= 1e-2 and worst_el <= el_bar, (case, f8, worst_mx, worst_el)
    assert (outbuf[:, Hq * D:] == 7.0).all()


def test_attn_plain_kernel_switch(dev, monkeypatch):
    """FLAGROT_KIVI_WIDE_PLAIN=1 (read at every call) sends every split through the plain fp32 kernel instead: same
    partial format, same merge, outputs within the bar of each other and of the fp64 reference"""
    from flagrot_releaser_amd import kivi as KV
    lens, Hkv, G, kv_start, (ns, chunk), tails = CASES[2]
    g = torch.Generator().manual_seed(77)
    B, Hq = len(lens), Hkv * G
    pool, bt, Ks, Vs = _filled_cache(dev, lens, Hkv, g, hd=D)
    T = 128
    ring = (torch.randn((B + 2) * T, 2 * Hkv, D, generator=g) * 1.5).bfloat16()
    tail_idx = torch.arange(B, dtype=torch.int32)
    tail_len = torch.tensor(tails, dtype=torch.int32)
    cached = torch.tensor(lens, dtype=torch.int32)
    q = (torch.randn(B, Hq, D, generator=g) * 1.2).bfloat16()
    ws = KV.Workspace(B * Hkv * (ns + 1), G, D, dev)
    scale = 1 / math.sqrt(D)
    outs = []
    for plain in ("0", "1"):
        monkeypatch.setenv("FLAGROT_KIVI_WIDE_PLAIN", plain)
        out = torch.zeros(B, Hq * D, dtype=torch.bfloat16, device=dev)
        KV.attn(q.to(dev), pool, bt.to(dev), cached.to(dev), out, ns, chunk, ws, scale * math.log2(math.e), kv_start, G,
                ring=ring.to(dev), tail_len=tail_len.to(dev), tail_idx=tail_idx.to(dev), T=T)
        torch.cuda.synchronize()
        outs.append(Q.bf16_to_f32(bits(out)).astype(np.float64).reshape(B, Hq, D))
    ringf = Q.bf16_to_f32(bits(ring)).astype(np.float64).reshape(B + 2, T, 2 * Hkv, D)
    for b in range(B):
        tb = ringf[b, :tails[b]]
        ref = _ref_attn(Q.bf16_to_f32(bits(q)).astype(np.float64)[b], Ks[b], Vs[b], min(kv_start, lens[b]), lens[b],
                        tb[:, :Hkv], tb[:, Hkv:], G, scale)
        for o in outs:
            assert (np.abs(o[b] - ref) / (2e-3 + 1e-2 * np.abs(ref))).max() <= 1.0



@F8
def test_dequant_and_torch_parser(dev, f8):
    from flagrot_releaser_amd import kivi as KV
    g = torch.Generator().manual_seed(11)
    Hkv = 3
    pool, bt, Ks, Vs = _filled_cache(dev, [416], Hkv, g, f8=f8, hd=D)
    row = bt[0].contiguous().to(dev)
    for a, n in ((0, 416), (40, 300), (64, 65)):
        k32, v32 = KV.dequant_cuda(pool, row, a, n, Hkv, D, dtype=torch.float32, f8=f8)
        kb, vb = KV.dequant_cuda(pool, row, a, n, Hkv, D, f8=f8)
        kt, vt = KV.dequant(pool, row, a, n, Hkv, D, f8=f8)
        torch.cuda.synchronize()
        for got, gotb, gott, ref in ((k32, kb, kt, Ks[0][a:n]), (v32, vb, vt, Vs[0][a:n])):
            assert got.shape == ref.shape == gotb.shape == gott.shape
            sc = np.abs(ref).max()
            assert np.abs(got.cpu().numpy() - ref).max() <= 2e-6 * sc
            assert np.abs(gott.cpu().numpy() - ref).max() <= 2e-6 * sc
            back = got.bfloat16()
            assert ((gotb.view(torch.int16).int() - back.view(torch.int16).int()).abs() <= 1).all()


def test_f8_value_flags_survive_interleaved_key_encoding(dev):
    """FP8-meta pages at head dim 256 keep a value row's whole-head flag in bit 7 of the key scale byte in slot 7 of
    the row's cell: value writes and key group encodings in any order leave the pool byte-equal to values first, keys
    after (the order of integrations/vllm_flagrot/tests/test_kivi.py:358-401)."""
    from flagrot_releaser_amd import kivi as KV
    g = torch.Generator().manual_seed(21)
    NG, Hkv, S = 4, 4, 4
    T = NG * 32
    kv = _kv(T, Hkv, g, hd=D).to(dev)
    qs, lz, co = (x.to(dev) for x in _calib(Hkv, 16, g, hd=D))
    perm = torch.randperm(2 * NG, generator=g)
    pos = torch.arange(T)
    slots = (perm[pos // 16] * 16 + pos % 16).long().to(dev)
    gp = pos.view(NG, 32)
    sid = torch.where(gp < S, -1, gp).contiguous().to(dev)
    ds = slots.view(NG, 32).contiguous()
    vfix = torch.tensor([1 << 16, 0b01100110, 1 << 16, 0], dtype=torch.int32, device=dev)
    kfix = torch.tensor([0b10011001, 1 << 16, 0, 0b11111111], dtype=torch.int32, device=dev)

    def venc(pool, a, b):
        KV.v_write(kv[a:b], slots[a:b].contiguous(), co, None, pool, Hkv, D, fix=vfix, f8=True)

    def kenc(pool, gs):
        KV.k_encode(kv, sid[gs].contiguous(), ds[gs].contiguous(), qs, lz, 0.09, pool, Hkv, D, fix=kfix, f8=True)

    pool = torch.zeros(2 * NG, Hkv, _cb(True, D), dtype=torch.uint8, device=dev)
    venc(pool, 0, 32)
    kenc(pool, [0])
    venc(pool, 32, T - 32)
    kenc(pool, list(range(1, NG - 1)))
    kenc(pool, [0])
    venc(pool, T - 32, T)
    kenc(pool, [NG - 1])
    ref = torch.zeros_like(pool)
    venc(ref, 0, T)
    kenc(ref, list(range(NG)))
    torch.cuda.synchronize()
    vf = OK.parse_chunks(ref.cpu().numpy(), D, True)[4]
    assert vf[:, 0].all() and vf[:, 2].all() and not vf[:, 1].any() and not vf[:, 3].any()
    assert torch.equal(pool, ref)
    venc(pool, 0, T)
    torch.cuda.synchronize()
    assert torch.equal(pool, ref)
