"""Oracle of the KIVI-style FlagRot INT2 pages: quantiser, value / key-group encoders, page layout, dequantiser.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Reference followed: integrations/vllm_flagrot/csrc/kivi.cu:1-35 (layout), :94-125 (quantiser), :164-328 (value
writer), :344-663 (key group encoder), vllm_flagrot/kivi.py:184-265 (page parser / dequantiser), and the simulator
semantics blockflag/formats.py:103-113 (fake_kivi).

Quantiser of a group with (mn, mx): s = (mx - mn) * fp32(1/3); code = rint(clamp((x - mn) / (s == 0 ? 1 : s), 0, 3));
rec = code * s + mn, every operation rounded to fp32.  Stored meta = fp16(s) (sign bit = flag) and fp16(mn); the
codes come from the fp32 values.  FP8-meta pages (f8; kivi.cu:28-35,84-88,123-128, blockflag/formats.py:195-205):
s and mn are rounded to E4M3 first (nearest even, saturating at +-448) and the codes come from the STORED values; a
10 D-byte chunk holds (s8 | flag << 7, m8) byte pairs, the value whole-head flag in bit 7 of a key scale byte.

Selection (identity / H32 per 32-dim sub-vector / whole-head H_D):
  values   per token, squared reconstruction error weighted by c_o per channel;
  keys     per 32-token group, rule 'att': w[t, q] = min(1, exp(qsc * x_t . q - lz_q)) over the calibration queries,
           error of a candidate = sum_{t, q} w (e_t . q)^2 (restricted to the sub-vector's channels for the local
           choice).
The reference accumulates these errors in fp32 with fused multiply-adds in a thread-dependent order, so a choice is
not reproducible bit for bit across implementations; the oracle evaluates them in fp64 and returns the decision
margins, and the parity tests (i) require bit-equal codes and meta GIVEN the stored flags, and (ii) allow a different
choice only where the fp64 margin is below 1e-3 relative.  "ident" and "fix" modes have no data-dependent choice and
are pinned bit for bit.

Parity status: PINNED by vectors the reference's own Python wrote (tests/golden/make_golden.py ->
tests/golden/kivi_layout.npz, kivi_select.npz; tests/test_oracle_golden.py): the page layout, the kbit interleave, the
meta cells, the flag positions and the dequantiser (both bases, FP16 and FP8 meta) against vllm_flagrot/kivi.py
parse_chunks / _kcodes / _codes / dequant_groups on random chunk bytes; the quantiser, the E4M3 conversion and the
selection rule against blockflag.qattention.dyn_quant (kivi2:32 and kivi2f8:32, rule att + F; keys per 32-token group
with sink tokens left out, values per token): same choices on every group of the vectors (the reference's own test
accepts 2 % mismatches between its kernels and that simulator, integrations/vllm_flagrot/tests/test_kivi.py:139-140)
and the same reconstruction up to the storage rounding of (scale, min).  At the bit level a choice near a tie stays
undetermined by construction (fp32 accumulation order of the reference's kernels), which the margins cover.
"""
from __future__ import annotations

import numpy as np

from . import quant as Q

F32 = np.float32
PAGE, GRP = 16, 32


def chunk_bytes(D: int, f8: bool = False) -> int:
    return 10 * D if f8 else 12 * D + 16


def kbit(i):
    return 2 * (i >> 1) + 16 * (i & 1)


# --------------------------------------------------------------------------------------------------- FP8 E4M3
# (kivi.cu:113-121 e4m3_bits / e4m3_val; blockflag/formats.py:189-192 _e4m3: clamp to +-448, round to nearest even)
def _e4m3_table():
    b = np.arange(127, dtype=np.int64)                    # non-negative finite patterns 0x00 .. 0x7E
    e, m = b >> 3, b & 7
    return np.where(e == 0, m * 2.0 ** -9, (8 + m) * 2.0 ** (e - 10.0))


_E4M3 = _e4m3_table()                                     # 0, 2^-9, ..., 448 (ascending; the pattern is the index)


def e4m3_bits(x):
    """fp32 -> E4M3 byte (sign | 4 exponent | 3 mantissa bits, bias 7, no infinities), round to nearest even,
    saturating at +-448."""
    x = np.asarray(x, F32)
    a = np.minimum(np.abs(x).astype(np.float64), 448.0)
    hi = np.clip(np.searchsorted(_E4M3, a, side="left"), 0, 126)         # first pattern >= a
    lo = np.maximum(hi - 1, 0)
    dl, dh = a - _E4M3[lo], _E4M3[hi] - a
    pick_lo = (dl < dh) | ((dl == dh) & ((lo & 1) == 0))
    idx = np.where(pick_lo, lo, hi).astype(np.uint8)
    return (idx | np.where(np.signbit(x), 0x80, 0).astype(np.uint8)).astype(np.uint8)


def e4m3_value(b):
    b = np.asarray(b).astype(np.int64)
    v = _E4M3[np.minimum(b & 0x7F, 126)]
    return np.where(b & 0x80, -v, v).astype(F32)


# --------------------------------------------------------------------------------------------------- quantiser
def kivi_params(mn, mx, f8: bool = False, true_div: bool = False):
    """(scale, min) the codes are computed from: fp32 values, or (f8) the stored E4M3 values (kivi.cu:123-128).
    true_div: the step as the simulator computes it on a CPU, (mx - mn) / 3 (blockflag/formats.py:109); the kernels,
    like torch on a GPU, multiply by fp32(1/3) (kivi.cu:97-99) -- one ulp apart at most."""
    d = (mx - mn).astype(F32)
    s, m = ((d / F32(3.0)) if true_div else (d * F32(1.0 / 3.0))).astype(F32), mn.astype(F32)
    if f8:
        s, m = e4m3_value(e4m3_bits(s)), e4m3_value(e4m3_bits(m))
    return s, m


def kivi_code(x, mn, s):
    d = np.where(s == 0, F32(1), s).astype(F32)
    q = np.clip(((x - mn) / d).astype(F32), F32(0), F32(3))
    return np.rint(q).astype(np.uint8)


def kivi_rec(code, mn, s):
    return (code.astype(F32) * s + mn).astype(F32)


def _cands(x):
    """x fp32 [..., D] -> the three candidate bases [3, ..., D]: identity, H32 per sub-vector, H_D."""
    D = x.shape[-1]
    return np.stack([x, Q.fwht(x, 32), Q.fwht(x, D)])


def _back(y, c):
    D = y.shape[-1]
    return y if c == 0 else Q.fwht(y, 32 if c == 1 else D)


# --------------------------------------------------------------------------------------------------- value encoder
def v_encode(x_bits, co, ident=False, fix=None, f8=False, true_div=False, M=None):
    """x_bits uint16 [T, H, D] bf16 V rows; co fp32 [H, D].  Returns dict: codes uint8 [3, T, H, D] per candidate,
    s, mn fp32 [3, T, H, NV], useH bool [T, H, NV], useF bool [T, H] (fp64 decision), margins (relative gaps).
    M fp32 [H, D, D] (kivi.cu:213-287; ignored with ident / fix, like the reference): the error e of a candidate, in the
    original basis, counts as e^T M e instead of sum co e^2 -- per sub-vector with the diagonal 32-block of M only, for
    the whole-head candidate and for the combination of the chosen sub-vector candidates with all of M.
    Parity of the M form: pinned by its reduction to the diagonal form for M = diag(co) and by a brute-force
    evaluation of the quadratic forms (tests/test_oracle_kivi.py); no reference-written vector covers it."""
    x = Q.bf16_to_f32(x_bits)
    T, H, D = x.shape
    NV = D // 32
    ys = _cands(x)
    g = ys.reshape(3, T, H, NV, 32)
    s, mn = kivi_params(g.min(-1), g.max(-1), f8, true_div)
    codes = kivi_code(g, mn[..., None], s[..., None])
    rec = kivi_rec(codes, mn[..., None], s[..., None]).reshape(3, T, H, D)
    ds = [(_back(rec[c], c) - x).astype(np.float64) for c in range(3)]
    if M is None or ident or fix is not None:
        err = [(d * d * np.asarray(co, np.float64)[None]).reshape(T, H, NV, 32).sum(-1) for d in ds]
        eI, eH, eF = err[0], err[1], err[2].sum(-1)
        useH = eH < eI
        eB = np.where(useH, eH, eI).sum(-1)
    else:
        Mh = np.asarray(M, np.float64)                                              # [H, D, D]
        Mb = np.stack([Mh[:, 32 * j:32 * j + 32, 32 * j:32 * j + 32] for j in range(NV)], 1)     # [H, NV, 32, 32]
        local = lambda d: np.einsum("thji,hjik,thjk->thj", d.reshape(T, H, NV, 32), Mb, d.reshape(T, H, NV, 32))  # noqa: E731
        whole = lambda d: np.einsum("thi,hik,thk->th", d, Mh, d)                                # noqa: E731
        eI, eH, eF = local(ds[0]), local(ds[1]), whole(ds[2])
        useH = eH < eI
        eB = whole(np.where(np.repeat(useH, 32, -1), ds[1], ds[0]))
    useF = eF < eB
    mH = np.abs(eH - eI) / np.maximum(eH + eI, 1e-300)
    mF = np.abs(eF - eB) / np.maximum(eF + eB, 1e-300)
    if ident:
        useH[:] = False
        useF[:] = False
    if fix is not None and not ident:
        fx = np.asarray(fix).astype(np.int64)
        useH = np.broadcast_to(((fx[:, None] >> np.arange(NV)[None]) & 1).astype(bool)[None], (T, H, NV)).copy()
        useF = np.broadcast_to(((fx >> 16) & 1).astype(bool)[None], (T, H)).copy()
    return dict(codes=codes.reshape(3, T, H, D), s=s, mn=mn, useH=useH, useF=useF, marginH=mH, marginF=mF)


def v_stored(enc, useH=None, useF=None, f8=False):
    """stored value fields for the given flags (default: the oracle's own): codes uint8 [T, H, D], meta uint16
    [T, H, NV, 2] (fp16 scale with sign = H32 and not H_D, fp16 min; f8: uint8 E4M3 bytes, flag in bit 7 of the
    scale byte), vf uint8 [T, H]."""
    useH = enc["useH"] if useH is None else useH
    useF = enc["useF"] if useF is None else useF
    T, H, NV = useH.shape
    cand = np.where(useF[..., None], 2, useH.astype(np.int64))                     # [T, H, NV]
    pick = lambda a: np.take_along_axis(a, cand[None], 0)[0]                       # noqa: E731
    s, mn = pick(enc["s"]), pick(enc["mn"])
    codes = np.take_along_axis(enc["codes"].reshape(3, T, H, NV, 32), cand[None, ..., None], 0)[0].reshape(T, H, -1)
    if f8:
        sb = np.where(cand == 1, e4m3_bits(s) | 0x80, e4m3_bits(s)).astype(np.uint8)
        return codes, np.stack([sb, e4m3_bits(mn)], -1).astype(np.uint8), useF.astype(np.uint8)
    sb = Q.f16_bits(s).astype(np.uint16) & 0x7FFF
    sb = np.where(cand == 1, sb | 0x8000, sb).astype(np.uint16)
    meta = np.stack([sb, Q.f16_bits(mn)], -1).astype(np.uint16)
    return codes, meta, useF.astype(np.uint8)


# --------------------------------------------------------------------------------------------------- key group encoder
def k_encode_group(x_bits, valid, qs, lz, qsc, ident=False, fix=None, f8=False, true_div=False):
    """one 32-token group of one KV head: x_bits uint16 [32, D] (rows of invalid tokens ignored), valid bool [32];
    qs fp32 [NQ, D], lz fp32 [NQ].  Returns dict: codes uint8 [3, 32, D], s, mn fp32 [3, D] (per channel over the valid
    tokens), useH bool [NV], useF bool, margins."""
    x = Q.bf16_to_f32(x_bits)
    x = np.where(valid[:, None], x, F32(0))
    D = x.shape[-1]
    NV = D // 32
    ys = _cands(x)                                                                # [3, 32, D]
    big = np.where(valid[None, :, None], ys, F32(np.inf))
    sml = np.where(valid[None, :, None], ys, F32(-np.inf))
    s, mn = kivi_params(big.min(1), sml.max(1), f8, true_div)                      # [3, D]
    codes = kivi_code(ys, mn[:, None], s[:, None])
    rec = kivi_rec(codes, mn[:, None], s[:, None])
    res = dict(codes=codes, s=s, mn=mn)
    if ident:
        res.update(useH=np.zeros(NV, bool), useF=False, marginH=np.ones(NV), marginF=1.0)
        return res
    if fix is not None:
        fx = int(fix)
        res.update(useH=np.array([(fx >> j) & 1 for j in range(NV)], bool), useF=bool((fx >> 16) & 1),
                   marginH=np.ones(NV), marginF=1.0)
        return res
    e = [np.where(valid[:, None], _back(rec[c], c) - x, F32(0)).astype(np.float64) for c in range(3)]
    qd = np.asarray(qs, np.float64)
    # the weight is min(1, e^(score - lz)): the exponent is capped at 0 first (the rows scaled x200 of the tests would overflow exp)
    w = np.exp(np.minimum(0.0, float(qsc) * (x.astype(np.float64) @ qd.T) - np.asarray(lz, np.float64)[None]))
    w = np.where(valid[:, None], w, 0.0)                                           # [32, NQ]
    loc = lambda ec: np.stack([(w * (ec[:, 32 * j:32 * j + 32] @ qd[:, 32 * j:32 * j + 32].T) ** 2).sum()  # noqa: E731
                               for j in range(NV)])
    EI, EH = loc(e[0]), loc(e[1])
    useH = EH < EI
    eb = np.where(np.repeat(useH, 32)[None], e[1], e[0])
    EB = (w * (eb @ qd.T) ** 2).sum()
    EF = (w * (e[2] @ qd.T) ** 2).sum()
    res.update(useH=useH, useF=bool(EF < EB), marginH=np.abs(EH - EI) / np.maximum(EH + EI, 1e-300),
               marginF=abs(EF - EB) / max(EF + EB, 1e-300))
    return res


def k_stored(enc, useH=None, useF=None, f8=False):
    """stored key fields of a group for the given flags: codes uint8 [32, D], meta uint16 [D, 2] per channel (fp16
    scale with the flag signs: channel j < NV carries 'sub-vector j is H32' (only when not H_D), channel NV carries
    'whole-head H_D'; fp16 min).  f8: meta uint8 [D, 2] E4M3 bytes; the flags sit in bit 7 of the scale bytes of
    channels j NV (slot 0 of cell j) and NV NV (slot 0 of cell NV); bit 7 of the channels k NV + NV - 1 (slot NV - 1
    of a cell) belongs to the value writer and is returned as 0 here (pack_key_group keeps what the page holds)."""
    useH = enc["useH"] if useH is None else np.asarray(useH, bool)
    useF = enc["useF"] if useF is None else bool(useF)
    D = enc["s"].shape[-1]
    NV = D // 32
    cand = np.full(D, 2) if useF else np.repeat(useH.astype(np.int64), 32)
    idx = np.arange(D)
    s, mn = enc["s"][cand, idx], enc["mn"][cand, idx]
    codes = enc["codes"][cand, :, idx].T                                            # [32, D]
    neg = np.zeros(D, bool)
    st = NV if f8 else 1                                                            # channel stride of the flag cells
    if useF:
        neg[NV * st] = True
    else:
        neg[0:NV * st:st] = useH
    if f8:
        sb = np.where(neg, e4m3_bits(s) | 0x80, e4m3_bits(s)).astype(np.uint8)
        return codes.astype(np.uint8), np.stack([sb, e4m3_bits(mn)], -1).astype(np.uint8)
    sb = Q.f16_bits(s).astype(np.uint16) & 0x7FFF
    sb = np.where(neg, sb | 0x8000, sb).astype(np.uint16)
    return codes.astype(np.uint8), np.stack([sb, Q.f16_bits(mn)], -1).astype(np.uint16)


# --------------------------------------------------------------------------------------------------- page layout
def pack_values(pool, slots, codes, meta, vf, f8=False):
    """pool uint8 [Np, H, CB] in place: value codes / meta / flag of tokens at slots (< 0 skipped).  f8: the whole-head
    flag goes to bit 7 of the KEY scale byte of the token's cell, slot NV - 1 (kivi.cu:312-315), other bits kept."""
    Np, H, CB = pool.shape
    D = codes.shape[-1]
    NV = D // 32
    assert CB == chunk_bytes(D, f8)
    vc0, vm0 = (5 * D, 9 * D) if f8 else (6 * D, 10 * D)
    for t, sl in enumerate(np.asarray(slots)):
        if sl < 0:
            continue
        pg, off = divmod(int(sl), PAGE)
        c = codes[t].reshape(H, D // 4, 4).astype(np.uint8)
        pool[pg, :, vc0 + off * (D // 4):vc0 + (off + 1) * (D // 4)] = c[..., 0] | (c[..., 1] << 2) | (c[..., 2] << 4) | (c[..., 3] << 6)
        if f8:
            pool[pg, :, vm0 + off * 2 * NV:vm0 + (off + 1) * 2 * NV] = meta[t].reshape(H, NV * 2).astype(np.uint8)
            kb = 4 * D + off * 2 * NV + 2 * (NV - 1)
            pool[pg, :, kb] = (pool[pg, :, kb] & 0x7F) | np.where(np.asarray(vf[t]) != 0, 0x80, 0).astype(np.uint8)
            continue
        m = meta[t].reshape(H, NV * 2).astype(np.uint16)
        pool[pg, :, vm0 + off * (D // 8):vm0 + (off + 1) * (D // 8)] = m.view(np.uint8).reshape(H, -1)
        pool[pg, :, 12 * D + off] = vf[t]


def pack_key_group(pool, head, dslot, valid, codes, meta, f8=False):
    """one group of one head: codes uint8 [32, D] at the page slots dslot [32] of the valid tokens, meta uint16 [D, 2]
    (f8: uint8 [D, 2]) spread over the 32 cells (cell i holds channels [i NV, (i + 1) NV)).  f8: bit 7 of a cell's
    last scale byte (slot NV - 1) is the value writer's and keeps what the page holds (kivi.cu:643)."""
    D = codes.shape[-1]
    NV = D // 32
    assert pool.shape[-1] == chunk_bytes(D, f8)
    for t in range(32):
        pg, off = divmod(int(dslot[t]), PAGE)
        if valid[t]:
            words = np.zeros(D // 16, np.uint32)
            for c in range(D):
                words[c // 16] |= np.uint32(int(codes[t, c]) & 3) << np.uint32(kbit(c % 16))
            pool[pg, head, off * (D // 4):(off + 1) * (D // 4)] = words.view(np.uint8)
        if f8:
            m = meta[t * NV:(t + 1) * NV].astype(np.uint8).reshape(-1).copy()
            kb = 4 * D + off * 2 * NV
            m[2 * (NV - 1)] = (m[2 * (NV - 1)] & 0x7F) | (pool[pg, head, kb + 2 * (NV - 1)] & 0x80)
            pool[pg, head, kb:kb + 2 * NV] = m
            continue
        m = meta[t * NV:(t + 1) * NV].astype(np.uint16)
        pool[pg, head, 4 * D + off * (D // 8):4 * D + (off + 1) * (D // 8)] = m.reshape(-1).view(np.uint8)


def parse_chunks(ch, D, f8=False):
    """chunks uint8 [np, H, CB] -> key codes [np, H, 16, D] uint8, key meta [np, H, 16, NV, 2] (uint16 fp16 patterns;
    f8: uint8 E4M3 bytes), value codes, value meta (same types), vf uint8 [np, H, 16] (f8: bit 7 of the key scale byte
    of the token's cell, slot NV - 1)."""
    npg, H, CB = ch.shape
    NV = D // 32
    assert CB == chunk_bytes(D, f8)
    kw = np.ascontiguousarray(ch[..., :4 * D]).view(np.uint32).reshape(npg, H, PAGE, D // 16)
    sh = np.array([kbit(i) for i in range(16)], np.uint32)
    kc = ((kw[..., None] >> sh) & 3).reshape(npg, H, PAGE, D).astype(np.uint8)
    vc0 = 5 * D if f8 else 6 * D
    vb = ch[..., vc0:vc0 + 4 * D].reshape(npg, H, PAGE, D // 4)
    vc = ((vb[..., None] >> np.array([0, 2, 4, 6], np.uint8)) & 3).reshape(npg, H, PAGE, D).astype(np.uint8)
    if f8:
        km = ch[..., 4 * D:5 * D].reshape(npg, H, PAGE, NV, 2)
        vm = ch[..., 9 * D:10 * D].reshape(npg, H, PAGE, NV, 2)
        return kc, km, vc, vm, (km[..., NV - 1, 0] >> 7).astype(np.uint8)
    km = np.ascontiguousarray(ch[..., 4 * D:6 * D]).view(np.uint16).reshape(npg, H, PAGE, NV, 2)
    vm = np.ascontiguousarray(ch[..., 10 * D:12 * D]).view(np.uint16).reshape(npg, H, PAGE, NV, 2)
    vf = ch[..., 12 * D:12 * D + PAGE]
    return kc, km, vc, vm, vf


def meta_values(m, f8=False):
    """meta patterns [..., 2] -> (flag bool, |scale|, min) as fp32"""
    if f8:
        return (m[..., 0] >> 7).astype(bool), e4m3_value(m[..., 0] & 0x7F), e4m3_value(m[..., 1])
    return (m[..., 0] >> 15).astype(bool), Q.f16_value(m[..., 0] & 0x7FFF), Q.f16_value(m[..., 1])


def dequant_groups(ch, D, dtype=np.float64, basis="orig", f8=False):
    """chunks of WHOLE groups [2 ng, H, CB] (pages 2 g, 2 g + 1 in order) -> K, V [2 ng 16, H, D]; basis "orig": in
    the original basis (inverse H32 / H_D applied), "stored": as the codes stand."""
    npg, H, _ = ch.shape
    ng = npg // 2
    NV = D // 32
    kc, km, vc, vm, vf = parse_chunks(ch, D, f8)
    kmg = km.reshape(ng, 2, H, PAGE, NV, 2).transpose(0, 2, 1, 3, 4, 5).reshape(ng, H, D, 2)
    flag, s, mn = meta_values(kmg, f8)
    st = NV if f8 else 1                            # f8: key flag j at channel j NV, whole head at channel NV NV
    lbits = flag[..., 0:NV * st:st]                                                # [ng, H, NV]
    fbit = flag[..., NV * st]                                                      # [ng, H]
    s, mn = s.astype(dtype), mn.astype(dtype)
    codes = kc.reshape(ng, 2, H, PAGE, D).transpose(0, 2, 1, 3, 4).reshape(ng, H, 32, D).astype(dtype)
    k = codes * s[:, :, None] + mn[:, :, None]
    H32, HD = Q.sylvester(32).astype(dtype), Q.sylvester(D).astype(dtype)
    if basis == "orig":
        kb = k.reshape(ng, H, 32, NV, 32)
        kh = np.where((lbits & ~fbit[..., None])[:, :, None, :, None], kb @ H32, kb).reshape(ng, H, 32, D)
        k = np.where(fbit[:, :, None, None], k @ HD, kh)
    k = k.transpose(0, 2, 1, 3).reshape(ng * 32, H, D)
    vl, vs, vmn = meta_values(vm, f8)
    v = vc.reshape(npg, H, PAGE, NV, 32).astype(dtype) * vs.astype(dtype)[..., None] + vmn.astype(dtype)[..., None]
    if basis == "orig":
        vh = np.where(vl[..., None], v @ H32, v).reshape(npg, H, PAGE, D)
        v = np.where((vf != 0)[..., None], v.reshape(npg, H, PAGE, D) @ HD, vh)
    v = v.reshape(npg, H, PAGE, D).transpose(0, 2, 1, 3).reshape(npg * PAGE, H, D)
    return k, v


def attention_reference(q, K, V, kv_start, cached, tailK, tailV, G, scale):
    """fp64 softmax attention of one sequence (the yardstick of kv_attn; reference test:
    integrations/vllm_flagrot/tests/test_kivi.py:235-247): q [Hq, D]; K, V [n, Hkv, D] dequantised page rows, of which
    rows [kv_start, cached) count; tailK, tailV [m, Hkv, D] BF16 ring rows.  Rows without any key give 0."""
    Hq, D = q.shape
    out = np.zeros((Hq, D))
    for hq in range(Hq):
        h = hq // G
        k = np.concatenate([K[kv_start:cached, h], tailK[:, h]])
        v = np.concatenate([V[kv_start:cached, h], tailV[:, h]])
        if len(k) == 0:
            continue
        sc = (k @ q[hq]) * scale
        p = np.exp(sc - sc.max())
        out[hq] = (p / p.sum()) @ v
    return out


def lse_merge(oa_bits, la, ob_bits, lb):
    """bf16 LSE merge of two partial attentions: oa, ob uint16 [n, H, D] bf16 patterns, la, lb fp32 [H, n] natural-log
    LSE (+inf treated as -inf).  fp32, every operation rounded on its own; exp in fp32 of the library."""
    oa, ob = Q.bf16_to_f32(oa_bits), Q.bf16_to_f32(ob_bits)
    a = np.where(np.isposinf(la), -np.inf, la).astype(F32).T[..., None]
    b = np.where(np.isposinf(lb), -np.inf, lb).astype(F32).T[..., None]
    m = np.maximum(a, b)
    with np.errstate(invalid="ignore"):
        wa, wb = np.exp((a - m).astype(F32)).astype(F32), np.exp((b - m).astype(F32)).astype(F32)
        num = ((oa * wa).astype(F32) + (ob * wb).astype(F32)).astype(F32)
        return Q.bf16_bits((num / (wa + wb).astype(F32)).astype(F32))
