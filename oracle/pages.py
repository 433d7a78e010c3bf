"""Byte-exact page layouts of the static / key-only FlagRot caches: packers and independent parsers (numpy).

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Reference followed: the layout comment kernels/csrc/attn_decode_v2.cuh:14-46, the writer's placement
kernels/csrc/attn_decode_v2.cu:1784-1880 and INT2 helpers kernels/csrc/attn_cb_common.cuh:142-156.  The parsers are
written as gather maps straight from the layout sentences (not from the packer), so a packer mistake shows up as a
pack -> parse mismatch; both are additionally pinned by hand-derived byte positions in tests/test_oracle_pages.py.

One contiguous chunk per (page, KV head): pool[(page * Hkv + head) * CHUNK + ...], P = tokens per page.

INT4 chunk (144 P bytes), element pairs A_i = d(32 j + 4 tg + i), B_i = d(32 j + 16 + 4 tg + i), tg, j, i in 0..3:
  [0, 64P)      K codes: token row at 64 t, 32-bit word (tg, j) at row byte 16 tg + 4 j, byte i <-> (A_i, B_i)
  [64P, 128P)   V^T codes: 16-byte entry e = (w * 8 + gid) * (P / 8) + c8; entry word `sub` <-> dim
                d = 64 (sub >> 1) + 16 w + gid + 8 (sub & 1); byte i: A_i = token 8 c8 + 2 i, B_i = token 8 c8 + 2 i + 1
  [128P, 136P)  K scale words: u16 at 8 t + 2 g
  [136P, 144P)  V scale words: u16 at (g * P + 8 c8 + slot8) * 2, slot8 = odd token ? 4 + (r8 >> 1) : r8 >> 1
  symmetric bit packing (sign-magnitude of q in [-7, 7]) of word byte k: bit 7 sign A_k, bits 6..4 |B_(k+1)%4|,
  bit 3 sign B_k, bits 2..0 |A_k|;  asymmetric (c in [0, 15]): low nibble A_k, high nibble B_k.
INT2 chunk (80 P bytes):
  [0, 32P)      K codes: token t's 32-byte row at physical row t ^ ((t >> 1) & 2); row byte 8 tg + 4 jp + i; the
                2-bit field at bit 4 h + 2 b is the element of group j = 2 jp + h, b = 0: A, b = 1: B
  [32P, 64P)    V^T codes: 8-byte entry e as above; entry word m <-> d = 64 m + 16 w + gid + 8 r; byte i, field at
                bit 4 r + 2 b = token 8 c8 + 2 i + b
  [64P, 72P)    K scale words, [72P, 80P) V scale words, as INT4.

Parity status: PINNED by vectors the reference's own parsers wrote (vllm_flagrot/kernels.py parse_pages /
dequant_v2_pages / dequant_cb_pages on pools of random bytes with packed tokens, six formats x pages of 16 and 32
tokens: tests/golden/pages_*.npz, tests/test_oracle_golden.py), plus hand-derived byte positions, pack/parse round
trips and whole-pool garbage preservation (tests/test_oracle_pages.py).
"""
from __future__ import annotations

import numpy as np

D = 128
NG = 4


def chunk_bytes(fmt: str, page: int) -> int:
    return page * (80 if fmt in ("int2a", "konlya2") else 144)


def is_int2(fmt: str) -> bool:
    return fmt in ("int2a", "konlya2")


def is_sym(fmt: str) -> bool:
    return fmt in ("int4", "konly")


# --------------------------------------------------------------------------------------------------- packer
def _k_pos(d: np.ndarray):
    """dim d -> (tg, j, i, isB) of the K row."""
    j = d // 32
    r = d % 32
    isB = r // 16
    tg = (r % 16) // 4
    i = r % 4
    return tg, j, i, isB


def _v_pos(d: np.ndarray):
    """dim d -> (w, gid, hi (= d / 64), r (= (d % 16) / 8)) of the V^T entry."""
    return (d % 64) // 16, d % 8, d // 64, (d % 16) // 8


def _rmw(flat: np.ndarray, idx: np.ndarray, mask: np.ndarray, bits: np.ndarray):
    np.bitwise_and.at(flat, idx, (~mask).astype(np.uint8))
    np.bitwise_or.at(flat, idx, bits.astype(np.uint8))


def pack_tokens(pool: np.ndarray, slots: np.ndarray, codes: np.ndarray, words: np.ndarray, fmt: str, page: int):
    """write tokens into pool (uint8 [Np, Hkv, CHUNK], modified in place, only the bytes / bit fields of the written
    tokens change).  slots int64 [T] (< 0: skipped); codes [T, 2*Hkv, 128] (K rows first; symmetric: signed q,
    asymmetric: unsigned); words [T, 2*Hkv, 4] 16-bit scale words (flag bits included)."""
    Np, Hkv, CH = pool.shape
    assert CH == chunk_bytes(fmt, page) and codes.shape[1] == 2 * Hkv and codes.shape[2] == D
    P = page
    keep = np.asarray(slots) >= 0
    slots = np.asarray(slots)[keep].astype(np.int64)
    codes = np.asarray(codes)[keep].astype(np.int64)
    words = np.asarray(words)[keep].astype(np.int64) & 0xFFFF
    T = slots.shape[0]
    if T == 0:
        return
    flat = pool.reshape(-1)
    pg, pos = slots // P, slots % P
    head = np.arange(Hkv)
    base = ((pg[:, None] * Hkv + head[None, :]) * CH)[..., None]              # [T, Hkv, 1]
    posb = pos[:, None, None]
    d = np.arange(D)[None, None, :]
    kc, vc = codes[:, :Hkv], codes[:, Hkv:]
    CB = 32 if is_int2(fmt) else 64                                             # code bytes per (token, row)
    ks_off, vs_off = 2 * CB * P, 2 * CB * P + 8 * P
    tg, j, i, isB = _k_pos(d)
    w, gid, hi, r = _v_pos(d)
    c8, r8 = posb // 8, posb % 8
    vi, vB = r8 >> 1, r8 & 1
    if is_int2(fmt):
        krow = 32 * (posb ^ ((posb >> 1) & 2))
        kbyte = base + krow + 8 * tg + 4 * (j >> 1) + i
        ksh = 4 * (j & 1) + 2 * isB
        _rmw(flat, np.broadcast_to(kbyte, kc.shape).ravel(), np.broadcast_to(3 << ksh, kc.shape).ravel(),
             (kc << ksh).ravel())
        vbyte = base + CB * P + ((w * 8 + gid) * (P // 8) + c8) * 8 + 4 * hi + vi
        vsh = 4 * r + 2 * vB
        _rmw(flat, np.broadcast_to(vbyte, vc.shape).ravel(), np.broadcast_to(3 << vsh, vc.shape).ravel(),
             (vc << vsh).ravel())
    else:
        kword = base + 64 * posb + 16 * tg + 4 * j
        vword = base + CB * P + ((w * 8 + gid) * (P // 8) + c8) * 16 + 4 * (2 * hi + r)
        for cd, word, bi, bB in ((kc, kword, i, isB), (vc, vword, vi, vB)):
            word = np.broadcast_to(word, cd.shape)
            bi = np.broadcast_to(bi, cd.shape)
            bB = np.broadcast_to(bB, cd.shape).astype(bool)
            if is_sym(fmt):
                sg, mag = (cd < 0).astype(np.int64), np.abs(cd)
                a, b = ~bB, bB
                # A: sign -> bit 7, |q| -> bits 2..0 of byte i
                _rmw(flat, (word + bi)[a], np.full(a.sum(), 0x87), (sg[a] << 7) | mag[a])
                # B: sign -> bit 3 of byte i, |q| -> bits 6..4 of byte (i + 3) % 4
                _rmw(flat, (word + bi)[b], np.full(b.sum(), 0x08), sg[b] << 3)
                _rmw(flat, (word + (bi + 3) % 4)[b], np.full(b.sum(), 0x70), mag[b] << 4)
            else:
                sh = 4 * bB.astype(np.int64)
                _rmw(flat, (word + bi).ravel(), (15 << sh).ravel(), (cd << sh).ravel())
    g = np.arange(NG)[None, None, :]
    kw, vw = words[:, :Hkv], words[:, Hkv:]
    kso = base + ks_off + 8 * posb + 2 * g
    slot8 = np.where(vB == 1, 4 + vi, vi)
    vso = base + vs_off + (g * P + 8 * c8 + slot8) * 2
    for wd, off in ((kw, kso), (vw, vso)):
        off = np.broadcast_to(off, wd.shape).ravel()
        flat[off] = (wd.ravel() & 0xFF).astype(np.uint8)
        flat[off + 1] = (wd.ravel() >> 8).astype(np.uint8)


# --------------------------------------------------------------------------------------------------- parser
_MAPS: dict = {}


def _maps(fmt: str, P: int):
    """gather maps [P, 128] for K and V codes: byte offset inside the chunk and shift, built by walking the chunk
    bytes in storage order (every stored field names the (token, dim) it holds)."""
    key = (is_int2(fmt), P)
    if key in _MAPS:
        return _MAPS[key]
    kb = np.zeros((P, D), np.int64)
    ksh = np.zeros((P, D), np.int64)
    vb = np.zeros((P, D), np.int64)
    vsh = np.zeros((P, D), np.int64)
    if is_int2(fmt):
        for t in range(P):
            row = 32 * (t ^ ((t >> 1) & 2))
            for tg in range(4):
                for jp in range(2):
                    for i in range(4):
                        for h in range(2):
                            for b in range(2):
                                dd = 32 * (2 * jp + h) + 16 * b + 4 * tg + i
                                kb[t, dd], ksh[t, dd] = row + 8 * tg + 4 * jp + i, 4 * h + 2 * b
        for w in range(4):
            for gid in range(8):
                for c8 in range(P // 8):
                    e = (w * 8 + gid) * (P // 8) + c8
                    for m in range(2):
                        for i in range(4):
                            for r in range(2):
                                for b in range(2):
                                    dd, t = 64 * m + 16 * w + gid + 8 * r, 8 * c8 + 2 * i + b
                                    vb[t, dd], vsh[t, dd] = 32 * P + 8 * e + 4 * m + i, 4 * r + 2 * b
    else:
        for t in range(P):
            for tg in range(4):
                for j in range(4):
                    for i in range(4):
                        word = 64 * t + 16 * tg + 4 * j
                        kb[t, 32 * j + 4 * tg + i], ksh[t, 32 * j + 4 * tg + i] = word + i, 0          # A_i
                        kb[t, 32 * j + 16 + 4 * tg + i], ksh[t, 32 * j + 16 + 4 * tg + i] = word + i, 1  # B_i
        for w in range(4):
            for gid in range(8):
                for c8 in range(P // 8):
                    e = (w * 8 + gid) * (P // 8) + c8
                    for sub in range(4):
                        dd = 64 * (sub >> 1) + 16 * w + gid + 8 * (sub & 1)
                        for i in range(4):
                            vb[8 * c8 + 2 * i, dd], vsh[8 * c8 + 2 * i, dd] = 64 * P + 16 * e + 4 * sub + i, 0
                            vb[8 * c8 + 2 * i + 1, dd], vsh[8 * c8 + 2 * i + 1, dd] = 64 * P + 16 * e + 4 * sub + i, 1
    _MAPS[key] = (kb, ksh, vb, vsh)
    return _MAPS[key]


def _sym_codes(ch: np.ndarray, byte: np.ndarray, isB: np.ndarray) -> np.ndarray:
    """sign-magnitude element of the 32-bit word containing `byte` (offsets inside the chunk)."""
    b0 = ch[..., byte].astype(np.int64)
    word = byte & ~3
    nb = ch[..., word + ((byte & 3) + 3) % 4].astype(np.int64)               # byte holding |B|
    sA, mA = (b0 >> 7) & 1, b0 & 7
    sB, mB = (b0 >> 3) & 1, (nb >> 4) & 7
    return np.where(isB.astype(bool), np.where(sB == 1, -mB, mB), np.where(sA == 1, -mA, mA))


def parse_pages(pool: np.ndarray, fmt: str, page: int):
    """pool uint8 [Np, Hkv, CHUNK] -> raw codes int16 [Np, Hkv, P, 2, 128] (0: K, 1: V; symmetric: signed q, asymmetric:
    unsigned c, zero point NOT subtracted) and raw 16-bit scale words int32 [Np, Hkv, P, 2, 4] (flag bits included)."""
    P = page
    Np, Hkv, CH = pool.shape
    assert CH == chunk_bytes(fmt, P)
    kb, ksh, vb, vsh = _maps(fmt, P)
    if is_int2(fmt):
        K = (pool[..., kb].astype(np.int64) >> ksh) & 3
        V = (pool[..., vb].astype(np.int64) >> vsh) & 3
        so = 64 * P
    elif is_sym(fmt):
        K = _sym_codes(pool, kb, ksh)
        V = _sym_codes(pool, vb, vsh)
        so = 128 * P
    else:
        K = (pool[..., kb].astype(np.int64) >> (4 * ksh)) & 15
        V = (pool[..., vb].astype(np.int64) >> (4 * vsh)) & 15
        so = 128 * P
    t = np.arange(P)[:, None]
    g = np.arange(NG)[None, :]
    ko = so + 8 * t + 2 * g
    r8 = t % 8
    slot8 = np.where(r8 & 1, 4 + (r8 >> 1), r8 >> 1)
    vo = so + 8 * P + (g * P + 8 * (t // 8) + slot8) * 2
    rd = lambda o: pool[..., o].astype(np.int32) | (pool[..., o + 1].astype(np.int32) << 8)  # noqa: E731
    codes = np.stack([K, V], 3).astype(np.int16)
    words = np.stack([rd(ko), rd(vo)], 3)
    return codes, words
