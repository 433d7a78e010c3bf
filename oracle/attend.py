"""Dequantise-then-attend reference of the paged decode path (numpy, fp64 softmax).

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Reference followed: the attention yardstick of the reference's tests,
integrations/vllm_flagrot/tests/test_kernels.py:37-56 (ref_attn: valid range [kv_start, len), tails appended), the
page dequantisers vllm_flagrot/kernels.py:687-743 (static: stored basis; key-only 2x2: original basis, H32 per flagged
key group / H_D when the token's group-0 V word carries the flag), the static q / output rotation
test_kernels.py:139-147, and the split merge kernels/csrc/attn_merge.cuh:23-84.

Parity status: pinned by textbook identities in tests/test_oracle_attend.py (orthonormal rotations leave scores
unchanged, all-identity flags reduce to plain group dequantisation, split merge == single pass, kv_start / tail ==
concatenation, shift invariance under key centring).
"""
from __future__ import annotations

import numpy as np

from . import pages as PG
from . import quant as Q


def dequant_pages(pool: np.ndarray, fmt: str, page: int, dtype=np.float64, Dh: int = 128):
    """pool uint8 [Np, Hkv, CHUNK] -> K, V [Np, P, Hkv, Dh].
    static formats (int4 / int4a / int2a): values in the STORED (rotated) basis;
    key-only kinds (konly / konlya / konlya2): keys in the ORIGINAL basis (inverse transform per flag bits), values as
    stored (they carry no transform).
    Dh = 256 (vllm_flagrot/kernels.py:598-603, 662-667): the chunk is two 128-d half chunks, half s = dims
    [128 s, 128 s + 128), each in the 128-d layout; key flags: H32 of group g (0..7) in its K scale word, whole-head
    H256 in the token's group-0 V scale word of half 0."""
    ng = Dh // 32
    if Dh == 256:
        Np, H, CB2 = pool.shape
        halves = pool.reshape(Np, 2 * H, CB2 // 2)                                # half chunks as heads 2 h + s
        codes, words = PG.parse_pages(halves, fmt, page)                          # [Np, 2 H, P, 2, 128], [.., 2, 4]
        join = lambda a: np.moveaxis(a.reshape(Np, H, 2, *a.shape[2:]), 2, 4).reshape(Np, H, *a.shape[2:4], -1)  # noqa: E731
        codes, words = join(codes), join(words)                                   # [Np, H, P, 2, 256], [.., 2, 8]
    else:
        assert Dh == 128
        codes, words = PG.parse_pages(pool, fmt, page)
    qk = Q.QK_OF_KIND[fmt]
    c = codes.astype(dtype)                                                       # [Np, H, P, 2, Dh]
    w = words.astype(np.int64)
    if qk != "sym":
        zmask = 15 if qk == "asym4" else 3
        c = c - np.repeat(w & zmask, 32, -1).astype(dtype)
    with np.errstate(invalid="ignore"):       # bytes that were never written parse as any pattern, NaN scale words among them
        mag = Q.word_scale(w).astype(dtype)
    x = (c.reshape(*c.shape[:-1], ng, 32) * mag[..., None])                       # [Np, H, P, 2, ng, 32]
    k, v = x[..., 0, :, :], x[..., 1, :, :]
    if fmt in ("konly", "konlya", "konlya2"):
        flag_h = ((w[..., 0, :] >> 15) & 1).astype(bool)                          # [Np, H, P, ng]
        flag_f = ((w[..., 1, 0] >> 15) & 1).astype(bool)                          # [Np, H, P]
        H32, HD = Q.sylvester(32).astype(dtype), Q.sylvester(Dh).astype(dtype)
        kl = np.where(flag_h[..., None], k @ H32, k).reshape(*k.shape[:-2], Dh)
        kf = k.reshape(*k.shape[:-2], Dh) @ HD
        k = np.where(flag_f[..., None], kf, kl)
    else:
        k = k.reshape(*k.shape[:-2], Dh)
    v = v.reshape(*v.shape[:-2], Dh)
    return np.swapaxes(k, 1, 2), np.swapaxes(v, 1, 2)


def rot_blocks(x: np.ndarray, mask: np.ndarray) -> np.ndarray:
    """x [..., H, Dh] fp64; mask [H, Dh / 32]: orthonormal H32 on flagged 32-blocks (its own inverse)."""
    H32 = Q.sylvester(32)
    xb = x.reshape(*x.shape[:-1], x.shape[-1] // 32, 32)
    return np.where(np.asarray(mask).astype(bool)[..., None], xb @ H32, xb).reshape(x.shape)


def attend(q: np.ndarray, Kc: np.ndarray, Vc: np.ndarray, lens, scale: float, tails=None, kv_start: int = 0):
    """q [B, Hq, Dh]; Kc, Vc [B, Lmax, Hkv, Dh]; valid cached range of row b is [min(kv_start, len_b), len_b);
    tails: optional list of (k [n, Hkv, Dh], v [n, Hkv, Dh]) or None per row.  Returns fp64 [B, Hq, Dh]; rows
    without any key are zero."""
    q = np.asarray(q, dtype=np.float64)
    B, Hq, Dh = q.shape
    G = Hq // Kc.shape[2]
    out = np.zeros((B, Hq, Dh))
    for b in range(B):
        n = int(lens[b])
        a = min(int(kv_start), n)
        ks, vs = [np.asarray(Kc[b, a:n], dtype=np.float64)], [np.asarray(Vc[b, a:n], dtype=np.float64)]
        if tails is not None and tails[b] is not None:
            ks.append(np.asarray(tails[b][0], dtype=np.float64))
            vs.append(np.asarray(tails[b][1], dtype=np.float64))
        k = np.repeat(np.concatenate(ks), G, 1)
        v = np.repeat(np.concatenate(vs), G, 1)
        if k.shape[0] == 0:
            continue
        s = np.einsum("hd,lhd->hl", q[b], k) * scale
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        out[b] = np.einsum("hl,lhd->hd", p, v)
    return out


def gather_cache(Kp: np.ndarray, Vp: np.ndarray, block_table: np.ndarray, Lmax: int, page: int):
    """Kp, Vp [Np, P, Hkv, Dh] + block_table int [B, n] -> Kc, Vc [B, npg * P, Hkv, Dh] (npg = ceil(Lmax / P))."""
    npg = max(1, -(-int(Lmax) // page))
    bt = np.asarray(block_table)[:, :npg].astype(np.int64)
    B = bt.shape[0]
    sh = (B, npg * page) + Kp.shape[2:]
    return Kp[bt].reshape(sh), Vp[bt].reshape(sh)


def decode_reference(q_bits, pool, fmt, page, block_table, lens, scale, kmask=None, vmask=None, tail=None,
                     tail_len=None, tail_idx=None, kv_start=0):
    """the full oracle of one decode launch: q_bits uint16 [B, Hq, Dh] bf16 patterns (Dh 128 | 256); tail uint16
    [R, W, 2*Hkv, Dh] bf16 patterns (original basis).  Static formats: q is rotated by kmask, tails by kmask / vmask,
    and the result is rotated back by vmask.  Returns fp64 [B, Hq, Dh]."""
    q = Q.bf16_to_f32(q_bits).astype(np.float64)
    B, Hq, Dh = q.shape
    Hkv = pool.shape[1]
    G = Hq // Hkv
    Lmax = max(int(max(lens)) if len(lens) else 1, 1)
    # only the pages the block table names are parsed: free pages may hold any bytes (scale words that read as NaN)
    npg = max(1, -(-Lmax // page))
    bt = np.asarray(block_table)[:, :npg].astype(np.int64)
    used, inv = np.unique(bt, return_inverse=True)
    with np.errstate(invalid="ignore"):       # slots past a sequence's end inside its last page are garbage as well
        Kp, Vp = dequant_pages(pool[used], fmt, page, Dh=Dh)
    Kc, Vc = gather_cache(Kp, Vp, inv.reshape(bt.shape), Lmax, page)
    tails = None
    if tail is not None:
        tails = []
        for b in range(B):
            row = int(tail_idx[b]) if tail_idx is not None else b
            n = int(tail_len[b])
            t = Q.bf16_to_f32(tail[row, :n]).astype(np.float64)
            tails.append((t[:, :Hkv], t[:, Hkv:]))
    static = fmt in ("int4", "int4a", "int2a")
    if static and kmask is not None:
        q = rot_blocks(q.reshape(B, Hkv, G, Dh).swapaxes(1, 2), kmask).swapaxes(1, 2).reshape(B, Hq, Dh)
        if tails is not None:
            tails = [(rot_blocks(k, kmask), v) for k, v in tails]
    if static and vmask is not None and tails is not None:
        tails = [(k, rot_blocks(v, vmask)) for k, v in tails]
    o = attend(q, Kc, Vc, lens, scale, tails, kv_start)
    if static and vmask is not None:
        o = rot_blocks(o.reshape(B, Hkv, G, Dh).swapaxes(1, 2), vmask).swapaxes(1, 2).reshape(B, Hq, Dh)
    return o


def merge_partials(o_parts: np.ndarray, m_parts: np.ndarray, l_parts: np.ndarray) -> np.ndarray:
    """log2-domain merge of split partials: o_parts [S, ..., Dh] (unnormalised sums), m_parts [S, ...] (running maxima,
    -inf for empty parts), l_parts [S, ...] (sums of 2^(s - m)).  Rows without any key give 0."""
    M = m_parts.max(0)
    with np.errstate(invalid="ignore"):
        w = np.where(np.isneginf(m_parts), 0.0, np.exp2(m_parts - np.where(np.isneginf(M), 0.0, M)))
    L = (w * l_parts).sum(0)
    o = (w[..., None] * o_parts).sum(0)
    return o * np.where(L > 0, 1.0 / np.where(L > 0, L, 1.0), 0.0)[..., None]
