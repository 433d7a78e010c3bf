"""Oracle of the prefix-cached multi-query prefill path: q preparation, masked attention over dequantised pages,
item merge, BF16 window gather and sink / window LSE merge.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Reference followed: integrations/vllm_flagrot/csrc/mq_prefill.cu:789-823 (k_mq_prep: fp32 butterflies, whole-head
H128 / 8, orthonormal H32 on flagged groups, * qscale, one rounding to fp16), :345-498 (row / key visibility of k_mq:
row r = token r / G, q head h G + r % G; key j visible iff kmin <= j <= max(p - shift, ext), j < nk), :716-772 (merge:
log2-domain maxima, natural-log LSE), :1350-1465 (window gather, sink + window merge), and the fp64 yardstick of the
reference's own check, integrations/vllm_flagrot/scripts/bench_mq_prefill.py:82-95.

Parity status: prep_q is an operation-by-operation fp32 restatement, pinned in tests/test_oracle_mq.py by the matrix
form (Sylvester matrices in fp64), by exactness on power-of-two inputs and by H (H x) = x; the attention yardstick is
pinned by brute force over explicit visibility sets and by the closed forms of uniform scores; merges by "merge of
parts == attention over the concatenation".
"""
from __future__ import annotations

import numpy as np

from . import quant as Q

F32 = np.float32
NO_EXT = -(1 << 30)


def _butterflies(x: np.ndarray, n: int) -> np.ndarray:
    """unnormalised Sylvester-Hadamard butterflies (a + b, a - b), partner distance 1, 2, 4, ..., fp32."""
    y = np.asarray(x, dtype=F32).reshape(-1, n).copy()
    lane = np.arange(n)
    h = 1
    while h < n:
        lo = lane[(lane & h) == 0]
        a, b = y[:, lo], y[:, lo + h]
        nxt = np.empty_like(y)
        nxt[:, lo] = a + b
        nxt[:, lo + h] = a - b
        y = nxt
        h *= 2
    return y.reshape(np.shape(x))


def prep_q(q, G: int, qscale: float, idx=None, kfull=None, kmask=None) -> np.ndarray:
    """q fp32 values [n, Hq, D] (bf16 inputs are passed as their exact fp32 values) -> fp16 bit patterns
    [m, Hq, D]: rows idx; whole-head unnormalised H_D times 0.125 (D = 128) or 0.0625 (D = 256; mq_prefill.cu:1319-1323)
    where kfull[kv head]; orthonormal H32 on the groups kmask[kv head, g]; times fp32(qscale); every step rounded to
    fp32, one final rounding to fp16."""
    x = np.asarray(q, dtype=F32)
    if idx is not None:
        x = x[np.asarray(idx, dtype=np.int64)]
    m, Hq, D = x.shape
    hk = np.arange(Hq) // G
    if kfull is not None:
        f = np.asarray(kfull).astype(bool)[hk]
        full = (_butterflies(x, D) * F32(0.125 if D == 128 else 0.0625)).astype(F32)
        x = np.where(f[None, :, None], full, x)
    if kmask is not None:
        km = np.asarray(kmask).astype(bool).reshape(-1, D // 32)[hk]                # [Hq, 4]
        rot = Q.fwht(x, 32)
        x = np.where(np.repeat(km, 32, -1)[None], rot, x)
    return Q.f16_bits((x * F32(qscale)).astype(F32))


def visible(pos: int, nk: int, shift: int, kmin: int = 0, ext: int = NO_EXT) -> np.ndarray:
    """indices of the page keys the row at position pos attends to"""
    hi = min(nk - 1, max(pos - shift, ext))
    return np.arange(max(kmin, 0), hi + 1) if hi >= kmin else np.zeros(0, np.int64)


def attention(q16_bits, K, V, reqs, G: int, shift: int, kmin: int = 0, ext=None):
    """fp64 yardstick.  q16_bits uint16 [m, Hq, 128] fp16 patterns in compact rows (pre-scaled: scores are in log2
    units); K, V: per block-table row r, float arrays [>= nk, Hkv, 128] (keys in the basis q16 was prepared for);
    reqs (r, q0, q1, L, s) in compact order.  Returns o fp64 [m, Hq, 128] (0 for rows without keys) and the
    natural-log LSE [Hq, m] (-inf for those rows)."""
    q = Q.f16_value(np.asarray(q16_bits)).astype(np.float64)
    m, Hq, D = q.shape
    o = np.zeros((m, Hq, D))
    lse = np.full((Hq, m), -np.inf)
    c = 0
    for (r, q0, q1, L, s) in reqs:
        e = ext.get(r, NO_EXT) if ext else NO_EXT
        nk = max(L - shift, e + 1, 0)
        k, v = np.asarray(K[r], np.float64), np.asarray(V[r], np.float64)
        for t in range(q1 - q0):
            js = visible(s + t, nk, shift, kmin, e)
            if len(js):
                lo, hi = int(js[0]), int(js[-1]) + 1
                sc = np.einsum("nhd,hgd->hgn", k[lo:hi], q[c + t].reshape(-1, G, D))
                mx = sc.max(-1, keepdims=True)
                p = np.exp2(sc - mx)
                den = p.sum(-1, keepdims=True)
                o[c + t] = (np.einsum("hgn,nhd->hgd", p, v[lo:hi]) / den).reshape(Hq, D)
                lse[:, c + t] = ((mx + np.log2(den)) * np.log(2.0)).reshape(Hq)
        c += q1 - q0
    return o, lse


def merge_items(opart, ml, tiles, G: int):
    """items of each tile -> (o fp64 [m, Hq, 128] compact rows, natural-log lse [Hq, m]); opart [ni, Hkv, rows, 128],
    ml [ni, Hkv, rows, 2] = (max in log2 units, sum)."""
    opart, ml = np.asarray(opart, np.float64), np.asarray(ml, np.float64)
    ni, Hkv, rows, D = opart.shape
    m = int(max(t[1] + t[3] for t in tiles)) if len(tiles) else 0
    Hq = Hkv * G
    o = np.zeros((m, Hq, D))
    lse = np.full((Hq, m), -np.inf)
    for tl in tiles:
        crow0, ntok, item0, nitem = int(tl[1]), int(tl[3]), int(tl[6]), int(tl[7])
        for r in range(min(rows, ntok * G)):
            t, g = divmod(r, G)
            for h in range(Hkv):
                mm = ml[item0:item0 + nitem, h, r, 0]
                ll = ml[item0:item0 + nitem, h, r, 1]
                M = mm.max()
                if np.isneginf(M):
                    continue
                w = np.where(np.isneginf(mm), 0.0, np.exp2(mm - M))
                Lsum = (w * ll).sum()
                o[crow0 + t, h * G + g] = (w[:, None] * opart[item0:item0 + nitem, h, r]).sum(0) / Lsum
                lse[h * G + g, crow0 + t] = (M + np.log2(Lsum)) * np.log(2.0)
    return o, lse


def win_gather(map_, sinkb, preb, kch, vch, Hkv: int):
    """rows [nk, Hkv, 128] of K and V: map_[d] = (kind << 32) | row; kind 0 sinkb [*, 2 Hkv, 128], 1 preb, 2 the batch
    rows kch / vch [n, Hkv, 128]."""
    kw, vw = [], []
    for code in np.asarray(map_, np.int64):
        kind, row = int(code >> 32), int(code & 0xFFFFFFFF)
        if kind == 2:
            kw.append(kch[row]); vw.append(vch[row])
        else:
            src = sinkb if kind == 0 else preb
            kw.append(src[row, :Hkv]); vw.append(src[row, Hkv:])
    return np.stack(kw), np.stack(vw)


def bf_merge(q, idx, o_p, lse_p, o_w, lse_w, sk, row_req, row_pos, sk_len, S: int, W: int, scale: float, Hkv: int):
    """fp64 LSE merge per (compact row c, q head): page part (o_p [m, Hq, 128], lse_p [Hq, m]), window part (o_w,
    lse_w; may be None), sink part (sk [nreq, S, 2 Hkv, 128], keys j < min(S, sk_len[req]) with j <= row_pos[c] - W;
    may be None).  q [n, Hq, 128] values; returns {batch row idx[c]: o [Hq, 128]}."""
    m, Hq, D = o_p.shape
    G = Hq // Hkv
    out = {}
    for c in range(m):
        res = np.zeros((Hq, D))
        for hq in range(Hq):
            parts = []
            for o, l in ((o_p, lse_p), (o_w, lse_w)):
                if o is not None and np.isfinite(l[hq, c]):
                    parts.append((np.asarray(o[c, hq], np.float64), float(l[hq, c])))
            if sk is not None:
                rq = int(row_req[c])
                n = min(S, int(sk_len[rq]), int(row_pos[c]) - W + 1)
                if n > 0:
                    k = np.asarray(sk[rq, :n, hq // G], np.float64)
                    v = np.asarray(sk[rq, :n, Hkv + hq // G], np.float64)
                    sc = (k @ np.asarray(q[int(idx[c]), hq], np.float64)) * scale
                    p = np.exp(sc - sc.max())
                    parts.append(((p @ v) / p.sum(), float(sc.max() + np.log(p.sum()))))
            if parts:
                M = max(l for _, l in parts)
                w = np.array([np.exp(l - M) for _, l in parts])
                res[hq] = sum(wi * o for wi, (o, _) in zip(w, parts)) / w.sum()
        out[int(idx[c])] = res
    return out
