"""Pins of the multi-query prefill oracle (oracle/mq.py) and of the host planner (prefill_mq.plan_arrays), CPU only."""
import math

import numpy as np

from oracle import mq as OM
from oracle import quant as Q

F32 = np.float32


def test_prep_q_matrix_form_and_exact_cases():
    rng = np.random.default_rng(0)
    n, Hkv, G, D = 5, 3, 2, 128
    Hq = Hkv * G
    q = Q.bf16_to_f32(Q.bf16_bits(rng.standard_normal((n, Hq, D)).astype(F32)))
    kfull = np.array([1, 0, 1], np.uint8)
    kmask = np.array([[1, 0, 0, 1], [0, 0, 0, 0], [1, 1, 1, 1]], np.uint8)
    idx = np.array([4, 0, 2], np.int32)
    qs = 0.1275
    got = Q.f16_value(OM.prep_q(q, G, qs, idx, kfull, kmask)).astype(np.float64)
    H128 = Q.sylvester(128).astype(np.float64) * math.sqrt(128) / 8.0
    H32 = Q.sylvester(32).astype(np.float64)
    want = np.zeros((3, Hq, D))
    for i, r in enumerate(idx):
        for hq in range(Hq):
            x = q[r, hq].astype(np.float64)
            hk = hq // G
            if kfull[hk]:
                x = x @ H128
            xb = x.reshape(4, 32)
            x = np.where(kmask[hk].astype(bool)[:, None], xb @ H32, xb).reshape(-1)
            want[i, hq] = x * float(F32(qs))
    assert np.abs(got - want).max() <= 2.0 ** -11 * np.abs(want).max() * 1.01 + 1e-7
    # small integers: every butterfly is exact in fp32, the result is the fp16 rounding of the exact value
    qi = rng.integers(-3, 4, (2, 2, D)).astype(F32)
    g2 = Q.f16_value(OM.prep_q(qi, 1, 0.25, None, np.array([1, 1], np.uint8), None)).astype(np.float64)
    ex = (qi.astype(np.float64) @ H128) * 0.25
    assert np.array_equal(g2, Q.f16_value(Q.f16_bits(ex.astype(F32))).astype(np.float64))
    # no flags: plain scaling; rotation twice by orthonormal H32 returns the input (up to fp32 rounding)
    g3 = OM.prep_q(q, G, 1.0)
    assert np.array_equal(g3, Q.f16_bits(q))
    once = Q.f16_value(OM.prep_q(q, G, 1.0, None, None, np.ones((Hkv, 4), np.uint8))).astype(F32)
    twice = Q.f16_value(OM.prep_q(once, G, 1.0, None, None, np.ones((Hkv, 4), np.uint8)))
    assert np.abs(twice - q).max() < 4e-3 * np.abs(q).max()


def _brute(q, K, V, pos, nk, shift, kmin, ext):
    js = [j for j in range(nk) if j >= kmin and (j <= pos - shift or j <= ext)]
    if not js:
        return None, js
    s = np.array([K[j] @ q for j in js])
    p = np.exp2(s - s.max())
    return (p[:, None] * V[js]).sum(0) / p.sum(), js


def test_attention_visibility_and_closed_forms():
    rng = np.random.default_rng(1)
    Hkv, G, D = 2, 2, 128
    Hq = Hkv * G
    cases = [  # (L, s, shift, kmin, ext)
        (40, 0, 0, 0, None), (40, 25, 0, 0, None), (50, 30, 8, 0, None), (50, 30, 8, 4, None), (60, 40, 16, 4, 33),
        (20, 0, 32, 0, None), (20, 10, 4, 8, None)]
    for (L, s, shift, kmin, e) in cases:
        nq = L - s
        K = [rng.standard_normal((L, Hkv, D))]
        V = [rng.standard_normal((L, Hkv, D))]
        q16 = Q.f16_bits((rng.standard_normal((nq, Hq, D)) * 0.3).astype(F32))
        ext = {0: e} if e is not None else None
        o, lse = OM.attention(q16, K, V, [(0, 0, nq, L, s)], G, shift, kmin, ext)
        qv = Q.f16_value(q16).astype(np.float64)
        ee = e if e is not None else OM.NO_EXT
        nk = max(L - shift, ee + 1, 0)
        for t in range(nq):
            for hq in range(Hq):
                want, js = _brute(qv[t, hq], K[0][:, hq // G], V[0][:, hq // G], s + t, nk, shift, kmin, ee)
                if want is None:
                    assert not o[t, hq].any() and np.isneginf(lse[hq, t])
                else:
                    assert np.allclose(o[t, hq], want, rtol=1e-12, atol=1e-12)
        # zero query: uniform weights -> mean of the visible values, lse = ln(count)
        o0, l0 = OM.attention(np.zeros_like(q16), K, V, [(0, 0, nq, L, s)], G, shift, kmin, ext)
        for t in range(nq):
            js = OM.visible(s + t, nk, shift, kmin, ee)
            if len(js):
                assert np.allclose(o0[t, 1], V[0][js, 0].mean(0)) and np.isclose(l0[1, t], math.log(len(js)))


def test_merge_items_equals_single_pass():
    rng = np.random.default_rng(2)
    Hkv, G, D, rows, L = 2, 4, 128, 64, 300
    TQ = rows // G
    K, V = rng.standard_normal((L, Hkv, D)), rng.standard_normal((L, Hkv, D))
    nq = 20
    q16 = Q.f16_bits((rng.standard_normal((nq, Hkv * G, D)) * 0.4).astype(F32))
    reqs = [(0, 0, nq, L, L - nq)]
    from flagrot_releaser_amd.prefill_mq import plan_arrays
    T, I, idx, rws = plan_arrays(reqs, G, Hkv, 0, ncu=2, kernel=1, waves=1.0, min_blocks=1)
    assert rws == rows and len(T) == 2 and len(I) > len(T)
    qv = Q.f16_value(q16).astype(np.float64)
    opart = np.zeros((len(I), Hkv, rows, D))
    ml = np.zeros((len(I), Hkv, rows, 2))
    ml[..., 0] = -np.inf
    for it, (ti, kb0, kb1, _) in enumerate(I):
        tl = T[ti]
        for r in range(tl[3] * G):
            t, g = divmod(r, G)
            pos = tl[4] + t
            js = [j for j in range(kb0 * 64, min(kb1 * 64, tl[5])) if j <= pos]
            for h in range(Hkv):
                if js:
                    s = K[js, h] @ qv[tl[1] + t, h * G + g]
                    p = np.exp2(s - s.max())
                    opart[it, h, r], ml[it, h, r] = p @ V[js, h], (s.max(), p.sum())
    o, lse = OM.merge_items(opart, ml, T, G)
    o1, lse1 = OM.attention(q16, [K], [V], reqs, G, 0)
    assert np.allclose(o, o1, atol=1e-12) and np.allclose(lse, lse1, atol=1e-12)


def test_plan_arrays_invariants():
    from flagrot_releaser_amd.prefill_mq import BN, KROWS, plan_arrays
    reqs = [(2, 0, 145, 9000, 9000 - 145), (0, 145, 445, 12000, 11700), (1, 445, 462, 5003, 4986), (3, 462, 1162, 700, 0)]
    for kernel in (1, 3, 4):
        for G in (1, 4, 5, 8):
            for shift, ext in ((0, None), (128, None), (128, {0: 11650})):
                T, I, idx, rows = plan_arrays(reqs, G, 8, shift, ncu=256, kernel=kernel, ext=ext)
                assert rows == KROWS[kernel]
                TQ = rows // G
                assert np.array_equal(idx, np.arange(1162))
                assert sum(int(t[3]) for t in T) == 1162 and all(1 <= t[3] <= TQ for t in T)
                assert np.array_equal(T[:, 6], np.concatenate([[0], np.cumsum(T[:, 7])[:-1]]))
                for ti, tl in enumerate(T):
                    its = I[tl[6]:tl[6] + tl[7]]
                    assert (its[:, 0] == ti).all()
                    kend = max(0, min(tl[5], max(tl[4] + tl[3] - shift, tl[8] + 1)))
                    nb = -(-kend // BN)
                    assert its[0, 1] == 0 and (its[1:, 1] == its[:-1, 2]).all()          # contiguous, no overlap
                    assert its[-1, 2] == nb or (nb == 0 and its[-1, 2] == 0)
                assert len(I) * 8 <= 4 * 2 * 4 * 256 + len(T) * 8                         # about `waves` rounds of the GPU


def test_split_items_equal_items_and_whole_rounds():
    from flagrot_releaser_amd.prefill_mq import BN, plan_arrays, split_items
    # the workload the bench measures: 64 tiles of 257 .. 264 key blocks, 8 KV heads, 256 resident workgroups
    reqs = [(r, r * 512, (r + 1) * 512, 16896, 16384) for r in range(4)]
    T, I, _, rows = plan_arrays(reqs, 8, 8, 0, ncu=256, kernel=4)
    assert rows == 256 and len(T) == 64 and len(I) == 64                     # one item per tile: 512 workgroups = 2 rounds
    assert (np.diff(I[:, 2] - I[:, 1]) <= 0).all()                          # longest tiles first
    # one request: 16 tiles x 8 heads = half a round -> two items per tile, of equal length
    T, I, _, _ = plan_arrays(reqs[:1], 8, 8, 0, ncu=256, kernel=4)
    assert len(I) == 32
    ln = (I[:, 2] - I[:, 1]).reshape(16, 2)
    assert (np.abs(ln[:, 0] - ln[:, 1]) <= 1).all() and ln.min() >= 128
    # properties on ragged inputs
    rng = np.random.default_rng(3)
    for _ in range(50):
        nb = rng.integers(0, 400, size=int(rng.integers(1, 40)))
        for waves in (None, 1.0, 2.5):
            n = split_items(nb, 8, 256, waves, 4)
            assert n.shape == nb.shape and (n >= 1).all()
            assert ((nb // n >= 4) | (n == 1)).all()                         # at least min_blocks blocks per item
    assert split_items(np.zeros(0, np.int64), 8, 256, None, 4).size == 0


def test_pick_kernel_by_rows_per_request():
    from flagrot_releaser_amd.prefill_mq import pick_kernel
    assert pick_kernel([(0, 0, 512, 16896, 16384)], 8) == 4          # 4096 rows
    assert pick_kernel([(0, 0, 16, 4096, 4080)], 8) == 3             # 128 rows: one 128-row tile
    assert pick_kernel([(0, 0, 16, 4096, 4080), (1, 16, 48, 900, 868)], 8) == 4
    assert pick_kernel([(0, 0, 100, 900, 800)], 1) == 3
    assert pick_kernel([], 4) == 3


def test_bf_merge_is_attention_over_the_union():
    rng = np.random.default_rng(3)
    Hkv, G, D, S, W = 2, 2, 128, 4, 8
    Hq = Hkv * G
    L, nq = 40, 6
    K, V = rng.standard_normal((L, Hkv, D)), rng.standard_normal((L, Hkv, D))
    q = rng.standard_normal((nq, Hq, D)) * 0.3
    scale = 1 / math.sqrt(D)
    pos = np.arange(L - nq, L)
    # page part: keys S <= j <= pos - W; sink part: j < S
    q16 = Q.f16_bits((q * scale * math.log2(math.e)).astype(F32))
    qv = Q.f16_value(q16).astype(np.float64) / (scale * math.log2(math.e))
    o_p, lse_p = OM.attention(q16, [K], [V], [(0, 0, nq, L, L - nq)], G, W, kmin=S)
    sk = np.concatenate([K[:S], V[:S]], 1)[None]
    out = OM.bf_merge(qv, np.arange(nq), o_p, lse_p, None, None, sk, np.zeros(nq, np.int64), pos, np.array([S]), S, W, scale, Hkv)
    for c in range(nq):
        for hq in range(Hq):
            js = list(range(0, pos[c] - W + 1))
            s = (K[js, hq // G] @ qv[c, hq]) * scale
            p = np.exp(s - s.max())
            assert np.allclose(out[c][hq], (p @ V[js, hq // G]) / p.sum(), atol=1e-10)
    kw, vw = OM.win_gather(np.array([(2 << 32) | 3, (0 << 32) | 1, (1 << 32) | 0]), sk[0], sk[0][::-1], K, V, Hkv)
    assert np.array_equal(kw[0], K[3]) and np.array_equal(vw[1], V[1]) and np.array_equal(kw[2], K[S - 1])
