"""Closed-form pins of the KIVI-style oracle (quantiser, layout, dequantiser, selection rules)."""
import numpy as np

from oracle import kivi as KV
from oracle import quant as Q

F32 = np.float32


def _x(rng, T, H, D=128):
    mu = rng.standard_normal((H, D)) * 2
    x = mu[None] + rng.standard_normal((T, H, D)) * (0.5 + rng.random((H, D)))
    return Q.bf16_bits(x.astype(F32))


def test_quantiser_closed_form():
    rng = np.random.default_rng(0)
    g = rng.standard_normal((50, 32)).astype(F32)
    g[0] = 1.5                                   # constant group: s = 0 -> code 0, rec = mn exactly
    s, mn = KV.kivi_params(g.min(-1), g.max(-1))
    c = KV.kivi_code(g, mn[:, None], s[:, None])
    r = KV.kivi_rec(c, mn[:, None], s[:, None])
    assert c.max() <= 3 and not c[0].any() and np.array_equal(r[0], g[0])
    assert (np.abs(r - g)[1:] <= 0.5 * s[1:, None] * 1.0001 + 1e-6).all()
    assert (c[np.arange(50), g.argmin(-1)] == 0).all() and (c[np.arange(1, 50), g[1:].argmax(-1)] == 3).all()
    assert np.array_equal(s, (g.max(-1) - g.min(-1)) * F32(1 / 3.0))


def test_value_rules_and_layout_round_trip():
    rng = np.random.default_rng(1)
    T, H, D = 40, 2, 128
    xb = _x(rng, T, H)
    co = rng.random((H, D)).astype(F32) + 0.1
    enc = KV.v_encode(xb, co)
    assert enc["useH"].any() and (~enc["useH"]).any()
    # brute force of the rule on one token / head in fp64
    x = Q.bf16_to_f32(xb)[3, 1].astype(np.float64)
    for c, n in ((0, None), (1, 32), (2, 128)):
        y = x if n is None else (x.reshape(-1, n) @ Q.sylvester(n)).reshape(-1)
        g = y.reshape(4, 32)
        s, mn = (g.max(-1) - g.min(-1)) / 3, g.min(-1)
        rec = np.rint(np.clip((g - mn[:, None]) / s[:, None], 0, 3)) * s[:, None] + mn[:, None]
        back = rec.reshape(-1) if n is None else (rec.reshape(-1, n) @ Q.sylvester(n)).reshape(-1)
        e = ((back - x) ** 2 * co[1]).reshape(4, 32).sum(-1)
        if c == 0: eI = e
        elif c == 1: eH = e
        else: eF = e.sum()
    clear = np.abs(eH - eI) > 1e-3 * (eH + eI)
    assert np.array_equal((eH < eI)[clear], enc["useH"][3, 1][clear])
    codes, meta, vf = KV.v_stored(enc)
    assert not ((meta[..., 0] >> 15).astype(bool) & vf.astype(bool)[..., None]).any()
    pool = rng.integers(0, 256, (5, H, KV.chunk_bytes(D)), dtype=np.uint8)
    before = pool.copy()
    slots = rng.permutation(5 * 16)[:T]
    slots[5] = -1
    KV.pack_values(pool, slots, codes, meta, vf)
    kc, km, vc, vm, vff = KV.parse_chunks(pool, D)
    kcb, kmb, *_ = KV.parse_chunks(before, D)
    assert np.array_equal(kc, kcb) and np.array_equal(km, kmb)          # key fields untouched
    for t, s in enumerate(slots):
        if s < 0:
            continue
        pg, off = divmod(int(s), 16)
        assert np.array_equal(vc[pg, :, off], codes[t]) and np.array_equal(vm[pg, :, off], meta[t])
        assert np.array_equal(vff[pg, :, off], vf[t])
    # ident: no flags at all; fix: the frozen bits
    e0 = KV.v_encode(xb, co, ident=True)
    assert not e0["useH"].any() and not e0["useF"].any()
    e1 = KV.v_encode(xb, co, fix=np.array([0b0101, 1 << 16]))
    assert e1["useH"][:, 0].tolist() == [[True, False, True, False]] * T and e1["useF"][:, 1].all()


def test_key_group_and_dequant():
    rng = np.random.default_rng(2)
    D, H, NQ = 128, 2, 64
    ng = 3
    xb = _x(rng, ng * 32, H)
    qs = (rng.standard_normal((H, NQ, D)) * 0.3).astype(F32)
    lz = np.full((H, NQ), 5.0, F32)
    pool = np.zeros((2 * ng + 2, H, KV.chunk_bytes(D)), np.uint8)
    bt = rng.permutation(2 * ng + 2)[:2 * ng]
    pos = np.arange(ng * 32)
    slots = bt[pos // 16] * 16 + pos % 16
    co = np.ones((H, D), F32)
    venc = KV.v_encode(xb, co)
    KV.pack_values(pool, slots, *KV.v_stored(venc))
    flags = []
    for g in range(ng):
        valid = np.ones(32, bool)
        if g == 0:
            valid[:4] = False
        for h in range(H):
            enc = KV.k_encode_group(xb[32 * g:32 * g + 32, h], valid, qs[h], lz[h], 0.0884)
            codes, meta = KV.k_stored(enc)
            KV.pack_key_group(pool, h, slots[32 * g:32 * g + 32], valid, codes, meta)
            flags.append((enc["useH"], enc["useF"]))
            # the per-channel range covers the valid tokens only
            y = Q.bf16_to_f32(xb[32 * g:32 * g + 32, h])[valid]
            assert np.array_equal(enc["mn"][0], y.min(0))
    k, v = KV.dequant_groups(pool[bt], D)
    x = Q.bf16_to_f32(xb).astype(np.float64)
    # reconstruction is close (2-bit): relative error well below 1, and exact structure checks on one group
    assert np.linalg.norm(k[4:] - x[4:]) / np.linalg.norm(x[4:]) < 0.35
    assert np.linalg.norm(v - x) / np.linalg.norm(x) < 0.45
    # flags in the stored meta
    _, km, *_ = KV.parse_chunks(pool[bt], D)
    kmg = km.reshape(ng, 2, H, 16, 4, 2).transpose(0, 2, 1, 3, 4, 5).reshape(ng, H, D, 2)
    i = 0
    for g in range(ng):
        for h in range(H):
            uh, uf = flags[i]; i += 1
            assert bool(kmg[g, h, 4, 0] >> 15) == uf
            assert ((kmg[g, h, :4, 0] >> 15).astype(bool) == (uh & (not uf))).all()


def test_lse_merge_matches_single_softmax():
    rng = np.random.default_rng(3)
    n, H, D = 5, 3, 128
    s1, s2 = rng.standard_normal((n, H, 7)), rng.standard_normal((n, H, 9))
    v1, v2 = rng.standard_normal((n, H, 7, D)), rng.standard_normal((n, H, 9, D))
    def part(s, v):
        m = s.max(-1, keepdims=True); p = np.exp(s - m)
        return (p[..., None] * v).sum(-2) / p.sum(-1)[..., None], (m[..., 0] + np.log(p.sum(-1))).T
    oa, la = part(s1, v1); ob, lb = part(s2, v2)
    full, _ = part(np.concatenate([s1, s2], -1), np.concatenate([v1, v2], -2))
    got = Q.bf16_to_f32(KV.lse_merge(Q.bf16_bits(oa.astype(F32)), la.astype(F32), Q.bf16_bits(ob.astype(F32)), lb.astype(F32)))
    assert np.abs(got - full).max() < 0.03


def test_value_selection_with_matrix_weight():
    """the M form of the value criterion: equals the diagonal form for M = diag(co); the quadratic forms agree with
    explicit loops; a rotation-mixing M changes some choices"""
    rng = np.random.default_rng(11)
    T, H, D = 24, 2, 128
    x = (rng.standard_normal((T, H, D)) * (0.3 + rng.random((H, D))) + rng.standard_normal((H, D))).astype(np.float32)
    xb = Q.f32_to_bf16_bits(x) if hasattr(Q, "f32_to_bf16_bits") else (x.view(np.uint32) >> 16).astype(np.uint16)
    co = (rng.random((H, D)) + 0.1).astype(np.float32)
    base = KV.v_encode(xb, co)
    Md = np.stack([np.diag(co[h]) for h in range(H)]).astype(np.float32)
    same = KV.v_encode(xb, co, M=Md)
    assert np.array_equal(base["useH"], same["useH"]) and np.array_equal(base["useF"], same["useF"])
    assert np.allclose(base["marginH"], same["marginH"], rtol=1e-9, atol=1e-12)
    A = rng.standard_normal((H, D, D)).astype(np.float32) * 0.2
    M = (np.einsum("hik,hjk->hij", A, A) + Md).astype(np.float32)                   # SPD, couples the sub-vectors
    enc = KV.v_encode(xb, co, M=M)
    # brute force of one (token, head): reconstruct the three candidates' errors and evaluate the forms by loops
    t, h = 5, 1
    xf = Q.bf16_to_f32(xb)[t, h].astype(np.float64)
    recs = []
    for c in range(3):
        codes = enc["codes"][c, t, h].reshape(4, 32).astype(np.float64)
        y = (codes * enc["s"][c, t, h][:, None].astype(np.float64) + enc["mn"][c, t, h][:, None].astype(np.float64)).astype(np.float32)
        y = y.reshape(D)
        back = y if c == 0 else Q.fwht(y, 32 if c == 1 else D)
        recs.append(back.astype(np.float64) - xf)
    Mh = M[h].astype(np.float64)
    quad = lambda e, lo, hi: sum(e[i] * Mh[i, k] * e[k] for i in range(lo, hi) for k in range(lo, hi))   # noqa: E731
    eI = [quad(recs[0], 32 * j, 32 * j + 32) for j in range(4)]
    eH = [quad(recs[1], 32 * j, 32 * j + 32) for j in range(4)]
    uH = [eH[j] < eI[j] for j in range(4)]
    assert uH == enc["useH"][t, h].tolist()
    comb = np.concatenate([recs[1][32 * j:32 * j + 32] if uH[j] else recs[0][32 * j:32 * j + 32] for j in range(4)])
    assert (quad(recs[2], 0, D) < quad(comb, 0, D)) == bool(enc["useF"][t, h])
    assert (enc["useH"] != base["useH"]).any() or (enc["useF"] != base["useF"]).any()
    # ident / fix ignore M
    assert not KV.v_encode(xb, co, M=M, ident=True)["useH"].any()
