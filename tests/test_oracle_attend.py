"""Pins of the attention oracle by textbook identities."""
import numpy as np

from oracle import attend as A
from oracle import pages as PG
from oracle import quant as Q

P = 16
F32 = np.float32


def _cache(fmt, rng, lens, Hkv=2, extra=3, C=None):
    npg = sum(-(-n // P) for n in lens) + extra
    pool = rng.integers(0, 256, (npg, Hkv, PG.chunk_bytes(fmt, P)), dtype=np.uint8)
    ids = rng.permutation(npg)
    bt = np.zeros((len(lens), max(1, max(-(-n // P) for n in lens))), np.int32)
    o = 0
    kvs = []
    mask = rng.integers(0, 2, (2 * Hkv, 4))
    for b, n in enumerate(lens):
        k = -(-n // P)
        bt[b, :k] = ids[o:o + k]
        o += k
        x = rng.standard_normal((n, 2 * Hkv, 128)).astype(F32)
        x[:, :Hkv, :4] *= 6
        xb = Q.bf16_bits(x)
        kvs.append(xb)
        pos = np.arange(n)
        slots = bt[b, pos // P].astype(np.int64) * P + pos % P
        if fmt in ("int4", "int4a", "int2a"):
            codes, words = Q.static_encode(xb, mask, fmt)
        else:
            codes, words, _ = Q.k2_encode(xb, C, fmt)
        PG.pack_tokens(pool, slots, codes, words, fmt, P)
    return pool, bt, kvs, mask


def test_k2_dequant_is_close_to_input_and_flags_matter():
    rng = np.random.default_rng(0)
    qs = rng.standard_normal((2, 64, 128)).astype(F32)
    C = np.einsum("hnd,hne->hde", qs, qs).astype(F32)
    lens = [37]
    pool, bt, kvs, _ = _cache("konlya", rng, lens, C=C)
    Kp, Vp = A.dequant_pages(pool, "konlya", P)
    Kc, Vc = A.gather_cache(Kp, Vp, bt, 37, P)
    x = Q.bf16_to_f32(kvs[0]).astype(np.float64)
    assert np.abs(Kc[0, :37] - x[:, :2]).max() < 0.9 and np.abs(Vc[0, :37] - x[:, 2:]).max() < 0.35
    rel = np.linalg.norm(Kc[0, :37] - x[:, :2]) / np.linalg.norm(x[:, :2])
    assert rel < 0.12
    # same bytes read with the flags ignored (as a static int4a cache) are a worse reconstruction
    Ks, _ = A.dequant_pages(pool, "int4a", P)
    Ks = A.gather_cache(Ks, Ks, bt, 37, P)[0]
    assert np.linalg.norm(Ks[0, :37] - x[:, :2]) > 2 * np.linalg.norm(Kc[0, :37] - x[:, :2])


def test_static_rotation_identity_and_split_merge():
    rng = np.random.default_rng(1)
    lens = [50, 1, 16]
    pool, bt, kvs, mask = _cache("int4a", rng, lens)
    Hkv, G = 2, 4
    qb = Q.bf16_bits(rng.standard_normal((3, Hkv * G, 128)).astype(F32))
    scale = 128 ** -0.5
    o = A.decode_reference(qb, pool, "int4a", P, bt, lens, scale, kmask=mask[:Hkv], vmask=mask[Hkv:])
    # un-rotate K and V first, attend in the original basis: identical in exact arithmetic
    Kp, Vp = A.dequant_pages(pool, "int4a", P)
    Kp = A.rot_blocks(Kp, mask[:Hkv])
    Vp = A.rot_blocks(Vp, mask[Hkv:])
    Kc, Vc = A.gather_cache(Kp, Vp, bt, 50, P)
    o2 = A.attend(Q.bf16_to_f32(qb), Kc, Vc, lens, scale)
    assert np.abs(o - o2).max() < 1e-12
    # split merge == single pass (log2 domain partials over two halves of row 0)
    q = Q.bf16_to_f32(qb)[0].astype(np.float64)
    k = np.repeat(Kc[0, :50], G, 1)
    v = np.repeat(Vc[0, :50], G, 1)
    parts = []
    for a, b in ((0, 32), (32, 50), (50, 50)):
        s = np.einsum("hd,lhd->hl", q, k[a:b]) * scale * np.log2(np.e)
        if b == a:
            parts.append((np.zeros((8, 128)), np.full(8, -np.inf), np.zeros(8)))
            continue
        m = s.max(-1)
        p = np.exp2(s - m[:, None])
        parts.append((np.einsum("hl,lhd->hd", p, v[a:b]), m, p.sum(-1)))
    mg = A.merge_partials(*[np.stack(x) for x in zip(*parts)])
    assert np.abs(mg - o2[0]).max() < 1e-12


def test_kv_start_and_tail_are_concatenation():
    rng = np.random.default_rng(2)
    lens = [40, 3]
    pool, bt, kvs, mask = _cache("int4", rng, lens)
    qb = Q.bf16_bits(rng.standard_normal((2, 8, 128)).astype(F32))
    ring = Q.bf16_bits(rng.standard_normal((4, 6, 4, 128)).astype(F32))
    tl, ti = np.array([5, 0]), np.array([2, 1])
    o = A.decode_reference(qb, pool, "int4", P, bt, lens, 0.1, tail=ring, tail_len=tl, tail_idx=ti, kv_start=4)
    Kp, Vp = A.dequant_pages(pool, "int4", P)
    Kc, Vc = A.gather_cache(Kp, Vp, bt, 40, P)
    t = Q.bf16_to_f32(ring[2, :5]).astype(np.float64)
    K0 = np.concatenate([Kc[0, 4:40], t[:, :2]])
    V0 = np.concatenate([Vc[0, 4:40], t[:, 2:]])
    o0 = A.attend(Q.bf16_to_f32(qb)[:1], K0[None], V0[None], [K0.shape[0]], 0.1)
    assert np.abs(o[0] - o0[0]).max() < 1e-12
    # row 1: len 3 < kv_start and empty tail -> no keys -> zeros
    assert not o[1].any()


def test_centring_shift_invariance():
    """softmax(q . (k - mu)) == softmax(q . k): a constant key shift moves every score of a head by q . mu."""
    rng = np.random.default_rng(3)
    k = rng.standard_normal((1, 30, 2, 128))
    v = rng.standard_normal((1, 30, 2, 128))
    q = rng.standard_normal((1, 8, 128))
    mu = rng.standard_normal((2, 128)) * 2
    a = A.attend(q, k, v, [30], 0.09)
    b = A.attend(q, k - mu[None, None], v, [30], 0.09)
    assert np.abs(a - b).max() < 1e-9
