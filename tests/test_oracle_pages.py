"""Page layout pins: byte positions derived by hand from the layout sentences, pack/parse round trips, and
whole-pool garbage preservation (a writer may touch only the bit fields of the tokens it writes)."""
import numpy as np
import pytest

from oracle import pages as PG

P, HKV = 16, 2


def _one_hot(fmt, pos, d, isv, val, word=None, g=0):
    pool = np.zeros((3, HKV, PG.chunk_bytes(fmt, P)), np.uint8)
    codes = np.zeros((1, 2 * HKV, 128), np.int64)
    words = np.zeros((1, 2 * HKV, 4), np.int64)
    head = 1
    codes[0, head + (HKV if isv else 0), d] = val
    if word is not None:
        words[0, head + (HKV if isv else 0), g] = word
    PG.pack_tokens(pool, np.array([2 * P + pos]), codes, words, fmt, P)
    assert not pool[:2].any() and not pool[2, 0].any()
    return pool[2, head]


def test_int4a_known_positions():
    # K, token 5, d = 37: group j = 1, r = 5 -> A, tg = 1, i = 1 -> byte 64*5 + 16*1 + 4*1 + 1, low nibble
    ch = _one_hot("int4a", 5, 37, False, 0xB)
    assert np.nonzero(ch)[0].tolist() == [64 * 5 + 16 + 4 + 1] and ch[341] == 0x0B
    # K, token 5, d = 37 + 16 = 53: the B element of the same byte -> high nibble
    ch = _one_hot("int4a", 5, 53, False, 0xB)
    assert np.nonzero(ch)[0].tolist() == [341] and ch[341] == 0xB0
    # V, token 11, d = 90: w = (90 % 64) / 16 = 1, gid = 2, sub = 2 * 1 + (90 % 16) / 8 = 3, c8 = 1, i = 1, odd -> B
    ch = _one_hot("int4a", 11, 90, True, 0x7)
    e = (1 * 8 + 2) * 2 + 1
    off = 64 * P + 16 * e + 4 * 3 + 1
    assert np.nonzero(ch)[0].tolist() == [off] and ch[off] == 0x70
    # K scale word of token 5 group 2; V scale word of token 11 (r8 = 3 -> slot8 = 4 + 1) group 3
    ch = _one_hot("int4a", 5, 0, False, 0, word=0xABCD, g=2)
    assert ch[128 * P + 8 * 5 + 4] == 0xCD and ch[128 * P + 8 * 5 + 5] == 0xAB
    ch = _one_hot("int4a", 11, 0, True, 0, word=0x1234, g=3)
    o = 136 * P + (3 * P + 8 + 5) * 2
    assert ch[o] == 0x34 and ch[o + 1] == 0x12 and np.count_nonzero(ch) == 2


def test_int4_sym_known_positions():
    # K, token 0, d = 2 (A_2 of word (0, 0)): -5 -> byte 2 = 0x80 | 5
    ch = _one_hot("int4", 0, 2, False, -5)
    assert np.nonzero(ch)[0].tolist() == [2] and ch[2] == 0x85
    # K, token 0, d = 18 (B_2 of word (0, 0)): -5 -> sign bit 3 of byte 2, magnitude bits 6..4 of byte (2 + 3) % 4 = 1
    ch = _one_hot("int4", 0, 18, False, -5)
    assert np.nonzero(ch)[0].tolist() == [1, 2] and ch[2] == 0x08 and ch[1] == 0x50
    # B_0: magnitude goes to byte 3
    ch = _one_hot("int4", 0, 16, False, 3)
    assert np.nonzero(ch)[0].tolist() == [3] and ch[3] == 0x30


def test_int2_known_positions():
    # K, token 6 -> physical row 6 ^ ((6 >> 1) & 2) = 4; d = 100: j = 3 (jp = 1, h = 1), r = 4 -> A, tg = 1, i = 0
    ch = _one_hot("konlya2", 6, 100, False, 3)
    off = 32 * 4 + 8 * 1 + 4 * 1 + 0
    assert np.nonzero(ch)[0].tolist() == [off] and ch[off] == 3 << 4
    # token 1 stays in row 1; B element (d = 116) of the same byte: shift 4 h + 2 = 6
    ch = _one_hot("konlya2", 1, 116, False, 2)
    assert np.nonzero(ch)[0].tolist() == [32 + 12] and ch[44] == 2 << 6
    # V, token 13, d = 77: m = 1, w = 0, gid = 5, r = 1; c8 = 1, i = 2, b = 1 -> entry (0*8+5)*2+1, byte 4*1+2, shift 6
    ch = _one_hot("int2a", 13, 77, True, 1)
    off = 32 * P + 8 * 11 + 4 + 2
    assert np.nonzero(ch)[0].tolist() == [off] and ch[off] == 1 << 6
    ch = _one_hot("int2a", 13, 0, True, 0, word=0x8123, g=1)
    o = 72 * P + (1 * P + 8 + 4 + 2) * 2
    assert ch[o] == 0x23 and ch[o + 1] == 0x81


@pytest.mark.parametrize("fmt", ["int4", "int4a", "int2a", "konly", "konlya", "konlya2"])
def test_round_trip_in_garbage_pool(fmt):
    rng = np.random.default_rng(hash(fmt) % 1000)
    Np, T = 9, 70
    pool = rng.integers(0, 256, (Np, HKV, PG.chunk_bytes(fmt, P)), dtype=np.uint8)
    before = pool.copy()
    slots = rng.permutation(Np * P)[:T].astype(np.int64)
    slots[3] = -1
    if PG.is_sym(fmt):
        codes = rng.integers(-7, 8, (T, 2 * HKV, 128))
    else:
        codes = rng.integers(0, 4 if PG.is_int2(fmt) else 16, (T, 2 * HKV, 128))
    words = rng.integers(0, 1 << 16, (T, 2 * HKV, 4))
    PG.pack_tokens(pool, slots, codes, words, fmt, P)
    c, w = PG.parse_pages(pool, fmt, P)
    cb, wb = PG.parse_pages(before, fmt, P)
    written = np.zeros(Np * P, bool)
    for t, s in enumerate(slots):
        if s < 0:
            continue
        written[s] = True
        pg, pos = divmod(int(s), P)
        assert np.array_equal(c[pg, :, pos, 0], codes[t, :HKV]) and np.array_equal(c[pg, :, pos, 1], codes[t, HKV:])
        assert np.array_equal(w[pg, :, pos, 0], words[t, :HKV]) and np.array_equal(w[pg, :, pos, 1], words[t, HKV:])
    # tokens not written keep their garbage (symmetric -0 vs +0 aside: compare raw bytes through a second pack)
    um = ~written.reshape(Np, P)
    cc, ccb = c.transpose(0, 2, 1, 3, 4), cb.transpose(0, 2, 1, 3, 4)
    ww, wwb = w.transpose(0, 2, 1, 3, 4), wb.transpose(0, 2, 1, 3, 4)
    assert np.array_equal(cc[um], ccb[um]) and np.array_equal(ww[um], wwb[um])
    # a page without any written token is byte-identical
    for pg in range(Np):
        if um[pg].all():
            assert np.array_equal(pool[pg], before[pg])
