"""Closed-form / brute-force pins of the oracle's arithmetic (no reference import, no GPU)."""
import math

import numpy as np
import pytest

from oracle import quant as Q

F32 = np.float32


@pytest.mark.parametrize("n", [2, 4, 8, 16, 32, 64, 128])
def test_fwht_is_sylvester_and_involutory(n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal((5, 2 * n)).astype(F32)
    y = Q.fwht(x, n)
    ref = (x.astype(np.float64).reshape(5, 2, n) @ Q.sylvester(n)).reshape(5, 2 * n)
    assert np.abs(y - ref).max() < 1e-5
    assert np.abs(Q.fwht(y, n) - x).max() < 1e-5
    S = Q.sylvester(n)
    assert np.allclose(S @ S, np.eye(n), atol=1e-12) and np.allclose(S, S.T)


def test_fwht_association_scalar_loop():
    """bit-exact against a scalar loop that spells the association out: stage h pairs (i, i + h), (a + b, a - b)."""
    rng = np.random.default_rng(0)
    x = rng.standard_normal(32).astype(F32)
    v = [F32(t) for t in x]
    h = 1
    while h < 32:
        nv = list(v)
        for i in range(32):
            if not i & h:
                nv[i], nv[i + h] = F32(v[i] + v[i + h]), F32(v[i] - v[i + h])
        v, h = nv, 2 * h
    v = np.array([F32(t * F32(1 / math.sqrt(32))) for t in v], dtype=F32)
    assert np.array_equal(Q.fwht(x, 32), v)


def test_sym4_invariants_and_edges():
    rng = np.random.default_rng(1)
    y = rng.standard_normal((64, 128)).astype(F32) * rng.uniform(0.01, 30, (64, 1)).astype(F32)
    y[0, :32] = 0
    y[1, 32:64] *= F32(1e-5)                      # fp16-subnormal scale
    y[2, 64:96] = 1.25
    q, w, deq = Q.quant_sym4(y)
    s = Q.f16_value(w)
    assert np.abs(q).max() <= 7
    assert np.array_equal(deq, q.astype(F32) * np.repeat(s, 32, -1))
    assert not q[0, :32].any() and w[0, 0] == 0
    # brute force: nearest grid point (ties to even) of y / s for s != 0
    g = y.reshape(64, 4, 32)
    ss = s[..., None]
    want = np.where(ss != 0, np.clip(np.rint(g / np.where(ss != 0, ss, 1)), -7, 7), 0).reshape(64, 128)
    assert np.array_equal(q, want.astype(np.int8))
    # the largest magnitude of a group maps to +-7 or +-6/7 (fp16 rounding of the scale can move it by one step)
    big = np.abs(q.reshape(64, 4, 32)).max(-1)
    assert ((big >= 6) | (s == 0) | (s < 1e-6)).all()


@pytest.mark.parametrize("bits", [4, 2])
def test_scale_word_exhaustive(bits):
    """for every positive fp16 pattern and zero point: the word carries z in its low bits, is the nearest such
    pattern (ties upwards), and never reaches the infinity pattern."""
    m = 1 << bits
    h = np.arange(0, 0x7C00, dtype=np.int32)
    s = h.astype(np.uint16).view(np.float16).astype(F32)
    for z in range(m):
        w = Q.scale_word(s, np.full(h.shape, z), bits)
        assert ((w & (m - 1)) == z).all() and (w < 0x7C00).all() and (w >= 0).all()
        cand = np.arange(z, 0x7C00, m)
        hs = h[::13]
        dist = np.abs(cand[None, :] - hs[:, None])
        best = dist.min(1)
        # nearest; on a tie the larger pattern
        pick = np.array([cand[np.nonzero(dist[i] == best[i])[0][-1]] for i in range(hs.size)])
        assert np.array_equal(w[::13], pick)


@pytest.mark.parametrize("bits", [4, 2])
def test_asym_stored_invariants(bits):
    lv = (1 << bits) - 1
    rng = np.random.default_rng(bits)
    y = rng.standard_normal((200, 128)).astype(F32) * rng.uniform(0.01, 10, (200, 1)).astype(F32)
    y[0, :32] = np.abs(y[0, :32]) + 1            # range excludes 0 -> widened
    y[1, :32] = -np.abs(y[1, :32]) - 1
    y[2, :32] = 0                                  # all-zero group
    q, w = Q.quant_asym_stored(y, bits)
    z = w & lv
    assert q.max() <= lv and (z <= lv).all()
    assert w[2, 0] == 0 and not q[2, :32].any()
    assert z[0, 0] == 0 and z[1, 0] == lv
    # the stored word is within half a zero-point step (in ulps) of fp16(step)
    g = y.reshape(200, 4, 32)
    mn, mx = np.minimum(g.min(-1), 0), np.maximum(g.max(-1), 0)
    s = np.maximum((mx - mn) * F32(1.0 / lv), F32(1e-12))
    assert (np.abs(w - Q.f16_bits(s).astype(np.int32)) <= (1 << (bits - 1))).all()
    # dequantised error bounded by one stored step
    deq = Q.dequant_stored(q, w, "asym4" if bits == 4 else "asym2")
    step = np.repeat(Q.word_scale(w), 32, -1).astype(np.float64)
    assert (np.abs(deq - y) <= 0.5 * step * 1.02 + 1e-6 + 2.0 ** -7 * np.abs(y) * lv).all()


def test_asym_error_form_reduces_to_stored_when_range_has_zero():
    rng = np.random.default_rng(5)
    y = rng.standard_normal((50, 128)).astype(F32)           # every group straddles 0
    q, w = Q.quant_asym_stored(y, 4)
    deq = Q.quant_asym_error(y, 4)
    g = y.reshape(50, 4, 32)
    s = np.maximum((g.max(-1) - g.min(-1)) * F32(1 / 15.0), F32(1e-12))
    z = (w & 15).astype(F32)
    want = ((q.reshape(50, 4, 32).astype(F32) - z[..., None]) * s[..., None]).reshape(50, 128)
    assert np.array_equal(deq, want)


def test_k2_rules_diagonal_weights():
    """C = c * I: the local rule is a plain squared-error comparison; ties keep the identity; the F flag and the
    local flags exclude each other."""
    rng = np.random.default_rng(9)
    x = rng.standard_normal((64, 2, 128)).astype(F32)
    x[:, :, 5] *= 8
    C = np.stack([np.eye(128, dtype=F32) * F32(c) for c in (1.0, 0.25)])
    r = Q.k2_encode_keys(x, C, "sym")
    ei = Q.quant_sym4(x)[2] - x
    eh = Q.fwht(Q.quant_sym4(Q.fwht(x, 32))[2], 32) - x
    mi = (ei.astype(np.float64) ** 2).reshape(64, 2, 4, 32).sum(-1)
    mh = (eh.astype(np.float64) ** 2).reshape(64, 2, 4, 32).sum(-1)
    clear = np.abs(mi - mh) > 1e-4 * (mi + mh)
    raw_local = r["err_local"][1] < r["err_local"][0]
    assert np.array_equal(raw_local[clear], (mh < mi)[clear])
    assert not (r["local"].astype(bool) & r["full"][..., None]).any()
    # chosen head error is the minimum, first index on ties
    assert np.array_equal(r["full"], r["err_head"][1] < r["err_head"][0])
    # identical inputs in both candidates (x = 0) -> identity everywhere
    z = Q.k2_encode_keys(np.zeros((3, 2, 128), F32), C, "asym4")
    assert not z["local"].any() and not z["full"].any()


def test_seq_matvec_and_tree_order():
    rng = np.random.default_rng(3)
    M = rng.standard_normal((1, 4, 6)).astype(F32)
    e = rng.standard_normal((1, 1, 6)).astype(F32)
    u = Q.seq_matvec(M, e, 1, 5)
    for i in range(4):
        acc = F32(M[0, i, 1] * e[0, 0, 1])
        for k in range(2, 5):
            acc = F32(acc + F32(M[0, i, k] * e[0, 0, k]))
        assert u[0, 0, i] == acc
    p = rng.standard_normal(8).astype(F32)
    t = F32(F32(F32(p[0] + p[4]) + F32(p[2] + p[6])) + F32(F32(p[1] + p[5]) + F32(p[3] + p[7])))
    assert Q.tree_sum(p) == t


def test_static_centring_exact_grid():
    """inputs on a 2^-6 grid: writer(k, kmu) == writer(bf16(k - mu)) because k - mu is exact in bf16."""
    rng = np.random.default_rng(11)
    k = (rng.integers(-128, 129, (20, 4, 128)) / 64.0).astype(F32)
    mu = (rng.integers(-64, 65, (2, 128)) / 64.0).astype(F32)
    kb = Q.bf16_bits(k)
    assert np.array_equal(Q.bf16_to_f32(kb), k)
    mask = rng.integers(0, 2, (4, 4))
    shifted = k.copy()
    shifted[:, :2] -= mu[None]
    sb = Q.bf16_bits(shifted)
    assert np.array_equal(Q.bf16_to_f32(sb), shifted)
    for fmt in ("int4", "int4a", "int2a"):
        a = Q.static_encode(kb, mask, fmt, kmu=mu)
        b = Q.static_encode(sb, mask, fmt)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_head_fwht_one_bf16_rounding():
    rng = np.random.default_rng(4)
    x = Q.bf16_bits(rng.standard_normal((7, 5, 128)).astype(F32))
    flags = np.array([1, 0, 1, 1, 0])
    y = Q.head_fwht(x, flags, 1 / 16)
    ref = Q.bf16_to_f32(x).astype(np.float64) @ (Q.sylvester(128) * math.sqrt(128)) / 16
    got = Q.bf16_to_f32(y).astype(np.float64)
    assert (np.abs(got - ref)[:, flags == 1] <= np.abs(ref[:, flags == 1]) * 2.0 ** -8 + 1e-30).all()
    assert np.array_equal(y[:, flags == 0], x[:, flags == 0])
