"""GPU parity of the paged writers through the C ABI (libflagrot_kernels.so) against the oracle: whole-pool byte
equality in garbage-filled pools (bit-exact bar: codes, scale words, flag bits, and no stray writes)."""
import numpy as np
import pytest
import torch

from oracle import pages as PG
from oracle import quant as Q
from tests.gpu_util import P, bits, make_kv, spd_calib

pytestmark = pytest.mark.gpu


def _pool(fmt, npg, Hkv, g):
    return torch.randint(0, 256, (npg, Hkv, PG.chunk_bytes(fmt, P)), dtype=torch.uint8, generator=g)


def _same(got, want, fmt):
    """whole-pool equality with a readable report of what differs."""
    if np.array_equal(got, want):
        return
    c, w = PG.parse_pages(got, fmt, P)
    cw, ww = PG.parse_pages(want, fmt, P)
    dc, dw = np.argwhere(c != cw), np.argwhere(w != ww)
    msg = [f"{int((got != want).sum())} bytes differ; codes {len(dc)}, words {len(dw)}"]
    for i in dc[:6]:
        msg.append(f"code [page,head,pos,kv,d]={i.tolist()} got {int(c[tuple(i)])} want {int(cw[tuple(i)])} "
                   f"word got {int(w[tuple(i[:4])][i[4] // 32]):#x} want {int(ww[tuple(i[:4])][i[4] // 32]):#x}")
    for i in dw[:6]:
        msg.append(f"word [page,head,pos,kv,g]={i.tolist()} got {int(w[tuple(i)]):#x} want {int(ww[tuple(i)]):#x}")
    raise AssertionError("\n".join(msg))


def _slots(T, npg, g, holes=True):
    s = torch.randperm(npg * P, generator=g)[:T].long()
    if holes and T >= 4:
        s[T // 3] = -1
    return s


@pytest.mark.parametrize("fmt", ["int4", "int4a", "int2a"])
@pytest.mark.parametrize("T", [1, 5, 64, 1000, -333, -90])
def test_static_writer_bytes(dev, fmt, T):
    """T < 0: |T| tokens at consecutive slots (aligned runs of 8 take the whole-word V^T store; ragged ends, a hole and a
    reversed stretch the atomic one)"""
    from flagrot_releaser_amd import kernels as K
    consecutive, T = T < 0, abs(T)
    g = torch.Generator().manual_seed(1000 + T)
    Hkv = 4
    npg = T // P + 5
    pool = _pool(fmt, npg, Hkv, g)
    base = torch.zeros(T, 2 * Hkv + 1, 128, dtype=torch.bfloat16)
    base[:, :2 * Hkv] = make_kv(T, Hkv, g)
    kv = base.to(dev)[:, :2 * Hkv]                                   # token stride (2 Hkv + 1) * 128
    slots = _slots(T, npg, g)
    if consecutive:
        slots = 13 + torch.arange(T).long()
        slots[T // 2] = -1
        slots[40:56] = slots[40:56].flip(0)
    mask = (torch.rand(2 * Hkv, 4, generator=g) < 0.5).to(torch.uint8)
    kmu = torch.randn(Hkv, 128, generator=g) if T != 5 else None
    dpool = pool.to(dev)
    K.v2_write(kv, slots.to(dev), mask.to(dev), 32, dpool, P, fmt=fmt, kmu=None if kmu is None else kmu.to(dev))
    torch.cuda.synchronize()
    want = pool.numpy().copy()
    codes, words = Q.static_encode(bits(base[:, :2 * Hkv]), mask.numpy(), fmt, None if kmu is None else kmu.numpy())
    PG.pack_tokens(want, slots.numpy(), codes, words, fmt, P)
    _same(dpool.cpu().numpy(), want, fmt)


@pytest.mark.parametrize("kind", ["konly", "konlya", "konlya2"])
@pytest.mark.parametrize("T", [1, 5, 64, 333, 700])
def test_selecting_writer_bytes(dev, kind, T):
    """T * Hkv <= 1024 runs the low-latency kernel (four half waves per token and head), T = 700 the one-half-wave kernel"""
    from flagrot_releaser_amd import kernels as K
    g = torch.Generator().manual_seed(2000 + T)
    Hkv = 2
    npg = T // P + 5
    pool = _pool(kind, npg, Hkv, g)
    kv = make_kv(T, Hkv, g)
    Cq, co = spd_calib(Hkv, g)
    slots = _slots(T, npg, g)
    kmu = torch.randn(Hkv, 128, generator=g) if T == 64 else None
    dpool = pool.to(dev)
    K.cb_write(kv.to(dev), slots.to(dev), Cq.transpose(1, 2).contiguous().to(dev), co.to(dev), kind, dpool, P,
               kmu=None if kmu is None else kmu.to(dev))
    torch.cuda.synchronize()
    want = pool.numpy().copy()
    codes, words, info = Q.k2_encode(bits(kv), Cq.numpy(), kind, None if kmu is None else kmu.numpy())
    PG.pack_tokens(want, slots.numpy(), codes, words, kind, P)
    _same(dpool.cpu().numpy(), want, kind)
    if T >= 64:
        assert info["local"].any() and info["full"].any()


@pytest.mark.parametrize("kind", ["konly", "konlya", "konlya2"])
@pytest.mark.parametrize("T,base", [(700, 0), (700, 5), (90, 8), (333, 16)])
def test_selecting_writer_consecutive_slots(dev, kind, T, base):
    """prefill-like slots (consecutive positions): aligned runs of 8 slots take the whole-word V^T store, the ragged
    ends, a hole and a token written twice the atomic one; whole-pool bytes against the oracle's packer"""
    from flagrot_releaser_amd import kernels as K
    g = torch.Generator().manual_seed(4000 + T + base)
    Hkv = 2
    npg = (T + base) // P + 3
    pool = _pool(kind, npg, Hkv, g)
    kv = make_kv(T, Hkv, g)
    Cq, co = spd_calib(Hkv, g)
    slots = base + torch.arange(T).long()
    slots[T // 2] = -1
    if T > 300:
        slots[200:216] = slots[200:216].flip(0)            # a run of 16 slots in reverse order
    dpool = pool.to(dev)
    CT = Cq.transpose(1, 2).contiguous().to(dev)
    K.cb_write(kv.to(dev), slots.to(dev), CT, co.to(dev), kind, dpool, P)
    torch.cuda.synchronize()
    want = pool.numpy().copy()
    codes, words, info = Q.k2_encode(bits(kv), Cq.numpy(), kind, None)
    PG.pack_tokens(want, slots.numpy(), codes, words, kind, P)
    _same(dpool.cpu().numpy(), want, kind)
    # the two-pass form (key-only and value-only launches) on the same slots
    C1, beta = K.w3_calib(Cq.to(dev))
    d2 = pool.to(dev)
    K.cb_write3(kv.to(dev), slots.to(dev), CT, co.to(dev), C1, beta, kind, d2, P, split=True)
    torch.cuda.synchronize()
    assert torch.equal(d2, dpool)


@pytest.mark.parametrize("fmt", ["int4a", "int2a", "konlya", "konlya2", "konly"])
@pytest.mark.parametrize("order", ["scattered", "consecutive"])
def test_writers_page_32(dev, fmt, order):
    """32-token pages (four runs of 8 slots per page): whole-pool bytes against the oracle's packer for both writers"""
    from flagrot_releaser_amd import kernels as K
    P32 = 32
    g = torch.Generator().manual_seed(5200 + len(fmt))
    Hkv, T = 2, 300
    npg = T // P32 + 4
    pool = torch.randint(0, 256, (npg, Hkv, PG.chunk_bytes(fmt, P32)), dtype=torch.uint8, generator=g)
    kv = make_kv(T, Hkv, g)
    slots = torch.randperm(npg * P32, generator=g)[:T].long() if order == "scattered" else 19 + torch.arange(T).long()
    slots[77] = -1
    dpool = pool.to(dev)
    want = pool.numpy().copy()
    if fmt in ("int4a", "int2a"):
        mask = (torch.rand(2 * Hkv, 4, generator=g) < 0.5).to(torch.uint8)
        K.v2_write(kv.to(dev), slots.to(dev), mask.to(dev), 32, dpool, P32, fmt=fmt)
        codes, words = Q.static_encode(bits(kv), mask.numpy(), fmt, None)
    else:
        Cq, co = spd_calib(Hkv, g)
        K.cb_write(kv.to(dev), slots.to(dev), Cq.transpose(1, 2).contiguous().to(dev), co.to(dev), fmt, dpool, P32)
        codes, words, _ = Q.k2_encode(bits(kv), Cq.numpy(), fmt, None)
    torch.cuda.synchronize()
    PG.pack_tokens(want, slots.numpy(), codes, words, fmt, P32)
    assert np.array_equal(dpool.cpu().numpy(), want)


@pytest.mark.parametrize("kind", ["konly", "konlya", "konlya2"])
def test_two_pass_writer_equals_one_pass(dev, kind):
    """fr_cb_write3: one launch, and key pass / value pass on two streams, write the same bytes as fr_cb_write."""
    from flagrot_releaser_amd import kernels as K
    g = torch.Generator().manual_seed(31)
    Hkv, T = 4, 200
    npg = T // P + 3
    pool = _pool(kind, npg, Hkv, g).to(dev)
    kv = make_kv(T, Hkv, g).to(dev)
    Cq, co = spd_calib(Hkv, g)
    CT, co = Cq.transpose(1, 2).contiguous().to(dev), co.to(dev)
    slots = _slots(T, npg, g).to(dev)
    kmu = torch.randn(Hkv, 128, generator=g).to(dev)
    C1, beta = K.w3_calib(Cq.to(dev))
    a, b, c = pool.clone(), pool.clone(), pool.clone()
    K.cb_write(kv, slots, CT, co, kind, a, P, kmu=kmu)
    K.cb_write3(kv, slots, CT, co, C1, beta, kind, b, P, split=False, kmu=kmu)
    K.cb_write3(kv, slots, CT, co, C1, beta, kind, c, P, split=True, kmu=kmu)
    torch.cuda.synchronize()
    assert torch.equal(a, b) and torch.equal(a, c)


@pytest.mark.parametrize("kind", ["konly", "konlya", "konlya2"])
@pytest.mark.parametrize("order", ["scattered", "consecutive"])
def test_screened_writer_equals_exact_writer(dev, kind, order):
    """fr_cb_write3 at prefill sizes runs the screened kernel (matrix-pipe estimates of the weighted errors, exact
    evaluation where the estimate cannot decide): whole-pool byte equality with fr_cb_write on ordinary rows, on the
    adversarial groups of the reference's tests, on rows that tie exactly (zeros, constants, repeated tokens) and on
    holes; key-only and value-only passes included."""
    from flagrot_releaser_amd import kernels as K
    g = torch.Generator().manual_seed(77)
    Hkv, T = 4, 3000
    npg = T // P + 9
    pool = _pool(kind, npg, Hkv, g).to(dev)
    kv = make_kv(T, Hkv, g, edge=True)
    kv[100:140] = 0                                        # every candidate reproduces the row: exact ties
    kv[140:180] = kv[140:141]                              # one token repeated
    kv[180:200] = 0.37                                     # constants
    kv[200:260, :, 32:64] = 0                              # ties in one 32-group only
    kv[260:300] = (kv[260:300].float() * 1e-4).bfloat16()  # tiny rows
    kv = kv.to(dev)
    Cq, co = spd_calib(Hkv, g)
    CT, co = Cq.transpose(1, 2).contiguous().to(dev), co.to(dev)
    slots = _slots(T, npg, g) if order == "scattered" else 11 + torch.arange(T).long()
    slots[500:523] = -1
    slots = slots.to(dev)
    C1, beta = K.w3_calib(Cq.to(dev))
    for kmu in (None, torch.randn(Hkv, 128, generator=g).to(dev)):
        a, b, c = pool.clone(), pool.clone(), pool.clone()
        K.cb_write(kv, slots, CT, co, kind, a, P, kmu=kmu)
        K.cb_write3(kv, slots, CT, co, C1, beta, kind, b, P, split=False, kmu=kmu)
        K.cb_write3(kv, slots, CT, co, C1, beta, kind, c, P, split=True, kmu=kmu)
        torch.cuda.synchronize()
        assert torch.equal(a, b) and torch.equal(a, c)


@pytest.mark.parametrize("fmt", ["int4", "int4a", "int2a"])
def test_fused_static_writer_equals_two_steps(dev, fmt):
    from flagrot_releaser_amd import kernels as K
    g = torch.Generator().manual_seed(41)
    Hkv, T = 4, 150
    npg = T // P + 3
    pool = _pool(fmt, npg, Hkv, g).to(dev)
    kv = make_kv(T, Hkv, g).to(dev)
    slots = _slots(T, npg, g).to(dev)
    mask = (torch.rand(2 * Hkv, 4, generator=g) < 0.5).to(torch.uint8).to(dev)
    hfull = (torch.rand(2 * Hkv, generator=g) < 0.5).to(torch.uint8).to(dev)
    kmu = torch.randn(Hkv, 128, generator=g).to(dev)
    a, b = pool.clone(), pool.clone()
    K.v2_write(K.head_fwht(kv, hfull, 1 / 16), slots, mask, 32, a, P, fmt=fmt, kmu=kmu)
    K.w3_static_write(kv, slots, mask, hfull, b, P, fmt=fmt, kmu=kmu)
    torch.cuda.synchronize()
    assert torch.equal(a, b)


@pytest.mark.parametrize("D", [128, 256])
def test_head_fwht(dev, D):
    from flagrot_releaser_amd import kernels as K
    g = torch.Generator().manual_seed(7)
    for T, H in ((1, 32), (5, 16), (300, 8)):
        base = torch.randn(T, H + 3, D, generator=g).bfloat16()
        x = base.to(dev)[:, 1:H + 1]
        flags = (torch.rand(H, generator=g) < 0.5).to(torch.uint8)
        y = K.head_fwht(x, flags.to(dev), 1 / 16)
        want = Q.head_fwht(bits(base[:, 1:H + 1]), flags.numpy(), 1 / 16)
        assert np.array_equal(bits(y), want)
        xc = x.contiguous()
        K.head_fwht(xc, flags.to(dev), 1 / 16, out=xc)
        assert torch.equal(xc, y)


def test_static_writer_head_dim_256(dev):
    """head dim 256 = two 128-d half chunks per (page, head), written as 2 * Hkv half heads."""
    from flagrot_releaser_amd import kernels as K
    g = torch.Generator().manual_seed(5)
    Hkv, T = 2, 40
    npg = 6
    pool = torch.randint(0, 256, (npg, Hkv, 2 * 144 * P), dtype=torch.uint8, generator=g)
    kv = torch.randn(T, 2 * Hkv, 256, generator=g).bfloat16()
    mask = (torch.rand(2 * Hkv, 8, generator=g) < 0.5).to(torch.uint8)
    kmu = torch.randn(Hkv, 256, generator=g)
    slots = _slots(T, npg, g)
    dpool = pool.to(dev)
    K.v2_write(kv.to(dev), slots.to(dev), mask.to(dev), 32, dpool, P, fmt="int4a", kmu=kmu.to(dev))
    torch.cuda.synchronize()
    want = pool.numpy().copy().reshape(npg, 2 * Hkv, 144 * P)
    codes, words = Q.static_encode(bits(kv).reshape(T, 4 * Hkv, 128), mask.numpy().reshape(4 * Hkv, 4), "int4a",
                                   kmu.numpy().reshape(2 * Hkv, 128))
    PG.pack_tokens(want, slots.numpy(), codes, words, "int4a", P)
    assert np.array_equal(dpool.cpu().numpy().reshape(want.shape), want)


@pytest.mark.parametrize("kind,P", [("konly", 16), ("konlya", 16), ("konlya2", 16), ("konlya", 32)])
def test_selecting_writer_head_dim_256(dev, kind, P):
    """fr_cb_write at head dim 256 (eight key groups, whole-head H256, C_q [Hkv, 256, 256]; two 128-d half chunks per
    (page, head); attn_codebook.cu:384-392,432): whole-pool bytes against the oracle (which reproduces the reference's
    own encoder at this head dim bit for bit, tests/golden/k2_encode_d256_*.npz), garbage pool, holes, centring"""
    from flagrot_releaser_amd import kernels as K
    g = torch.Generator().manual_seed(900 + len(kind) + P)
    Hkv, T, Dh = 2, 75, 256
    npg = T // P + 3
    cb = PG.chunk_bytes(kind, P)
    pool = torch.randint(0, 256, (npg, Hkv, 2 * cb), dtype=torch.uint8, generator=g)
    kv = torch.randn(T, 2 * Hkv, Dh, generator=g)
    kv[:, :Hkv, 7] *= 6
    kv[:, :Hkv, 200] *= 5
    kv = (kv * (0.5 + torch.rand(T, 1, 1, generator=g)))
    kv[3, :, 32:64] *= 300.0
    kv[4] = 0.0
    kv[5, :, 128:160] = 1.25
    kv = kv.bfloat16()
    qs = torch.randn(Hkv, 512, Dh, generator=g)
    qs[:, :, :8] *= 4
    Cq = torch.einsum("hnd,hne->hde", qs, qs).contiguous()
    co = torch.rand(Hkv, Dh, generator=g) + 0.1
    kmu = torch.randn(Hkv, Dh, generator=g) * 0.5
    slots = torch.randperm(npg * P, generator=g)[:T].long()
    slots[11] = -1
    for use_mu in (False, True):
        dpool = pool.to(dev)
        K.cb_write(kv.to(dev), slots.to(dev), Cq.transpose(1, 2).contiguous().to(dev), co.to(dev), kind, dpool, P,
                   kmu=kmu.to(dev) if use_mu else None)
        torch.cuda.synchronize()
        codes, words, info = Q.k2_encode(bits(kv), Cq.numpy(), kind, kmu.numpy() if use_mu else None)
        want = pool.numpy().copy().reshape(npg, 2 * Hkv, cb)
        PG.pack_tokens(want, slots.numpy(), codes.reshape(T, 4 * Hkv, 128), words.reshape(T, 4 * Hkv, 4), kind, P)
        assert np.array_equal(dpool.cpu().numpy().reshape(want.shape), want), (kind, P, use_mu)
        assert info["full"].any() and (~info["full"]).any() and info["local"].any()
    # the two-pass writer has no 256-d form
    with pytest.raises(AssertionError, match="head dim"):
        K.cb_write3(kv.to(dev), slots.to(dev), Cq.to(dev), co.to(dev), None, None, kind, pool.to(dev), P)


def test_centring_exact_grid_all_writers(dev):
    """writer(k, kmu) == writer(bf16(k - mu)) byte for byte when k and mu sit on a 2^-6 grid."""
    from flagrot_releaser_amd import kernels as K
    g = torch.Generator().manual_seed(9)
    Hkv, T = 2, 48
    k = (torch.randint(-128, 129, (T, 2 * Hkv, 128), generator=g) / 64.0)
    mu = (torch.randint(-64, 65, (Hkv, 128), generator=g) / 64.0)
    sh = k.clone()
    sh[:, :Hkv] -= mu[None]
    kb, sb = k.bfloat16().to(dev), sh.bfloat16().to(dev)
    assert torch.equal(sb.float().cpu(), sh)
    slots = torch.randperm(4 * P, generator=g)[:T].long().to(dev)
    mask = (torch.rand(2 * Hkv, 4, generator=g) < 0.5).to(torch.uint8).to(dev)
    Cq, co = spd_calib(Hkv, g)
    CT, co = Cq.transpose(1, 2).contiguous().to(dev), co.to(dev)
    for fmt in ("int4", "int4a", "int2a"):
        a = torch.zeros(4, Hkv, PG.chunk_bytes(fmt, P), dtype=torch.uint8, device=dev)
        b = a.clone()
        K.v2_write(kb, slots, mask, 32, a, P, fmt=fmt, kmu=mu.to(dev))
        K.v2_write(sb, slots, mask, 32, b, P, fmt=fmt)
        assert torch.equal(a, b)
    for kind in ("konly", "konlya", "konlya2"):
        a = torch.zeros(4, Hkv, PG.chunk_bytes(kind, P), dtype=torch.uint8, device=dev)
        b = a.clone()
        K.cb_write(kb, slots, CT, co, kind, a, P, kmu=mu.to(dev))
        K.cb_write(sb, slots, CT, co, kind, b, P)
        assert torch.equal(a, b)


def test_error_codes(dev):
    from flagrot_releaser_amd import kernels as K
    L = K.lib()
    z = torch.zeros(64, dtype=torch.uint8, device=dev)
    assert L.fr_v2_write(77, z.data_ptr(), 256, z.data_ptr(), 1, 1, 16, z.data_ptr(), 32, z.data_ptr(), None, 128, None) == -4
    assert L.fr_v2_write(4, z.data_ptr(), 256, z.data_ptr(), 1, 1, 24, z.data_ptr(), 32, z.data_ptr(), None, 128, None) == -5
    assert L.fr_v2_write(4, z.data_ptr(), 256, z.data_ptr(), 1, 1, 16, z.data_ptr(), 32, z.data_ptr(), None, 96, None) == -8
    assert L.fr_v2_write(4, z.data_ptr(), 256, z.data_ptr(), 0, 1, 16, z.data_ptr(), 32, z.data_ptr(), None, 128, None) == 0
    assert L.fr_head_fwht(z.data_ptr(), 128, z.data_ptr(), 128, 1, 1, z.data_ptr(), 1.0, None, 64) == -8
    assert L.fr_last_error().decode() != ""
