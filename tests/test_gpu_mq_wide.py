"""GPU parity of libflagrot_mq.so at head dim 256 (integrations/vllm_flagrot/csrc/mq_prefill.cu:825-1203 k_mq3, :1205-1273
merge, :1275-1339 q preparation; the reference's shape (G, D, Hkv) = (6, 256, 4), tests/test_kernels.py:366-374) against
oracle/mq.py over the oracle's dequantised pages (two 128-d half chunks per page and head).

Bars as at head dim 128 (tests/test_gpu_mq.py): prep_q bit-equal to the oracle; merged attention within 1e-3 relative L2
of fp64 for static pages and 1.5e-3 for key-only pages, LSE within 5e-3 / 1e-2; rows without a visible key are zeros with
LSE -inf; bf16 rows equal the rounding of the fp32 result; the BF16 window gather copies exactly and the sink / window
merge stays within 1e-2.  Pools: unused block-table entries poisoned, free pages random bytes.
"""
import math

import numpy as np
import pytest
import torch

from oracle import attend as OA
from oracle import mq as OM
from oracle import quant as Q
from tests.gpu_util import bits
from tests.test_gpu_mq import FMT, LOG2E, _rel

pytestmark = pytest.mark.gpu
D, PAGE = 256, 16


def _rand_kv(L, Hkv, g):
    k = torch.randn(L, Hkv, D, generator=g)
    v = torch.randn(L, Hkv, D, generator=g)
    k[..., 5] *= 8
    k[..., 70] += 4
    k[..., 200] *= 5
    v[..., 3] += 2
    return torch.cat([k, v], 1).bfloat16()


def _make_pool(dev, Ls, Hkv, fmt, g, kmask=None, kfull=None):
    from flagrot_releaser_amd import kernels as K
    cell = FMT[fmt][2]
    npg = [(L + PAGE - 1) // PAGE for L in Ls]
    total = sum(npg) + 11
    perm = torch.randperm(total, generator=g)
    bt = torch.full((len(Ls), max(npg) + 3), 1 << 30, dtype=torch.int32)
    pool = torch.randint(0, 256, (total, Hkv, 2 * cell * PAGE), generator=g, dtype=torch.uint8).to(dev)
    o = 0
    Ks, Vs = [], []
    for i, (L, n) in enumerate(zip(Ls, npg)):
        bt[i, :n] = perm[o:o + n].int()
        o += n
        kv = _rand_kv(L, Hkv, g).to(dev)
        slots = (bt[i].long()[torch.arange(L) // PAGE] * PAGE + torch.arange(L) % PAGE).to(dev)
        if fmt in ("konlya", "konlya2"):
            w = 0.5 + 1.5 * torch.rand(Hkv, D, generator=g)
            K.cb_write(kv, slots, torch.diag_embed(w).contiguous().to(dev), w.to(dev), fmt, pool, PAGE)
        else:
            mask = torch.zeros(2 * Hkv, 8, dtype=torch.uint8)
            mask[:Hkv] = torch.as_tensor(kmask)
            hfull = torch.zeros(2 * Hkv, dtype=torch.uint8)
            hfull[:Hkv] = torch.as_tensor(kfull)
            K.v2_write(K.head_fwht(kv, hfull.to(dev), 1 / 16), slots, mask.to(dev), 32, pool, PAGE, fmt=fmt)
    torch.cuda.synchronize()
    hp = pool.cpu().numpy()
    for i, (L, n) in enumerate(zip(Ls, npg)):
        with np.errstate(all="ignore"):
            Kp, Vp = OA.dequant_pages(hp[bt[i, :n].numpy()], fmt, PAGE, Dh=D)
        Ks.append(Kp.reshape(n * PAGE, Hkv, D)[:L])
        Vs.append(Vp.reshape(n * PAGE, Hkv, D)[:L])
    return pool, bt.to(dev), Ks, Vs


CASES = [  # (requests [(L, nq)], shift, sink, G, fmt, ext[, min_blocks])
    ([(1000, 1000)], 0, 0, 6, "int4a", None),
    ([(777, 300)], 0, 0, 6, "konlya", None),
    ([(3000, 1)], 0, 0, 4, "int4a", None),
    ([(17, 17)], 0, 0, 4, "konlya", None),
    ([(16, 5)], 0, 0, 6, "int2a", None),
    ([(64, 64)], 0, 0, 6, "konlya2", None),
    ([(2000, 145), (1200, 300), (503, 17), (700, 700), (4000, 64)], 0, 0, 6, "konlya", None),
    ([(2048, 600)], 128, 0, 6, "int4a", None),
    ([(130, 70)], 64, 0, 4, "konlya2", None),
    ([(1191, 300), (600, 600)], 128, 4, 6, "konlya", None),
    ([(1500, 200), (300, 300)], 0, 0, 5, "int2a", None),
    ([(1500, 200)], 0, 0, 1, "konlya", None),
    ([(900, 200), (400, 100)], 128, 4, 8, "konlya", {0: 650}),
    ([(20000, 40)], 0, 0, 2, "konlya", None, 300),          # an item longer than the page-id window: it slides
]


@pytest.mark.parametrize("case", range(len(CASES)))
def test_mq_attention_against_fp64(dev, case):
    from flagrot_releaser_amd import prefill_mq as MQ
    reqs_in, shift, sink, G, fmt, ext = CASES[case][:6]
    min_blocks = CASES[case][6] if len(CASES[case]) > 6 else None
    k2, int2, _ = FMT[fmt]
    g = torch.Generator().manual_seed(700 + case)
    Hkv = 2
    Hq = Hkv * G
    kmask = (torch.rand(Hkv, 8, generator=g) < 0.5).to(torch.uint8) if not k2 else None
    kfull = torch.tensor([1, 0], dtype=torch.uint8) if not k2 else None
    Ls = [L for L, _ in reqs_in]
    pool, bt, Ks, Vs = _make_pool(dev, Ls, Hkv, fmt, g, kmask, kfull)
    reqs, row = [], 3
    for r, (L, nq) in enumerate(reqs_in):
        reqs.append((r, row, row + nq, L, L - nq))
        row += nq
    n = row + 2
    q = (torch.randn(n, Hq, D, generator=g) * 1.5).bfloat16()
    scale = 1 / math.sqrt(D)
    plan = MQ.build_plan(reqs, G, Hkv, shift, dev, sink=sink, kernel=4, ext=ext, min_blocks=min_blocks, D=D)
    assert plan.rows == 128 and plan.kernel == 3 and plan.D == D          # one kernel at this head dim, whatever was asked
    if min_blocks:
        it = plan.items.cpu().numpy().reshape(-1, 4)
        assert (it[:, 2] - it[:, 1]).max() > 256
    q16 = MQ.prep_q(q.to(dev), scale * LOG2E, G, plan.idx, None if k2 else kfull.to(dev), None if k2 else kmask.to(dev))
    want16 = OM.prep_q(Q.bf16_to_f32(bits(q)), G, scale * LOG2E, plan.idx.cpu().numpy(),
                       None if k2 else kfull.numpy(), None if k2 else kmask.numpy())
    got16 = q16.cpu().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got16, want16), "prep_q differs from the oracle"
    creqs, c = [], 0
    for (r, q0, q1, L, s) in reqs:
        creqs.append((r, c, c + q1 - q0, L, s))
        c += q1 - q0
    ref, ref_lse = OM.attention(want16, Ks, Vs, creqs, G, shift, sink, ext)
    outbuf = torch.full((n, Hq * D + 32), 3.0, dtype=torch.bfloat16, device=dev)
    out = outbuf[:, :Hq * D]
    for rep in range(2):
        opart, ml = MQ.attn(q16, pool, bt, plan, G, shift, k2, int2)
        o32, lse = MQ.merge(plan, opart, ml, G, fp32=True, want_lse=True)
        MQ.merge(plan, opart, ml, G, out=out)
        torch.cuda.synchronize()
        got, gl = o32.cpu().numpy().astype(np.float64), lse.cpu().numpy().astype(np.float64)
        assert np.isfinite(got).all()
        empty = np.isneginf(ref_lse)
        assert np.array_equal(np.isneginf(gl), empty)
        assert not got[empty.T].any()
        c, worst = 0, 0.0
        for (r, q0, q1, L, s) in reqs:
            nq = q1 - q0
            e = _rel(got[c:c + nq], ref[c:c + nq])
            assert e <= (1.5e-3 if k2 else 1e-3), (case, rep, r, e)
            worst = max(worst, e)
            c += nq
        fin = ~empty
        lerr = np.abs(gl[fin] - ref_lse[fin]).max() if fin.any() else 0.0
        el = float((np.abs(got - ref) / (2e-3 + 1e-2 * np.abs(ref))).max())
        print(f"case {case} rep {rep}: lse abs err {lerr:.2e}, worst rel l2 {worst:.2e}, element-wise "
              f"|err| / (2e-3 + 1e-2 |ref|) = {el:.2f} (fp32 output)", flush=True)
        assert lerr <= (1e-2 if k2 else 5e-3), (case, rep, lerr)
        ob = outbuf.float().cpu()
        idx = plan.idx.cpu().long()
        back = o32.cpu().bfloat16().float().reshape(plan.m, Hq * D)
        assert (ob[idx, :Hq * D] - back).abs().max() <= 2 ** -7 * back.abs().max()
        keep = torch.ones(n, dtype=torch.bool)
        keep[idx] = False
        assert (ob[keep] == 3.0).all() and (ob[:, Hq * D:] == 3.0).all()


def test_prep_q_fp32_rows(dev):
    from flagrot_releaser_amd import prefill_mq as MQ
    g = torch.Generator().manual_seed(5)
    Hkv, G = 3, 2
    q = torch.randn(9, Hkv * G, D, generator=g)
    kfull = torch.tensor([0, 1, 1], dtype=torch.uint8)
    kmask = (torch.rand(Hkv, 8, generator=g) < 0.5).to(torch.uint8)
    idx = torch.tensor([8, 1, 1, 4], dtype=torch.int32)
    got = MQ.prep_q(q.to(dev), 0.3, G, idx.to(dev), kfull.to(dev), kmask.to(dev)).cpu().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, OM.prep_q(q.numpy(), G, 0.3, idx.numpy(), kfull.numpy(), kmask.numpy()))
    got = MQ.prep_q(q.to(dev), 1.7, G).cpu().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, OM.prep_q(q.numpy(), G, 1.7))


def test_win_gather_and_bf_merge(dev):
    from flagrot_releaser_amd import prefill_mq as MQ
    g = torch.Generator().manual_seed(8)
    Hkv, G, S, W = 2, 3, 4, 16
    Hq = Hkv * G
    nreq, n, m = 2, 12, 9
    sinkb = torch.randn(nreq * S, 2 * Hkv, D, generator=g).bfloat16()
    preb = torch.randn(7, 2 * Hkv, D, generator=g).bfloat16()
    kbuf = torch.randn(n, Hkv * D + 64, generator=g).bfloat16()
    vbuf = torch.randn(n, Hkv * D + 64, generator=g).bfloat16()
    kch, vch = kbuf[:, :Hkv * D], vbuf[:, 64:]
    codes = [(0, 5), (1, 6), (2, 11), (2, 0), (1, 0), (0, 0)]
    map_ = torch.tensor([(k << 32) | r for k, r in codes], dtype=torch.int64)
    kw, vw = MQ.win_gather(map_.to(dev), len(codes), sinkb.to(dev), preb.to(dev), kch.to(dev), vch.to(dev), Hkv, D)
    wk, wv = OM.win_gather(map_.numpy(), bits(sinkb), bits(preb), bits(kch.contiguous()).reshape(n, Hkv, D),
                           bits(vch.contiguous()).reshape(n, Hkv, D), Hkv)
    assert np.array_equal(bits(kw), wk) and np.array_equal(bits(vw), wv)
    q = torch.randn(n, Hq, D, generator=g).bfloat16()
    idx = torch.tensor([2, 3, 4, 5, 6, 7, 8, 9, 10], dtype=torch.int64)
    o_p = torch.randn(m, Hq, D, generator=g)
    lse_p = torch.randn(Hq, m, generator=g) * 2
    lse_p[0, 0] = float("-inf")
    lse_p[1, 1] = float("inf")
    o_w = torch.randn(m, Hq, D, generator=g).bfloat16()
    lse_w = torch.randn(Hq, m, generator=g) * 2
    sk = sinkb.view(nreq, S, 2 * Hkv, D)
    row_req = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1, 1], dtype=torch.int64)
    row_pos = torch.tensor([14, 17, 18, 30, 16, 19, 40, 41, 15], dtype=torch.int64)
    sk_len = torch.tensor([4, 2], dtype=torch.int64)
    scale = 1 / math.sqrt(D)
    for use_w, use_s in ((True, True), (False, True), (True, False)):
        outbuf = torch.full((n, Hq * D + 16), 5.0, dtype=torch.bfloat16, device=dev)
        out = outbuf.as_strided((n, Hq, D), (Hq * D + 16, D, 1))
        MQ.bf_merge(q.to(dev), idx.to(dev), o_p.to(dev), lse_p.to(dev), o_w.to(dev) if use_w else None,
                    lse_w.to(dev) if use_w else None, sk.to(dev) if use_s else None, row_req.to(dev), row_pos.to(dev),
                    sk_len.to(dev), S, W, scale, out, Hkv)
        torch.cuda.synchronize()
        want = OM.bf_merge(Q.bf16_to_f32(bits(q)), idx.numpy(), o_p.numpy(), lse_p.numpy(),
                           Q.bf16_to_f32(bits(o_w)) if use_w else None, lse_w.numpy() if use_w else None,
                           Q.bf16_to_f32(bits(sk)) if use_s else None, row_req.numpy(), row_pos.numpy(), sk_len.numpy(),
                           S, W, scale, Hkv)
        got = out.float().cpu().numpy()
        for r, w in want.items():
            assert np.abs(got[r] - w).max() <= 1e-2 * max(np.abs(w).max(), 1.0), (use_w, use_s, r)
        assert (outbuf[:2] == 5.0).all() and (outbuf[11:] == 5.0).all()
