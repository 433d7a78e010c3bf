"""GPU parity of libflagrot_mq.so (through the C-ABI, via flagrot_releaser_amd.prefill_mq) against oracle/mq.py.

Bars:
  prep_q     fp16 bit patterns equal to the oracle's (an operation-by-operation fp32 restatement);
  attention  relative L2 error of the merged output against fp64 attention over the oracle's dequantised pages
             <= 1e-3 per request and natural-log LSE within 5e-3 for static pages (measured 4e-4 / 3e-3), <= 1.5e-3 and
             1e-2 for key-only pages, whose keys go through packed-fp16 inverse transforms like the reference's
             (measured 9e-4 / 5.5e-3).  Scores reach +-40 here; FP16 operands, fp32 accumulation: the reference accepts
             anything not worse than BF16 FlashAttention (integrations/vllm_flagrot/scripts/bench_mq_prefill.py:225-242),
             whose error is about 3e-3.  Rows without a visible key: zeros and LSE -inf;
  bf16 out   equals the bf16 rounding of the fp32 output; rows of the layer output outside the plan keep their bytes;
  win_gather exact copies; bf_merge within 1e-2 of the fp64 oracle (bf16 output).
The pools follow the reference's check: unused block-table entries are poisoned with 2^30 and free pages hold random
bytes, so an over-read faults or produces NaNs.
"""
import math

import numpy as np
import pytest
import torch

from oracle import attend as OA
from oracle import mq as OM
from oracle import quant as Q
from tests.gpu_util import bits

pytestmark = pytest.mark.gpu
D, PAGE = 128, 16
LOG2E = 1.4426950408889634
FMT = {"int4a": (False, False, 144), "konlya": (True, False, 144), "int2a": (False, True, 80), "konlya2": (True, True, 80)}


def _rand_kv(L, Hkv, g):
    k = torch.randn(L, Hkv, D, generator=g)
    v = torch.randn(L, Hkv, D, generator=g)
    k[..., 5] *= 8
    k[..., 70] += 4
    v[..., 3] += 2
    return torch.cat([k, v], 1).bfloat16()


def _make_pool(dev, Ls, Hkv, fmt, g, kmask=None, kfull=None):
    """pages of sequences of lengths Ls written by the HIP writers; returns pool, block table (poisoned), and the fp64
    K / V of every sequence as the oracle reads them back from the same bytes."""
    from flagrot_releaser_amd import kernels as K
    cell = FMT[fmt][2]
    npg = [(L + PAGE - 1) // PAGE for L in Ls]
    total = sum(npg) + 11
    perm = torch.randperm(total, generator=g)
    bt = torch.full((len(Ls), max(npg) + 3), 1 << 30, dtype=torch.int32)
    pool = torch.randint(0, 256, (total, Hkv, cell * PAGE), generator=g, dtype=torch.uint8).to(dev)
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
            mask = torch.zeros(2 * Hkv, 4, dtype=torch.uint8)
            mask[:Hkv] = torch.as_tensor(kmask)
            hfull = torch.zeros(2 * Hkv, dtype=torch.uint8)
            if kfull is not None:
                hfull[:Hkv] = torch.as_tensor(kfull)
            K.w3_static_write(kv, slots, mask.to(dev), hfull.to(dev), pool, PAGE, fmt=fmt)
    torch.cuda.synchronize()
    hp = pool.cpu().numpy()
    for i, (L, n) in enumerate(zip(Ls, npg)):
        with np.errstate(all="ignore"):
            Kp, Vp = OA.dequant_pages(hp[bt[i, :n].numpy()], fmt, PAGE)
        Ks.append(Kp.reshape(n * PAGE, Hkv, D)[:L])
        Vs.append(Vp.reshape(n * PAGE, Hkv, D)[:L])
    return pool, bt.to(dev), Ks, Vs


def _rel(a, b):
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


CASES = [  # (requests [(L, nq)], shift, sink, G, fmt, kernel, ext)
    ([(1000, 1000)], 0, 0, 4, "int4a", 3, None),
    ([(777, 300)], 0, 0, 4, "konlya", 3, None),
    ([(10145, 145)], 0, 0, 4, "konlya", 3, None),
    ([(3000, 1)], 0, 0, 4, "int4a", 1, None),
    ([(17, 17)], 0, 0, 4, "konlya", 1, None),
    ([(16, 5)], 0, 0, 4, "int2a", 3, None),
    ([(64, 64)], 0, 0, 4, "konlya2", 3, None),
    ([(2000, 145), (1200, 300), (503, 17), (700, 700), (4000, 64)], 0, 0, 4, "konlya", 3, None),
    ([(2048, 600)], 128, 0, 4, "int4a", 3, None),
    ([(130, 70)], 64, 0, 4, "konlya2", 1, None),
    ([(1191, 300), (600, 600)], 128, 4, 4, "konlya", 3, None),
    ([(140, 140)], 128, 4, 4, "int2a", 3, None),
    ([(1500, 200), (300, 300)], 0, 0, 5, "konlya", 3, None),
    ([(1500, 200), (300, 300)], 0, 0, 8, "konlya2", 1, None),
    ([(1500, 200)], 0, 0, 1, "int4a", 3, None),
    ([(900, 200), (400, 100)], 128, 4, 8, "konlya", 3, {0: 650}),
    # kernel 4: 256-row tiles, two wavefront groups half a block apart
    ([(1000, 1000)], 0, 0, 4, "int4a", 4, None),
    ([(10145, 145)], 0, 0, 4, "konlya", 4, None),
    ([(16, 5)], 0, 0, 4, "int2a", 4, None),
    ([(64, 64)], 0, 0, 4, "konlya2", 4, None),
    ([(3000, 1)], 0, 0, 4, "int4a", 4, None),
    ([(2000, 145), (1200, 300), (503, 17), (700, 700), (4000, 64)], 0, 0, 4, "konlya", 4, None),
    ([(2048, 600)], 128, 0, 4, "int4a", 4, None),
    ([(1191, 300), (600, 600)], 128, 4, 4, "konlya", 4, None),
    ([(1500, 200), (300, 300)], 0, 0, 5, "konlya", 4, None),
    ([(1500, 200), (300, 300)], 0, 0, 8, "konlya2", 4, None),
    ([(1500, 200)], 0, 0, 1, "int4a", 4, None),
    ([(900, 200), (400, 100)], 128, 4, 8, "konlya", 4, {0: 650}),
    # items longer than the page-id window of the kernels (256 blocks): the window slides
    ([(30000, 40)], 0, 0, 4, "int4a", 4, None, 400),
    ([(30000, 40)], 0, 0, 4, "konlya", 3, None, 400),
    # ... and in the 64-row kernel, which fetches one block ahead (the others two)
    ([(30000, 12)], 0, 0, 4, "konlya", 1, None, 400),
    ([(20000, 16)], 0, 0, 4, "int2a", 1, None, 300),
]


def _random_cases(n, seed):
    """seeded shapes for the 256-row kernel: every format, odd group sizes, ragged lengths, shift / sink / ext, the
    planner's own kernel choice (None) among them"""
    rng = np.random.default_rng(seed)
    fmts = ["int4a", "konlya", "int2a", "konlya2"]
    out = []
    for i in range(n):
        G = int(rng.choice([1, 2, 3, 4, 6, 7, 8]))
        nreq = int(rng.integers(1, 4))
        reqs = []
        for _ in range(nreq):
            nq = int(rng.integers(1, 400))
            reqs.append((nq + int(rng.integers(0, 1200)), nq))
        shift = int(rng.choice([0, 0, 64, 128]))
        sink = int(rng.choice([0, 4])) if shift else 0
        ext = {0: int(rng.integers(0, reqs[0][0]))} if shift and rng.random() < 0.5 else None
        out.append((reqs, shift, sink, G, fmts[i % 4], None if i % 5 == 4 else 4, ext))
    return out


CASES += _random_cases(12, 77)


@pytest.mark.parametrize("case", range(len(CASES)))
def test_mq_attention_against_fp64(dev, case):
    from flagrot_releaser_amd import prefill_mq as MQ
    reqs_in, shift, sink, G, fmt, kernel, ext = CASES[case][:7]
    min_blocks = CASES[case][7] if len(CASES[case]) > 7 else None
    k2, int2, _ = FMT[fmt]
    g = torch.Generator().manual_seed(200 + case)
    Hkv = 2
    Hq = Hkv * G
    kmask = (torch.rand(Hkv, 4, generator=g) < 0.5).to(torch.uint8) if not k2 else None
    kfull = torch.tensor([1, 0], dtype=torch.uint8) if not k2 else None
    Ls = [L for L, _ in reqs_in]
    pool, bt, Ks, Vs = _make_pool(dev, Ls, Hkv, fmt, g, kmask, kfull)
    # batch rows: the requests' new tokens back to back, with 3 foreign rows in front
    reqs, row = [], 3
    for r, (L, nq) in enumerate(reqs_in):
        reqs.append((r, row, row + nq, L, L - nq))
        row += nq
    n = row + 2
    q = (torch.randn(n, Hq, D, generator=g) * 1.5).bfloat16()
    scale = 1 / math.sqrt(D)
    plan = MQ.build_plan(reqs, G, Hkv, shift, dev, sink=sink, kernel=kernel, ext=ext, min_blocks=min_blocks)
    assert plan.m == sum(nq for _, nq in reqs_in)
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
              f"|err| / (2e-3 + 1e-2 |ref|) = {el:.2f} (fp32 output)")
        assert lerr <= (1e-2 if k2 else 5e-3), (case, rep, lerr)
        # bf16 rows of the layer output
        ob = outbuf.float().cpu()
        idx = plan.idx.cpu().long()
        back = o32.cpu().bfloat16().float().reshape(plan.m, Hq * D)
        assert (ob[idx, :Hq * D] - back).abs().max() <= 2 ** -7 * back.abs().max()
        keep = torch.ones(n, dtype=torch.bool)
        keep[idx] = False
        assert (ob[keep] == 3.0).all() and (ob[:, Hq * D:] == 3.0).all()


def test_prep_q_fp32_rows_and_rejects(dev):
    from flagrot_releaser_amd import prefill_mq as MQ
    g = torch.Generator().manual_seed(5)
    Hkv, G = 3, 2
    q = torch.randn(9, Hkv * G, D, generator=g)
    kfull = torch.tensor([0, 1, 1], dtype=torch.uint8)
    kmask = (torch.rand(Hkv, 4, generator=g) < 0.5).to(torch.uint8)
    idx = torch.tensor([8, 1, 1, 4], dtype=torch.int32)
    got = MQ.prep_q(q.to(dev), 0.3, G, idx.to(dev), kfull.to(dev), kmask.to(dev)).cpu().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, OM.prep_q(q.numpy(), G, 0.3, idx.numpy(), kfull.numpy(), kmask.numpy()))
    got = MQ.prep_q(q.to(dev), 1.7, G).cpu().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, OM.prep_q(q.numpy(), G, 1.7))
    L = MQ.lib()
    assert L.frmq_attn(None, None, 0, None, 0, None, None, 1, 2, 4, 0, 0, None, None, 3, 64, None, 0) == -4
    assert L.frmq_attn(None, None, 0, None, 0, None, None, 1, 2, 200, 0, 0, None, None, 3, 128, None, 0) == -3
    assert b"head dim" in L.frmq_last_error() or b"G out" in L.frmq_last_error()
    assert L.frmq_smem_bytes() > 0


def test_win_gather_and_bf_merge(dev):
    from flagrot_releaser_amd import prefill_mq as MQ
    g = torch.Generator().manual_seed(8)
    Hkv, G, S, W = 2, 4, 4, 16
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
    # sink + window + page parts
    q = torch.randn(n, Hq, D, generator=g).bfloat16()
    idx = torch.tensor([2, 3, 4, 5, 6, 7, 8, 9, 10], dtype=torch.int64)
    o_p = torch.randn(m, Hq, D, generator=g)
    lse_p = torch.randn(Hq, m, generator=g) * 2
    lse_p[0, 0] = float("-inf")                   # no page key for this row
    lse_p[1, 1] = float("inf")
    o_w = torch.randn(m, Hq, D, generator=g).bfloat16()
    lse_w = torch.randn(Hq, m, generator=g) * 2
    sk = sinkb.view(nreq, S, 2 * Hkv, D)
    row_req = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1, 1], dtype=torch.int64)
    row_pos = torch.tensor([14, 17, 18, 30, 16, 19, 40, 41, 15], dtype=torch.int64)     # pos - W < 0: no sink key
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
