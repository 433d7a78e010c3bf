"""The host-side decode harness on the GPU: prompts prefilled into pages and BF16 rows, then decode steps (cache update
+ attention of one layer) captured once in a HIP graph and replayed with the builder's persistent buffers updated in
place; every step is checked against fp64 attention over the oracle's parse of the pages and the ring."""
import math

import numpy as np
import pytest
import torch

from oracle import attend as A
from oracle import pages as PG
from tests.gpu_util import P, bits, make_kv, spd_calib

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind,S,W,center", [("konlya2", 4, 16, True), ("konlya", 0, 0, False), ("int4a", 0, 8, False),
                                              ("konly", 2, 0, True)])
def test_decode_steps_in_graph(dev, kind, S, W, center):
    from flagrot_releaser_amd import backend as BK
    from flagrot_releaser_amd import kernels as K
    Hkv, G, R, rows, steps = 2, 4, 3, 4, 6
    g = torch.Generator().manual_seed(41)
    prompts, req = [37, 70], np.array([2, 0])
    nreal, nrows = len(prompts), 3                                   # one padding row in the captured batch
    max_len = max(prompts) + steps
    nblk = (max_len + P - 1) // P
    num_pages = nreal * nblk + 3
    pool = torch.randint(0, 256, (num_pages, Hkv, PG.chunk_bytes(kind, P)), dtype=torch.uint8, generator=g).to(dev)
    ids = torch.randperm(num_pages, generator=g)[:nreal * nblk].int().view(nreal, nblk)
    bt = torch.zeros(nrows, nblk, dtype=torch.int32)
    bt[:nreal] = ids
    static = BK.is_static(kind)
    kw = {}
    if static:
        kw["wmask"] = (torch.rand(2 * Hkv, 4, generator=g) < 0.5).to(torch.uint8).to(dev)
    else:
        Cq, co = spd_calib(Hkv, g)
        kw.update(CT=Cq.transpose(1, 2).contiguous().to(dev), co=co.to(dev))
    if center:
        kw["kmu"] = (1.5 * torch.randn(Hkv, 128, generator=g)).to(dev)
    builder = BK.StepPlanner(kind, Hkv, G, max_len, rows, R, S, W, dev)
    layer = BK.DecodeLayer(kind, Hkv, G, pool, builder, **kw)

    def slot_of(b, p):
        return int(bt[b, p // P]) * P + p % P

    for b, n in enumerate(prompts):
        kv = make_kv(n, Hkv, g, edge=False).to(dev)
        layer.prefill(kv, torch.tensor([slot_of(b, p) for p in range(n)], dtype=torch.int64, device=dev), int(req[b]))
    # persistent step inputs
    seq = torch.zeros(nrows, dtype=torch.int32, device=dev)
    slots = torch.full((nrows,), -1, dtype=torch.int64, device=dev)
    dbt = bt.to(dev)
    q = torch.zeros(nrows, G * Hkv, 128, dtype=torch.bfloat16, device=dev)
    kvn = torch.zeros(nrows, 2 * Hkv, 128, dtype=torch.bfloat16, device=dev)
    out = torch.zeros(nrows, G * Hkv * 128, dtype=torch.bfloat16, device=dev)
    lens = list(prompts)
    graph = None
    T = S + W
    for step in range(steps):
        lens = [n + 1 for n in lens]
        seq.copy_(torch.tensor(lens + [0], dtype=torch.int32))
        slots.copy_(torch.tensor([slot_of(b, lens[b] - 1) for b in range(nreal)] + [-1], dtype=torch.int64))
        q.copy_((torch.randn(q.shape, generator=g) * 0.8).bfloat16())
        kvn.copy_(make_kv(nrows, Hkv, g, edge=False))
        md = builder.prepare(seq, dbt, slots, homes=req)
        if graph is None:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            ring0 = None if layer.ring is None else layer.ring.clone()
            pool0 = pool.clone()
            with torch.cuda.stream(side):
                layer.step(q, kvn, md, out)                          # warm-up; the same step is replayed below
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            pool.copy_(pool0)
            if ring0 is not None:
                layer.ring.copy_(ring0)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                layer.step(q, kvn, md, out)
            pool.copy_(pool0)
            if ring0 is not None:
                layer.ring.copy_(ring0)
        graph.replay()
        torch.cuda.synchronize()
        # the new tokens sit in their BF16 slots (key rows centred)
        if T:
            want = layer.center_rows(kvn[:nreal])
            for b in range(nreal):
                s = BK.ring_slot(lens[b] - 1, S, W)
                if s >= 0:
                    assert torch.equal(layer.ring[int(req[b]), s], want[b]), (step, b)
        cached = md.page_tokens[:nreal].cpu().tolist() if T else lens
        ref = A.decode_reference(bits(q[:nreal]), pool.cpu().numpy(), kind, P, bt[:nreal].numpy(), cached, 1 / math.sqrt(128),
                                 kmask=kw["wmask"][:Hkv].cpu().numpy() if static else None,
                                 vmask=kw["wmask"][Hkv:].cpu().numpy() if static else None,
                                 tail=None if not T else bits(layer.ring),
                                 tail_len=None if not T else md.ring_tokens[:nreal].cpu().numpy(),
                                 tail_idx=None if not T else md.ring_home[:nreal].cpu().numpy(), kv_start=S)
        got = out[:nreal].view(nreal, G * Hkv, 128).float().cpu().numpy().astype(np.float64)
        assert not np.isnan(got).any()
        lim = 2e-3 + 1e-2 * np.abs(ref) + 1e-5 * np.abs(ref).max(axis=(1, 2), keepdims=True)
        assert (np.abs(got - ref) <= lim).all(), (kind, step, float(np.abs(got - ref).max()))
    assert int(layer.ws.counter.abs().sum()) == 0


@pytest.mark.parametrize("f8,big", [(False, 200.0), (True, 20.0), (True, 200.0)], ids=["f16meta", "f8meta", "f8meta-saturated"])
def test_kivi_decode_steps_in_graph(dev, f8, big):
    """KIVI-style pages: prompts prefilled (values per token, whole key groups), then decode steps replayed from one
    captured graph; steps that complete a 32-token key group encode it from the BF16 ring inside the graph (FP8-meta
    pages: after the group's value rows have put their whole-head flags into the key meta bytes).  The scores are sums
    of fp16 products q' * scale * code and q' * min per channel, so their absolute error grows with |min|: the prompt's
    large row is scaled by 20 for the FP8 pages (inside the E4M3 range) instead of 200, which saturates scale and min at
    448 in every channel and leaves a handful of tokens with near-equal scores of ~100 log2 units whose weights then move
    by more than the bar (an ill-conditioned case, not a format property)."""
    from flagrot_releaser_amd import backend as BK
    from flagrot_releaser_amd import kivi as KV
    from oracle import kivi as OK
    from oracle import quant as Q
    from tests.test_gpu_kivi import _calib, _kv, _ref_attn
    Hkv, G, R, rows, steps, S, W = 2, 4, 3, 4, 7, 4, 32
    T = S + W
    g = torch.Generator().manual_seed(43)
    prompts, req = [61, 90], np.array([1, 2])                          # groups complete at lengths 64 and 96
    nreal, nrows = len(prompts), 3
    max_len = max(prompts) + steps
    nblk = 2 * (-(-max_len // 32))
    num_pages = nreal * nblk + 2
    pool = torch.zeros(num_pages, Hkv, KV.chunk_bytes(128, f8), dtype=torch.uint8, device=dev)
    bt = torch.zeros(nrows, nblk, dtype=torch.int32)
    bt[:nreal] = torch.randperm(num_pages, generator=g)[:nreal * nblk].int().view(nreal, nblk)
    qs, lz, co = _calib(Hkv, 24, g)
    builder = BK.StepPlanner("kivi2", Hkv, G, max_len, rows, R, S, W, dev)
    layer = BK.KiviDecodeLayer(Hkv, G, pool, builder, qs.to(dev), lz.to(dev), co.to(dev), f8=f8)

    def slot_of(b, p):
        return int(bt[b, p // P]) * P + p % P

    for b, n in enumerate(prompts):
        layer.prefill(_kv(n, Hkv, g, big=big).to(dev), torch.tensor([slot_of(b, p) for p in range(n)], dtype=torch.int64, device=dev),
                      int(req[b]))
    seq = torch.zeros(nrows, dtype=torch.int32, device=dev)
    slots = torch.full((nrows,), -1, dtype=torch.int64, device=dev)
    dbt = bt.to(dev)
    q = torch.zeros(nrows, G * Hkv, 128, dtype=torch.bfloat16, device=dev)
    kvn = torch.zeros(nrows, 2 * Hkv, 128, dtype=torch.bfloat16, device=dev)
    out = torch.zeros(nrows, G * Hkv * 128, dtype=torch.bfloat16, device=dev)
    lens = list(prompts)
    graph = None
    encoded = 0
    worst = 0.0
    for step in range(steps):
        lens = [n + 1 for n in lens]
        seq.copy_(torch.tensor(lens + [0], dtype=torch.int32))
        slots.copy_(torch.tensor([slot_of(b, lens[b] - 1) for b in range(nreal)] + [-1], dtype=torch.int64))
        q.copy_((torch.randn(q.shape, generator=g) * 1.2).bfloat16())
        kvn.copy_(_kv(nrows, Hkv, g))
        md = builder.prepare(seq, dbt, slots, homes=req)
        encoded += int((md.group_dst[:, 0] >= 0).sum())
        if graph is None:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            ring0, pool0 = layer.ring.clone(), pool.clone()
            with torch.cuda.stream(side):
                layer.step(q, kvn, md, out)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            pool.copy_(pool0); layer.ring.copy_(ring0)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                layer.step(q, kvn, md, out)
            pool.copy_(pool0); layer.ring.copy_(ring0)
        graph.replay()
        torch.cuda.synchronize()
        pnp = pool.cpu().numpy()
        ringf = Q.bf16_to_f32(bits(layer.ring)).astype(np.float64).reshape(R + 1, T, 2 * Hkv, 128)
        qf = Q.bf16_to_f32(bits(q)).astype(np.float64)
        got = Q.bf16_to_f32(bits(out)).astype(np.float64).reshape(nrows, G * Hkv, 128)
        for b in range(nreal):
            L = lens[b]
            cached, tl = int(md.page_tokens[b]), int(md.ring_tokens[b])
            assert cached == (L - W if L - W > S else 0) and tl == min(L, T) and cached <= 32 * (L // 32)
            Kp, Vp = OK.dequant_groups(pnp[bt[b, :2 * (-(-max(cached, 1) // 32))].numpy()], 128, f8=f8)
            tb = ringf[int(req[b]), :tl]
            ref = _ref_attn(qf[b], Kp, Vp, min(S, cached), cached, tb[:, :Hkv], tb[:, Hkv:], G, 1 / math.sqrt(128))
            tol = 1e-2 * np.abs(ref).max() + 1e-6
            worst = max(worst, float(np.abs(got[b] - ref).max() / tol))
            assert np.abs(got[b] - ref).max() <= tol, (step, b, float(np.abs(got[b] - ref).max()), tol)
    print(f"\nkivi backend steps (f8={f8}, large row x{big:g}): worst max |err| / (1e-2 max |ref|) = {worst:.3f}", flush=True)
    assert encoded == 2                                               # lengths 64 and 96 were reached


@pytest.mark.parametrize("kind,S,W,center", [("konlya2", 4, 16, True), ("int4a", 0, 8, False), ("konly", 2, 0, False)])
def test_chunked_prefill_equals_whole_prompt(dev, kind, S, W, center):
    """a prompt that arrives in chunks leaves the same page bytes and the same BF16 rows as the prompt in one piece"""
    from flagrot_releaser_amd import backend as BK
    Hkv, G, R, n, cuts = 2, 4, 2, 150, [0, 50, 87, 88, 150]
    g = torch.Generator().manual_seed(51)
    nblk = (n + P - 1) // P
    init = torch.randint(0, 256, (nblk + 3, Hkv, PG.chunk_bytes(kind, P)), dtype=torch.uint8, generator=g)
    row = torch.randperm(nblk + 3, generator=g)[:nblk].int()
    slots = (row.long()[torch.arange(n) // P] * P + torch.arange(n) % P).to(dev)
    kw = {}
    if BK.is_static(kind):
        kw["wmask"] = (torch.rand(2 * Hkv, 4, generator=g) < 0.5).to(torch.uint8).to(dev)
    else:
        Cq, co = spd_calib(Hkv, g)
        kw.update(CT=Cq.transpose(1, 2).contiguous().to(dev), co=co.to(dev))
    if center:
        kw["kmu"] = (1.5 * torch.randn(Hkv, 128, generator=g)).to(dev)
    kv = make_kv(n, Hkv, g, edge=True).to(dev)
    layers = []
    for _ in range(2):
        planner = BK.StepPlanner(kind, Hkv, G, n + 8, 4, R, S, W, dev)
        layers.append(BK.DecodeLayer(kind, Hkv, G, init.clone().to(dev), planner, **kw))
    whole, chunked = layers
    whole.prefill(kv, slots, 1)
    for a, b in zip(cuts[:-1], cuts[1:]):
        chunked.prefill_chunk(kv[a:b], slots[a:b], 1, a)
    torch.cuda.synchronize()
    assert torch.equal(whole.pool, chunked.pool)
    if S + W:
        assert torch.equal(whole.ring, chunked.ring)


@pytest.mark.parametrize("f8", [False, True], ids=["f16meta", "f8meta"])
def test_kivi_chunked_prefill_equals_whole_prompt(dev, f8):
    """KIVI-style pages: a prompt in chunks -- a chunk may start inside a 32-token key group, whose earlier positions
    the encoder then reads from the BF16 ring -- leaves the same page bytes (values, key codes, key meta, flags) and the
    same BF16 rows as the prompt in one piece"""
    from flagrot_releaser_amd import backend as BK
    from flagrot_releaser_amd import kivi as KV
    from tests.test_gpu_kivi import _calib, _kv
    Hkv, G, R, S, W, n = 2, 4, 2, 4, 32, 150
    g = torch.Generator().manual_seed(52)
    nblk = (n + P - 1) // P
    row = torch.randperm(nblk + 3, generator=g)[:nblk].int()
    slots = (row.long()[torch.arange(n) // P] * P + torch.arange(n) % P).to(dev)
    qs, lz, co = _calib(Hkv, 24, g)
    kv = _kv(n, Hkv, g, big=20.0).to(dev)
    for cuts in ([0, 50, 87, 88, 150], [0, 31, 33, 64, 97, 150], [0, 150]):
        layers = []
        for _ in range(2):
            pool = torch.zeros(nblk + 3, Hkv, KV.chunk_bytes(128, f8), dtype=torch.uint8, device=dev)
            planner = BK.StepPlanner("kivi2", Hkv, G, n + 8, 4, R, S, W, dev)
            layers.append(BK.KiviDecodeLayer(Hkv, G, pool, planner, qs.to(dev), lz.to(dev), co.to(dev), f8=f8))
        whole, chunked = layers
        whole.prefill(kv, slots, 1)
        for a, b in zip(cuts[:-1], cuts[1:]):
            chunked.prefill_chunk(kv[a:b], slots[a:b], 1, a, row.to(dev))
        torch.cuda.synchronize()
        assert torch.equal(whole.pool, chunked.pool), cuts
        assert torch.equal(whole.ring, chunked.ring), cuts
