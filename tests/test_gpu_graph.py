"""The decode step inside a HIP graph: the selecting writer and the paged decode captured once and replayed with new
inputs (the plugin captures its decode step, `backend.py` of the reference; every entry point must be capturable: no
allocation, no synchronisation, counters that reset themselves).  Every replay is checked against the eager result of
the same inputs, with eager work and synchronisations between the replays."""
import math

import pytest
import torch

from tests.gpu_util import P, alloc_tables, make_kv, slots_of, spd_calib

pytestmark = pytest.mark.gpu
LOG2E = 1.4426950408889634


@pytest.mark.parametrize("lens,Hkv,nsplit", [([700, 120, 333], 4, None), ([2300, 2100], 2, 1)])
def test_decode_step_in_graph(dev, lens, Hkv, nsplit):
    from flagrot_releaser_amd import kernels as K
    kind, G = "konlya", 4
    g = torch.Generator().manual_seed(31)
    B = len(lens)
    num_pages = sum((n + 1 + P - 1) // P for n in lens) + 5
    pool = torch.randint(0, 256, (num_pages, Hkv, K.cb_chunk_bytes(kind, P)), dtype=torch.uint8, generator=g).to(dev)
    bt = alloc_tables([n + 1 for n in lens], num_pages, g)
    Cq, co = spd_calib(Hkv, g)
    CT, co = Cq.transpose(1, 2).contiguous().to(dev), co.to(dev)
    for b in range(B):
        K.cb_write(make_kv(lens[b], Hkv, g, edge=False).to(dev), slots_of(bt, b, lens[b]).to(dev), CT, co, kind, pool, P)
    dbt = bt.to(dev)
    seq = torch.tensor([n + 1 for n in lens], dtype=torch.int32, device=dev)       # the step's token included
    new_slots = torch.stack([slots_of(bt, b, lens[b] + 1)[-1] for b in range(B)]).to(dev)
    ns, ch = K.plan_cb(B, max(lens) + 1, Hkv, P, kind, nsplit=nsplit)
    ws = K.Workspace(B, Hkv, B * Hkv * (ns + 1), dev)
    scale = LOG2E / math.sqrt(128)
    q = torch.zeros(B, G * Hkv, 128, dtype=torch.bfloat16, device=dev)
    kv = torch.zeros(B, 2 * Hkv, 128, dtype=torch.bfloat16, device=dev)
    out = torch.zeros(B, G * Hkv * 128, dtype=torch.bfloat16, device=dev)

    def step(o):
        K.cb_write(kv, new_slots, CT, co, kind, pool, P)
        K.cb_attn(q, pool, dbt, seq, o, ns, ch, ws, scale, kind)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(out)                                   # warm-up outside the capture (library loading, caches)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(out)
    eager = torch.zeros_like(out)
    for rep in range(4):
        q.copy_((torch.randn(q.shape, generator=g) * 0.8).bfloat16())
        kv.copy_(make_kv(B, Hkv, g, edge=False))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        pool_after = pool.clone()
        step(eager)                                 # the same step eagerly: same pool bytes, same output up to the
        torch.cuda.synchronize()                    # order in which wavefronts happened to draw their pages
        assert torch.equal(pool, pool_after)
        assert not torch.isnan(got.float()).any()
        err = (got.float() - eager.float()).abs().max().item()
        assert err <= 2e-3 + 1e-2 * eager.float().abs().max().item(), (rep, err)
    assert int(ws.counter.abs().sum()) == 0


@pytest.mark.parametrize("name,B,Hkv,G,L,nsplit", [
    ("large workgroups, 32 splits of 1024 tokens", 2, 2, 4, 32768, 32),
    ("4-wavefront workgroups sharing ranges, 64 splits of 128 tokens", 3, 2, 4, 8192, 64),
    ("8-head tiles, 64 splits of 128 tokens", 2, 2, 8, 8192, 64),
    ("8-head tiles, large workgroups, 32 splits", 1, 2, 8, 32768, 32),
])
def test_split_merge_200_replays(dev, name, B, Hkv, G, L, nsplit):
    """The merge of split partials under replay pressure.  Every split workgroup stores its partials, waits for the
    stores, and takes a ticket; the last arriver of a (sequence, head tile) reads all partials back and writes the
    output.  Were a ticket to overtake its stores, the merger would read what the PREVIOUS launch left in the workspace.
    So 200 replays of one captured launch cycle through four very different queries: a stale partial would show as an
    O(1) error, while the legitimate run-to-run difference (the order in which wavefronts draw page quads changes fp32
    sums in their last bits) stays within two bf16 units of the largest output.  Stops at the first replay that
    differs; the tickets must all be back at zero."""
    from flagrot_releaser_amd import kernels as K
    kind, W, S = "konlya", 16, 4
    g = torch.Generator().manual_seed(77)
    npg = -(-L // P)
    pool = torch.randint(0, 256, (B * npg + 3, Hkv, K.cb_chunk_bytes(kind, P)), dtype=torch.uint8, generator=g).to(dev)
    bt = alloc_tables([L] * B, B * npg + 3, g).to(dev)
    w = 0.5 + 1.5 * torch.rand(Hkv, 128, generator=g)
    CT, co = torch.diag_embed(w).contiguous().to(dev), w.contiguous().to(dev)
    for b in range(B):
        for s0 in range(0, L, 8192):
            n = min(8192, L - s0)
            pos = torch.arange(s0, s0 + n, device=dev)
            K.cb_write(make_kv(n, Hkv, g, edge=False).to(dev), bt[b].long()[pos // P] * P + pos % P, CT, co, kind, pool, P)
    seq = torch.full((B,), L, dtype=torch.int32, device=dev)
    ring = torch.randn(B, S + W, 2 * Hkv, 128, generator=g).bfloat16().to(dev)
    tkw = dict(tail=ring, tail_len=torch.full((B,), S + W, dtype=torch.int32, device=dev),
               tail_idx=torch.arange(B, dtype=torch.int32, device=dev), tail_bs=ring.stride(0), tail_ts=ring.stride(1),
               kv_start=S)
    ns, ch = K.plan_cb(B, L, Hkv, P, kind, nsplit=nsplit, G=G)
    assert ns == nsplit
    HV, GT = (K.vheads(Hkv, G, 128, kind), K.tile_of(K.v2_variant(kind, G, 128))) if G != 4 else (Hkv, 4)
    ws = K.Workspace(B, HV, B * HV * (ns + 1), dev, GT, 128)
    scale = LOG2E / math.sqrt(128)
    bank = [(torch.randn(B, G * Hkv, 128, generator=g) * (0.5 + i)).bfloat16().to(dev) for i in range(4)]
    q = torch.zeros_like(bank[0])
    out = torch.zeros(B, G * Hkv * 128, dtype=torch.bfloat16, device=dev)

    def launch():
        K.cb_attn(q, pool, bt, seq, out, ns, ch, ws, scale, kind, **tkw)

    want = []
    for qb in bank:                                     # eager results, one per query
        q.copy_(qb)
        launch()
        torch.cuda.synchronize()
        want.append(out.float().clone())
    assert min((want[0] - want[i]).abs().max().item() for i in (1, 2, 3)) > 0.05, "queries too alike to expose stale partials"
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
    for rep in range(200):
        k = (rep * 7 + rep // 3) % 4
        q.copy_(bank[k])
        graph.replay()
        torch.cuda.synchronize()
        diff = (out.float() - want[k]).abs().max().item()
        assert diff <= 2 ** -7 * want[k].abs().max().item(), f"{name}: replay {rep} (query {k}) differs by {diff}"
    assert int(ws.counter.abs().sum()) == 0
