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
