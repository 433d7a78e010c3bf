"""GPU test of the entry point that allocates nothing, fr_cb_attn_noalloc, through the C ABI against fr_cb_attn /
fr_v2_attn (the entry points whose caller-owned workspace it replaces by an array built into the library).

Two calls in a row on one GPU, the second with a smaller input: the second call meets whatever the first left in the
shared array.  Both launch shapes are covered (4-wavefront workgroups that share a sequence's page range, and large
workgroups with fixed token ranges).  In either shape the wavefronts draw their pages from a counter, so the fp32
summation order depends on the draw order and two runs of even the same entry point are not bit-identical: the two
entry points are held to the decode bar (|a - b| <= 2e-3 + 1e-2 |b|) against each other and against the fp64 oracle.
The last test checks the size limit and the error codes."""
import math

import numpy as np
import pytest
import torch

from oracle import attend as A
from oracle import pages as PG
from tests.gpu_util import P as P16, alloc_tables, bits, make_kv, slots_of, spd_calib

pytestmark = pytest.mark.gpu
LOG2E = 1.4426950408889634
ATOL, RTOL = 2e-3, 1e-2


def _cache(dev, lens, kind, Hkv, seed):
    from flagrot_releaser_amd import kernels as K
    g = torch.Generator().manual_seed(seed)
    num_pages = sum((n + P16 - 1) // P16 for n in lens) + 5
    pool = torch.randint(0, 256, (num_pages, Hkv, PG.chunk_bytes(kind, P16)), dtype=torch.uint8, generator=g).to(dev)
    bt = alloc_tables(lens, num_pages, g, P16)
    Cq, co = spd_calib(Hkv, g)
    CT, co = Cq.transpose(1, 2).contiguous().to(dev), co.to(dev)
    for b, n in enumerate(lens):
        kv = make_kv(n, Hkv, g, edge=False).to(dev)
        K.cb_write(kv, slots_of(bt, b, n, P16).to(dev), CT, co, kind, pool, P16)
    return pool, bt, g


def _both(dev, kind, lens, Hkv, G, nsplit, seed, win=None, kv_start=0):
    """runs the workspace entry point and the allocation-free one on the same inputs; returns (a, b, ref, large)"""
    from flagrot_releaser_amd import kernels as K
    pool, bt, g = _cache(dev, lens, kind, Hkv, seed)
    B, HQ = len(lens), G * Hkv
    q = (torch.randn(B, HQ, 128, generator=g) * 0.8).bfloat16()
    scale = 1 / math.sqrt(128)
    tail = tail_len = tail_idx = None
    tkw = {}
    if win is not None:
        W, R = win
        tail = torch.randn(R, W, 2 * Hkv, 128, generator=g).bfloat16()
        tail_idx = torch.randperm(R, generator=g)[:B].int()
        tail_len = torch.randint(1, W + 1, (B,), generator=g).int()
        dt = tail.to(dev)
        tkw = dict(tail=dt, tail_len=tail_len.to(dev), tail_idx=tail_idx.to(dev), tail_bs=dt.stride(0), tail_ts=dt.stride(1))
    ref = A.decode_reference(bits(q), pool.cpu().numpy(), kind, P16, bt.numpy(), lens, scale,
                             tail=None if tail is None else bits(tail),
                             tail_len=None if tail is None else tail_len.numpy(),
                             tail_idx=None if tail is None else tail_idx.numpy(), kv_start=kv_start)
    ns, ch = K.plan_cb(B, max(lens), Hkv, P16, kind, nsplit=nsplit, G=G)
    HV = Hkv * -(-G // 4)                         # (KV head, 4-head q tile) pairs: what the launch shape depends on
    if G != 4:                                    # the workspace entry point routes other groups through fr_v2_attn
        WV, GT = K.vheads(Hkv, G, 128, kind), K.tile_of(K.v2_variant(kind, G, 128))
    else:
        WV, GT = Hkv, 4
    ws = K.Workspace(B, WV, B * WV * (ns + 1), dev, GT, 128)
    dq, dbt, dseq = q.to(dev), bt.to(dev), torch.tensor(lens, dtype=torch.int32, device=dev)
    out_a = torch.full((B, HQ * 128), float("nan"), dtype=torch.bfloat16, device=dev)
    out_b = torch.full((B, HQ * 128), float("nan"), dtype=torch.bfloat16, device=dev)
    K.cb_attn(dq, pool, dbt, dseq, out_a, ns, ch, ws, scale * LOG2E, kind, kv_start=kv_start, **tkw)
    K.cb_attn_noalloc(dq, pool, dbt, dseq, out_b, ns, ch, scale * LOG2E, kind, kv_start=kv_start, **tkw)
    torch.cuda.synchronize()
    # large workgroups with fixed ranges: chunks of >= 1024 tokens on at most one round of CUs
    large = ch >= K.BIG_CHUNK and B * HV * ns <= torch.cuda.get_device_properties(dev).multi_processor_count
    return out_a, out_b, ref, large


def _check(out_a, out_b, ref, large, what):
    B = ref.shape[0]
    a = out_a.view(B, -1, 128).float().cpu().numpy().astype(np.float64)
    b = out_b.view(B, -1, 128).float().cpu().numpy().astype(np.float64)
    assert not np.isnan(b).any(), what
    assert (np.abs(b - a) <= ATOL + RTOL * np.abs(a)).all(), f"{what}: differs from the workspace entry point"
    assert (np.abs(b - ref) <= ATOL + RTOL * np.abs(ref) + 1e-5 * np.abs(ref).max(axis=(1, 2), keepdims=True)).all(), \
        f"{what}: differs from the oracle"


@pytest.mark.parametrize("kind", ["konlya", "konlya2"])
def test_noalloc_matches_workspace_entry_point_twice(dev, kind):
    # first call: splits + BF16 tail rows + two q tiles (G = 8); second call, smaller, right behind it
    _check(*_both(dev, kind, [900, 333, 64, 1500], Hkv=2, G=8, nsplit=4, seed=71, win=(40, 6), kv_start=4), f"{kind} first")
    _check(*_both(dev, kind, [200, 17], Hkv=2, G=4, nsplit=2, seed=72), f"{kind} second (smaller)")


def test_noalloc_large_workgroups_twice(dev):
    a = _both(dev, "konlya", [4300, 2100], Hkv=2, G=4, nsplit=2, seed=73, win=(24, 3))
    assert a[3], "expected the large-workgroup launch shape"
    _check(*a, "large first")
    b = _both(dev, "konlya", [2300], Hkv=2, G=4, nsplit=2, seed=74)
    assert b[3]
    _check(*b, "large second (smaller)")


def test_noalloc_allocates_nothing_and_replays_from_a_graph(dev):
    """after one warm-up call (the first call on a device looks the built-in array up and must not be made under
    capture) a call changes neither the device's free memory nor torch's allocator; captured into a HIP graph it replays
    with new queries and matches the eager call each time"""
    from flagrot_releaser_amd import kernels as K
    kind, lens, Hkv, G = "konlya", [900, 333, 1500], 2, 4
    pool, bt, g = _cache(dev, lens, kind, Hkv, 75)
    B, HQ = len(lens), G * Hkv
    dq = (torch.randn(B, HQ, 128, generator=g) * 0.8).bfloat16().to(dev)
    dbt, dseq = bt.to(dev), torch.tensor(lens, dtype=torch.int32, device=dev)
    ns, ch = K.plan_cb(B, max(lens), Hkv, P16, kind, nsplit=3)
    out = torch.zeros(B, HQ * 128, dtype=torch.bfloat16, device=dev)
    scale = LOG2E / math.sqrt(128)
    call = K.cb_attn_noalloc(dq, pool, dbt, dseq, out, ns, ch, scale, kind, bound=True)
    call()                                                   # warm-up: address lookup, module load
    torch.cuda.synchronize()
    free0, held0, peak0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.max_memory_allocated()
    call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_allocated() == held0
    assert torch.cuda.max_memory_allocated() == peak0
    eager = out.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        K.cb_attn_noalloc(dq, pool, dbt, dseq, out, ns, ch, scale, kind)      # the capture stream's first use
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        K.cb_attn_noalloc(dq, pool, dbt, dseq, out, ns, ch, scale, kind)
    for rep in range(3):
        if rep:
            dq.copy_((torch.randn(B, HQ, 128, generator=g) * 0.8).bfloat16())
            call()                                           # eager work and a synchronisation between the replays
            torch.cuda.synchronize()
            eager = out.clone()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        a, b = eager.float().cpu().numpy().astype(np.float64), out.float().cpu().numpy().astype(np.float64)
        assert (np.abs(b - a) <= ATOL + RTOL * np.abs(a)).all(), f"replay {rep} differs from the eager call"


def test_noalloc_rejects_sizes_beyond_the_built_in_workspace(dev):
    from flagrot_releaser_amd import kernels as K
    L = K.lib()
    z = torch.zeros(1024, dtype=torch.uint8, device=dev)
    zp = z.data_ptr()
    # B * Hkv * ceil(gqa / 4) * (nsplit + 1) = 64 * 8 * 1 * 17 = 8704 > 8192
    rc = L.fr_cb_attn_noalloc(zp, 512, zp, zp, 1, zp, 64, 8, 16, 16, 1024, 1.0, 10, zp, 512, None, None, None, 0, 0,
                              None, 4, 0)
    assert rc == -2 and b"exceed" in L.fr_last_error()
    assert L.fr_cb_attn_noalloc(zp, 512, zp, zp, 1, zp, 1, 1, 16, 1, 64, 1.0, 3, zp, 512, None, None, None, 0, 0, None,
                                4, 0) == -4
