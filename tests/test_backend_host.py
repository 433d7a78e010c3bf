"""Host bookkeeping of the decode step (flagrot_releaser_amd.backend) on the CPU: batch buckets, the BF16 ring slot
formula against a token-by-token simulation, and the metadata builder against a per-row restatement."""
import numpy as np
import pytest
import torch

from flagrot_releaser_amd import backend as BK


def test_plan_bucket():
    assert [BK.plan_bucket(b) for b in (1, 2, 3, 4, 5, 8, 9, 255, 256, 257, 300)] == [1, 2, 4, 4, 8, 8, 16, 256, 256, 272, 304]
    for b in range(1, 600):
        assert BK.plan_bucket(b) >= b and BK.plan_bucket(BK.plan_bucket(b)) == BK.plan_bucket(b)


@pytest.mark.parametrize("S,W", [(4, 128), (4, 8), (0, 16), (3, 0), (1, 1)])
def test_ring_slot_keeps_sinks_and_window(S, W):
    """writing every position p to ring_slot(p) leaves, after L tokens, exactly the sinks [0, min(L, S)) and the window
    [max(S, L - W), L) in the slots [0, min(L, S + W)) -- what the decode kernel reads as its BF16 rows"""
    T = S + W
    row = [-1] * max(T, 1)
    for L in range(1, 3 * T + 40):
        p = L - 1
        s = BK.ring_slot(p, S, W)
        assert s == int(BK.ring_slot(torch.tensor([p]), S, W)[0])
        if s >= 0:
            row[s] = p
        held = sorted(x for x in row[:min(L, T)] if x >= 0)
        want = sorted(set(range(min(L, S))) | set(range(max(S, L - W), L)))
        assert held == want, (L, held, want)
        assert all(x >= 0 for x in row[:min(L, T)])


@pytest.mark.parametrize("S,W", [(0, 0), (4, 128), (4, 0), (0, 16)])
def test_metadata_builder_rows(S, W):
    R, rows = 5, 8
    b = BK.StepPlanner("konlya", 8, 4, 4096, rows, R, S, W, "cpu", plan_fn=lambda B: (3, 1408))
    lens = torch.tensor([1, 3, 4, 5, 131, 132, 133, 1000], dtype=torch.int32)
    req = np.array([2, 0, 4, 1, 3, 2])                     # two rows more than request slots: padding rows
    md = b.prepare(lens, torch.zeros(8, 4, dtype=torch.int32), torch.zeros(8, dtype=torch.int64), homes=req)
    assert (md.nsplit, md.chunk, md.rows) == (3, 1408, 8)
    if S == 0 and W == 0:
        assert md.page_tokens is lens and md.ring_tokens is None
        return
    T = S + W
    for i, L in enumerate(lens.tolist()):
        row = int(req[i]) if i < len(req) else R
        assert int(md.ring_home[i]) == row
        assert int(md.page_tokens[i]) == (L - W if L - W > S else 0)
        assert int(md.ring_tokens[i]) == min(L, T)
        s = BK.ring_slot(L - 1, S, W)
        assert int(md.ring_dest[i]) == (row * T + s if s >= 0 else R * T)
    # the buffers are persistent: a second, shorter build reuses them
    md2 = b.prepare(lens[:3] + 1, md.block_table[:3], md.slots[:3], homes=req[:3])
    assert md2.ring_home.data_ptr() == md.ring_home.data_ptr() and md2.ring_dest.shape[0] == 3


def test_kivi_decode_groups():
    """the key group a decode step completes: ring rows of its 32 positions (sinks excluded) and their page slots"""
    S, W, R = 4, 64, 3
    T = S + W
    b = BK.StepPlanner("kivi2", 2, 4, 4096, 6, R, S, W, "cpu", plan_fn=lambda B: (2, 512))
    lens = torch.tensor([32, 33, 64, 31, 96, 128], dtype=torch.int32)
    bt = torch.arange(6 * 16, dtype=torch.int32).view(6, 16) * 3 % 97
    req = np.array([1, 0, 2, 1])                                           # rows 4, 5: padding (ring row R)
    md = b.prepare(lens, bt, torch.zeros(6, dtype=torch.int64), homes=req)
    for i, L in enumerate(lens.tolist()):
        act = L % 32 == 0 and L >= 32 and i < len(req)
        if not act:
            assert int(md.group_dst[i, 0]) < 0 and (md.group_src[i] == -1).all()
            continue
        for j in range(32):
            p = L - 32 + j
            assert int(md.group_dst[i, j]) == int(bt[i, p // 16]) * 16 + p % 16
            assert int(md.group_src[i, j]) == (-1 if p < S else int(req[i]) * T + BK.ring_slot(p, S, W))


@pytest.mark.parametrize("S,W", [(4, 32), (0, 64), (4, 128)])
def test_chunk_key_groups_against_a_position_walk(S, W):
    """the key groups a prompt chunk completes: every position's source (chunk row, ring row of an earlier chunk, or
    sink) and page slot, against a walk over positions with a model of which chunk brought which position"""
    geo = BK.RingGeometry(S, W)
    T = S + W
    rng = np.random.default_rng(5 + S + W)
    bt = torch.from_numpy(rng.permutation(64).astype(np.int32))
    for req, cuts in ((0, [0, 150]), (2, [0, 50, 87, 150]), (1, [0, 31, 32, 33, 97, 128, 129]), (3, [0, 64, 65, 200, 201, 233])):
        for a, b in zip(cuts[:-1], cuts[1:]):
            got = BK.chunk_key_groups(geo, a, b - a, req * T, bt)
            groups = [g for g in range(b // 32) if 32 * g + 31 >= a]          # completed by [a, b): last position inside it
            if not groups:
                assert got is None
                continue
            src, dst = got
            assert src.shape == dst.shape == (len(groups), 32) and src.dtype == dst.dtype == torch.int64
            for i, g in enumerate(groups):
                for j in range(32):
                    p = 32 * g + j
                    assert int(dst[i, j]) == int(bt[p // 16]) * 16 + p % 16
                    if p < S:
                        want = -1
                    elif p >= a:
                        want = p - a
                    else:
                        assert a - p <= W, "an earlier position must still be in the window"
                        want = -2 - (req * T + S + (p - S) % W)
                    assert int(src[i, j]) == want, (req, a, b, g, j)
