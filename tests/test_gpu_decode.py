"""GPU parity of paged decode attention through the C ABI against the oracle's dequantise-then-attend reference.

Bar (floating point, the tolerance of the build's north star: max-abs 2e-3 / rel 1e-2):
  * rows of ordinary data: |out - ref| <= 2e-3 + 1e-2 * |ref| element-wise;
  * row 0 (and every row when the sequences share one block-table row), which carries the reference tests'
    adversarial groups (values x300, x1e-5, constants, one-hots: log2 scores of +-1000, outputs of several hundred, so
    that a 1e-5 relative change of one score moves a weight by percents): |out - ref| <= 2e-3 + 1e-2 * max |ref[row]|
    (the reference's own tests measure every row against the global max |ref| with a 4e-3 floor,
    test_kernels.py:173), AND element-wise within TWICE the bar of the ordinary rows (measured on these cases: at most
    0.99 times; randomised shapes: 0.3-0.5 % of such rows above 1, on the 2-bit pages; up to 15 times before the value
    products of quads with large V scales were rescaled and the scores of quads with very large scores formed a second
    time -- beside a group scaled x300 the matrix pipe's 24-bit window cut its neighbours short).  The query variants
    enter the score products as fp16 value + fp16 remainder (22 bits).
Every case prints its worst element-wise ratio |err| / (2e-3 + 1e-2 |ref|), ordinary and adversarial rows apart.
ref = fp64 softmax attention over the pages parsed by the oracle's independent layout parser (the cache bytes are
written by the HIP writers, whose bit-exactness tests/test_gpu_writers.py establishes)."""
import contextlib
import math
import os

import numpy as np
import pytest
import torch

from oracle import attend as A
from oracle import pages as PG
from tests.gpu_util import P as P16, alloc_tables, bits, make_kv, slots_of, spd_calib

pytestmark = pytest.mark.gpu
LOG2E = 1.4426950408889634
ATOL, RTOL = 2e-3, 1e-2
HARD_ROWS = 2.0      # element-wise bound of the rows that read the adversarial tokens, in units of the ordinary bar


@contextlib.contextmanager
def as_planned(on):
    """the library runs the caller's split plan unchanged inside this block (if `on`)"""
    before = os.environ.get("FLAGROT_REPLAN")
    if on:
        os.environ["FLAGROT_REPLAN"] = "0"
    try:
        yield
    finally:
        if on:
            if before is None:
                del os.environ["FLAGROT_REPLAN"]
            else:
                os.environ["FLAGROT_REPLAN"] = before


def run_case(dev, mode, lens, fmt, win=None, bt_shared=False, seed=0, G=4, Hkv=4, kv_start=0, nsplit=None, P=P16,
             hard_rows=None, twin=None):
    from flagrot_releaser_amd import kernels as K
    g = torch.Generator().manual_seed(seed)
    B = len(lens)
    HQ = G * Hkv
    num_pages = sum((n + P - 1) // P for n in lens) + 7
    pool = torch.randint(0, 256, (num_pages, Hkv, PG.chunk_bytes(fmt, P)), dtype=torch.uint8, generator=g).to(dev)
    bt = alloc_tables(lens, num_pages, g, P)
    if bt_shared:
        # every sequence reads the table row of the longest one (a shorter row would name page 0 for the positions past
        # its end, and the writer below would be handed the same slot several times)
        first = max(range(B), key=lambda b: lens[b])
        bt = bt[first:first + 1].expand(B, -1)
        if bt_shared != "stride0":
            bt = bt.contiguous()
    mask = (torch.rand(2 * Hkv, 4, generator=g) < 0.5).to(torch.uint8)
    if mode == "codebook":
        Cq, co = spd_calib(Hkv, g)
        CT, co = Cq.transpose(1, 2).contiguous().to(dev), co.to(dev)
    for b in range(B if not bt_shared else 1):
        n = max(lens) if bt_shared else lens[b]
        if n == 0:
            continue
        kv = make_kv(n, Hkv, g, edge=(b == 0))
        if twin is not None and b == 0:
            # a second token with token 4's key (x 300 group included) up to a small change in another group, and values of
            # its own: two keys whose scores are in the hundreds and a few hundredths apart, so the weights between the
            # two value rows hang on the last bits of those scores
            kv[twin] = kv[4]
            kv[twin, :Hkv, 64:96] += (0.05 * torch.randn(Hkv, 32, generator=g)).bfloat16()
            kv[twin, Hkv:] = torch.randn(Hkv, 128, generator=g).bfloat16()
        kv = kv.to(dev)
        sl = slots_of(bt, b, n, P).to(dev)
        if mode == "static":
            K.v2_write(kv, sl, mask.to(dev), 32, pool, P, fmt=fmt)
        else:
            K.cb_write(kv, sl, CT, co, fmt, pool, P)
    q = (torch.randn(B, HQ, 128, generator=g) * 0.8).bfloat16()
    scale = 1 / math.sqrt(128)
    tail = tail_len = tail_idx = None
    if win is not None:
        W, R = win
        tail = torch.randn(R, W, 2 * Hkv, 128, generator=g).bfloat16()
        tail_idx = torch.randperm(R, generator=g)[:B].int()
        tail_len = torch.randint(0, W + 1, (B,), generator=g).int()
    Lmax = max(max(lens), 1)
    seq = torch.tensor(lens, dtype=torch.int32)
    ref = A.decode_reference(bits(q), pool.cpu().numpy(), fmt, P, bt.numpy(), lens, scale,
                             kmask=mask[:Hkv].numpy() if mode == "static" else None,
                             vmask=mask[Hkv:].numpy() if mode == "static" else None,
                             tail=None if tail is None else bits(tail),
                             tail_len=None if tail is None else tail_len.numpy(),
                             tail_idx=None if tail is None else tail_idx.numpy(), kv_start=kv_start)
    out = torch.full((B, HQ * 128), float("nan"), dtype=torch.bfloat16, device=dev)
    if mode == "static":
        ns, ch = K.plan_v2(B, Lmax, Hkv, P, nsplit=nsplit, fmt=fmt, G=G)
    else:
        ns, ch = K.plan_cb(B, Lmax, Hkv, P, fmt, nsplit=nsplit, G=G)
    gfmt = fmt
    if mode == "static" or G != 4:
        HV, GT = K.vheads(Hkv, G, 128, gfmt), K.tile_of(K.v2_variant(gfmt, G, 128))
    else:
        HV, GT = Hkv, 4
    ws = K.Workspace(B, HV, B * HV * (ns + 1), dev, GT, 128)
    tkw = {}
    if tail is not None:
        dt = tail.to(dev)
        tkw = dict(tail=dt, tail_len=tail_len.to(dev), tail_idx=tail_idx.to(dev), tail_bs=dt.stride(0), tail_ts=dt.stride(1))
    dq, dbt, dseq = q.to(dev), bt.to(dev) if bt_shared != "stride0" else bt.to(dev)[:1].expand(B, -1), seq.to(dev)
    # Two calls: the second finds the self-resetting tickets back at zero.  The first runs the plan as the library
    # re-shapes it (fewer, longer splits; short splits as large workgroups), the second exactly as the caller planned it
    # (FLAGROT_REPLAN=0, read at every call): both launch shapes of every case.
    for rep in range(2):
        out.fill_(float("nan"))
        with as_planned(rep == 1):
            if mode == "static":
                K.v2_attn(dq, pool, dbt, dseq, out, ns, ch, ws, scale * LOG2E, kmask=mask[:Hkv].to(dev),
                          vmask=mask[Hkv:].to(dev), fmt=fmt, kv_start=kv_start, page=P, **tkw)
            else:
                K.cb_attn(dq, pool, dbt, dseq, out, ns, ch, ws, scale * LOG2E, fmt, kv_start=kv_start, page=P, **tkw)
        torch.cuda.synchronize()
        got = out.view(B, HQ, 128).float().cpu().numpy().astype(np.float64)
        valid = np.array([min(kv_start, lens[b]) < lens[b] or (tail is not None and int(tail_len[b]) > 0) for b in range(B)])
        assert not np.isnan(got[valid]).any(), (fmt, lens, "NaN in output")
        # ordinary rows: element-wise; rows that read the adversarial tokens (row 0, or every row when the block-table
        # row is shared): the row's largest |ref| in place of |ref|
        lim = ATOL + RTOL * np.abs(ref)
        hard = np.zeros(B, bool)
        hard[0] = True
        if bt_shared:
            hard[:] = True
        lim[hard] = ATOL + RTOL * np.abs(ref[hard]).max(axis=(1, 2), keepdims=True)
        err = np.where(valid[:, None, None], np.abs(got - ref), 0.0)
        worst = np.unravel_index(np.argmax(err / lim), err.shape)
        strict = err / (ATOL + RTOL * np.abs(ref))
        print(f"\n{fmt} G={G} lens={lens[:4]}.. ns={ns}: worst |err| / (2e-3 + 1e-2 |ref|) = "
              f"{strict[~hard].max() if (~hard).any() else 0.0:.3f} on ordinary rows, {strict[hard].max():.3f} on rows with "
              f"adversarial tokens ({(err / lim)[hard].max():.3f} of their row-max bar)", flush=True)
        assert (err <= lim).all(), (f"{fmt} {lens} ns={ns} ch={ch} worst(b,head,d)={tuple(int(i) for i in worst)} "
                                    f"got={got[worst]:.5f} ref={ref[worst]:.5f} limit={lim[worst]:.5f}")
        assert strict[hard].max() <= (HARD_ROWS if hard_rows is None else hard_rows), (fmt, lens, ns, float(strict[hard].max()))
    assert int(ws.counter.abs().sum()) == 0
    return ns, ch


LENS = [1, 15, 16, 17, 63, 64, 65, 200, 1000, 3, 511]


@pytest.mark.parametrize("mode,fmt", [("codebook", "konlya2"), ("static", "int2a"), ("codebook", "konlya"), ("static", "int4a")])
def test_two_keys_with_very_large_scores(dev, mode, fmt):
    """Two tokens share a key group scaled x 300 and differ a little in another group: scores in the hundreds of log2
    units, a few hundredths apart, value rows of their own.  On the 2-bit pages every quad that holds such a score is
    scored a second time with the code operands eight bits higher (decode_tiles.hpp: rescore_fine); this test runs that
    pass in 4- and 8-head tiles, on pages of 16 and 32, with one and several splits, and holds its rows to the bars of
    the other adversarial rows.  (It does not by itself show what the second pass gains: two tokens with the same codes
    in the scaled group lose the same bits.  The randomised runs do.)"""
    for seed, (G, Hkv), P, nsplit, twin in ((31, (4, 2), 16, None, 21), (32, (8, 2), 16, 2, 70), (33, (4, 4), 32, None, 40),
                                           (34, (6, 2), 16, None, 9), (35, (4, 2), 16, 3, 130)):
        run_case(dev, mode, [300, 40], fmt, seed=seed, G=G, Hkv=Hkv, P=P, nsplit=nsplit, twin=twin)


@pytest.mark.parametrize("mode,fmt", [("codebook", "konlya"), ("static", "int2a")])
def test_plans_the_library_runs_as_fewer_longer_splits(dev, mode, fmt):
    """A plan of more workgroups than CUs whose (sequence, KV head, q tile) pairs fit the CUs by themselves (256 pairs
    here) is run as one large workgroup per pair over the whole sequence (csrc/capi.hip: fr_v2_attn) -- the reference
    front end never plans chunks beyond 8192 tokens, so every longer context reaches the library like this.  Ragged
    lengths, an empty and a one-page sequence, BF16 rows, kv_start; the caller's workspace is sized for ITS plan."""
    lens = [2300 - 37 * (b % 9) for b in range(32)]
    lens[5], lens[17] = 0, 9
    ns, ch = run_case(dev, mode, lens, fmt, seed=41, G=4, Hkv=8, nsplit=3, win=(20, 33), kv_start=4)
    assert (ns, ch) == (3, 768)


@pytest.mark.parametrize("mode,fmt", [("codebook", "konlya"), ("codebook", "konlya2"), ("static", "int4a")])
def test_short_splits_run_as_large_workgroups(dev, mode, fmt):
    """Plans of short splits (the reference planner's answer to short contexts: 6 x 384 tokens for one sequence of
    2048) are run as large workgroups where those fit the CUs once (csrc/capi.hip: fr_v2_attn): one of them up to 1024
    tokens, splits of 512 tokens beyond, never more splits than planned.  Ragged and empty sequences, BF16 rows,
    kv_start, tiles of 8 heads; the second call of every case runs the plan as given (run_case)."""
    ns, ch = run_case(dev, mode, [2040, 1300, 0, 7], fmt, seed=71, Hkv=2, nsplit=6, win=(40, 6), kv_start=4)
    assert ch < 512 and ns * ch >= 2040                 # 6 x 352 -> run as 5 x 512
    ns, ch = run_case(dev, mode, [1000, 513, 1], fmt, seed=72, Hkv=2, nsplit=4)
    assert ch == 256                                    # 4 x 256 -> run as 1 x 1024
    run_case(dev, mode, [520, 100], fmt, seed=73, Hkv=1, G=8, nsplit=2, win=(17, 3))
    run_case(dev, mode, [1500], fmt, seed=74, Hkv=4, nsplit=5, P=32)


def test_large_workgroups_in_full_rounds(dev):
    """4-bit pages, more pairs than CUs (40 sequences x 4 KV heads x 3 q tiles = 480), sequences of >= 4096 tokens: the
    library runs large workgroups in rounds that fill the CUs to >= 90 % (here one split per pair, 480 of 512) instead
    of the plan's small ones"""
    lens = [4200 - 11 * (b % 7) for b in range(40)]
    ns, ch = run_case(dev, "codebook", lens, "konlya", seed=42, G=12, Hkv=4)
    assert ns * 480 > 256 and ns * ch >= 4200


@pytest.mark.parametrize("kind", ["konly", "konlya", "konlya2"])
def test_codebook_decode(dev, kind):
    run_case(dev, "codebook", LENS, kind, seed=1)


@pytest.mark.parametrize("fmt", ["int4", "int4a", "int2a"])
def test_static_decode(dev, fmt):
    run_case(dev, "static", LENS, fmt, seed=2)


@pytest.mark.parametrize("kind", ["konlya", "konlya2"])
def test_codebook_decode_long_and_splits(dev, kind):
    run_case(dev, "codebook", [4097, 33, 2500], kind, seed=3, Hkv=2)
    run_case(dev, "codebook", [700, 120], kind, seed=4, Hkv=2, nsplit=3)
    run_case(dev, "codebook", [700, 120], kind, seed=5, Hkv=2, nsplit=1)


@pytest.mark.parametrize("mode,fmt", [("codebook", "konlya"), ("codebook", "konlya2"), ("codebook", "konly"),
                                      ("static", "int4a"), ("static", "int4"), ("static", "int2a")])
def test_window_and_kv_start(dev, mode, fmt):
    run_case(dev, mode, [300, 5, 0, 64, 37], fmt, win=(132, 7), seed=6, Hkv=2, kv_start=4)
    run_case(dev, mode, [300, 5, 17], fmt, win=(32, 4), seed=7, Hkv=2, kv_start=16)
    run_case(dev, mode, [90, 40], fmt, seed=8, Hkv=2, kv_start=37)


@pytest.mark.parametrize("mode,fmt", [("codebook", "konlya"), ("codebook", "konlya2"), ("codebook", "konly"),
                                      ("static", "int4a"), ("static", "int2a")])
def test_large_workgroup_shape(dev, mode, fmt):
    """chunks of >= 1024 tokens on few (sequence, head) pairs: one large (16- or 12-wavefront) workgroup per split, quads drawn from
    a counter in LDS (the other tests run the 4-wavefront shapes); with splits, tail rows, kv_start and a q tile pair."""
    ns, ch = run_case(dev, mode, [2300, 2100], fmt, seed=20, Hkv=2, nsplit=1)
    assert (ns, ch) == (1, 2304)
    run_case(dev, mode, [4500, 2049, 70], fmt, seed=21, Hkv=2, nsplit=2, win=(40, 5), kv_start=4)
    run_case(dev, mode, [2200], fmt, seed=22, Hkv=1, G=8, nsplit=1)
    # one split of large workgroups with BF16 rows: the body's wavefronts take the rows themselves
    # (an empty sequence that has rows only, one of five tokens behind kv_start = 4, padding heads in the q tile)
    run_case(dev, mode, [2300, 0, 5, 2100], fmt, seed=25, G=3, Hkv=2, nsplit=1, win=(132, 6), kv_start=4)
    run_case(dev, mode, [2049, 2049], fmt, seed=26, Hkv=2, nsplit=1, win=(7, 3), bt_shared=True)
    # two splits of 4544 tokens: the first split's workgroup takes the rows, its partial and the second split's are merged
    run_case(dev, mode, [9000, 4200, 0], fmt, seed=27, Hkv=2, nsplit=2, win=(40, 5), kv_start=4)


def test_block_table_beyond_the_lds_cache(dev):
    """more than 1024 pages per sequence: the block-table entries past the workgroup's LDS cache are read from memory
    (shared-range workgroups and, with one split of 17 k tokens, the large workgroup)"""
    run_case(dev, "codebook", [17000, 40], "konlya", seed=23, Hkv=1)
    run_case(dev, "codebook", [16500], "konlya2", seed=24, Hkv=1, nsplit=3)


@pytest.mark.parametrize("mode,fmt", [("codebook", "konlya"), ("codebook", "konlya2"), ("static", "int4a")])
def test_long_contexts(dev, mode, fmt):
    """33 000 and 65 536 tokens (the lengths of the reference's own long cases, kernels/test_attn_v2.py:144,354-382, and
    of its decode benchmark, scripts/bench_attn_int2.py:30): 2063 and 4096 pages per sequence, so three quarters of the
    block table is read past the workgroup's LDS window; the planner's split, the fewest splits a chunk of 8192 tokens
    allows, and BF16 rows with a masked sink range"""
    run_case(dev, mode, [33000], fmt, seed=50, Hkv=1)
    run_case(dev, mode, [33000, 700], fmt, seed=51, Hkv=1, nsplit=5)
    run_case(dev, mode, [65536, 40], fmt, seed=52, Hkv=1, win=(132, 3), kv_start=4)
    run_case(dev, mode, [65536], fmt, seed=53, Hkv=1, nsplit=8)


@pytest.mark.parametrize("shared", ["copy", "stride0"])
def test_shared_block_table_row(dev, shared):
    run_case(dev, "codebook", [100, 37, 64], "konlya", bt_shared=shared, seed=9, Hkv=2)
    if shared == "copy":
        run_case(dev, "static", [100, 37, 64], "int4a", bt_shared=shared, seed=10, Hkv=2)


@pytest.mark.parametrize("G,Hkv", [(8, 8), (5, 8), (12, 4), (6, 2), (1, 4)])
def test_gqa_groups(dev, G, Hkv):
    run_case(dev, "codebook", [130, 31, 700], "konlya", seed=11, G=G, Hkv=Hkv, win=(40, 5), kv_start=4)
    run_case(dev, "static", [130, 31, 700], "int4a", seed=12, G=G, Hkv=Hkv)
    run_case(dev, "codebook", [130, 31], "konlya2", seed=13, G=G, Hkv=Hkv)


@pytest.mark.parametrize("mode,fmt", [("codebook", "konlya"), ("codebook", "konlya2"), ("codebook", "konly"),
                                      ("static", "int4a"), ("static", "int2a"), ("static", "int4")])
def test_tiles_of_8_heads(dev, mode, fmt):
    """GQA groups of 5 .. 8 heads: one workgroup serves all heads of a KV head on one unpacking of the pages (the
    reference's GT = 8 kernels, kernels/csrc/attn_decode_v2g.cuh:5-10).  Ragged lengths, groups that do not fill the
    tile (heads past the group are padding), splits with BF16 rows and a masked sink range, the large workgroup, and
    32-token pages."""
    run_case(dev, mode, LENS, fmt, seed=60, G=8, Hkv=2)
    run_case(dev, mode, [700, 120, 2300], fmt, seed=61, G=7, Hkv=2, nsplit=3, win=(40, 5), kv_start=4)
    ns, ch = run_case(dev, mode, [2300, 2100], fmt, seed=62, G=8, Hkv=1, nsplit=1)
    assert (ns, ch) == (1, 2304)
    run_case(dev, mode, [200, 1000, 33], fmt, seed=63, G=5, Hkv=2, P=32)
    run_case(dev, mode, [4500, 2049], fmt, seed=64, G=6, Hkv=1, nsplit=2, win=(24, 3), P=32)


@pytest.mark.parametrize("mode,fmt", [("codebook", "konlya"), ("codebook", "konlya2"), ("codebook", "konly"),
                                      ("static", "int4a"), ("static", "int2a")])
def test_pages_of_32_tokens(dev, mode, fmt):
    """32-token pages: a quad is two pages of four 8-token runs each; ragged lengths, splits, the large workgroup,
    tail rows and kv_start"""
    run_case(dev, mode, [1, 31, 32, 33, 65, 200, 1000, 511], fmt, seed=40, P=32)
    run_case(dev, mode, [700, 120], fmt, seed=41, Hkv=2, nsplit=3, win=(40, 5), kv_start=37, P=32)
    run_case(dev, mode, [2300, 2100], fmt, seed=42, Hkv=2, nsplit=1, P=32)


def test_decode_error_codes(dev):
    from flagrot_releaser_amd import kernels as K
    L = K.lib()
    z = torch.zeros(1024, dtype=torch.uint8, device=dev)
    zp = z.data_ptr()
    base = [zp, 512, zp, zp, 1, zp, 1, 1, 16, 1, 64, 1.0, None, None, 32, 0, 0, 264, 4, zp, zp, zp, zp, 512, None, None,
            None, 0, 0, None]
    assert L.fr_v2_attn(99, *base, 4, 0) == -4
    bad_page = list(base); bad_page[8] = 64
    assert L.fr_v2_attn(5, *bad_page, 4, 0) == -5
    assert L.fr_v2_attn(5, *base, 8, 0) == -7            # gqa 8 without the generalised variant bits
    no_ws = list(base); no_ws[9] = 2; no_ws[19] = None                # two splits, no partial buffer: an error code, not a fault
    assert L.fr_v2_attn(5, *no_ws, 4, 0) == -3 and b"opart" in L.fr_last_error()
    no_ctr = list(base); no_ctr[9] = 2; no_ctr[21] = None
    assert L.fr_v2_attn(5, *no_ctr, 4, 0) == -3
    hd = list(base); hd[17] = 264 | 1024 | 2048 | 4096
    assert L.fr_v2_attn(5, *hd, 4, 0) == -3              # head dim 256 takes q tiles of 4 heads, not 8
    odd = list(base); odd[24] = zp + 2; odd[25] = zp; odd[27] = 2048; odd[28] = 2048     # BF16 rows off a 16-byte boundary
    assert L.fr_v2_attn(5, *odd, 4, 0) == -3 and b"16-byte" in L.fr_last_error()
    odd[24] = zp; odd[28] = 2052                                                         # ... or a row stride that leaves it
    assert L.fr_v2_attn(5, *odd, 4, 0) == -3 and b"16-byte" in L.fr_last_error()
    assert L.fr_cb_attn(zp, 512, zp, zp, 1, zp, 1, 1, 16, 1, 64, 1.0, K.sign_words(), 3, 0, 4, zp, zp, zp, zp, 512, None,
                        None, None, 0, 0, None, 0) == -4
    assert L.fr_v2_attn(5, *(base[:6] + [0] + base[7:]), 4, 0) == 0     # B = 0: nothing to do


@pytest.mark.parametrize("fmt", ["konly", "konlya", "konlya2", "int4", "int4a", "int2a"])
@pytest.mark.parametrize("P", [16, 32])
def test_head_dim_256(dev, fmt, P):
    """head dim 256 (`variant | 4096`; the reference's shape (G, D, Hkv) = (6, 256, 4), test_kernels.py:366-374): pages
    of two 128-d half chunks written by the 256-d writers, q tiles of 4 + 2 heads, splits, BF16 window rows, kv_start,
    ragged lengths; against the oracle's dequantise-then-attend at that head dim, element-wise bar."""
    _head_dim_256(dev, fmt, P, 6, 4)


@pytest.mark.parametrize("fmt", ["konlya2", "int4a"])
@pytest.mark.parametrize("G,Hkv", [(1, 4), (4, 2), (8, 2), (12, 1), (5, 8)])
def test_head_dim_256_groups(dev, fmt, G, Hkv):
    """other GQA groups at head dim 256: one, two and three q tiles per KV head (with and without the placement of a
    KV head's tiles on one XCD, which needs (KV heads x splits x sequences) to be a multiple of 8)"""
    _head_dim_256(dev, fmt, 16, G, Hkv)


def _head_dim_256(dev, fmt, P, G, Hkv, lens=None, seed=None):
    from flagrot_releaser_amd import kernels as K
    Dh = 256
    static = fmt in ("int4", "int4a", "int2a")
    g = torch.Generator().manual_seed(600 + len(fmt) + P if seed is None else seed)
    lens = [1, 17, 64, 65, 333, 700, 0] if lens is None else list(lens) + [0]      # the last sequence is empty
    B, HQ = len(lens), G * Hkv
    num_pages = sum((n + P - 1) // P for n in lens) + 5
    pool = torch.randint(0, 256, (num_pages, Hkv, 2 * PG.chunk_bytes(fmt, P)), dtype=torch.uint8, generator=g).to(dev)
    bt = alloc_tables(lens, num_pages, g, P)
    mask = (torch.rand(2 * Hkv, 8, generator=g) < 0.5).to(torch.uint8)
    qs = torch.randn(Hkv, 384, Dh, generator=g)
    qs[:, :, :8] *= 4
    CT = torch.einsum("hnd,hne->hde", qs, qs).transpose(1, 2).contiguous().to(dev)
    co = torch.ones(Hkv, Dh, device=dev)
    for b, n in enumerate(lens):
        if n == 0:
            continue
        kv = torch.randn(n, 2 * Hkv, Dh, generator=g)
        kv[:, :Hkv, 9] *= 6
        kv[:, :Hkv, 130] *= 5
        kv[:, :Hkv] *= (0.5 + torch.rand(n, 1, 1, generator=g))
        kv = kv.bfloat16().to(dev)
        sl = slots_of(bt, b, n, P).to(dev)
        if static:
            K.v2_write(kv, sl, mask.to(dev), 32, pool, P, fmt=fmt)
        else:
            K.cb_write(kv, sl, CT, co, fmt, pool, P)
    q = (torch.randn(B, HQ, Dh, generator=g) * 0.8).bfloat16()
    scale = 1 / math.sqrt(Dh)
    W, R, kv_start = 20, B + 1, 3
    tail = torch.randn(R, W, 2 * Hkv, Dh, generator=g).bfloat16()
    tail_idx = torch.randperm(R, generator=g)[:B].int()
    tail_len = torch.randint(0, W + 1, (B,), generator=g).int()
    tail_len[-1] = 0                                   # the empty sequence has no window rows either: output 0
    seq = torch.tensor(lens, dtype=torch.int32)
    ref = A.decode_reference(bits(q), pool.cpu().numpy(), fmt, P, bt.numpy(), lens, scale,
                             kmask=mask[:Hkv].numpy() if static else None, vmask=mask[Hkv:].numpy() if static else None,
                             tail=bits(tail), tail_len=tail_len.numpy(), tail_idx=tail_idx.numpy(), kv_start=kv_start)
    dt = tail.to(dev)
    tkw = dict(tail=dt, tail_len=tail_len.to(dev), tail_idx=tail_idx.to(dev), tail_bs=dt.stride(0), tail_ts=dt.stride(1))
    for nsplit in (1, 3):
        ns, ch = (K.plan_v2 if static else K.plan_cb)(B, max(lens), Hkv, P, *((fmt,) if not static else ()), nsplit=nsplit,
                                                     **({"fmt": fmt} if static else {}), G=G, Dh=Dh)
        HV, GT = K.vheads(Hkv, G, Dh, fmt), K.tile_of(K.v2_variant(fmt, G, Dh))
        assert (HV, GT) == (Hkv * ((G + 3) // 4), 4)
        ws = K.Workspace(B, HV, B * HV * (ns + 1), dev, GT, Dh)
        out = torch.full((B, HQ * Dh), float("nan"), dtype=torch.bfloat16, device=dev)
        if static:
            K.v2_attn(q.to(dev), pool, bt.to(dev), seq.to(dev), out, ns, ch, ws, scale * LOG2E, kmask=mask[:Hkv].to(dev),
                      vmask=mask[Hkv:].to(dev), fmt=fmt, kv_start=kv_start, page=P, **tkw)
        else:
            K.cb_attn(q.to(dev), pool, bt.to(dev), seq.to(dev), out, ns, ch, ws, scale * LOG2E, fmt, kv_start=kv_start,
                      page=P, **tkw)
        torch.cuda.synchronize()
        got = out.view(B, HQ, Dh).float().cpu().numpy().astype(np.float64)
        assert not np.isnan(got).any()
        strict = np.abs(got - ref) / (ATOL + RTOL * np.abs(ref))
        print(f"\n{fmt} P={P} D=256 G={G} ns={ns}: worst |err| / (2e-3 + 1e-2 |ref|) = {strict.max():.3f}", flush=True)
        assert strict.max() <= 1.0, (fmt, P, ns, np.unravel_index(np.argmax(strict), strict.shape))
        assert not got[-1].any()
        assert int(ws.counter.abs().sum()) == 0


@pytest.mark.parametrize("fmt,P", [("konlya", 16), ("int2a", 32)])
def test_head_dim_256_plain_switch(dev, fmt, P, monkeypatch):
    """FLAGROT_WIDE_PLAIN=1 (read at every call) sends every split through the plain fp32 kernel instead of the
    matrix-pipe one: same partial format, same bar"""
    monkeypatch.setenv("FLAGROT_WIDE_PLAIN", "1")
    test_head_dim_256(dev, fmt, P)
