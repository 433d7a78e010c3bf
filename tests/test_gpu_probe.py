"""The page-read probe (a measurement aid beside the decode kernel in bench.py): it must read exactly the chunks the
block table addresses.  A lane whose words or to one marker value writes the sink word, so a marker planted in an
addressed page shows in the sink and one planted in a page outside the block table does not."""
import pytest
import torch

pytestmark = pytest.mark.gpu
MARK = 0x9E3779B9 - (1 << 32)


@pytest.mark.parametrize("chunk,page,hkv", [(2304, 16, 8), (1280, 16, 4), (1552, 32, 2), (4608, 32, 2)])
def test_probe_reads_the_addressed_pages_only(chunk, page, hkv):
    from flagrot_releaser_amd import probe
    dev = torch.device("cuda:0")
    B, npages = 3, 200
    seq = torch.tensor([1, 37 * page - 5, 90 * page], dtype=torch.int32, device=dev)
    g = torch.Generator().manual_seed(5)
    perm = torch.randperm(npages, generator=g).to(torch.int32)
    bt = torch.zeros(B, 96, dtype=torch.int32)
    bt[0, :1], bt[1, :37], bt[2, :90] = perm[:1], perm[1:38], perm[38:128]
    bt = bt.to(dev)
    unused = int(perm[150])
    for pg, head, word, hit in ((int(perm[0]), 0, 0, True), (int(perm[37]), hkv - 1, chunk // 4 - 1, True),
                                (int(perm[127]), 1, 17, True), (unused, 0, 3, False)):
        pool = torch.zeros(npages, hkv, chunk // 4, dtype=torch.int32, device=dev)
        pool[pg, head, word] = MARK
        sink = torch.zeros(4, dtype=torch.int32, device=dev)
        probe.read_pages(pool.view(torch.uint8).view(npages, hkv, chunk), bt, seq, sink, page)
        torch.cuda.synchronize()
        assert (int(sink[0]) == MARK) == hit, (pg, head, word, hit)


def test_probe_rejects_bad_arguments():
    from flagrot_releaser_amd import probe
    dev = torch.device("cuda:0")
    pool = torch.zeros(4, 2, 1288, dtype=torch.uint8, device=dev)
    bt = torch.zeros(1, 4, dtype=torch.int32, device=dev)
    seq = torch.ones(1, dtype=torch.int32, device=dev)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError):
        probe.read_pages(pool, bt, seq, sink, 16)          # chunk bytes not a multiple of 16


def test_mfma_probe_runs_and_reports_a_plausible_rate():
    """the matrix-pipe probe: both modes launch, finish, and land between 5 % and 110 % of the nominal dense fp16 rate"""
    import bench
    dev = torch.device("cuda:0")
    r = bench.mfma_probe(torch, dev, iters=800)
    print(f"\nmfma probe: {r}", flush=True)
    for key in ("registers_TFLOPs", "lds_operand_TFLOPs"):
        assert 0.05 * r["nominal_TFLOPs"] < r[key] < 1.1 * r["nominal_TFLOPs"], r
