"""helpers shared by the GPU parity tests (torch <-> numpy bf16, synthetic caches)."""
import numpy as np
import torch

P = 16


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> uint16 bit patterns (numpy)."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(a: np.ndarray, dev) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).to(dev)


def make_kv(T, Hkv, g, outliers=4, gain=6.0, edge=True):
    """LLM-like rows: K with a few outlier channels per head and a per-token scale spread, plus the edge groups the
    reference's tests use (all-positive, all-negative, zero, tiny, large, constant, one-hot)."""
    kv = torch.randn(T, 2 * Hkv, 128, generator=g)
    for h in range(Hkv):
        ch = torch.randint(0, 128, (outliers,), generator=g)
        kv[:, h, ch] *= gain
    kv[:, :Hkv] *= (0.5 + torch.rand(T, 1, 1, generator=g))
    kv[:, Hkv:] *= (0.25 + 1.5 * torch.rand(T, 1, 1, generator=g))
    if edge and T >= 8:
        kv[0, :, 0:32] = kv[0, :, 0:32].abs() + 0.1
        kv[1, :, 32:64] = -kv[1, :, 32:64].abs() - 0.1
        kv[2, :, 64:96] = 0.0
        kv[3, :, 96:128] *= 1e-5
        kv[4, :, 0:32] *= 300.0
        kv[5, :, 32:64] = 1.25
        kv[6, :, 64:96] = 0.0
        kv[6, :, 70] = 3.0
        kv[7] = 0.0
    return kv.bfloat16()


def spd_calib(Hkv, g, nq=256):
    qs = torch.randn(Hkv, nq, 128, generator=g)
    qs[:, :, :8] *= 4
    Cq = torch.einsum("hnd,hne->hde", qs, qs).contiguous()
    co = torch.rand(Hkv, 128, generator=g) + 0.1
    return Cq, co


def alloc_tables(lens, num_pages, g, P=P):
    need = [(n + P - 1) // P for n in lens]
    ids = torch.randperm(num_pages, generator=g)[:sum(need)]
    bt = torch.zeros(len(lens), max(max(need), 1), dtype=torch.int32)
    o = 0
    for b, n in enumerate(need):
        bt[b, :n] = ids[o:o + n].int()
        o += n
    return bt


def slots_of(bt, b, n, P=P):
    pos = torch.arange(n)
    return bt[b].long()[pos // P] * P + pos % P
