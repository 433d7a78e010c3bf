"""Writes the golden vectors tests/golden/k2_encode_<kind>.npz by running the reference's own PyTorch encoder
(kernels/codebook_ref.encode of the reference tree, on the CPU) on small seeded inputs.

Run once in the build container (the reference tree does not exist anywhere else):
    python tests/golden/make_golden.py [/root/reference]

Only the function that nothing else pins bit for bit is imported: codebook_ref.encode, end to end near ties.  Through
it the vectors also cover ref.fwht, ref.int4_quant, formats.quant_asym_dep and formats.scale_word, which encode calls.
The reference runs on the CPU here, so its asymmetric step is an IEEE division ((max - min) / levels); the oracle
reproduces these vectors with true_div=True, and differs from its kernel form (true_div=False) in that one
expression only.

Inputs per kind (all from torch.Generator().manual_seed(seed)):
  x   bf16 [T, 2*Hkv, 128]: N(0,1), 4 outlier channels x6 on the K rows, per-token scale 0.5 + U(0,1), plus the
      edge groups of the reference's tests (all-positive, all-negative, zero, x1e-5, x300, constant 1.25, one-hot)
  C   fp32 [Hkv, 128, 128] = sum of 256 outer products of N(0,1) queries with 8 channels x4  (dense SPD)
  co  fp32 [Hkv, 128] = U(0,1) + 0.1
Stored: x as bf16 bit patterns, C, co, and for K and V rows the encoder's q, s (word values), local, mode.
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

REF = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
OUT = Path(__file__).resolve().parent
T, HKV, DH = 40, 2, 128
QK = {"konly": "cache", "konlya": "asym", "konlya2": "asym2"}


def inputs(seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, 2 * HKV, DH, generator=g)
    for h in range(HKV):
        ch = torch.randint(0, DH, (4,), generator=g)
        x[:, h, ch] *= 6
    x = x * (0.5 + torch.rand(T, 1, 1, generator=g))
    # edge groups (one 32-group each, K and V rows of head 0 / 1)
    x[0, :, 0:32] = x[0, :, 0:32].abs() + 0.1
    x[1, :, 32:64] = -x[1, :, 32:64].abs() - 0.1
    x[2, :, 64:96] = 0.0
    x[3, :, 96:128] *= 1e-5
    x[4, :, 0:32] *= 300.0
    x[5, :, 32:64] = 1.25
    x[6, :, 64:96] = 0.0
    x[6, :, 70] = 3.0
    x[7] = 0.0
    x = x.bfloat16()
    qs = torch.randn(HKV, 256, DH, generator=g)
    qs[:, :, :8] *= 4
    C = torch.einsum("hnd,hne->hde", qs, qs).contiguous()
    co = torch.rand(HKV, DH, generator=g) + 0.1
    return x, C, co


def main():
    sys.path.insert(0, str(REF / "kernels"))
    sys.path.insert(0, str(REF))
    import codebook_ref as CR  # the reference's encoder (pulls blockflag.qattention -> transformers)

    torch.set_num_threads(4)
    for n, (kind, qk) in enumerate(QK.items()):
        x, C, co = inputs(100 + n)
        k = CR.encode(x[:, :HKV], C, co, "k", cfg=kind, qk=qk)
        v = CR.encode(x[:, HKV:], C, co, "v", cfg=kind, qk=qk)
        np.savez_compressed(
            OUT / f"k2_encode_{kind}.npz",
            x_bits=x.view(torch.int16).numpy().view(np.uint16), C=C.numpy(), co=co.numpy(),
            kq=k["q"].numpy(), ks=k["s"].numpy(), klocal=k["local"].numpy().astype(np.uint8),
            kmode=k["mode"].numpy().astype(np.uint8), kherr=k["head_errs"].numpy(),
            vq=v["q"].numpy(), vs=v["s"].numpy(), vmode=v["mode"].numpy().astype(np.uint8))
        print(kind, "local H32 fraction", float(k["local"].float().mean()), "F fraction",
              float((k["mode"] == 2).float().mean()))


if __name__ == "__main__":
    main()
