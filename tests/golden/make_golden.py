"""Writes the golden vectors under tests/golden/ by running the reference's own PyTorch code (CPU) on small seeded
inputs.  Only data is stored (inputs and the reference's outputs): nothing of the reference's source travels.

Run once in the build container (the reference tree does not exist anywhere else):
    python tests/golden/make_golden.py [/root/reference] [k2|k2d256|pages|pages256|static|kivi_layout|kivi_select ...]

Files and the reference functions that wrote them:
  k2_encode_<kind>.npz     kernels/codebook_ref.encode                                     (selecting writer, below)
  k2_encode_d256_<kind>.npz  the same at head dim 256 (eight 32-groups, whole-head H256; 24 tokens, one dense SPD C_q
                           [Hkv, 256, 256]; konly and konlya)
  pages_<fmt>_p<P>.npz     vllm_flagrot/kernels.py parse_pages / dequant_v2_pages / dequant_cb_pages on a pool of random
                           bytes into which oracle.pages.pack_tokens has packed seeded tokens (six formats x pages of 16
                           and 32 tokens): pins the oracle's parser on arbitrary bytes and its packer through the
                           reference's parser
  pages_d256.npz           vllm_flagrot/kernels.py dequant_v2_pages / dequant_cb_pages with Dh = 256 on random chunk bytes
                           (two 128-d half chunks per page and head; six formats, 16-token pages)
  static_writer.npz        kernels/ref.py kv_selrot_quant(fmt="int4") and int4a_quant (and formats.quant_asym_dep with
                           2 bits + scale_word_b for int2a) on seeded rows with a random rotation mask
  kivi_layout.npz          vllm_flagrot/kivi.py _kcodes / _codes / parse_chunks / dequant_groups on random chunk bytes
                           (FP16 meta and FP8 meta chunks; both bases); kivi_layout_d256.npz: the same at head dim 256
  kivi_select.npz          blockflag.qattention.dyn_quant("kivi2:32" and "kivi2f8:32", att + F rule) reconstructions and
                           the per-group / per-token choices (the internals test_kivi.py's sim_choice_k uses) for keys
                           (token axis, with 4 sink tokens excluded from the first group) and values (head axis)

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

import math
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


def write_k2():
    import codebook_ref as CR  # the reference's encoder (pulls blockflag.qattention -> transformers)

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


def write_k2_d256():
    import codebook_ref as CR

    for n, kind in enumerate(("konly", "konlya")):
        g = torch.Generator().manual_seed(300 + n)
        Tn, Dn = 24, 256
        x = torch.randn(Tn, 2 * HKV, Dn, generator=g)
        for h in range(HKV):
            x[:, h, torch.randint(0, Dn, (6,), generator=g)] *= 6
        x = x * (0.5 + torch.rand(Tn, 1, 1, generator=g))
        x[0, :, 0:32] = x[0, :, 0:32].abs() + 0.1
        x[1, :, 160:192] *= 300.0
        x[2, :, 224:256] = 0.0
        x[3] = 0.0
        x = x.bfloat16()
        qs = torch.randn(HKV, 512, Dn, generator=g)
        qs[:, :, :8] *= 4
        qs[:, :, 130:136] *= 3
        C = torch.einsum("hnd,hne->hde", qs, qs).contiguous()
        co = torch.rand(HKV, Dn, generator=g) + 0.1
        k = CR.encode(x[:, :HKV], C, co, "k", cfg=kind, qk=QK[kind])
        v = CR.encode(x[:, HKV:], C, co, "v", cfg=kind, qk=QK[kind])
        np.savez_compressed(
            OUT / f"k2_encode_d256_{kind}.npz",
            x_bits=x.view(torch.int16).numpy().view(np.uint16), C=C.numpy(), co=co.numpy(),
            kq=k["q"].numpy(), ks=k["s"].numpy(), klocal=k["local"].numpy().astype(np.uint8),
            kmode=k["mode"].numpy().astype(np.uint8), kherr=k["head_errs"].numpy(),
            vq=v["q"].numpy(), vs=v["s"].numpy(), vmode=v["mode"].numpy().astype(np.uint8))
        print(kind, "D=256 local H32 fraction", float(k["local"].float().mean()), "F fraction",
              float((k["mode"] == 2).float().mean()))


# ------------------------------------------------------------------------------------------------ page parsers
def _here_oracle():
    root = str(OUT.parents[1])
    if root not in sys.path:
        sys.path.insert(0, root)
    from oracle import pages as PG
    from oracle import quant as Q
    return PG, Q


def write_pages():
    """pool = random bytes + tokens packed by the oracle's packer; outputs = the reference's parsers on those bytes"""
    from vllm_flagrot import kernels as RK   # top level imports ctypes, fcntl, torch only; lib() is never called
    PG, Q = _here_oracle()
    for n, fmt in enumerate(("int4", "int4a", "int2a", "konly", "konlya", "konlya2")):
        for P in (16, 32):
            rng = np.random.default_rng(1000 + 10 * n + P)
            Np, H, T = 3, 2, 37
            pool = rng.integers(0, 256, (Np, H, PG.chunk_bytes(fmt, P)), dtype=np.uint8)
            x, C, _ = inputs(200 + n)
            xb = x.view(torch.int16).numpy().view(np.uint16)[:T]
            if fmt in QK:
                codes, words, _ = Q.k2_encode(xb, C.numpy(), fmt)
            else:
                mask = rng.integers(0, 2, (2 * HKV, 4)).astype(np.uint8)
                codes, words = Q.static_encode(xb, mask, fmt)
            slots = rng.permutation(Np * P)[:T].astype(np.int64)
            slots[3] = -1
            PG.pack_tokens(pool, slots, codes, words, fmt, P)
            ch = torch.from_numpy(pool.copy())
            c, m, sb = RK.parse_pages(ch, P, fmt)
            if fmt in QK:
                k, v = RK.dequant_cb_pages(ch, P, fmt, dtype=torch.float32)
            else:
                k, v = RK.dequant_v2_pages(ch, P, dtype=torch.float32, fmt=fmt)
            np.savez_compressed(OUT / f"pages_{fmt}_p{P}.npz", pool=pool, slots=slots,
                                packed_codes=codes.astype(np.int16), packed_words=words.astype(np.int32),
                                codes=c.numpy(), mag_bits=m.numpy().view(np.uint32), sbits=sb.numpy(),
                                k=k.contiguous().numpy().view(np.uint32), v=v.contiguous().numpy().view(np.uint32))
            print("pages", fmt, P, tuple(c.shape), tuple(k.shape))


def write_pages_d256():
    """head dim 256 (two 128-d half chunks per page and head): the reference's parsers on random chunk bytes"""
    from vllm_flagrot import kernels as RK
    PG, _ = _here_oracle()
    out = {}
    for n, fmt in enumerate(("int4", "int4a", "int2a", "konly", "konlya", "konlya2")):
        rng = np.random.default_rng(4000 + n)
        P, Np, H = 16, 2, 2
        pool = rng.integers(0, 256, (Np, H, 2 * PG.chunk_bytes(fmt, P)), dtype=np.uint8)
        # keep every scale word's FP16 exponent finite (random bytes would make infinities / NaNs)
        half = PG.chunk_bytes(fmt, P)
        for s0 in (0, half):
            sw = pool[..., s0 + half - 16 * P:s0 + half].view(np.uint16)
            sw &= np.uint16(0xBBFF)
        ch = torch.from_numpy(pool.copy())
        if fmt in QK:
            k, v = RK.dequant_cb_pages(ch, P, fmt, dtype=torch.float32, Dh=256)
        else:
            k, v = RK.dequant_v2_pages(ch, P, dtype=torch.float32, fmt=fmt, Dh=256)
        out[f"{fmt}_pool"] = pool
        out[f"{fmt}_k"] = k.contiguous().numpy()
        out[f"{fmt}_v"] = v.contiguous().numpy()
        print("pages d256", fmt, tuple(k.shape))
    np.savez_compressed(OUT / "pages_d256.npz", **out)


# ------------------------------------------------------------------------------------------------ static writers
def write_static():
    import ref as R
    import blockflag.formats as FM
    x, _, _ = inputs(300)
    g = torch.Generator().manual_seed(301)
    mask = (torch.rand(2 * HKV, 4, generator=g) < 0.5)
    T, H, D = x.shape
    qp, s = R.kv_selrot_quant(x, mask, 32, "int4")                      # packed (q + 8) nibbles, fp16 scales
    y = R.sel_fwht_rb(x.float().reshape(T, H * D), mask, 32).reshape(T, H, D)
    q4a, w4a = R.int4a_quant(y)
    q2, z2, s2, _ = FM.quant_asym_dep(y.float(), 32, False, 2)
    w2 = FM.scale_word_b(s2, z2, 2)
    np.savez_compressed(OUT / "static_writer.npz", x_bits=x.view(torch.int16).numpy().view(np.uint16),
                        mask=mask.numpy().astype(np.uint8), y_bits=y.numpy().view(np.uint32),
                        int4_q=(R.unpack_nibbles(qp).to(torch.int16) - 8).numpy(),
                        int4_s_bits=s.view(torch.int16).numpy().view(np.uint16),
                        int4a_q=q4a.numpy().astype(np.int16), int4a_w=w4a.numpy().astype(np.int32),
                        int2a_q=q2.reshape(y.shape).numpy().astype(np.int16),
                        int2a_w=(w2.squeeze(-1).long() & 0xFFFF).numpy().astype(np.int32))
    print("static", tuple(x.shape), "mask", mask.int().tolist())


# ------------------------------------------------------------------------------------------------ KIVI page layout
def write_kivi_layout(D=128, name="kivi_layout.npz"):
    from vllm_flagrot import kivi as RKV     # top level imports ctypes, fcntl, torch only; lib() is never called
    H, npg = 2, 4
    NV = D // 32
    rng = np.random.default_rng(77)
    out = {}
    for f8 in (False, True):
        CB = 10 * D if f8 else 12 * D + 16
        ch = rng.integers(0, 256, (npg, H, CB), dtype=np.uint8)
        if f8:
            meta = ch[..., 4 * D:5 * D], ch[..., 9 * D:10 * D]
            for m in meta:                       # no NaN patterns (0x7F / 0xFF) in the E4M3 bytes
                m[(m & 0x7F) == 0x7F] ^= 0x01
        else:                                    # fp16 meta: finite, magnitudes 2^-6 .. 2^3, random signs (= flags)
            for lo in (4 * D, 10 * D):
                n = 2 * D // 2
                mag = np.exp2(rng.uniform(-6, 3, (npg, H, n))).astype(np.float16)
                sgn = rng.integers(0, 2, (npg, H, n)).astype(bool)
                ch[..., lo:lo + 2 * D] = np.where(sgn, -mag, mag).astype(np.float16).view(np.uint8).reshape(npg, H, 2 * D)
            ch[..., 12 * D:12 * D + 16] = rng.integers(0, 2, (npg, H, 16))
        t = torch.from_numpy(ch.copy())
        kc, km, vc, vm, vf = RKV.parse_chunks(t, D, f8=f8)
        tag = "f8" if f8 else "f16"
        out[f"{tag}_chunks"] = ch
        out[f"{tag}_kcodes"] = RKV._kcodes(kc, D).numpy().astype(np.uint8)
        out[f"{tag}_vcodes"] = RKV._codes(vc, D).numpy().astype(np.uint8)
        out[f"{tag}_km"] = km.float().numpy()
        out[f"{tag}_vm"] = vm.float().numpy()
        out[f"{tag}_vf"] = vf.numpy().astype(np.uint8)
        for basis in ("orig", "stored"):
            k, v = RKV.dequant_groups(t, D, basis=basis, f8=f8)
            out[f"{tag}_k_{basis}"], out[f"{tag}_v_{basis}"] = k.numpy(), v.numpy()
        print("kivi layout", tag, tuple(kc.shape), tuple(km.shape), tuple(vf.shape))
    np.savez_compressed(OUT / name, **out)


def write_kivi_layout_d256():
    write_kivi_layout(256, "kivi_layout_d256.npz")


# ------------------------------------------------------------------------------------------------ KIVI selection
def kivi_keys(T, Hkv, D, g):
    """the generator of the reference's KIVI test (integrations/vllm_flagrot/tests/test_kivi.py:42-48)"""
    mu = torch.randn(Hkv, D, generator=g) * 2.0
    mu[:, torch.randint(0, D, (6,), generator=g)] *= 6
    x = mu[None] + torch.randn(T, Hkv, D, generator=g) * (0.5 + torch.rand(Hkv, D, generator=g))
    x[torch.randint(0, T, (3,), generator=g)] *= 3
    return x.bfloat16()


def write_kivi_select():
    from blockflag import qattention as QA
    from blockflag.hadamard import fwht
    D, H, NQ, S, NG = 128, 2, 64, 4, 6
    T = NG * 32
    g = torch.Generator().manual_seed(4242)
    xk = kivi_keys(T, H, D, g)
    xv = (kivi_keys(100, H, D, g).float() * 0.3).bfloat16()
    qs = (torch.randn(H, NQ, D, generator=g) * 0.3).contiguous()
    lz = torch.full((H, NQ), 5.0)
    co = torch.rand(H, D, generator=g) + 0.1
    qscale = 1.0 / math.sqrt(D)
    out = dict(xk_bits=xk.view(torch.int16).numpy().view(np.uint16), xv_bits=xv.view(torch.int16).numpy().view(np.uint16),
               qs=qs.numpy(), lz=lz.numpy(), co=co.numpy(), qscale=np.float32(qscale), S=np.int32(S))
    for spec, tag in (("kivi2:32", "f16"), ("kivi2f8:32", "f8")):
        QA.KV.update(dyn=dict(rule="att", local=["H"], head=["F"], group=1, only=None), sink=0, qs={0: qs}, lz={0: lz},
                     qscale=qscale, co={0: co}, xf=None, dynstat={})
        xf = xk.float().permute(1, 0, 2)[None]                       # [1, H, T, D]
        rec = torch.empty_like(xf)
        rec[:, :, :S] = xf[:, :, :S]
        loc, full = [], []
        for a, b in ((S, 32), (32, T)):                              # first group without its sinks, then whole groups
            u = xf[:, :, a:b]
            rec[:, :, a:b] = QA.dyn_quant(u, spec, 32, "k", 0, "token")
            W = QA._weights("k", 0, u)
            Q = lambda y: QA._fake_tok(y, spec)  # noqa: E731
            recs = [Q(u), fwht(Q(fwht(u, 32)), 32)]
            errs = QA._pool_tokens(torch.stack([QA._vec_err(r - u, W, 32) for r in recs]), 32, 3)
            chs = errs.argmin(0)
            sel = chs[..., None].expand(*chs.shape, 32).reshape(u.shape)
            r = torch.where(sel == 1, recs[1], recs[0])
            F = fwht(Q(fwht(u, D)), D)
            he = QA._pool_tokens(torch.stack([QA._head_err(h - u, W) for h in (r, F)]), 32, 3)
            hs = he.argmin(0)
            idx = torch.arange(0, u.shape[2], 32)
            loc.append(chs[0][:, idx].permute(1, 0, 2).bool())       # [groups, H, NV]
            full.append(hs[0][:, idx].permute(1, 0).bool())          # [groups, H]
        out[f"{tag}_k_rec"] = rec[0].permute(1, 0, 2).contiguous().numpy()          # [T, H, D]
        out[f"{tag}_k_local"] = torch.cat(loc).numpy().astype(np.uint8)
        out[f"{tag}_k_full"] = torch.cat(full).numpy().astype(np.uint8)
        xvf = xv.float().permute(1, 0, 2)[None]
        out[f"{tag}_v_rec"] = QA.dyn_quant(xvf, spec, 32, "v", 0)[0].permute(1, 0, 2).contiguous().numpy()
        print("kivi select", tag, "local H32 fraction", float(torch.cat(loc).float().mean()), "F fraction",
              float(torch.cat(full).float().mean()))
    np.savez_compressed(OUT / "kivi_select.npz", **out)


WRITERS = {"k2": write_k2, "k2d256": write_k2_d256, "pages": write_pages, "pages256": write_pages_d256, "kivi_layout256": write_kivi_layout_d256, "static": write_static, "kivi_layout": write_kivi_layout,
           "kivi_select": write_kivi_select}


def main():
    sys.path.insert(0, str(REF / "kernels"))
    sys.path.insert(0, str(REF / "integrations" / "vllm_flagrot"))
    sys.path.insert(0, str(REF))
    torch.set_num_threads(4)
    names = [a for a in sys.argv[2:]] or list(WRITERS)
    for n in names:
        WRITERS[n]()


if __name__ == "__main__":
    main()
