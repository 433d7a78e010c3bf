"""The binding tables a maintainer of the reference plugin is told to use, taken literally out of the integration
notes at the repository root (NOTES below): every `L.<entry point>.argtypes = [...]` line is parsed from the document, compared type by type with the declaration
in include/*.h (CPU), and used -- on a fresh ctypes handle, without this package's own loader -- for one writer call
and one decode call checked against the oracle (GPU).  A typo in the document fails here."""
import ctypes
import math
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CT = {"P": ctypes.c_void_p, "I": ctypes.c_int, "LL": ctypes.c_longlong, "F": ctypes.c_float}
LIB_OF_PREFIX = {"fr": "kernels", "kv": "kivi", "frmq": "mq"}
NOTES = "INTEGRATION.md"


def documented_tables():
    text = open(os.path.join(ROOT, NOTES)).read()
    out = {}
    for name, body in re.findall(r"L\.(\w+)\.argtypes\s*=\s*\[([^\]]*)\]", text):
        out[name] = [t.strip() for t in body.split(",") if t.strip()]
    return out


def declared_parameters():
    """entry point -> list of parameter classes ('P', 'I', 'LL', 'F') read from the headers"""
    decl = {}
    for header in ("flagrot_kernels.h", "flagrot_kivi.h", "flagrot_mq.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        for name, params in re.findall(r"\b((?:fr|kv|frmq)_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
            kinds = []
            for prm in params.split(","):
                prm = " ".join(prm.split())
                if prm in ("", "void"):
                    continue
                if "*" in prm:
                    kinds.append("P")
                elif prm.startswith("long long"):
                    kinds.append("LL")
                elif prm.startswith("float"):
                    kinds.append("F")
                elif prm.startswith(("int", "unsigned")):
                    kinds.append("I")
                else:
                    raise AssertionError(f"{header}: cannot classify parameter '{prm}' of {name}")
            decl[name] = kinds
    return decl


def test_documented_tables_match_the_headers():
    tables, decl = documented_tables(), declared_parameters()
    must = {"fr_v2_attn", "fr_v2_write", "fr_cb_write", "fr_cb_write3", "fr_w3_static_write", "fr_cb_attn", "fr_head_fwht",
            "fr_cb_attn_noalloc", "kv_v_write", "kv_k_encode", "kv_attn", "kv_dequant", "kv_lse_merge", "frmq_prep_q",
            "frmq_attn", "frmq_merge", "frmq_win_gather", "frmq_bf_merge"}
    assert must <= set(tables), sorted(must - set(tables))
    for name, types in tables.items():
        assert name in decl, f"{name} is documented but not declared in include/"
        assert all(t in CT for t in types), (name, types)
        assert types == decl[name], f"{name}: the notes say {types}, the header declares {decl[name]}"


def test_documented_tables_match_the_front_ends():
    """the package's own signature strings say the same as the document"""
    from flagrot_releaser_amd import kernels, kivi, prefill_mq
    letter = {"p": "P", "i": "I", "l": "LL", "f": "F"}
    own = {}
    for mod in (kernels, kivi, prefill_mq):
        for name, sig in mod.NATIVE.table.items():
            own[name] = [letter[c] for c in sig.partition("->")[0].split()]
    for name, types in documented_tables().items():
        assert own[name] == types, name


@pytest.mark.gpu
def test_writer_and_decode_through_the_documented_binding(dev):
    import torch

    from flagrot_releaser_amd import build
    from oracle import attend as A
    from oracle import pages as PG
    from oracle import quant as Q
    from tests.gpu_util import P, alloc_tables, bits, make_kv, slots_of, spd_calib
    tables = documented_tables()
    L = ctypes.CDLL(str(build.lib_path("kernels")))           # a handle of its own: nothing of native.py is in play
    for name in ("fr_cb_write", "fr_cb_attn"):
        getattr(L, name).argtypes = [CT[t] for t in tables[name]]
        getattr(L, name).restype = ctypes.c_int
    L.fr_last_error.restype = ctypes.c_char_p
    assert L.fr_abi_version() == 9
    kind, kid, Hkv, G = "konlya", 10, 2, 4
    lens = [150, 33, 700]
    g = torch.Generator().manual_seed(77)
    npg = sum(-(-n // P) for n in lens) + 3
    pool = torch.randint(0, 256, (npg, Hkv, PG.chunk_bytes(kind, P)), dtype=torch.uint8, generator=g)
    want = pool.numpy().copy()
    dpool = pool.to(dev)
    bt = alloc_tables(lens, npg, g, P)
    Cq, co = spd_calib(Hkv, g)
    CTm, dco = Cq.transpose(1, 2).contiguous().to(dev), co.to(dev)
    sg = (ctypes.c_uint * 60)()
    stream = torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())
    for b, n in enumerate(lens):
        kv = make_kv(n, Hkv, g, edge=(b == 0))
        dkv, sl = kv.to(dev), slots_of(bt, b, n, P).to(dev)
        rc = L.fr_cb_write(dkv.data_ptr(), dkv.stride(0), sl.data_ptr(), 0, n, Hkv, P, 0, CTm.data_ptr(), dco.data_ptr(),
                           sg, kid, dpool.data_ptr(), stream, 128, None)
        assert rc == 0, L.fr_last_error()
        codes, words, _ = Q.k2_encode(bits(kv), Cq.numpy(), kind)
        PG.pack_tokens(want, slots_of(bt, b, n, P).numpy(), codes, words, kind, P)
    torch.cuda.synchronize()
    assert np.array_equal(dpool.cpu().numpy(), want), "writer bytes differ from the oracle"
    B, HQ = len(lens), G * Hkv
    q = (torch.randn(B, HQ, 128, generator=g) * 0.8).bfloat16()
    dq, dbt = q.to(dev), bt.to(dev)
    dseq = torch.tensor(lens, dtype=torch.int32, device=dev)
    ns, chunk = 2, 384
    opart = torch.zeros(B * Hkv * (ns + 1) * 4 * 128, dtype=torch.float32, device=dev)
    mlpart = torch.zeros(B * Hkv * (ns + 1) * 4 * 2, dtype=torch.float32, device=dev)
    counter = torch.zeros(B * Hkv, dtype=torch.int32, device=dev)
    out = torch.zeros(B, HQ * 128, dtype=torch.bfloat16, device=dev)
    scale = 1 / math.sqrt(128)
    rc = L.fr_cb_attn(dq.data_ptr(), dq.stride(0), dpool.data_ptr(), dbt.data_ptr(), dbt.stride(0), dseq.data_ptr(), B, Hkv,
                      P, ns, chunk, scale * 1.4426950408889634, sg, kid, 0, 4, opart.data_ptr(), mlpart.data_ptr(),
                      counter.data_ptr(), out.data_ptr(), out.stride(0), None, None, None, 0, 0, stream, 0)
    assert rc == 0, L.fr_last_error()
    torch.cuda.synchronize()
    ref = A.decode_reference(bits(q), want, kind, P, bt.numpy(), lens, scale)
    got = out.view(B, HQ, 128).float().cpu().numpy().astype(np.float64)
    lim = 2e-3 + 1e-2 * np.abs(ref)
    lim[0] = 2e-3 + 1e-2 * np.abs(ref[0]).max()          # row 0 reads the adversarial tokens: its row maximum
    assert (np.abs(got - ref) <= lim).all(), float((np.abs(got - ref) / lim).max())
    assert int(counter.abs().sum()) == 0
