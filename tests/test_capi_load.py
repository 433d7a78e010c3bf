"""CPU-side checks of the drop-in boundary: the library builds/loads and exports every symbol the header declares
(no compute calls here: there is no GPU)."""
import ctypes
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b((?:fr|kv|frmq)_[a-z0-9_]+)\s*\(", text)


def test_kernels_library_exports_header_symbols():
    from flagrot_releaser_amd import build, kernels
    path = build.lib_path("kernels")
    if not path.exists():
        build.build("kernels", verbose=False)
    L = ctypes.CDLL(str(path))
    names = _declared("flagrot_kernels.h")
    assert set(names) == set(kernels.EXPORTS)
    for n in names:
        assert hasattr(L, n), n
    L.fr_abi_version.restype = ctypes.c_int
    assert L.fr_abi_version() == 9
    assert L.fr_cb_nsg() == 15
    assert L.fr_v2_chunk_bytes(5, 16) == 2304 and L.fr_v2_chunk_bytes(8, 16) == 1280
    assert L.fr_cb_chunk_bytes(10, 16) == 2304 and L.fr_cb_chunk_bytes(11, 16) == 1280


def test_kivi_library_exports_header_symbols():
    from flagrot_releaser_amd import build, kivi
    path = build.lib_path("kivi")
    if not path.exists():
        build.build("kivi", verbose=False)
    L = ctypes.CDLL(str(path))
    names = _declared("flagrot_kivi.h")
    assert set(names) == set(kivi.EXPORTS)
    for n in names:
        assert hasattr(L, n), n
    L.kv_abi_version.restype = ctypes.c_int
    assert L.kv_abi_version() == 9
    assert L.kv_chunk_bytes(128) == 1552 and L.kv_chunk_bytes8(128) == 1280
    assert kivi.plan(16, 32768, 8, sms=256) == (6, 5472) and kivi.plan(1, 100, 8, sms=256)[1] == 256
    # few pairs or short contexts: half the slots, 24 splits at most, 1024 tokens per split at least
    assert kivi.plan(1, 32640, 8, sms=256) == (24, 1376) and kivi.plan(8, 8064, 8, sms=256) == (7, 1152)
    assert kivi.plan(64, 2048, 8, sms=256) == (2, 1024)
    assert kivi.plan(16, 8192, 4, sms=256, D=256) == (7, 1184)         # two workgroups per CU at head dim 256, one of the 8 slots for the ring rows


def test_mq_library_exports_header_symbols():
    from flagrot_releaser_amd import build, prefill_mq
    path = build.lib_path("mq")
    if not path.exists():
        build.build("mq", verbose=False)
    L = ctypes.CDLL(str(path))
    names = _declared("flagrot_mq.h")
    assert set(names) == set(prefill_mq.EXPORTS)
    for n in names:
        assert hasattr(L, n), n
    L.frmq_abi_version.restype = ctypes.c_int
    assert L.frmq_abi_version() == 7
    assert 0 < L.frmq_smem_bytes() <= 160 * 1024


def test_probe_library_exports_header_symbols():
    from flagrot_releaser_amd import build, probe
    path = build.lib_path("probe")
    if not path.exists():
        build.build("probe", verbose=False)
    L = ctypes.CDLL(str(path))
    names = _declared("flagrot_probe.h")
    assert set(names) == set(probe.EXPORTS) == {"fr_probe_abi_version", "fr_probe_last_error", "fr_probe_read",
                                                      "fr_probe_mfma", "fr_probe_mfma_flops"}
    for n in names:
        assert hasattr(L, n), n
    L.fr_probe_abi_version.restype = ctypes.c_int
    assert L.fr_probe_abi_version() == probe.ABI


def test_c_caller_compiles_links_and_runs(tmp_path):
    """tests/c_abi/abi_check.c, a plain C99 caller: the headers compile as C (-Wall -Wextra -Werror -pedantic), every
    declared entry point of the three boundary libraries resolves at link time, and the calls that need no GPU
    (versions, sizes, argument checks that return before any launch) give the documented answers"""
    from flagrot_releaser_amd import build
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    libdir = build.lib_path("kernels").parent
    for lib in ("kernels", "kivi", "mq"):
        if not build.lib_path(lib).exists():
            build.build(lib, verbose=False)
    exe = tmp_path / "abi_check"
    cmd = [gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "c_abi", "abi_check.c"), "-o", str(exe), "-L", str(libdir), "-lflagrot_kernels",
           "-lflagrot_kivi", "-lflagrot_mq", f"-Wl,-rpath,{libdir}", "-Wl,-rpath-link,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.returncode, r.stderr[-500:])
    assert "all checks passed" in r.stdout


def test_host_planner_invariants():
    from flagrot_releaser_amd import kernels as K
    for B, L in ((1, 1), (1, 2048), (32, 8192), (64, 16384), (3, 33000), (8, 65536)):
        for slots in (256, 512, 1024):
            ns, ch = K.plan_splits(B, L, 8, 16, slots)
            assert ch % 64 == 0 and ch <= K.MAX_CHUNK and ns == -(-L // ch) and ns <= K.MAX_SPLITS
    assert K.plan_splits(4, 1000, 8, 16, 512, nsplit=3) == (3, 384)
    # pairs that fill the CUs with long chunks: one large workgroup each; else one round of shared-range workgroups
    assert K.plan_splits(32, 8192, 8, 16, 1024, ncu=256) == (1, 8192)
    assert K.plan_splits(8, 32768, 8, 16, 1024, ncu=256) == (4, 8192)
    assert K.plan_splits(64, 16256, 8, 16, 1024, ncu=256) == (2, 8128)
    assert K.plan_splits(2, 4097, 8, 16, 1024, ncu=256) == (4, 1088)
    # short contexts on few pairs: one large workgroup up to 1024 tokens, splits of 512 tokens beyond; below 512 tokens
    # (and where such splits would not fit the CUs) the small workgroups' plan
    assert K.plan_splits(1, 1024, 8, 16, 1024, ncu=256) == (1, 1024)
    assert K.plan_splits(1, 2048, 8, 16, 1024, ncu=256) == (4, 512)
    assert K.plan_splits(2, 1500, 8, 16, 1024, ncu=256) == (3, 512)
    assert K.plan_splits(1, 4096, 8, 16, 1024, ncu=256) == (8, 512)
    assert K.plan_splits(8, 2048, 8, 16, 1024, ncu=256) == (4, 512)
    assert K.plan_splits(8, 4096, 8, 16, 1024, ncu=256) == (4, 1024)
    assert K.plan_splits(1, 300, 8, 16, 1024, ncu=256) == (1, 320)
    assert K.plan_splits(32, 2000, 8, 16, 1024, ncu=256) == (1, 2048)
    assert K.plan_splits(40, 800, 8, 16, 1024, ncu=256) == (3, 320)
    assert K.plan_splits(1, 2048, 8, 16, 512, ncu=0) == (6, 384)                     # head dim 256: small workgroups only
    assert K.plan_splits(1, 32768, 8, 16, 1024, ncu=256) == (32, 1024)
    assert K.plan_splits(64, 2048, 8, 16, 1024, ncu=256) == (2, 1024)
    assert K.v2_variant("int4a", 4) == 264 and K.tile_of(K.v2_variant("konlya", 8)) == 8
    assert K.vheads(8, 8, 128, "konlya") == 8 and K.vheads(4, 12, 128, "int4") == 12


def test_key_loops_keep_their_registers():
    """No kernel with a software-pipelined page loop may spill: a reload from scratch is a vector-memory load, and the
    wait for it is a wait for every page fetch in flight.  Read from the register reports of the in-tree build."""
    from flagrot_releaser_amd import build
    hot = ("k_decode", "k_wide_parts_mma", "k_attn_pages", "k_mq")
    seen = 0
    for lib in ("kernels", "kivi", "mq"):
        rep = build.spills(lib)
        if not rep:
            pytest.skip("no register report: the libraries were not built in this tree")
        for kernel, n in rep.items():
            if any(h in kernel for h in hot):
                seen += 1
                assert n == 0, (kernel, n)
    assert seen >= 40


def test_decode_front_end_rejects_a_pool_of_another_page_size():
    """a pool of 32-token pages read with page = 16 would send the kernels past the ends of the block-table rows: the
    front end compares the chunk size with (format, page, head dim) before anything is launched"""
    import torch
    from flagrot_releaser_amd import kernels as K
    q = torch.zeros(2, 32, 128, dtype=torch.bfloat16)
    out = torch.zeros(2, 32 * 128, dtype=torch.bfloat16)
    bt = torch.zeros(2, 4, dtype=torch.int32)
    lens = torch.zeros(2, dtype=torch.int32)
    pool32 = torch.zeros(8, 8, K.cb_chunk_bytes("konlya", 32), dtype=torch.uint8)
    with pytest.raises(AssertionError, match="not pages of 16 tokens"):
        K.cb_attn(q, pool32, bt, lens, out, 1, 64, None, 1.0, "konlya")
    with pytest.raises(AssertionError, match="not pages of 16 tokens"):
        K.v2_attn(q, pool32, bt, lens, out, 1, 64, None, 1.0, fmt="int4a")
    with pytest.raises(AssertionError, match="not pages of 16 tokens"):
        K.cb_attn_noalloc(q, pool32, bt, lens, out, 1, 64, 1.0, "konlya")
