"""ctypes front end of libflagrot_kernels.so (gfx950): paged FlagRot KV-cache writers + paged decode attention.

Host-side mirror of the reference plugin's front end (integrations/vllm_flagrot/vllm_flagrot/kernels.py of the
reference): same function names, argument meaning and error behaviour, so callers written against it
(`v2_write`, `v2_attn`, `cb_write`, `cb_write3`, `w3_static_write`, `cb_attn`, `head_fwht`, `plan_v2`, `plan_cb`,
`Workspace`) run unchanged.  PyTorch-ROCm only supplies device memory and the current HIP stream; every launch is
asynchronous on that stream and allocates nothing.

The shared library is built in-tree by `flagrot_releaser_amd.build` (hipcc, --offload-arch=gfx950).  It is rebuilt on
first use when it is missing or older than a source (file lock; set FLAGROT_NO_REBUILD=1 to forbid), and a missing
compiler or a failed build raises: there is no fallback path.
"""
from __future__ import annotations

import ctypes
import fcntl
import math
import os
from pathlib import Path

import torch

from . import build as _build

ABI = 9
D, RB, NG = 128, 32, 4
V2_FMT = {"int4": 4, "int4a": 5, "konly": 6, "konlya": 7, "int2a": 8, "konlya2": 9}
INT2_FMTS = ("int2a", "konlya2")
GEN, GT8, HD256 = 1024, 2048, 4096
CB_KINDS = {"konly": 6, "konlya": 10, "konlya2": 11}
K2 = ("konly", "konlya", "konlya2")
STAGES = 4
MAX_CHUNK, MAX_SPLITS = 8192, 512
SEEDS = (0,) + tuple(range(2, 16))
W3_SPLIT_T = int(os.environ.get("W3_SPLIT_T", "256"))


# ------------------------------------------------------------------------------------------------ library
def _lib_path() -> Path:
    return Path(os.environ.get("FLAGROT_LIB", _build.lib_path("kernels")))


def _stale(lib: Path) -> bool:
    if not lib.exists():
        return True
    if os.environ.get("FLAGROT_NO_REBUILD") or "FLAGROT_LIB" in os.environ:
        return False
    t = lib.stat().st_mtime
    return any(s.exists() and s.stat().st_mtime > t for s in _build.sources("kernels"))


_LIB = None


def lib():
    """the loaded library (built first when missing or out of date); raises when it cannot be had."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = _lib_path()
    if _stale(path):
        if os.environ.get("FLAGROT_NO_REBUILD"):
            raise RuntimeError(f"{path} is missing and FLAGROT_NO_REBUILD is set")
        path.parent.mkdir(parents=True, exist_ok=True)
        with open(str(path) + ".lock", "w") as lk:
            fcntl.flock(lk, fcntl.LOCK_EX)
            try:
                if _stale(path):
                    _build.build("kernels", verbose=False)
            finally:
                fcntl.flock(lk, fcntl.LOCK_UN)
    L = ctypes.CDLL(str(path))
    P, I, LL, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong, ctypes.c_float
    L.fr_abi_version.restype = I
    if L.fr_abi_version() != ABI:
        raise RuntimeError(f"libflagrot_kernels ABI {L.fr_abi_version()} != {ABI}: rebuild ({path})")
    sig = {
        "fr_v2_attn": [I, P, LL, P, P, I, P, I, I, I, I, I, F, P, P, I, I, I, I, I, P, P, P, P, LL, P, P, P, LL, LL, P,
                       I, I],
        "fr_v2_write": [I, P, LL, P, I, I, I, P, I, P, P, I, P],
        "fr_v2_occupancy": [I, I, I, I],
        "fr_v2_chunk_bytes": [I, I],
        "fr_cb_nsg": [],
        "fr_cb_write": [P, LL, P, I, I, I, I, I, P, P, P, I, P, P, I, P],
        "fr_cb_write3": [P, LL, P, I, I, I, I, P, P, P, P, P, I, P, I, I, P, P],
        "fr_w3_static_write": [P, LL, P, I, I, I, P, P, I, P, I, P, P],
        "fr_cb_attn": [P, LL, P, P, I, P, I, I, I, I, I, F, P, I, I, I, P, P, P, P, LL, P, P, P, LL, LL, P, I],
        "fr_cb_occupancy": [I, I, I, I],
        "fr_cb_chunk_bytes": [I, I],
        "fr_cb_write_smem": [I, I, I],
        "fr_head_fwht": [P, LL, P, LL, I, I, P, F, P, I],
        "fr_cb_attn_noalloc": [P, LL, P, P, I, P, I, I, I, I, I, F, I, P, LL, P, P, P, LL, LL, P, I, I],
    }
    for name, args in sig.items():
        fn = getattr(L, name)
        fn.argtypes, fn.restype = args, I
    L.fr_last_error.restype = ctypes.c_char_p
    _LIB = L
    return L


EXPORTS = ("fr_abi_version", "fr_v2_attn", "fr_v2_write", "fr_v2_occupancy", "fr_v2_chunk_bytes", "fr_cb_nsg",
           "fr_cb_write", "fr_cb_write3", "fr_w3_static_write", "fr_cb_attn", "fr_cb_occupancy", "fr_cb_chunk_bytes",
           "fr_cb_write_smem", "fr_last_error", "fr_head_fwht", "fr_cb_attn_noalloc")
NOALLOC_MAX_PARTS = 8192     # FR_NOALLOC_MAX_PARTS of include/flagrot_kernels.h


def _check(rc: int, what: str):
    if rc != 0:
        raise RuntimeError(f"{what}: launch failed (code {rc}, {lib().fr_last_error().decode()})")


def _ptr(t):
    return None if t is None else t.data_ptr()


_DEV_IDX: list = []


def _stream():
    """raw hipStream_t of torch's current stream (the device index is cached: one device per process)."""
    if not _DEV_IDX:
        _DEV_IDX.append(torch.cuda.current_device())
    return torch._C._cuda_getCurrentRawStream(_DEV_IDX[0])


_SG = None


def sign_words():
    """uint32[15 * 4] sign table argument of the codebook entry points.  The key-only kinds never read it; it is
    passed as zeros to keep the reference signature."""
    global _SG
    if _SG is None:
        _SG = (ctypes.c_uint * (len(SEEDS) * 4))()
    return _SG


# ------------------------------------------------------------------------------------------------ shapes / variants
def qtile(G: int, Dh: int = 128) -> int:
    return 8 if Dh == 128 and 5 <= G <= 8 else 4


def v2_variant(fmt: str, G: int = 4, Dh: int = 128) -> int:
    if G == 4 and Dh == 128 and fmt in ("int4", "int4a", "int2a"):
        return 264
    return 264 | GEN | (GT8 if qtile(G, Dh) == 8 else 0) | (HD256 if Dh == 256 else 0)


def tile_of(variant: int) -> int:
    return 8 if (variant & GEN) and (variant & GT8) else 4


def vheads(Hkv: int, G: int, Dh: int = 128, fmt: str = "int4") -> int:
    return Hkv * -(-G // tile_of(v2_variant(fmt, G, Dh)))


def v2_chunk_bytes(page: int, Dh: int = 128, fmt: str = "int4") -> int:
    return page * (80 if fmt in INT2_FMTS else 144) * Dh // 128


def cb_chunk_bytes(kind: str, page: int, Dh: int = 128) -> int:
    return page * (80 if kind in INT2_FMTS else 144) * Dh // 128


# ------------------------------------------------------------------------------------------------ split planner
_NUM_CU = None
# 4-wavefront workgroups resident per CU (what the small launch shape's planner fills): 4 (every format's loop fits
# 128 registers).  The library's own occupancy entry points answer 1 on purpose (one LARGE workgroup per CU: the number
# a caller written against the reference should plan with).
def _slots(fmt) -> int:
    """4-wavefront workgroups resident on the GPU at once."""
    global _NUM_CU
    if _NUM_CU is None:
        _NUM_CU = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
    return 4 * _NUM_CU


BIG_CHUNK = int(os.environ.get("FLAGROT_BIG_CHUNK", "1024"))   # tokens per split from which the library launches large workgroups


def plan_splits(B: int, Lmax: int, HV: int, page: int, slots: int, nsplit=None, ncu: int = None):
    """(nsplit, chunk) for B sequences x HV (KV head, q tile) pairs: chunk a multiple of 64 tokens, <= 8192,
    nsplit = ceil(Lmax / chunk).  Mirrors the two launch shapes of the library: when the pairs alone nearly fill the
    CUs allow chunks of >= 1024 tokens, large workgroups, one per CU at most (nsplit = min(CUs // pairs, Lmax // 1024));
    otherwise workgroups of 4 wavefronts that share a pair's page range, at most `slots` (= CUs x resident workgroups)
    of them and about sqrt(quads of pages) per pair."""
    gran = max(64, page)
    Lmax = max(1, int(Lmax))
    ncu = ncu or max(1, slots // 4)

    def plan(ns):
        ns = max(1, min(MAX_SPLITS, ns, math.ceil(Lmax / gran)))
        ns = max(ns, math.ceil(Lmax / MAX_CHUNK))
        chunk = min(MAX_CHUNK, math.ceil(Lmax / ns / gran) * gran)
        return math.ceil(Lmax / chunk), chunk

    if nsplit is not None:
        return plan(nsplit)
    pairs = B * HV
    if pairs <= ncu and Lmax >= BIG_CHUNK:          # as many large workgroups as keep >= 1024 tokens each (measured best
        ns, chunk = plan(min(ncu // pairs, Lmax // BIG_CHUNK))     # even when they fill only part of the CUs)
        if chunk >= BIG_CHUNK and 24 <= pairs * ns <= ncu:
            return ns, chunk
    # small workgroups: one round at most; a short job is a trade of pages per wavefront against partials to merge
    quads = math.ceil(Lmax / 64)
    return plan(min(max(1, slots // pairs), max(1, quads // 4), max(1, round(math.sqrt(quads)))))


def plan_v2(B, Lmax, Hkv, page, nsplit=None, fmt="int4", G=4, Dh=128):
    HV = Hkv * -(-G // 4)                                  # workgroups per (row, split): q tiles of 4 heads
    s = _slots(fmt)
    return plan_splits(B, Lmax, HV, page, s, nsplit, ncu=_NUM_CU)


def plan_cb(B, Lmax, Hkv, page, kind, nsplit=None, G=4, Dh=128):
    if kind in K2 and (G != 4 or Dh != 128):
        return plan_v2(B, Lmax, Hkv, page, nsplit, fmt=kind, G=G, Dh=Dh)
    s = _slots(kind)
    return plan_splits(B, Lmax, Hkv, page, s, nsplit, ncu=_NUM_CU)


class Workspace:
    """split-K partials for up to `parts` (row, kv head / q tile, split) partials of GT q heads x Dh dims, plus the
    per-(row, kv head / q tile) merge tickets (zeroed once, self-resetting).  Allocate before graph capture."""

    def __init__(self, rows: int, Hkv: int, parts: int, device, GT: int = 4, Dh: int = 128):
        self.rows, self.parts, self.HV, self.GT, self.Dh = rows, parts, Hkv, GT, Dh
        self.opart = torch.empty(parts * GT * Dh, device=device, dtype=torch.float32)
        self.mlpart = torch.empty(parts * GT * 2, device=device, dtype=torch.float32)
        self.counter = torch.zeros(rows * Hkv, device=device, dtype=torch.int32)

    def fits(self, B, Hkv, nsplit_total, GT=4, Dh=128):
        return (B <= self.rows and B * Hkv * nsplit_total <= self.parts and Hkv <= self.HV
                and GT * Dh <= self.GT * self.Dh
                and B * Hkv * nsplit_total * GT * Dh <= self.parts * self.GT * self.Dh)


# ------------------------------------------------------------------------------------------------ launches
def _kmu(kmu, kv):
    if kmu is None:
        return None
    Hkv, Dh = kv.shape[1] // 2, kv.shape[2]
    assert kmu.dtype == torch.float32 and kmu.is_contiguous() and tuple(kmu.shape) == (Hkv, Dh) \
        and kmu.device == kv.device, (kmu.dtype, tuple(kmu.shape), (Hkv, Dh))
    return kmu.data_ptr()


def _rows_ok(kv):
    """bf16 rows contiguous over (head, dim) and 8-byte aligned (the kernels load 4 elements at a time)."""
    Dh = kv.shape[2]
    if kv.stride(2) != 1 or kv.stride(1) != Dh or kv.stride(0) % 4 or kv.data_ptr() % 8:
        kv = kv.contiguous()
    return kv


def v2_write(kv, slots, mask, rb, pool, page, fmt="int4", kmu=None):
    """kv bf16 [T, 2*Hkv, Dh] (Dh 128 | 256) -> pool [num_pages, Hkv, chunk] at slots int64 [T] (< 0 skipped);
    mask uint8 [2*Hkv, Dh/rb] (K rows first); fmt "int4" | "int4a" | "int2a"."""
    T = kv.shape[0]
    if T == 0:
        return
    Dh = kv.shape[2]
    assert kv.dtype == torch.bfloat16 and slots.dtype == torch.int64
    kv = _rows_ok(kv)
    _check(lib().fr_v2_write(V2_FMT[fmt], kv.data_ptr(), kv.stride(0), slots.data_ptr(), T, kv.shape[1] // 2, page,
                             mask.data_ptr(), rb, pool.data_ptr(), _stream(), Dh, _kmu(kmu, kv)), "fr_v2_write")


def _launcher(fn, args, what, bound):
    """launch now, or (bound) return a zero-argument callable that launches with these very arguments: the checks and
    the pointer marshalling are done once, as under graph capture; the tensors must stay alive and in place"""
    if not bound:
        _check(fn(*args), what)
        return None

    def launch():
        rc = fn(*args)
        if rc:
            _check(rc, what)
    return launch


def v2_attn(q, pool, block_table, seq_lens, out, nsplit, chunk, ws, qscale, kmask=None, vmask=None, rb=32,
            tail=None, tail_len=None, tail_idx=None, tail_bs=None, tail_ts=None, page=16, fmt="int4", kv_start=0,
            bound=False):
    """q bf16 [B, G*Hkv, Dh] -> out bf16 [B, G*Hkv*Dh].  block_table int32 [B, *] (row stride may be 0), seq_lens int32
    [B]; tail: bf16 window rows (strides tail_bs / tail_ts elements) with tail_len int32 [B] (+ tail_idx int32 [B]).
    qscale = softmax scale * log2(e).  kv_start: tokens [0, kv_start) are masked in the paged body."""
    B, Hq, Dh = q.shape
    Hkv = pool.shape[1]
    G = Hq // Hkv
    assert Hq == G * Hkv and q.stride(2) == 1 and q.stride(1) == Dh and out.stride(1) == 1
    v = v2_variant(fmt, G, Dh)
    GT = tile_of(v)
    assert ws.fits(B, vheads(Hkv, G, Dh, fmt), nsplit + (tail is not None), GT, Dh), "split-K workspace too small"
    args = (V2_FMT[fmt], q.data_ptr(), q.stride(0), pool.data_ptr(), block_table.data_ptr(),
            block_table.stride(0), seq_lens.data_ptr(), B, Hkv, page, nsplit, chunk, qscale,
            _ptr(kmask), _ptr(vmask), rb, int(kmask is not None), int(vmask is not None), v, STAGES,
            ws.opart.data_ptr(), ws.mlpart.data_ptr(), ws.counter.data_ptr(), out.data_ptr(),
            out.stride(0), _ptr(tail), _ptr(tail_len), _ptr(tail_idx),
            0 if tail is None else tail_bs, 0 if tail is None else tail_ts, _stream(), G, int(kv_start))
    return _launcher(lib().fr_v2_attn, args, "fr_v2_attn", bound)


def cb_write(kv, slots, CT, co, kind, pool, page, tg=None, kmu=None):
    """kv bf16 [T, 2*Hkv, 128] -> pool at slots int64 [T]; CT fp32 [Hkv, 128, 128] = C_q^T, co fp32 [Hkv, 128]."""
    T = kv.shape[0]
    if T == 0:
        return
    Dh = kv.shape[2]
    assert kv.dtype == torch.bfloat16 and slots.dtype == torch.int64
    kv = _rows_ok(kv)
    if tg is None:
        tg = 1 if T <= 16 else (2 if T <= 64 or kind not in K2 else 4)
    _check(lib().fr_cb_write(kv.data_ptr(), kv.stride(0), slots.data_ptr(), 0, T, kv.shape[1] // 2, page, tg,
                             CT.data_ptr(), co.data_ptr(), sign_words(), CB_KINDS[kind], pool.data_ptr(), _stream(),
                             Dh, _kmu(kmu, kv)), "fr_cb_write")


_SIDE: dict = {}


def side_stream(device=None):
    """second stream of the two-pass writer (one per device, default priority; create before graph capture)."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    if dev not in _SIDE:
        _SIDE[dev] = torch.cuda.Stream(dev)
    return _SIDE[dev]


def w3_nchunk(Hkv, per_cu):
    global _NUM_CU
    if _NUM_CU is None:
        _NUM_CU = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
    return max(1, (per_cu * _NUM_CU) // Hkv)


def w3_calib(Cq, kappa=None, nd=8):
    """the reference's writer v3 takes tensor-core screening constants (C1 fp16 [H, 168, 128], aux fp32 [H, 48]).
    This library's writer evaluates the exact fp32 criterion directly and ignores them; zero tensors of the reference
    shapes keep callers unchanged."""
    H = Cq.shape[0]
    return (torch.zeros(H, 168, 128, dtype=torch.float16, device=Cq.device),
            torch.zeros(H, 48, dtype=torch.float32, device=Cq.device))


def cb_write3(kv, slots, CT, co, C1, beta, kind, pool, page, split=None, kmu=None):
    """= cb_write (same pool bytes).  split (default: T <= W3_SPLIT_T): key pass on the current stream, value pass on
    the side stream (fork / join by stream waits, graph capturable), else both in one launch."""
    T = kv.shape[0]
    if T == 0:
        return
    assert kv.dtype == torch.bfloat16 and slots.dtype == torch.int64
    assert kv.shape[2] == D, f"writer v3: head dim {D} only (got {kv.shape[2]}; use cb_write)"
    kv = _rows_ok(kv)
    slots = slots.contiguous()
    Hkv = kv.shape[1] // 2
    L = lib()
    nk, nv = w3_nchunk(Hkv, 2), w3_nchunk(Hkv, 3)
    km = _kmu(kmu, kv)
    args = (kv.data_ptr(), kv.stride(0), slots.data_ptr(), 0, T, Hkv, page, CT.data_ptr(), co.data_ptr(),
            _ptr(C1), _ptr(beta), sign_words(), CB_KINDS[kind], pool.data_ptr())
    if split is None:
        split = T <= W3_SPLIT_T
    if not split:
        _check(L.fr_cb_write3(*args, nk, nv, _stream(), km), "fr_cb_write3")
        return
    cur = torch.cuda.current_stream()
    side = side_stream(kv.device)
    side.wait_stream(cur)
    _check(L.fr_cb_write3(*args, nk, -1, cur.cuda_stream, km), "fr_cb_write3 (keys)")
    _check(L.fr_cb_write3(*args, -1, nv, side.cuda_stream, None), "fr_cb_write3 (values)")
    cur.wait_stream(side)


def w3_static_write(kv, slots, mask, hfull, pool, page, fmt="int4", path=0, kmu=None):
    """= head_fwht(kv, hfull, 1/16) + v2_write(.., mask, rb 32, ..) in one launch (same pool bytes)."""
    T = kv.shape[0]
    if T == 0:
        return
    assert kv.dtype == torch.bfloat16 and slots.dtype == torch.int64
    assert kv.shape[2] == D, f"writer v3: head dim {D} only (got {kv.shape[2]}; use v2_write)"
    kv = _rows_ok(kv)
    slots = slots.contiguous()
    _check(lib().fr_w3_static_write(kv.data_ptr(), kv.stride(0), slots.data_ptr(), T, kv.shape[1] // 2, page,
                                    _ptr(mask), _ptr(hfull), {"int4": 0, "int4a": 1, "int2a": 2}[fmt],
                                    pool.data_ptr(), path, _stream(), _kmu(kmu, kv)), "fr_w3_static_write")


def cb_attn(q, pool, block_table, seq_lens, out, nsplit, chunk, ws, qscale, kind, tail=None, tail_len=None,
            tail_idx=None, tail_bs=None, tail_ts=None, page=16, kv_start=0, bound=False):
    B, Hq, Dh = q.shape
    if kind in K2 and (Hq != 4 * pool.shape[1] or Dh != 128):
        return v2_attn(q, pool, block_table, seq_lens, out, nsplit, chunk, ws, qscale, tail=tail, tail_len=tail_len,
                       tail_idx=tail_idx, tail_bs=tail_bs, tail_ts=tail_ts, page=page, fmt=kind, kv_start=kv_start,
                       bound=bound)
    Hkv = Hq // 4
    assert Hq == 4 * pool.shape[1] and Dh == D, f"codebook {kind}: GQA 4, head dim 128 only"
    assert q.stride(2) == 1 and q.stride(1) == D and out.stride(1) == 1
    assert ws.fits(B, Hkv, nsplit + (tail is not None)), "split-K workspace too small"
    args = (q.data_ptr(), q.stride(0), pool.data_ptr(), block_table.data_ptr(), block_table.stride(0),
            seq_lens.data_ptr(), B, Hkv, page, nsplit, chunk, qscale, sign_words(), CB_KINDS[kind], 0,
            STAGES, ws.opart.data_ptr(), ws.mlpart.data_ptr(), ws.counter.data_ptr(), out.data_ptr(),
            out.stride(0), _ptr(tail), _ptr(tail_len), _ptr(tail_idx),
            0 if tail is None else tail_bs, 0 if tail is None else tail_ts, _stream(), int(kv_start))
    return _launcher(lib().fr_cb_attn, args, "fr_cb_attn", bound)


def cb_attn_noalloc(q, pool, block_table, seq_lens, out, nsplit, chunk, qscale, kind, tail=None, tail_len=None,
                    tail_idx=None, tail_bs=None, tail_ts=None, page=16, kv_start=0, bound=False):
    """cb_attn for callers that cannot allocate: no workspace argument, the split partials live in an array built
    into the library (shared by all calls on the GPU: do not overlap calls).  Raises when
    B * Hkv * ceil(G / 4) * (nsplit + 1) exceeds NOALLOC_MAX_PARTS.  No counterpart in the reference front end."""
    B, Hq, Dh = q.shape
    Hkv = pool.shape[1]
    G = Hq // Hkv
    assert kind in K2 and Hq == G * Hkv and Dh == D, f"{kind}: key-only 2x2 kinds, head dim 128 only"
    assert q.stride(2) == 1 and q.stride(1) == D and out.stride(1) == 1
    args = (q.data_ptr(), q.stride(0), pool.data_ptr(), block_table.data_ptr(), block_table.stride(0),
            seq_lens.data_ptr(), B, Hkv, page, nsplit, chunk, qscale, CB_KINDS[kind], out.data_ptr(), out.stride(0),
            _ptr(tail), _ptr(tail_len), _ptr(tail_idx), 0 if tail is None else tail_bs,
            0 if tail is None else tail_ts, _stream(), G, int(kv_start))
    return _launcher(lib().fr_cb_attn_noalloc, args, "fr_cb_attn_noalloc", bound)


def head_fwht(x, flags, scale, out=None):
    """x bf16 [T, H, Dh] (Dh 128 | 256) -> scale * H_Dh x (unnormalised +-1 Sylvester) for heads with flags[h] != 0,
    a copy otherwise; out may alias x."""
    T, H, Dh = x.shape
    assert x.dtype == torch.bfloat16 and x.stride(2) == 1 and x.stride(1) == Dh
    if out is None:
        out = torch.empty(T, H, Dh, dtype=x.dtype, device=x.device)
    assert out.stride(2) == 1 and out.stride(1) == Dh
    if T:
        _check(lib().fr_head_fwht(x.data_ptr(), x.stride(0), out.data_ptr(), out.stride(0), T, H, flags.data_ptr(),
                                  scale, _stream(), Dh), "fr_head_fwht")
    return out


# ------------------------------------------------------------------------------------------------ torch page parsers
# Host-side readers of the page bytes (any device, no library call): what the plugin's PyTorch prefill path and tests use
# to look inside a cache.  Mirrors parse_int4_pages / parse_int2_pages / parse_pages / dequant_v2_pages / hadamard /
# dequant_cb_pages of the reference front end (vllm_flagrot/kernels.py:591-765); the key-only 2x2 kinds only.
_MAPS: dict = {}


def _layout_maps(fmt: str, page: int, device):
    """gather maps of one 128-d chunk: for every (token, K|V, dim) the byte holding its code and the bit position, and
    for every (token, K|V, group) the byte offset of its 16-bit scale word.  INT4 symmetric additionally: byte / bit of
    the sign and of the 3-bit magnitude."""
    key = (fmt, page, str(device))
    if key in _MAPS:
        return _MAPS[key]
    P = page
    int2, sym = fmt in INT2_FMTS, fmt in ("int4", "konly")
    cb = 32 if int2 else 64
    t = torch.arange(P).view(P, 1)
    d = torch.arange(128).view(1, 128)
    g, r = d // 32, d % 32
    isB, tg, i = r // 16, (r % 16) // 4, r % 4
    # V^T entry of a dim and position of a token inside it
    e = ((d % 64) // 16) * 8 + d % 8
    sub = 2 * (d // 64) + (d % 16) // 8
    c8, ii, odd = t // 8, (t % 8) // 2, t % 2
    if int2:
        kbyte = 32 * (t ^ ((t >> 1) & 2)) + 8 * tg + 4 * (g // 2) + i
        kshift = 4 * (g % 2) + 2 * isB + 0 * t
        vbyte = cb * P + (e * (P // 8) + c8) * 8 + 4 * (d // 64) + ii
        vshift = 4 * ((d % 16) // 8) + 2 * odd
        maps = dict(byte=torch.stack([kbyte, vbyte], 1), shift=torch.stack([kshift.expand(P, 128), vshift], 1))
    else:
        kbyte = 64 * t + 16 * tg + 4 * g + i
        vbyte = cb * P + (e * (P // 8) + c8) * 16 + 4 * sub + ii
        if not sym:
            kshift = (4 * isB).expand(P, 128)
            vshift = (4 * odd).expand(P, 128)
            maps = dict(byte=torch.stack([kbyte, vbyte], 1), shift=torch.stack([kshift, vshift], 1))
        else:
            # A element: sign bit 7, magnitude bits 0-2 of its byte; B element: sign bit 3 of its byte, magnitude bits
            # 4-6 of the byte (k + 3) % 4 of the same word
            kB = isB.expand(P, 128).bool()
            vB = odd.expand(P, 128).bool()
            kmagb = torch.where(kB, 64 * t + 16 * tg + 4 * g + (i + 3) % 4, kbyte)
            vmagb = torch.where(vB, cb * P + (e * (P // 8) + c8) * 16 + 4 * sub + (ii + 3) % 4, vbyte)
            B2 = torch.stack([kB, vB], 1)
            maps = dict(byte=torch.stack([kbyte, vbyte], 1), magbyte=torch.stack([kmagb, vmagb], 1),
                        signbit=torch.where(B2, 3, 7), magshift=torch.where(B2, 4, 0))
    gg = torch.arange(4).view(1, 4)
    slot8 = torch.where(t % 2 == 1, 4 + (t % 8) // 2, (t % 8) // 2)
    ks = 2 * cb * P + 8 * t + 2 * gg
    vs = 2 * cb * P + 8 * P + (gg * P + 8 * (t // 8) + slot8) * 2
    maps["scale"] = torch.stack([ks, vs], 1)                                        # [P, 2, 4] byte offsets
    maps = {k: v.to(device) for k, v in maps.items()}
    _MAPS[key] = maps
    return maps


def parse_pages(chunks, page, fmt, Dh=128):
    """chunks uint8 [Np, H, >= chunk bytes] of a static format ("int4" | "int4a" | "int2a") or key-only kind ("konly" |
    "konlya" | "konlya2") -> codes int16 [Np, H, P, 2, Dh] (K then V, stored coordinates, zero point already subtracted
    for the asymmetric formats), scale magnitudes fp32 [Np, H, P, 2, Dh / 32] (the word read as FP16 without its sign
    bit), raw scale words int16 [Np, H, P, 2, Dh / 32] (zero point in the low bits, flags in the sign bits).
    Dh 256: the chunk is two 128-d half chunks (dims 0-127, then 128-255)."""
    Np, H = chunks.shape[:2]
    if Dh == 256:
        half = (80 if fmt in INT2_FMTS else 144) * page
        c, m, sb = parse_pages(chunks[..., :2 * half].reshape(Np, 2 * H, half), page, fmt)
        join = lambda x: x.reshape(Np, H, 2, page, 2, x.shape[-1]).permute(0, 1, 3, 4, 2, 5).reshape(Np, H, page, 2, -1)  # noqa: E731
        return join(c), join(m), join(sb)
    assert Dh == 128
    mp = _layout_maps(fmt, page, chunks.device)
    by = chunks.to(torch.int16)
    if "shift" in mp:
        width = 3 if fmt in INT2_FMTS else 15
        codes = (by[..., mp["byte"]] >> mp["shift"]) & width
    else:
        sign = (by[..., mp["byte"]] >> mp["signbit"]) & 1
        mag = (by[..., mp["magbyte"]] >> mp["magshift"]) & 7
        codes = torch.where(sign == 1, -mag, mag)
    so = mp["scale"]
    lo, hi = chunks[..., so].to(torch.int32), chunks[..., so + 1].to(torch.int32)
    word = lo | (hi << 8)
    sbits = torch.where(word >= 32768, word - 65536, word).to(torch.int16)              # [Np, H, P, 2, 4]
    mag = (sbits & 0x7FFF).view(torch.float16).float()
    if fmt not in ("int4", "konly"):
        zmask = 3 if fmt in INT2_FMTS else 15
        codes = codes - (sbits & zmask).repeat_interleave(RB, -1)
    return codes.to(torch.int16), mag, sbits


def parse_int4_pages(chunks, page, asym=False, Dh=128):
    return parse_pages(chunks, page, "int4a" if asym else "int4", Dh)


def parse_int2_pages(chunks, page, Dh=128):
    return parse_pages(chunks, page, "int2a", Dh)


def dequant_v2_pages(chunks, page, dtype=torch.bfloat16, fmt="int4", Dh=128):
    """static pages -> K, V [Np, P, H, Dh] in the STORED (rotated) basis: codes times the group's scale magnitude."""
    codes, mag, _ = parse_pages(chunks, page, fmt, Dh)
    x = codes.float().reshape(*codes.shape[:-1], Dh // RB, RB) * mag[..., None]
    x = x.reshape(codes.shape).to(dtype)
    return x[..., 0, :].transpose(1, 2), x[..., 1, :].transpose(1, 2)


_HM: dict = {}


def hadamard(n, device, dtype=torch.float32):
    """orthonormal Sylvester-Hadamard matrix (symmetric)."""
    key = (n, str(device), dtype)
    if key not in _HM:
        h = torch.ones(1, 1, dtype=torch.float64)
        while h.shape[0] < n:
            h = torch.cat([torch.cat([h, h], 1), torch.cat([h, -h], 1)], 0)
        _HM[key] = (h / math.sqrt(n)).to(device=device, dtype=dtype)
    return _HM[key]


def dequant_cb_pages(chunks, page, kind, dtype=torch.bfloat16, Dh=128):
    """key-only 2x2 pages -> K, V [Np, P, H, Dh]: keys in the ORIGINAL basis (H32 on the groups whose K scale word has
    its sign bit set, whole-head H_Dh when the token's group-0 V scale word has), values as stored."""
    if kind not in K2:
        raise NotImplementedError(f"codebook kind {kind}: only the key-only 2x2 kinds are built")
    Np, H = chunks.shape[:2]
    codes, mag, sbits = parse_pages(chunks, page, kind, Dh)
    ng = Dh // RB
    dev = chunks.device
    x = codes.float().reshape(*codes.shape[:-1], ng, RB) * mag[..., None]                # [Np, H, P, 2, ng, 32]
    whole = sbits[..., 1, 0] < 0                                                         # [Np, H, P]
    local = sbits[..., 0, :] < 0                                                         # [Np, H, P, ng]
    k = x[..., 0, :, :]
    kl = torch.where(local[..., None], k @ hadamard(RB, dev), k).reshape(Np, H, page, Dh)
    kf = k.reshape(Np, H, page, Dh) @ hadamard(Dh, dev)
    k = torch.where(whole[..., None], kf, kl).to(dtype)
    v = x[..., 1, :, :].reshape(Np, H, page, Dh).to(dtype)
    return k.transpose(1, 2), v.transpose(1, 2)
