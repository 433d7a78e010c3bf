"""Front end of libflagrot_kernels.so (gfx950): the paged FlagRot KV-cache writers and the paged decode attention.

What a caller of the reference plugin's front end (integrations/vllm_flagrot/vllm_flagrot/kernels.py) finds here under
the same names and with the same arguments: the static-format writer and decode (`v2_write`, `v2_attn`), the selecting
writers of the key-only kinds (`cb_write`, `cb_write3`, `w3_static_write`, `head_fwht`) and their decode (`cb_attn`), the
split planners (`plan_v2`, `plan_cb`) and the split-K `Workspace`.  `cb_attn_noalloc` exists on this build only.

PyTorch lends device memory and the current HIP stream; each call is one or two asynchronous kernel launches on that
stream, and none of them allocates.  The library is built in-tree by flagrot_releaser_amd.build (hipcc,
--offload-arch=gfx950) and rebuilt on first use when a source is newer (FLAGROT_NO_REBUILD=1 forbids that); when it
cannot be had the call raises -- there is no other path to a result.
"""
from __future__ import annotations

import ctypes
import math
import os

import torch

from .native import Library, as_arg, current_stream

ABI = 9
D, RB, NG = 128, 32, 4
# numbers the C ABI shares with the reference: format ids, kind ids, variant bits
V2_FMT = {"int4": 4, "int4a": 5, "konly": 6, "konlya": 7, "int2a": 8, "konlya2": 9}
INT2_FMTS = ("int2a", "konlya2")
GEN, GT8, HD256 = 1024, 2048, 4096
CB_KINDS = {"konly": 6, "konlya": 10, "konlya2": 11}
K2 = ("konly", "konlya", "konlya2")
STAGES = 4
MAX_CHUNK, MAX_SPLITS = 8192, 512
SEEDS = (0,) + tuple(range(2, 16))
W3_SPLIT_T = int(os.environ.get("W3_SPLIT_T", "256"))
NOALLOC_MAX_PARTS = 8192     # FR_NOALLOC_MAX_PARTS of include/flagrot_kernels.h

NATIVE = Library("kernels", "FLAGROT_LIB", "fr_abi_version", ABI, "fr_last_error", {
    "fr_v2_attn": "i p l p p i p i i i i i f p p i i i i i p p p p l p p p l l p i i",
    "fr_v2_write": "i p l p i i i p i p p i p",
    "fr_v2_occupancy": "i i i i",
    "fr_v2_chunk_bytes": "i i",
    "fr_cb_nsg": "",
    "fr_cb_write": "p l p i i i i i p p p i p p i p",
    "fr_cb_write3": "p l p i i i i p p p p p i p i i p p",
    "fr_w3_static_write": "p l p i i i p p i p i p p",
    "fr_cb_attn": "p l p p i p i i i i i f p i i i p p p p l p p p l l p i",
    "fr_cb_occupancy": "i i i i",
    "fr_cb_chunk_bytes": "i i",
    "fr_cb_write_smem": "i i i",
    "fr_last_error": "->s",
    "fr_head_fwht": "p l p l i i p f p i",
    "fr_cb_attn_noalloc": "p l p p i p i i i i i f i p l p p p l l p i i",
})
EXPORTS = NATIVE.exports


def lib():
    """the ctypes handle (the library is built first when it is missing or older than its sources)"""
    return NATIVE.dll


_SIGN_TABLE = (ctypes.c_uint * (len(SEEDS) * 4))()


def sign_words():
    """The sign-table argument (uint32 [15 * 4]) of the codebook entry points.  Only codebook kinds that this build
    does not have read it; the key-only kinds get zeros, so that the reference's signatures stay as they are."""
    return _SIGN_TABLE


# ------------------------------------------------------------------------------------------------ shapes / variants
def qtile(G: int, Dh: int = 128) -> int:
    """query heads one decode workgroup serves: 8 for GQA groups of 5 .. 8 at head dim 128, else 4"""
    return 8 if (Dh == 128 and 4 < G <= 8) else 4


def v2_variant(fmt: str, G: int = 4, Dh: int = 128) -> int:
    """the `variant` argument of fr_v2_attn: 264 = the GQA-4, head-128 kernels of the static formats; every other shape
    (and every key-only kind) adds GEN, plus GT8 for 8-head tiles and HD256 for head dim 256"""
    if (G, Dh) == (4, 128) and fmt not in K2:
        return 264
    bits = GEN
    if qtile(G, Dh) == 8:
        bits |= GT8
    if Dh == 256:
        bits |= HD256
    return 264 | bits


def tile_of(variant: int) -> int:
    """query heads per partial slot of a variant"""
    return 8 if variant & GEN and variant & GT8 else 4


def vheads(Hkv: int, G: int, Dh: int = 128, fmt: str = "int4") -> int:
    """workgroups per (sequence, split): one per (KV head, tile of query heads)"""
    tile = tile_of(v2_variant(fmt, G, Dh))
    return Hkv * ((G + tile - 1) // tile)


def _token_bytes(fmt: str) -> int:
    return 80 if fmt in INT2_FMTS else 144                    # codes + scale words of K and V of one 128-d token


def v2_chunk_bytes(page: int, Dh: int = 128, fmt: str = "int4") -> int:
    return page * _token_bytes(fmt) * Dh // 128


def cb_chunk_bytes(kind: str, page: int, Dh: int = 128) -> int:
    return page * _token_bytes(kind) * Dh // 128


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
    ncu = max(1, slots // 4) if ncu is None else ncu          # 0: no large workgroups

    def plan(ns):
        ns = max(1, min(MAX_SPLITS, ns, math.ceil(Lmax / gran)))
        ns = max(ns, math.ceil(Lmax / MAX_CHUNK))
        chunk = min(MAX_CHUNK, math.ceil(Lmax / ns / gran) * gran)
        return math.ceil(Lmax / chunk), chunk

    if nsplit is not None:
        return plan(nsplit)
    pairs = B * HV
    # short contexts on few pairs: large workgroups, one up to 1024 tokens, splits of 512 tokens up to 4096 tokens where
    # they fit the CUs once (these launches are chains of latencies: one sequence of 2048 tokens 4 x 512 11.9 us, 6 x 384
    # in workgroups of 4 wavefronts 15.0; of 4096 tokens 8 x 512 12.5 us, 4 x 1024 13.4; the library runs plans of
    # short splits as large workgroups whoever made them)
    if ncu and 512 <= Lmax <= 4 * BIG_CHUNK:
        ns = 1 if Lmax <= 2 * 512 else math.ceil(Lmax / 512)
        if pairs * ns <= ncu:
            return plan(ns)
    if pairs <= ncu and Lmax >= BIG_CHUNK:          # as many large workgroups as keep >= 1024 tokens each (measured best
        ns, chunk = plan(min(ncu // pairs, Lmax // BIG_CHUNK))     # even when they fill only part of the CUs)
        if chunk >= BIG_CHUNK and 24 <= pairs * ns <= ncu:
            return ns, chunk
    # small workgroups: one round at most; a short job is a trade of pages per wavefront against partials to merge
    quads = math.ceil(Lmax / 64)
    return plan(min(max(1, slots // pairs), max(1, quads // 4), max(1, round(math.sqrt(quads)))))


def plan_v2(B, Lmax, Hkv, page, nsplit=None, fmt="int4", G=4, Dh=128):
    """(nsplit, chunk) of a static-format decode: a workgroup per (KV head, tile of 4 -- or, for GQA groups of 5 .. 8
    heads at head dim 128, of 8 -- query heads)"""
    tile = qtile(G, Dh)
    tiles = Hkv * ((G + tile - 1) // tile)
    slots = _slots(fmt)
    if Dh == 256:      # workgroups of 4 wavefronts only, two resident per CU (256 registers): one round of them
        return plan_splits(B, Lmax, tiles, page, slots // 2, nsplit, ncu=0)
    if tile == 8:      # tiles of 8 heads: three small workgroups resident per CU (two for the sign-magnitude INT4 format)
        slots = slots * (2 if fmt == "int4" else 3) // 4
    return plan_splits(B, Lmax, tiles, page, slots, nsplit, ncu=_NUM_CU)


def plan_cb(B, Lmax, Hkv, page, kind, nsplit=None, G=4, Dh=128):
    """(nsplit, chunk) of a key-only-kind decode (shapes other than GQA 4 / head 128 run the general kernels)"""
    if kind in K2 and (G, Dh) != (4, 128):
        return plan_v2(B, Lmax, Hkv, page, nsplit, fmt=kind, G=G, Dh=Dh)
    return plan_splits(B, Lmax, Hkv, page, _slots(kind), nsplit, ncu=_NUM_CU)


class Workspace:
    """Device memory of the split-K decode: unnormalised partial outputs and (maximum, sum) pairs for `parts`
    (sequence, KV head or head tile, split) workgroups of GT query heads x Dh channels, and one arrival counter per
    (sequence, KV head or head tile) that the kernels leave at zero.  Create it before capturing a graph."""

    def __init__(self, rows: int, Hkv: int, parts: int, device, GT: int = 4, Dh: int = 128):
        self.rows, self.parts, self.HV, self.GT, self.Dh = rows, parts, Hkv, GT, Dh
        fp32 = dict(dtype=torch.float32, device=device)
        self.opart = torch.empty(parts * GT * Dh, **fp32)
        self.mlpart = torch.empty(parts * GT * 2, **fp32)
        self.counter = torch.zeros(rows * Hkv, dtype=torch.int32, device=device)

    def fits(self, B, Hkv, nsplit_total, GT=4, Dh=128):
        """whether a launch of B sequences x Hkv (head, tile) pairs x nsplit_total splits has room"""
        need = B * Hkv * nsplit_total
        return (B <= self.rows and Hkv <= self.HV and need <= self.parts and GT * Dh <= self.GT * self.Dh
                and need * GT * Dh <= self.parts * self.GT * self.Dh)


# ------------------------------------------------------------------------------------------------ launches
def _centre(kmu, kv):
    """the optional per-(KV head, channel) key centring vector, checked against the rows it will be subtracted from"""
    if kmu is not None:
        want = (kv.shape[1] // 2, kv.shape[2])
        assert kmu.dtype == torch.float32 and kmu.device == kv.device and kmu.is_contiguous(), "kmu: fp32, contiguous, on the rows' device"
        assert tuple(kmu.shape) == want, (tuple(kmu.shape), want)
    return kmu


def _loadable(kv):
    """the writers read four bf16 at a time: heads and channels of a row must be dense, rows 8-byte aligned"""
    dense = kv.stride(2) == 1 and kv.stride(1) == kv.shape[2]
    aligned = kv.stride(0) % 4 == 0 and kv.data_ptr() % 8 == 0
    return kv if dense and aligned else kv.contiguous()


def _new_rows(kv, slots):
    """common checks of the writers' inputs: bf16 rows [T, 2 Hkv, Dh] and int64 slots; returns (rows to read, Hkv, Dh)"""
    assert kv.dtype == torch.bfloat16 and slots.dtype == torch.int64
    return _loadable(kv), kv.shape[1] // 2, kv.shape[2]


def v2_write(kv, slots, mask, rb, pool, page, fmt="int4", kmu=None):
    """Static formats ("int4" | "int4a" | "int2a"): quantise the rows kv bf16 [T, 2 Hkv, Dh] (K heads, then V heads;
    Dh 128 or 256) into pool uint8 [pages, Hkv, chunk bytes] at the page slots `slots` int64 [T] (negative: skip).
    mask uint8 [2 Hkv, Dh / rb] marks the rb-channel groups stored Hadamard-rotated."""
    if kv.shape[0] == 0:
        return
    rows, Hkv, Dh = _new_rows(kv, slots)
    NATIVE.run("fr_v2_write", V2_FMT[fmt], rows, rows.stride(0), slots, rows.shape[0], Hkv, page, mask, rb, pool,
               current_stream(), Dh, _centre(kmu, rows))


class _Bound:
    """A decode launch with every argument already marshalled: calling it launches again with the very same pointers
    (what a captured graph would replay), so the tensors have to stay alive and in place."""

    def __init__(self, entry: str, args: tuple):
        self.entry, self.args = entry, args
        self.fn = getattr(NATIVE.dll, entry)

    def __call__(self):
        if self.fn(*self.args):
            raise RuntimeError(f"{self.entry}: launch failed ({NATIVE.last_error()})")


def _decode(entry: str, args: tuple, bound: bool):
    if bound:
        return _Bound(entry, tuple(map(as_arg, args)))
    NATIVE.run(entry, *args)
    return None


def _tail_args(tail, tail_len, tail_idx, tail_bs, tail_ts):
    """(rows, lengths, block per sequence, block stride, row stride) of the BF16 window; strides are 0 without one"""
    if tail is None:
        return None, tail_len, tail_idx, 0, 0
    return tail, tail_len, tail_idx, tail_bs, tail_ts


def v2_attn(q, pool, block_table, seq_lens, out, nsplit, chunk, ws, qscale, kmask=None, vmask=None, rb=32,
            tail=None, tail_len=None, tail_idx=None, tail_bs=None, tail_ts=None, page=16, fmt="int4", kv_start=0,
            bound=False):
    """Paged decode attention of B one-token queries: q bf16 [B, G Hkv, Dh] -> out bf16 [B, G Hkv Dh] (any row stride).
    block_table int32 [B, pages] (row stride 0 shares one row) and seq_lens int32 [B] describe the cached tokens, of
    which [0, kv_start) are skipped; the newest tokens may sit in BF16 rows `tail` (block / row strides tail_bs /
    tail_ts in elements, tail_len int32 [B] rows used, tail_idx int32 [B] the block of each sequence).  qscale = softmax
    scale x log2 e; (nsplit, chunk) from plan_v2 / plan_cb; ws a Workspace.  kmask / vmask uint8 [Hkv, Dh / rb] tell the
    static formats which groups are stored rotated.  bound: return a callable that repeats the launch."""
    B, Hq, Dh = q.shape
    Hkv = pool.shape[1]
    G = Hq // Hkv
    assert G * Hkv == Hq and q.stride(2) == 1 and q.stride(1) == Dh and out.stride(1) == 1
    # (a pool of pages of another size read with this `page` sends the kernel past the ends of the block-table rows)
    assert pool.shape[-1] == v2_chunk_bytes(page, Dh, fmt), \
        f"the pool's chunks hold {pool.shape[-1]} bytes: not pages of {page} tokens of format {fmt} at head dim {Dh}"
    variant = v2_variant(fmt, G, Dh)
    splits = nsplit + (tail is not None)
    assert ws.fits(B, vheads(Hkv, G, Dh, fmt), splits, tile_of(variant), Dh), "split-K workspace too small"
    args = (V2_FMT[fmt], q, q.stride(0), pool, block_table, block_table.stride(0), seq_lens, B, Hkv, page, nsplit, chunk,
            qscale, kmask, vmask, rb, kmask is not None, vmask is not None, variant, STAGES, ws.opart, ws.mlpart,
            ws.counter, out, out.stride(0), *_tail_args(tail, tail_len, tail_idx, tail_bs, tail_ts), current_stream(), G,
            int(kv_start))
    return _decode("fr_v2_attn", args, bound)


def cb_write(kv, slots, CT, co, kind, pool, page, tg=None, kmu=None):
    """Key-only kinds: choose per token and KV head between the stored bases (as is / H32 per group / whole-head
    Hadamard), quantise and pack.  kv bf16 [T, 2 Hkv, 128] at slots int64 [T]; the choice minimises the key error as
    seen through CT fp32 [Hkv, 128, 128] (the transposed query covariance factor) and the value error weighted by co
    fp32 [Hkv, 128].  tg: token-group size hint of the reference's launch (1 | 2 | 4), chosen from T when None."""
    if kv.shape[0] == 0:
        return
    rows, Hkv, Dh = _new_rows(kv, slots)
    T = rows.shape[0]
    if tg is None:
        tg = 1 if T <= 16 else 4 if (T > 64 and kind in K2) else 2
    NATIVE.run("fr_cb_write", rows, rows.stride(0), slots, 0, T, Hkv, page, tg, CT, co, sign_words(), CB_KINDS[kind], pool,
               current_stream(), Dh, _centre(kmu, rows))


_SECOND: dict = {}


def side_stream(device=None):
    """the stream the value pass of the two-pass writer runs on: one per device, ordinary priority; ask for it before
    capturing a graph"""
    where = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    if where not in _SECOND:
        _SECOND[where] = torch.cuda.Stream(where)
    return _SECOND[where]


def w3_nchunk(Hkv, per_cu):
    """token chunks per KV head that give `per_cu` workgroups per CU"""
    _slots(None)
    return max(1, per_cu * _NUM_CU // Hkv)


def w3_calib(Cq, kappa=None, nd=8):
    """The reference's third writer screens candidates with tensor-core products and wants constants for that (C1 fp16
    [H, 168, 128], aux fp32 [H, 48]).  This build evaluates the selection criterion itself in fp32 and never reads
    them: zeros of those shapes are returned so that calling code needs no change."""
    heads = Cq.shape[0]
    return Cq.new_zeros((heads, 168, 128), dtype=torch.float16), Cq.new_zeros((heads, 48), dtype=torch.float32)


def cb_write3(kv, slots, CT, co, C1, beta, kind, pool, page, split=None, kmu=None):
    """Writes the same pool bytes as cb_write.  split (default: up to W3_SPLIT_T tokens): the key pass launches on the
    current stream and the value pass on side_stream(), forked and joined by stream waits, which a graph capture
    records; otherwise one launch does both."""
    if kv.shape[0] == 0:
        return
    assert kv.shape[2] == D, f"writer v3: head dim {D} only (got {kv.shape[2]}; use cb_write)"
    rows, Hkv, _ = _new_rows(kv, slots)
    T = rows.shape[0]
    common = (rows, rows.stride(0), slots.contiguous(), 0, T, Hkv, page, CT, co, C1, beta, sign_words(), CB_KINDS[kind],
              pool)
    key_chunks, value_chunks = w3_nchunk(Hkv, 2), w3_nchunk(Hkv, 3)
    centre = _centre(kmu, rows)
    if split is None:
        split = T <= W3_SPLIT_T
    if not split:
        NATIVE.run("fr_cb_write3", *common, key_chunks, value_chunks, current_stream(), centre)
        return
    main, other = torch.cuda.current_stream(), side_stream(rows.device)
    other.wait_stream(main)
    NATIVE.run("fr_cb_write3", *common, key_chunks, -1, main.cuda_stream, centre)           # keys
    NATIVE.run("fr_cb_write3", *common, -1, value_chunks, other.cuda_stream, None)          # values
    main.wait_stream(other)


def w3_static_write(kv, slots, mask, hfull, pool, page, fmt="int4", path=0, kmu=None):
    """One launch for head_fwht(kv, hfull, 1 / 16) followed by v2_write(.., mask, rb = 32, ..): same pool bytes."""
    if kv.shape[0] == 0:
        return
    assert kv.shape[2] == D, f"writer v3: head dim {D} only (got {kv.shape[2]}; use v2_write)"
    rows, Hkv, _ = _new_rows(kv, slots)
    NATIVE.run("fr_w3_static_write", rows, rows.stride(0), slots.contiguous(), rows.shape[0], Hkv, page, mask, hfull,
               ("int4", "int4a", "int2a").index(fmt), pool, path, current_stream(), _centre(kmu, rows))


def cb_attn(q, pool, block_table, seq_lens, out, nsplit, chunk, ws, qscale, kind, tail=None, tail_len=None,
            tail_idx=None, tail_bs=None, tail_ts=None, page=16, kv_start=0, bound=False):
    """v2_attn for the key-only kinds (arguments as there).  GQA 4 at head dim 128 has its own kernels; other shapes
    go through the general ones."""
    B, Hq, Dh = q.shape
    Hkv = pool.shape[1]
    if kind in K2 and (Hq, Dh) != (4 * Hkv, 128):
        return v2_attn(q, pool, block_table, seq_lens, out, nsplit, chunk, ws, qscale, tail=tail, tail_len=tail_len,
                       tail_idx=tail_idx, tail_bs=tail_bs, tail_ts=tail_ts, page=page, fmt=kind, kv_start=kv_start,
                       bound=bound)
    assert (Hq, Dh) == (4 * Hkv, D), f"codebook {kind}: GQA 4, head dim 128 only"
    assert q.stride(2) == 1 and q.stride(1) == D and out.stride(1) == 1
    assert pool.shape[-1] == cb_chunk_bytes(kind, page), \
        f"the pool's chunks hold {pool.shape[-1]} bytes: not pages of {page} tokens of kind {kind}"
    assert ws.fits(B, Hkv, nsplit + (tail is not None)), "split-K workspace too small"
    args = (q, q.stride(0), pool, block_table, block_table.stride(0), seq_lens, B, Hkv, page, nsplit, chunk, qscale,
            sign_words(), CB_KINDS[kind], 0, STAGES, ws.opart, ws.mlpart, ws.counter, out, out.stride(0),
            *_tail_args(tail, tail_len, tail_idx, tail_bs, tail_ts), current_stream(), int(kv_start))
    return _decode("fr_cb_attn", args, bound)


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
    assert pool.shape[-1] == cb_chunk_bytes(kind, page), \
        f"the pool's chunks hold {pool.shape[-1]} bytes: not pages of {page} tokens of kind {kind}"
    args = (q, q.stride(0), pool, block_table, block_table.stride(0), seq_lens, B, Hkv, page, nsplit, chunk, qscale,
            CB_KINDS[kind], out, out.stride(0), *_tail_args(tail, tail_len, tail_idx, tail_bs, tail_ts), current_stream(),
            G, int(kv_start))
    return _decode("fr_cb_attn_noalloc", args, bound)


def head_fwht(x, flags, scale, out=None):
    """scale x H x per head of x bf16 [T, H, Dh] (Dh 128 or 256; H the +-1 Sylvester matrix, not normalised) where
    flags[h] is set, a plain copy of the head where it is not.  out may be x itself."""
    T, H, Dh = x.shape
    dense = lambda t: t.stride(2) == 1 and t.stride(1) == Dh            # noqa: E731
    assert x.dtype == torch.bfloat16 and dense(x)
    if out is None:
        out = torch.empty_like(x, memory_format=torch.contiguous_format)
    assert dense(out)
    if T:
        NATIVE.run("fr_head_fwht", x, x.stride(0), out, out.stride(0), T, H, flags, scale, current_stream(), Dh)
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
