"""Host side of a decode step, as the serving plugin drives the libraries: split plans per batch bucket, the shared
split-K workspace, the BF16 sink / window ring bookkeeping, and the write -> attend call sequence of one attention layer.

It mirrors, without vLLM, the decode-row part of the reference's attention backend
(integrations/vllm_flagrot/vllm_flagrot/attention/backend.py): `plan_bucket` (:638-644), `tile_layout` (:657-662),
`decode_plan` (:665-676), `decode_workspace` / `kivi_workspace` (:684-711), `FlagRotMetadataBuilder.build` and
`_kivi_decode_groups` (:564-636), `_write` (:1234-1248), the decode rows of `_kv_cache_update` / `_kivi_update`
(:1266-1325) and `_decode` (:1513-1547).  Everything the builder
touches per step is a persistent device buffer written in place, so that a captured graph of `DecodeLayer.step` can be
replayed with new lengths, slots and ring positions.  Kinds: the key-only 2x2 codebooks (konly, konlya, konlya2) and the
static formats (int4, int4a, int2a) through `DecodeLayer`, the KIVI-style pages ("kivi2") through `KiviDecodeLayer`;
the transform-before-write variants of the reference are out of scope here.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np
import torch

from . import kernels as K
from . import kivi as KIVI

PAGE = 16
D = 128
LOG2E = 1.4426950408889634
STATIC_KINDS = ("int4", "int4a", "int2a")


def is_static(kind: str) -> bool:
    return kind in STATIC_KINDS


def plan_bucket(B: int) -> int:
    """decode batch size a split plan is made for: 1, 2, 4, then multiples of 8 up to 256, of 16 beyond (the graph
    capture sizes), so that a padded graph batch and the same batch run eagerly sum in the same order."""
    if B <= 4:
        return 1 << (B - 1).bit_length()
    return -(-B // 8) * 8 if B <= 256 else -(-B // 16) * 16


def tile_layout(kind: str, Hkv: int, G: int, Dh: int = D):
    """(workgroups per (row, split), q heads per partial slot, head dim) of the decode kernel of `kind`."""
    if is_static(kind) or (kind in K.K2 and (G != 4 or Dh != D)):
        return K.vheads(Hkv, G, Dh, kind), K.tile_of(K.v2_variant(kind, G, Dh)), Dh
    return Hkv, 4, D


def decode_plan(kind: str, B: int, max_len: int, Hkv: int, G: int = 4, Dh: int = D):
    """(nsplit, chunk) of a decode batch of B rows: fixed per (batch bucket, longest context), no device sync."""
    Bp = plan_bucket(B)
    if kind == "kivi2":
        return KIVI.plan(Bp, max_len, Hkv, D=Dh)
    if is_static(kind):
        return K.plan_v2(Bp, max_len, Hkv, PAGE, fmt=kind, G=G, Dh=Dh)
    return K.plan_cb(Bp, max_len, Hkv, PAGE, kind, G=G, Dh=Dh)


_WS: dict = {}


def decode_workspace(device, layout, rows: int, plan_fn):
    """one split-K workspace per device and tile layout, sized once for every decode batch size <= rows (graphs bake
    the pointers in; layers run one after the other and share it)."""
    HV, GT, Dh = layout
    key = (str(device), HV, GT, Dh)
    ws = _WS.get(key)
    if ws is None or ws.rows < rows:
        parts = max(plan_bucket(B) * HV * (plan_fn(B)[0] + 1) for B in range(1, rows + 1))
        ws = _WS[key] = K.Workspace(rows, HV, parts, device, GT, Dh)
    return ws


_KWS: dict = {}


def kivi_workspace(device, rows: int, Hkv: int, G: int, Dh: int, plan_fn):
    """KIVI split-K workspace, sized once for every decode batch size <= rows"""
    key = (str(device), Hkv, G, Dh)
    parts = max(plan_bucket(B) * Hkv * (plan_fn(B)[0] + 1) for B in range(1, rows + 1))
    ws = _KWS.get(key)
    if ws is None or ws.parts < parts:
        ws = _KWS[key] = KIVI.Workspace(parts, G, Dh, device)
    return ws


def ring_slot(p, S: int, W: int):
    """BF16 slot of position p inside a request's row of S sink slots followed by a W-slot window ring, or -1 when the
    position keeps no BF16 copy (W = 0 and p >= S).  p: int or integer tensor."""
    if isinstance(p, torch.Tensor):
        if W > 0:
            return torch.where(p < S, p, S + torch.remainder(p - S, W))
        return torch.where(p < S, p, torch.full_like(p, -1))
    if p < S:
        return p
    return S + (p - S) % W if W > 0 else -1


@dataclass
class DecodeMetadata:
    seq_lens: torch.Tensor                   # [n] int32 context lengths including the step's token
    block_table: torch.Tensor                # [n, max_blocks] int32
    slot_mapping: torch.Tensor               # [n] int64 page slots of the step's tokens (< 0: padding row)
    num_decodes: int
    nsplit: int = 1
    chunk: int = 64
    dec_cached: torch.Tensor | None = None   # int32 page tokens read: [0, L - W) with [0, S) masked; 0 if L - W <= S
    dec_tail_len: torch.Tensor | None = None  # int32 BF16 slots read: min(L, S + W)
    dec_tail_idx: torch.Tensor | None = None  # int32 ring row (request slot; R = the padding row)
    dec_ring_pos: torch.Tensor | None = None  # int64 flat BF16 slot of the new token (row * (S + W) + slot)
    kivi_sidx: torch.Tensor | None = None    # kivi2: [nd, 32] int64 ring rows of the key group the step completes
    kivi_dslot: torch.Tensor | None = None   # (-1: sinks) and its page slots ([:, 0] < 0: no group completes)


class MetadataBuilder:
    """per-step bookkeeping of the decode rows (every row has one query token)."""

    def __init__(self, kind: str, Hkv: int, G: int, max_len: int, max_rows: int, ring_rows: int, sink: int, window: int,
                 device, Dh: int = D, plan_fn=None):
        self.kind, self.Hkv, self.G, self.Dh = kind, Hkv, G, Dh
        self._plan_fn = plan_fn          # B -> (nsplit, chunk); default: the library's planner (needs the GPU)
        self.max_len, self.max_rows, self.R, self.S, self.W = max_len, max_rows, ring_rows, sink, window
        i32 = dict(dtype=torch.int32, device=device)
        self._cached = torch.zeros(max_rows, **i32)
        self._tail_len = torch.zeros(max_rows, **i32)
        self._tail_idx = torch.full((max_rows,), ring_rows, **i32)
        self._ring_pos = torch.zeros(max_rows, dtype=torch.int64, device=device)
        self._plans: dict = {}
        if kind == "kivi2":
            self._ksidx = torch.full((max_rows, 32), -1, dtype=torch.int64, device=device)
            self._kdslot = torch.full((max_rows, 32), -1, dtype=torch.int64, device=device)
            self._k32 = torch.arange(32, dtype=torch.int64, device=device)

    def plan(self, B: int):
        if B not in self._plans:
            self._plans[B] = (self._plan_fn(B) if self._plan_fn is not None else
                              decode_plan(self.kind, B, self.max_len, self.Hkv, self.G, self.Dh))
        return self._plans[B]

    def build(self, seq_lens, block_table, slot_mapping, req_idx=None) -> DecodeMetadata:
        """seq_lens [n] int32 (device); req_idx: host array of request slots of the first rows (rows beyond it, and
        dummy runs without it, are padding: they read and write the extra ring row R)."""
        nd = int(seq_lens.shape[0])
        md = DecodeMetadata(seq_lens=seq_lens, block_table=block_table, slot_mapping=slot_mapping, num_decodes=nd)
        if nd == 0:
            return md
        md.nsplit, md.chunk = self.plan(nd)
        L = seq_lens
        S, W = self.S, self.W
        if S == 0 and W == 0:
            md.dec_cached = L
            return md
        T = S + W
        self._tail_idx[:nd].fill_(self.R)
        if req_idx is not None:
            k = min(len(req_idx), nd)
            self._tail_idx[:k].copy_(torch.from_numpy(np.ascontiguousarray(np.asarray(req_idx)[:k], dtype=np.int32)),
                                     non_blocking=True)
        # the pages hold every position; the kernel reads [S, L - W) of them and the BF16 slots [0, min(L, T)) =
        # the sinks [0, min(L, S)) and the window [max(S, L - W), L)
        torch.where(L - W > S, L - W, torch.zeros_like(L), out=self._cached[:nd])
        torch.clamp(L, max=T, out=self._tail_len[:nd])
        p = L.long() - 1                                                     # the new token
        row = self._tail_idx[:nd].long() * T
        slot = ring_slot(p, S, W)
        torch.where(slot >= 0, row + slot, torch.full_like(p, self.R * T), out=self._ring_pos[:nd])
        md.dec_cached, md.dec_tail_len = self._cached[:nd], self._tail_len[:nd]
        md.dec_tail_idx, md.dec_ring_pos = self._tail_idx[:nd], self._ring_pos[:nd]
        if self.kind == "kivi2":
            self._kivi_decode_groups(md, L, block_table[:nd], nd)
        return md

    def _kivi_decode_groups(self, md, L, bt, nd):
        """kivi2: the key group [32 g, 32 g + 32) a decode step completes (new token p = L - 1 = 32 g + 31) is encoded
        from the BF16 ring in the same step (device operations on persistent buffers)"""
        S, W, T = self.S, self.W, self.S + self.W
        Ll = L.long()
        act = (Ll % 32 == 0) & (Ll >= 32) & (self._tail_idx[:nd] < self.R)
        pos = ((Ll - 1) // 32 * 32)[:, None] + self._k32[None]                          # [nd, 32]
        row = self._tail_idx[:nd].long()[:, None] * T
        slot = ring_slot(pos, S, W)
        torch.where((pos < S) | ~act[:, None], torch.full_like(pos, -1), row + slot, out=self._ksidx[:nd])
        pg = torch.clamp(pos // PAGE, min=0, max=bt.shape[1] - 1)
        ds = bt.gather(1, pg).long() * PAGE + pos % PAGE
        torch.where(act[:, None], ds, torch.full_like(ds, -1), out=self._kdslot[:nd])
        md.kivi_sidx, md.kivi_dslot = self._ksidx[:nd], self._kdslot[:nd]


class DecodeLayer:
    """cache state and call sequence of one attention layer: pages + BF16 ring, writer then decode."""

    def __init__(self, kind: str, Hkv: int, G: int, pool: torch.Tensor, builder: MetadataBuilder, scale: float = None,
                 CT=None, co=None, wmask=None, kmu=None):
        self.kind, self.Hkv, self.G = kind, Hkv, G
        self.static = is_static(kind)
        self.pool = pool                                   # uint8 [num_pages, Hkv, chunk bytes]
        self.b = builder
        self.S, self.W, self.T, self.R = builder.S, builder.W, builder.S + builder.W, builder.R
        self.qscale = (scale if scale is not None else 1.0 / math.sqrt(D)) * LOG2E
        self.CT, self.co, self.wmask, self.kmu = CT, co, wmask, kmu
        if self.static:
            if wmask is None:
                raise ValueError("static formats need the [2 Hkv, 4] rotation mask")
        elif CT is None or co is None:
            raise ValueError("codebook kinds need the calibration (CT, co)")
        dev = pool.device
        self.layout = tile_layout(kind, Hkv, G)
        self.kmask = wmask[:Hkv].contiguous() if self.static else None
        self.vmask = wmask[Hkv:].contiguous() if self.static else None
        self.ring = torch.zeros(self.R + 1, max(self.T, 1), 2 * Hkv, D, dtype=torch.bfloat16, device=dev) if self.T else None
        self.ws = decode_workspace(dev, self.layout, builder.max_rows, builder.plan)

    # -- the BF16 slots hold bf16(k - mu) (fp32 subtraction), V rows unchanged
    def center_rows(self, kv):
        if self.kmu is None:
            return kv
        H = self.Hkv
        return torch.cat([(kv[:, :H].float() - self.kmu).to(torch.bfloat16), kv[:, H:]], 1)

    def write_pages(self, kv, slots):
        """kv bf16 [n, 2 Hkv, 128] -> pages at slots (< 0 skipped); the kernels subtract kmu from the K rows"""
        if self.static:
            K.v2_write(kv, slots, self.wmask, 32, self.pool, PAGE, fmt=self.kind, kmu=self.kmu)
        else:
            # same bytes either way; fr_cb_write3 runs the screened kernel on prompt-sized launches
            if kv.shape[0] * self.Hkv > 1024:
                K.cb_write3(kv, slots, self.CT, self.co, None, None, self.kind, self.pool, PAGE, split=False, kmu=self.kmu)
            else:
                K.cb_write(kv, slots, self.CT, self.co, self.kind, self.pool, PAGE, kmu=self.kmu)

    def prefill(self, kv, slots, req: int):
        """a prompt of n tokens of request slot `req`: every token to its page, sinks and the newest W tokens also to
        the request's BF16 row"""
        self.write_pages(kv, slots)
        if self.T:
            n = kv.shape[0]
            pos = torch.arange(n, device=kv.device)
            keep = (pos < self.S) | (pos >= n - self.W) if self.W > 0 else pos < self.S
            sl = ring_slot(pos[keep], self.S, self.W)
            self.ring[req].index_copy_(0, sl, self.center_rows(kv[keep]))

    def update(self, kv, md: DecodeMetadata):
        """cache update of a decode step: the new tokens to their pages and to their BF16 slots"""
        self.write_pages(kv, md.slot_mapping)
        if self.T:
            self.ring.view(-1, 2 * self.Hkv, D).index_copy_(0, md.dec_ring_pos, self.center_rows(kv))

    def decode(self, q, md: DecodeMetadata, out):
        nd = q.shape[0]
        tkw = {}
        if self.T:
            r = self.ring
            tkw = dict(tail=r, tail_len=md.dec_tail_len, tail_idx=md.dec_tail_idx, tail_bs=r.stride(0),
                       tail_ts=r.stride(1), kv_start=self.S)        # the sinks are in the pages too, read in BF16
        if q.stride(1) != D or q.stride(2) != 1:
            q = q.contiguous()
        if self.static:
            K.v2_attn(q, self.pool, md.block_table[:nd], md.dec_cached, out, md.nsplit, md.chunk, self.ws, self.qscale,
                      kmask=self.kmask, vmask=self.vmask, rb=32, fmt=self.kind, **tkw)
        else:
            K.cb_attn(q, self.pool, md.block_table[:nd], md.dec_cached, out, md.nsplit, md.chunk, self.ws, self.qscale,
                      self.kind, **tkw)

    def step(self, q, kv, md: DecodeMetadata, out):
        """what a captured decode step of this layer contains"""
        self.update(kv, md)
        self.decode(q, md, out)


class KiviDecodeLayer:
    """KIVI-style pages: values written per token, key groups of 32 tokens encoded when they complete (from the prompt
    rows at prefill, from the BF16 ring at decode: the window must hold a whole group, W >= 32)."""

    def __init__(self, Hkv: int, G: int, pool: torch.Tensor, builder: MetadataBuilder, qs, lz, co, scale: float = None,
                 f8: bool = False):
        """f8: FP8-meta pages (the reference's `kivi_f8` option, attention/backend.py:365-366): pool chunks of
        KIVI.chunk_bytes(D, True) bytes."""
        assert builder.kind == "kivi2" and builder.W >= 32, "kivi2 needs a BF16 window of at least one key group"
        assert pool.shape[-1] == KIVI.chunk_bytes(D, f8), "pool chunk size does not match the page format"
        self.Hkv, self.G, self.pool, self.b, self.f8 = Hkv, G, pool, builder, f8
        self.S, self.W, self.T, self.R = builder.S, builder.W, builder.S + builder.W, builder.R
        self.scale = scale if scale is not None else 1.0 / math.sqrt(D)
        self.qs, self.lz, self.co = qs, lz, co             # calibration queries, their log normalisers, value weights
        dev = pool.device
        self.ring = torch.zeros((self.R + 1) * self.T, 2 * Hkv, D, dtype=torch.bfloat16, device=dev)
        self.ws = kivi_workspace(dev, builder.max_rows, Hkv, G, D, builder.plan)

    def prefill(self, kv, slots, req: int):
        """a fresh prompt of n tokens: values of every token, the whole key groups, sinks and newest W rows in BF16"""
        n = kv.shape[0]
        dev = kv.device
        KIVI.v_write(kv, slots, self.co, None, self.pool, self.Hkv, D, f8=self.f8)
        pos = torch.arange(n, device=dev)
        keep = (pos < self.S) | (pos >= n - self.W)
        self.ring.view(self.R + 1, self.T, 2 * self.Hkv, D)[req].index_copy_(0, ring_slot(pos[keep], self.S, self.W), kv[keep])
        ng = n // 32
        if ng:
            gp = pos[:32 * ng].view(ng, 32)
            sidx = torch.where(gp < self.S, torch.full_like(gp, -1), gp).contiguous()
            KIVI.k_encode(kv, sidx, slots[:32 * ng].view(ng, 32).contiguous(), self.qs, self.lz, self.scale, self.pool,
                          self.Hkv, D, f8=self.f8)

    def update(self, kv, md: DecodeMetadata):
        KIVI.v_write(kv, md.slot_mapping, self.co, None, self.pool, self.Hkv, D, f8=self.f8)
        self.ring.index_copy_(0, md.dec_ring_pos, kv)
        KIVI.k_encode(self.ring, md.kivi_sidx, md.kivi_dslot, self.qs, self.lz, self.scale, self.pool, self.Hkv, D,
                      f8=self.f8)

    def decode(self, q, md: DecodeMetadata, out):
        nd = q.shape[0]
        if q.stride(1) != D or q.stride(2) != 1:
            q = q.contiguous()
        KIVI.attn(q, self.pool, md.block_table[:nd], md.dec_cached, out, md.nsplit, md.chunk, self.ws,
                  self.scale * LOG2E, self.S, self.G, ring=self.ring, tail_len=md.dec_tail_len,
                  tail_idx=md.dec_tail_idx, T=self.T, f8=self.f8)

    def step(self, q, kv, md: DecodeMetadata, out):
        self.update(kv, md)
        self.decode(q, md, out)
