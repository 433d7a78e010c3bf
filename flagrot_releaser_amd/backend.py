"""Host side of a decode step over the three libraries: which split plan a batch gets, where the split-K partials live,
which BF16 rows a request keeps beside its pages, and the order of calls of one attention layer (write, then attend).

This is the part of the reference's serving plugin that sits between the scheduler and the kernels
(integrations/vllm_flagrot/vllm_flagrot/attention/backend.py: metadata builder :564-636, batch buckets and workspaces
:638-711, `_write` :1234-1248, decode rows of the cache update :1266-1325, `_decode` :1513-1547), rebuilt without vLLM
around three small objects:

  RingGeometry   S sink rows + a W-row window ring of BF16 tokens per request: the slot of a position, what a sequence
                 of length L reads from pages and what from the ring.  The slot rule `p < S ? p : S + (p - S) % W` and
                 the read ranges (pages [S, L - W), ring rows [0, min(L, S + W))) are the contract with the kernels.
  StepPlanner    owns every per-step device buffer (allocated once, rewritten in place), so that a HIP graph captured
                 around `layer.step` can be replayed with new lengths, slots and ring positions.
  DecodeLayer /  pages + ring of one layer and the call sequence of a step, for FlagRot pages (key-only 2x2 kinds and
  KiviDecodeLayer static formats) and for KIVI-style pages ("kivi2": a key group is encoded from the ring by the step that
                 completes it).
The transform-before-write variants of the reference are out of scope here.
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
GROUP = 32                      # tokens per KIVI key group


def is_static(kind: str) -> bool:
    return kind in STATIC_KINDS


# ------------------------------------------------------------------------------------------------ batch buckets
def plan_bucket(B: int) -> int:
    """The batch size whose split plan a batch of B rows uses.  Plans are shared by all batches that a serving stack
    pads to one captured graph size -- 1, 2, 4, every 8th size up to 256, every 16th beyond -- because the split count
    fixes the summation order: a batch must get the same bits whether it runs padded inside a graph or on its own."""
    if B <= 1:
        return 1
    if B <= 4:
        return 2 if B == 2 else 4
    step = 8 if B <= 256 else 16
    return (B + step - 1) // step * step


def buckets_upto(rows: int):
    """the distinct bucket sizes batches of 1 .. rows map to"""
    seen, out = set(), []
    for B in range(1, rows + 1):
        b = plan_bucket(B)
        if b not in seen:
            seen.add(b)
            out.append(b)
    return out


def tile_layout(kind: str, Hkv: int, G: int, Dh: int = D):
    """(workgroups per (row, split), q heads per partial slot, head dim) of the decode kernel of `kind`."""
    generalised = is_static(kind) or G != 4 or Dh != D
    if not generalised:
        return Hkv, 4, D
    variant = K.v2_variant(kind, G, Dh)
    return K.vheads(Hkv, G, Dh, kind), K.tile_of(variant), Dh


def decode_plan(kind: str, B: int, max_len: int, Hkv: int, G: int = 4, Dh: int = D):
    """(nsplit, chunk) for a batch of B rows of at most max_len tokens; depends on the bucket only (no device sync)."""
    rows = plan_bucket(B)
    if kind == "kivi2":
        return KIVI.plan(rows, max_len, Hkv, D=Dh)
    if is_static(kind):
        return K.plan_v2(rows, max_len, Hkv, PAGE, fmt=kind, G=G, Dh=Dh)
    return K.plan_cb(rows, max_len, Hkv, PAGE, kind, G=G, Dh=Dh)


class WorkspacePool:
    """Split-K workspaces shared by the layers of a model: layers run one after the other, and captured graphs keep the
    pointers, so there is one workspace per (device, partial shape), grown only before anything was captured.  Sized
    for the largest `rows x heads x (splits + 1)` any bucket up to `rows` asks for (+ 1: the BF16 rows' partial)."""

    def __init__(self):
        self._held = {}

    @staticmethod
    def parts_needed(rows: int, heads: int, plan_fn) -> int:
        return max(b * heads * (plan_fn(b)[0] + 1) for b in buckets_upto(rows))

    def flagrot(self, device, layout, rows: int, plan_fn):
        heads, tile, Dh = layout
        key = ("fr", str(device), heads, tile, Dh)
        ws = self._held.get(key)
        if ws is None or ws.rows < rows:
            ws = self._held[key] = K.Workspace(rows, heads, self.parts_needed(rows, heads, plan_fn), device, tile, Dh)
        return ws

    def kivi(self, device, rows: int, Hkv: int, G: int, Dh: int, plan_fn):
        key = ("kv", str(device), Hkv, G, Dh)
        need = self.parts_needed(rows, Hkv, plan_fn)
        ws = self._held.get(key)
        if ws is None or ws.parts < need:
            ws = self._held[key] = KIVI.Workspace(need, G, Dh, device)
        return ws


WORKSPACES = WorkspacePool()


def decode_workspace(device, layout, rows: int, plan_fn):
    return WORKSPACES.flagrot(device, layout, rows, plan_fn)


def kivi_workspace(device, rows: int, Hkv: int, G: int, Dh: int, plan_fn):
    return WORKSPACES.kivi(device, rows, Hkv, G, Dh, plan_fn)


# ------------------------------------------------------------------------------------------------ BF16 rows
@dataclass(frozen=True)
class RingGeometry:
    """S sink slots followed by a ring of W window slots; a request's row of the ring tensor has S + W slots."""
    S: int
    W: int

    @property
    def slots(self) -> int:
        return self.S + self.W

    @property
    def active(self) -> bool:
        return self.slots > 0

    def slot(self, p):
        """slot of position p (int or integer tensor); -1 where the position keeps no BF16 copy (past the sinks of a
        ring without window)"""
        S, W = self.S, self.W
        if isinstance(p, torch.Tensor):
            beyond = S + (p - S) % W if W > 0 else torch.full_like(p, -1)
            return torch.where(p < S, p, beyond)
        if p < S:
            return p
        return S + (p - S) % W if W > 0 else -1

    def kept(self, n: int, device):
        """positions of an n-token prompt that stay in BF16 (sinks and the newest W), and their slots"""
        pos = torch.arange(n, device=device)
        keep = pos < self.S
        if self.W > 0:
            keep = keep | (pos >= n - self.W)
        pos = pos[keep]
        return keep, self.slot(pos)

    def paged_tokens(self, L, out=None):
        """tokens of a length-L sequence that decode reads from pages: [S, L - W) with the sinks masked by kv_start,
        nothing while the sequence still fits the BF16 rows"""
        body = L - self.W
        return torch.mul(body, body > self.S, out=out)

    def ring_tokens(self, L, out=None):
        """BF16 rows read for a length-L sequence: the sinks it has and its window"""
        return torch.clamp(L, max=self.slots, out=out)


def ring_slot(p, S: int, W: int):
    """BF16 slot of position p for S sinks and a W-slot window (RingGeometry.slot)"""
    return RingGeometry(S, W).slot(p)


def chunk_key_groups(geo: RingGeometry, start: int, n: int, ring_row0: int, table_row, page: int = PAGE):
    """The 32-token key groups that a prompt chunk of n tokens at positions [start, start + n) completes, as the
    (sources, page slots) pair the key group encoder takes: int64 [N, 32] each, or None when the chunk completes no
    group.  A position of such a group comes from the chunk (its row index), from the BF16 ring of the request when an
    earlier chunk brought it (encoded -2 - ring row; ring_row0 = the request's first row of the flattened ring), or is
    a sink that stays BF16 only (-1).  A group that straddles the chunk's start has at most 31 earlier positions, all
    still in a window of W >= 32 slots -- so the groups must be encoded BEFORE the chunk's own rows go into the ring.
    table_row: the request's block-table row (int tensor).  Reference: attention/backend.py:1327-1371."""
    g0, g1 = start // GROUP, (start + n) // GROUP
    if g1 <= g0:
        return None
    dev = table_row.device
    pos = torch.arange(g0 * GROUP, g1 * GROUP, device=dev).view(g1 - g0, GROUP)
    from_ring = -2 - (ring_row0 + geo.slot(pos))
    src = torch.where(pos < geo.S, torch.full_like(pos, -1), torch.where(pos >= start, pos - start, from_ring))
    dst = table_row[pos // page].long() * page + pos % page
    return src.contiguous(), dst.contiguous()


@dataclass
class StepPlan:
    """what one decode step of a batch needs on the device (views of the planner's persistent buffers)"""
    lengths: torch.Tensor                    # [n] int32 context lengths including the step's token
    block_table: torch.Tensor                # [n, max_blocks] int32
    slots: torch.Tensor                      # [n] int64 page slots of the step's tokens (< 0: padding row)
    rows: int
    nsplit: int = 1
    chunk: int = 64
    page_tokens: torch.Tensor | None = None  # [n] int32 tokens read from pages (the kernels' seq_lens)
    ring_tokens: torch.Tensor | None = None  # [n] int32 BF16 rows read
    ring_home: torch.Tensor | None = None    # [n] int32 row of the ring tensor (the request's; the spare row for padding)
    ring_dest: torch.Tensor | None = None    # [n] int64 flat ring index the step's token is copied to
    group_src: torch.Tensor | None = None    # kivi2: [n, 32] int64 flat ring rows of the key group this step completes (-1: sink)
    group_dst: torch.Tensor | None = None    # kivi2: [n, 32] int64 page slots of that group ([:, 0] < 0: none completes)


class StepPlanner:
    """per-step bookkeeping of a decode batch (one query token per row).  `ring_rows` request rows + one spare row that
    padding rows read and write."""

    def __init__(self, kind: str, Hkv: int, G: int, max_len: int, max_rows: int, ring_rows: int, sink: int, window: int,
                 device, Dh: int = D, plan_fn=None):
        self.kind, self.Hkv, self.G, self.Dh = kind, Hkv, G, Dh
        self.max_len, self.max_rows = max_len, max_rows
        self.geo = RingGeometry(sink, window)
        self.spare = ring_rows                          # index of the extra ring row
        self.S, self.W, self.R = sink, window, ring_rows
        self._plan_fn = plan_fn                         # B -> (nsplit, chunk); default: the libraries' planners (need the GPU)
        self._plan_of_bucket = {}
        self._i32 = torch.zeros(3, max_rows, dtype=torch.int32, device=device)     # page tokens | ring tokens | home
        self._i32[2].fill_(ring_rows)
        self._dest = torch.zeros(max_rows, dtype=torch.int64, device=device)
        self._group = None
        if kind == "kivi2":
            self._group = torch.full((2, max_rows, GROUP), -1, dtype=torch.int64, device=device)
            self._lane = torch.arange(GROUP, dtype=torch.int64, device=device)

    def plan(self, B: int):
        b = plan_bucket(B)
        if b not in self._plan_of_bucket:
            fn = self._plan_fn or (lambda rows: decode_plan(self.kind, rows, self.max_len, self.Hkv, self.G, self.Dh))
            self._plan_of_bucket[b] = fn(b)
        return self._plan_of_bucket[b]

    def _assign_homes(self, n: int, homes):
        home = self._i32[2, :n]
        home.fill_(self.spare)
        if homes is None:
            return home
        real = np.ascontiguousarray(np.asarray(homes)[:n], dtype=np.int32)
        if real.size:
            # asynchronous: the host must not wait for the queue once per step
            home[:real.size].copy_(torch.from_numpy(real), non_blocking=True)
        return home

    def prepare(self, lengths, block_table, slots, homes=None) -> StepPlan:
        """lengths [n] int32 on the device; homes: host array with the ring row of the leading rows (rows past it, and
        dry runs without it, are padding)."""
        n = int(lengths.shape[0])
        sp = StepPlan(lengths=lengths, block_table=block_table, slots=slots, rows=n)
        if n == 0:
            return sp
        sp.nsplit, sp.chunk = self.plan(n)
        geo = self.geo
        if not geo.active:
            sp.page_tokens = lengths
            return sp
        home = self._assign_homes(n, homes)
        sp.page_tokens = geo.paged_tokens(lengths, out=self._i32[0, :n])
        sp.ring_tokens = geo.ring_tokens(lengths, out=self._i32[1, :n])
        sp.ring_home = home
        # where the step's own token goes: its slot in the request's row, or the spare row's slot 0 if it keeps none
        newest = lengths.long() - 1
        where = geo.slot(newest)
        base = home.long() * geo.slots
        torch.where(where < 0, torch.full_like(base, self.spare * geo.slots), base + where, out=self._dest[:n])
        sp.ring_dest = self._dest[:n]
        if self._group is not None:
            self._completed_groups(sp, lengths.long(), base, block_table[:n], n)
        return sp

    def _completed_groups(self, sp: StepPlan, L, base, table, n: int):
        """kivi2: a step whose token closes a key group (L a multiple of 32) has the group's 32 rows encoded from the
        ring in the same step.  Sources are flat ring rows (-1 for sink positions, which stay BF16 only), destinations
        the page slots of the 32 positions; rows that close no group, and padding rows, get -1 throughout."""
        geo = self.geo
        closes = (L >= GROUP) & (L % GROUP == 0) & (sp.ring_home < self.spare)
        first = torch.clamp(L - GROUP, min=0)
        pos = first[:, None] + self._lane                                   # [n, 32] positions of the group
        src = base[:, None] + geo.slot(pos)
        src = torch.where(pos < geo.S, torch.full_like(src, -1), src)
        page = torch.clamp(torch.div(pos, PAGE, rounding_mode="floor"), max=table.shape[1] - 1)
        dst = table.gather(1, page).long() * PAGE + pos % PAGE
        off = ~closes[:, None]
        self._group[0, :n] = torch.where(off, torch.full_like(src, -1), src)
        self._group[1, :n] = torch.where(off, torch.full_like(dst, -1), dst)
        sp.group_src, sp.group_dst = self._group[0, :n], self._group[1, :n]


class DecodeLayer:
    """cache state and call sequence of one attention layer over FlagRot pages: pages + BF16 ring, writer then decode."""

    def __init__(self, kind: str, Hkv: int, G: int, pool: torch.Tensor, planner: StepPlanner, scale: float = None,
                 CT=None, co=None, wmask=None, kmu=None):
        self.kind, self.Hkv, self.G = kind, Hkv, G
        self.static = is_static(kind)
        if self.static and wmask is None:
            raise ValueError("static formats need the [2 Hkv, 4] rotation mask")
        if not self.static and (CT is None or co is None):
            raise ValueError("codebook kinds need the calibration (CT, co)")
        self.pool = pool                                   # uint8 [num_pages, Hkv, chunk bytes]
        self.planner = planner
        self.geo = planner.geo
        self.qscale = (scale if scale is not None else 1.0 / math.sqrt(D)) * LOG2E
        self.CT, self.co, self.wmask, self.kmu = CT, co, wmask, kmu
        self.kmask = wmask[:Hkv].contiguous() if self.static else None
        self.vmask = wmask[Hkv:].contiguous() if self.static else None
        dev = pool.device
        self.ring = None
        if self.geo.active:
            self.ring = torch.zeros(planner.spare + 1, self.geo.slots, 2 * Hkv, D, dtype=torch.bfloat16, device=dev)
        self.ws = decode_workspace(dev, tile_layout(kind, Hkv, G), planner.max_rows, planner.plan)

    def center_rows(self, kv):
        """what the BF16 slots hold: key rows with the static mean removed (fp32 subtraction, one bf16 rounding)"""
        if self.kmu is None:
            return kv
        H = self.Hkv
        keys = (kv[:, :H].float() - self.kmu).to(torch.bfloat16)
        return torch.cat([keys, kv[:, H:]], dim=1)

    def write_pages(self, kv, slots):
        """kv bf16 [n, 2 Hkv, 128] -> pages at slots (< 0 skipped); the kernels subtract kmu from the K rows"""
        if self.static:
            K.v2_write(kv, slots, self.wmask, 32, self.pool, PAGE, fmt=self.kind, kmu=self.kmu)
        elif kv.shape[0] * self.Hkv > 1024:
            # prompt-sized: the screened two-pass writer (same bytes as fr_cb_write)
            K.cb_write3(kv, slots, self.CT, self.co, None, None, self.kind, self.pool, PAGE, split=False, kmu=self.kmu)
        else:
            K.cb_write(kv, slots, self.CT, self.co, self.kind, self.pool, PAGE, kmu=self.kmu)

    def prefill(self, kv, slots, req: int):
        """a prompt of request row `req`: every token to its page; sinks and the newest W tokens also to the BF16 row"""
        self.write_pages(kv, slots)
        if self.ring is not None:
            keep, where = self.geo.kept(kv.shape[0], kv.device)
            self.ring[req].index_copy_(0, where, self.center_rows(kv[keep]))

    def prefill_chunk(self, kv, slots, req: int, start: int):
        """the next n tokens of request row `req`'s prompt, positions [start, start + n): every token to its page; the
        sinks among them and the newest W of the prompt so far also to the BF16 row"""
        self.write_pages(kv, slots)
        if self.ring is not None:
            n = kv.shape[0]
            pos = start + torch.arange(n, device=kv.device)
            keep = (pos < self.geo.S) | (pos >= start + n - self.geo.W)
            self.ring[req].index_copy_(0, self.geo.slot(pos[keep]), self.center_rows(kv[keep]))

    def update(self, kv, sp: StepPlan):
        """cache update of a decode step: the new tokens to their pages and to their BF16 slots"""
        self.write_pages(kv, sp.slots)
        if self.ring is not None:
            self.ring.view(-1, 2 * self.Hkv, D).index_copy_(0, sp.ring_dest, self.center_rows(kv))

    def decode(self, q, sp: StepPlan, out):
        n = q.shape[0]
        extra = {}
        if self.ring is not None:      # the sinks are in the pages too, but read in BF16: kv_start masks them there
            extra = dict(tail=self.ring, tail_len=sp.ring_tokens, tail_idx=sp.ring_home, tail_bs=self.ring.stride(0),
                         tail_ts=self.ring.stride(1), kv_start=self.geo.S)
        if q.stride(1) != D or q.stride(2) != 1:
            q = q.contiguous()
        if self.static:
            K.v2_attn(q, self.pool, sp.block_table[:n], sp.page_tokens, out, sp.nsplit, sp.chunk, self.ws, self.qscale,
                      kmask=self.kmask, vmask=self.vmask, rb=32, fmt=self.kind, **extra)
        else:
            K.cb_attn(q, self.pool, sp.block_table[:n], sp.page_tokens, out, sp.nsplit, sp.chunk, self.ws, self.qscale,
                      self.kind, **extra)

    def step(self, q, kv, sp: StepPlan, out):
        """what a captured decode step of this layer contains"""
        self.update(kv, sp)
        self.decode(q, sp, out)


class KiviDecodeLayer:
    """KIVI-style pages: values written per token, key groups of 32 tokens encoded when they complete (from the prompt
    rows at prefill, from the BF16 ring at decode: the window must hold a whole group, W >= 32)."""

    def __init__(self, Hkv: int, G: int, pool: torch.Tensor, planner: StepPlanner, qs, lz, co, scale: float = None,
                 f8: bool = False):
        """f8: FP8-meta pages (the reference's `kivi_f8` option, attention/backend.py:365-366): pool chunks of
        KIVI.chunk_bytes(D, True) bytes."""
        if planner.kind != "kivi2" or planner.geo.W < GROUP:
            raise ValueError("kivi2 needs a BF16 window of at least one key group")
        if pool.shape[-1] != KIVI.chunk_bytes(D, f8):
            raise ValueError("pool chunk size does not match the page format")
        self.Hkv, self.G, self.pool, self.planner, self.f8 = Hkv, G, pool, planner, f8
        self.geo = planner.geo
        self.scale = scale if scale is not None else 1.0 / math.sqrt(D)
        self.qs, self.lz, self.co = qs, lz, co             # calibration queries, their log normalisers, value weights
        dev = pool.device
        self.ring = torch.zeros((planner.spare + 1) * self.geo.slots, 2 * Hkv, D, dtype=torch.bfloat16, device=dev)
        self.ws = kivi_workspace(dev, planner.max_rows, Hkv, G, D, planner.plan)

    def prefill(self, kv, slots, req: int):
        """a fresh prompt of n tokens: values of every token, the whole key groups, sinks and newest W rows in BF16"""
        n = kv.shape[0]
        KIVI.v_write(kv, slots, self.co, None, self.pool, self.Hkv, D, f8=self.f8)
        keep, where = self.geo.kept(n, kv.device)
        row = self.ring.view(self.planner.spare + 1, self.geo.slots, 2 * self.Hkv, D)[req]
        row.index_copy_(0, where, kv[keep])
        whole = n // GROUP
        if whole:
            pos = torch.arange(whole * GROUP, device=kv.device).view(whole, GROUP)
            src = torch.where(pos < self.geo.S, torch.full_like(pos, -1), pos).contiguous()     # sinks stay BF16 only
            KIVI.k_encode(kv, src, slots[:whole * GROUP].view(whole, GROUP).contiguous(), self.qs, self.lz, self.scale,
                          self.pool, self.Hkv, D, f8=self.f8)

    def prefill_chunk(self, kv, slots, req: int, start: int, table_row):
        """the next n tokens of request `req`'s prompt, positions [start, start + n): values of every token, the key
        groups the chunk completes (their earlier positions read from the ring, which therefore takes the chunk's own
        rows only afterwards), then the sinks and the newest W rows of the prompt so far in BF16"""
        n = kv.shape[0]
        KIVI.v_write(kv, slots, self.co, None, self.pool, self.Hkv, D, f8=self.f8)
        flat = self.ring.view(-1, 2 * self.Hkv, D)
        groups = chunk_key_groups(self.geo, start, n, req * self.geo.slots, table_row)
        if groups is not None:
            KIVI.k_encode(kv, groups[0], groups[1], self.qs, self.lz, self.scale, self.pool, self.Hkv, D, src2=flat,
                          f8=self.f8)
        pos = start + torch.arange(n, device=kv.device)
        keep = (pos < self.geo.S) | (pos >= start + n - self.geo.W)
        flat.index_copy_(0, req * self.geo.slots + self.geo.slot(pos[keep]), kv[keep])

    def update(self, kv, sp: StepPlan):
        KIVI.v_write(kv, sp.slots, self.co, None, self.pool, self.Hkv, D, f8=self.f8)
        self.ring.index_copy_(0, sp.ring_dest, kv)
        KIVI.k_encode(self.ring, sp.group_src, sp.group_dst, self.qs, self.lz, self.scale, self.pool, self.Hkv, D,
                      f8=self.f8)

    def decode(self, q, sp: StepPlan, out):
        n = q.shape[0]
        if q.stride(1) != D or q.stride(2) != 1:
            q = q.contiguous()
        KIVI.attn(q, self.pool, sp.block_table[:n], sp.page_tokens, out, sp.nsplit, sp.chunk, self.ws,
                  self.scale * LOG2E, self.geo.S, self.G, ring=self.ring, tail_len=sp.ring_tokens,
                  tail_idx=sp.ring_home, T=self.geo.slots, f8=self.f8)

    def step(self, q, kv, sp: StepPlan, out):
        self.update(kv, sp)
        self.decode(q, sp, out)
