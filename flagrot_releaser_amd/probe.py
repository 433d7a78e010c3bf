"""Measurement aid (no counterpart in the reference, not part of the drop-in boundary): `read_pages` launches a kernel
that only reads the (page, KV head) chunks a paged decode launch over the same block table reads, with the decode kernel's
workgroup layout.  bench.py times it beside the decode kernel: the rate the memory system gives that access pattern,
measured in the same run on the same cache.  Asynchronous on torch's current stream."""
import torch

from .native import Library, current_stream

ABI = 1
NATIVE = Library("probe", "FLAGROT_PROBE_LIB", "fr_probe_abi_version", ABI, "fr_probe_last_error", {
    "fr_probe_last_error": "->s",
    "fr_probe_read": "p p i p i i i i p p",
    "fr_probe_mfma": "i i i p p",
    "fr_probe_mfma_flops": "i i",
})
EXPORTS = NATIVE.exports


def lib():
    return NATIVE.dll


def read_pages(pool, block_table, seq_lens, sink, page=16):
    """pool uint8 [num_pages, Hkv, chunk_bytes]; block_table int32 [B, pages]; seq_lens int32 [B]; sink int32 [>= 1]"""
    assert pool.dtype == torch.uint8 and pool.is_contiguous() and block_table.dtype == torch.int32 and seq_lens.dtype == torch.int32
    B, Hkv, chunk = block_table.shape[0], pool.shape[1], pool.shape[2]
    NATIVE.run("fr_probe_read", pool, block_table, block_table.stride(0), seq_lens, B, Hkv, page, chunk, sink, current_stream())


def mfma_burst(mode: int, iters: int, workgroups: int, sink):
    """launches the matrix-pipe probe (mode 0: register operands, 1: one LDS operand per instruction); returns its flops"""
    NATIVE.run("fr_probe_mfma", mode, iters, workgroups, sink, current_stream())
    return 2 * 32 * 32 * 16 * 4 * 8 * (iters + (iters & 1)) * workgroups
