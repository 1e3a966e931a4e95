"""Vertical/slash index conversion -- host side.

Mirror of ``minference.cuda.convert_vertical_slash_indexes`` (reference
csrc/kernels.cpp:7-18, csrc/vertical_slash_index.cu:127-167): same name,
argument order and return order; outputs are int32 tensors on the inputs'
device.  The work is done by ``minf_vs_index_build_ws`` in libminf_hip.so (the
table-driven builder; ``use_tables=False`` selects the plain wave-per-row
``minf_vs_index_build``) on the caller's current stream (the reference used
the legacy default stream).
"""
from __future__ import annotations

import torch

from . import _lib


def _i32_contig(t: torch.Tensor) -> torch.Tensor:
    if t.dtype != torch.int32:
        t = t.to(torch.int32)
    return t.contiguous()


def convert_vertical_slash_indexes(seqlens, vertical_indexes, slash_indexes, context_size,
                                   block_size_M=64, block_size_N=64, zero_fill=True,
                                   error_flag=None, use_tables=True):
    """-> [block_count, block_offset, column_count, column_index].

    seqlens [B] int32, vertical_indexes [B,H,V] ascending, slash_indexes [B,H,S]
    descending (all int32, on the GPU).  ``zero_fill=False`` leaves everything
    past the per-row counts unwritten (torch.empty) instead of zero; the
    attention kernels never read past the counts.
    """
    if block_size_M != 64 or block_size_N != 64:
        # the reference only asserts this (csrc/vertical_slash_index.cu:135-136)
        raise ValueError("only 64x64 blocks are supported")
    if not vertical_indexes.is_cuda:
        raise RuntimeError("convert_vertical_slash_indexes needs GPU tensors (no CPU path)")
    if vertical_indexes.dim() != 3 or slash_indexes.dim() != 3:
        raise ValueError("vertical_indexes / slash_indexes must be [B, H, nnz]")
    seqlens = _i32_contig(seqlens)
    v = _i32_contig(vertical_indexes)
    s = _i32_contig(slash_indexes)
    B, H, S = s.shape
    V = v.shape[2]
    if v.shape[0] != B or v.shape[1] != H or seqlens.numel() != B:
        raise ValueError("batch/head sizes of seqlens, vertical_indexes, slash_indexes differ")
    rows = (int(context_size) + 63) // 64
    dev = v.device
    alloc = torch.empty                              # the kernel writes every element itself
    block_count = alloc((B, H, rows), dtype=torch.int32, device=dev)
    block_offset = alloc((B, H, rows, S), dtype=torch.int32, device=dev)
    column_count = alloc((B, H, rows), dtype=torch.int32, device=dev)
    column_index = alloc((B, H, rows, V), dtype=torch.int32, device=dev)
    if not zero_fill:
        # counts of rows past seqlen are not written by the kernel in this mode
        block_count.zero_()
        column_count.zero_()
    lib = _lib.load()
    args = (seqlens.data_ptr(), v.data_ptr(), s.data_ptr(), block_count.data_ptr(),
            block_offset.data_ptr(), column_count.data_ptr(), column_index.data_ptr(),
            B, H, rows, V, S, 1 if zero_fill else 0,
            error_flag.data_ptr() if error_flag is not None else None)
    with torch.cuda.device(dev):
        if use_tables:
            ws_bytes = lib.minf_vs_index_workspace_bytes(B, H, S, rows)
            ws = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=dev)
            st = lib.minf_vs_index_build_ws(*args, ws.data_ptr(), ws_bytes, _lib.stream_ptr(dev))
        else:
            st = lib.minf_vs_index_build(*args, _lib.stream_ptr(dev))
    _lib.check(st, "minf_vs_index_build")
    return [block_count, block_offset, column_count, column_index]
