"""Offline pattern search -- host side.

Counterpart of ``search_pattern`` (reference minference/modules/minference_forward.py:129-227),
the routine that produces the per-head entries of the ``best_pattern`` JSON the prefill
dispatcher consumes.  The reference scores a candidate by multiplying an N x N mask into the
N x N softmax of one head; here the candidates of all heads are turned into per-column,
per-diagonal and per-32x32-block flag bytes (top-k and flag kernels of libminf_hip.so) and one
sweep over the causal score matrix (``minf_pattern_recall``) returns the kept softmax mass of up
to eight candidates at once, so the search also runs at context lengths whose N x N matrix would
not fit anywhere.
"""
from __future__ import annotations

import torch

from . import _lib
from .estimate import _prep16, topk_indices, vertical_slash_scores
from .ops import _check_qkv

ROW_BEGIN = 2500                  # minference_forward.py:161: attn_weights_x[:, :, 2500:]
SEARCH_FORCE = 30                 # :140 and :144: first 30 verticals, last 30 slash entries
CANDIDATES = (                    # :209-215
    ("stream_llm", 100, 800),
    ("vertical_and_slash", 30, 800), ("vertical_and_slash", 100, 750),
    ("vertical_and_slash", 500, 700), ("vertical_and_slash", 3500, 100),
    ("block_sparse", 8, 1),
)
MAX_CANDIDATES = 8


def _dtype_code(t):
    return _lib.MINF_BF16 if t.dtype == torch.bfloat16 else _lib.MINF_F16


def _search_block_index(q16, k16, keep):
    """Top ``keep`` key blocks (32 tokens) per query block of the pooled scores, :175-186."""
    B, H, N, _ = q16.shape
    Hk = k16.shape[1]
    rows = (N + 31) // 32
    keep = min(keep, rows)
    lib = _lib.load()
    dev = q16.device
    out = torch.empty((B, H, rows, keep), dtype=torch.int32, device=dev)
    ws_bytes = lib.minf_search_block_index_workspace_bytes(B, H, Hk, N)
    ws = torch.empty((ws_bytes + 15) // 16 * 16, dtype=torch.uint8, device=dev)
    i64x3 = _lib.c_i64 * 3
    with torch.cuda.device(dev):
        st = lib.minf_search_block_index(
            q16.data_ptr(), k16.data_ptr(), i64x3(*q16.stride()[:3]), i64x3(*k16.stride()[:3]),
            B, H, Hk, N, 128, _dtype_code(q16), keep, out.data_ptr(), ws.data_ptr(), ws_bytes,
            _lib.stream_ptr(dev))
    _lib.check(st, "minf_search_block_index")
    return out


def pattern_recall(q, k, candidates=CANDIDATES, row_begin=ROW_BEGIN):
    """-> [B, H, len(candidates)] fp32: for every head and candidate ``(type, a, b)`` the mean over
    query rows >= row_begin of the exact causal softmax mass inside the candidate's mask, with the
    masks of the reference's search (element-granular, not the kernels' 64-wide blocks):

    * ``("stream_llm", v, s)``          diagonals 0..s plus the first v columns (:164-173)
    * ``("vertical_and_slash", v, s)``  the v best columns and the s best single diagonals of the
      last-64-query estimate, first 30 columns and diagonals 0..29 forced (:133-162)
    * ``("block_sparse", ratio, _)``    32 x 32 blocks: the ceil(N/32) // ratio best key blocks of
      every query block by mean-pooled score (:175-195)

    q [B,H,N,D], k [B,Hk,N,D] on the GPU (fewer kv heads are read in place).  NaN when
    N <= row_begin, like the reference's mean over an empty slice."""
    if not 1 <= len(candidates) <= MAX_CANDIDATES:
        raise ValueError(f"1..{MAX_CANDIDATES} candidates per call")
    _check_qkv(q, k, k)
    head_dim = q.shape[-1]
    q16, k16 = _prep16(q, k)
    B, H, N, _ = q16.shape
    Hk = k16.shape[1]
    dev = q16.device
    lib = _lib.load()
    stream = _lib.stream_ptr(dev)
    pitch = (N + 63) // 64 * 64
    rows32 = (N + 31) // 32
    bpitch = (rows32 + 3) // 4 * 4
    col = torch.zeros((B * H, pitch), dtype=torch.uint8, device=dev)
    diag = torch.zeros((B * H, pitch), dtype=torch.uint8, device=dev)
    blk = None
    scores = None
    with torch.cuda.device(dev):
        for bit, (ty, a, b) in enumerate(candidates):
            a, b = int(a), int(b)
            if ty == "stream_llm":
                _lib.check(lib.minf_flags_set_range(0, min(a, N), B * H, bit, col.data_ptr(), pitch, stream),
                           "minf_flags_set_range")
                _lib.check(lib.minf_flags_set_range(0, min(b + 1, N), B * H, bit, diag.data_ptr(), pitch, stream),
                           "minf_flags_set_range")
            elif ty == "vertical_and_slash":
                if scores is None:
                    scores = vertical_slash_scores(q, k, 64, SEARCH_FORCE, SEARCH_FORCE, reference_rounding=False)
                v_idx = topk_indices(scores[0], min(a, N))
                s_idx = topk_indices(scores[1], min(b, N), reverse_base=N - 1)
                for idx, flags in ((v_idx, col), (s_idx, diag)):
                    kk = idx.shape[-1]
                    _lib.check(lib.minf_flags_set_indices(idx.data_ptr(), B * H, kk, kk, bit, flags.data_ptr(),
                                                          pitch, N, stream), "minf_flags_set_indices")
            elif ty == "block_sparse":
                keep = rows32 // a
                if blk is None:
                    blk = torch.zeros((B * H * rows32, bpitch), dtype=torch.uint8, device=dev)
                if keep > 0:
                    bi = _search_block_index(q16, k16, keep)
                    kk = bi.shape[-1]
                    _lib.check(lib.minf_flags_set_indices(bi.data_ptr(), B * H * rows32, kk, kk, bit,
                                                          blk.data_ptr(), bpitch, rows32, stream),
                               "minf_flags_set_indices")
            else:
                raise ValueError(f"unknown pattern type {ty!r}")
        recall = torch.empty((B * H, MAX_CANDIDATES), dtype=torch.float32, device=dev)
        ws_bytes = lib.minf_pattern_recall_workspace_bytes(B, H, N)
        ws = torch.empty((ws_bytes + 15) // 16 * 16, dtype=torch.uint8, device=dev)
        i64x3 = _lib.c_i64 * 3
        st = lib.minf_pattern_recall(
            q16.data_ptr(), k16.data_ptr(), i64x3(*q16.stride()[:3]), i64x3(*k16.stride()[:3]),
            B, H, Hk, N, 128, _dtype_code(q16), float(head_dim) ** -0.5,
            col.data_ptr(), diag.data_ptr(), pitch,
            blk.data_ptr() if blk is not None else None, bpitch, int(row_begin),
            recall.data_ptr(), ws.data_ptr(), ws_bytes, stream)
    _lib.check(st, "minf_pattern_recall")
    return recall.view(B, H, MAX_CANDIDATES)[..., :len(candidates)]


def _choose(candidates, scores):
    """:205-227: the best score wins (first on ties, must exceed 0); a stream_llm winner is
    relabelled vertical_and_slash with its own sizes, a block_sparse winner becomes
    vertical_and_slash (1000, 6096)."""
    best_ty, best_v, best_s, best = "", 0, 0, 0.0
    for (ty, v_size, s_size), sc in zip(candidates, scores):
        if sc > best:
            best_ty, best_v, best_s, best = ty, v_size, s_size, sc
    if best_ty == "stream_llm":
        best_ty = "vertical_and_slash"
    if best_ty == "block_sparse":
        best_ty, best_v, best_s = "vertical_and_slash", 1000, 6096
    return best_ty, best_v, best_s, best


def search_pattern(q, k, head=None, candidates=CANDIDATES, row_begin=ROW_BEGIN):
    """Same call as the reference's ``search_pattern(q, k, head)``: q, k [1, 1, N, D] of one head
    -> ``(type, vertical_size, slash_size, score)``.  ``head`` is only echoed by the reference's
    print and is ignored."""
    if q.shape[0] != 1 or q.shape[1] != 1:
        raise ValueError("search_pattern takes one head: q [1, 1, N, D]; use search_patterns for a layer")
    rec = pattern_recall(q, k, candidates, row_begin)[0, 0].tolist()
    return _choose(candidates, rec)


def search_patterns(q, k, candidates=CANDIDATES, row_begin=ROW_BEGIN):
    """All heads of a layer in one sweep: q [1,H,N,D], k [1,Hk,N,D] -> ``{str(head): [type, v, s,
    score]}``, one layer of the ``best_pattern`` table (the loop at minference_forward.py:566-571)."""
    if q.shape[0] != 1:
        raise ValueError("one sequence at a time")
    rec = pattern_recall(q, k, candidates, row_begin)[0].tolist()
    return {str(h): list(_choose(candidates, rec[h])) for h in range(q.shape[1])}
