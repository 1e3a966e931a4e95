"""ORACLE -- TEST INFRASTRUCTURE ONLY.

CPU restatement of the dynamic sparse prefill attention path of
microsoft/MInference.  Nothing under ``minference_amd/`` may import this
module; only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` use it, and only as the checker / the timed CPU baseline.

Every function cites the reference lines it restates.  Parity status:

* ``vs_index_build``      pinned (hand KATs, set-based specification, properties)
* ``estimate_vs``         pinned (brute-force double loops, sum invariants, Q=0 closed form)
* ``vs_mask`` / ``masked_attention``  pinned (special cases that reduce to
  torch's scaled_dot_product_attention, brute force on tiny inputs)
* ``bs_block_index`` / ``bs_mask``    pinned (properties, top_k>=rows -> causal SDPA)
* ``ashape_mask``         pinned (closed form vs per-element loop, n_local>=N -> causal SDPA)
* ``search_candidate_mask`` / ``search_pattern_scores``  pinned (Q=0 closed forms counted by
  explicit loops, all-kept candidates -> 1, brute force on tiny inputs)
* ``estimate_scores(reference_rounding=True)`` / ``bs_block_scores(reference_rounding=True)``: the
  rounding points of the reference's torch code on 16-bit inputs; pinned by per-element loops that
  round with ``.to(dtype)`` at exactly those points (tests/test_oracle_rounding.py)
* ``torch.topk`` tie order and Triton's bf16 rounding points inside the attention kernels are
  implementation defined in the reference (not in its source): "parity unpinned" for those;
  tests compare top-k *sets* away from ties and outputs within tolerance.
"""
from __future__ import annotations

import ctypes
import math
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build_c_oracle(force: bool = False) -> str:
    """Compile oracle/vs_index_ref.c into oracle/_build/liboracle.so (gcc)."""
    so = os.path.join(_HERE, "_build", "liboracle.so")
    src = os.path.join(_HERE, "vs_index_ref.c")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-C", _HERE] + (["-B"] if force else []))
    return so


def _lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "_build", "liboracle.so")
        if not os.path.exists(so):
            so = build_c_oracle()
        lib = ctypes.CDLL(so)
        i32p = ctypes.POINTER(ctypes.c_int32)
        lib.oracle_vs_index_build.argtypes = [i32p] * 7 + [ctypes.c_int] * 5
        lib.oracle_vs_index_build.restype = ctypes.c_int
        _LIB = lib
    return _LIB


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))


# --------------------------------------------------------------------------
# a-2  index builder            csrc/vertical_slash_index.cu:27-167
# --------------------------------------------------------------------------
def vs_index_build(seqlens, vertical, slash, context_size, block_m=64, block_n=64):
    """C restatement (oracle/vs_index_ref.c) of convert_vertical_slash_indexes.

    seqlens [B] i32, vertical [B,H,V] i32 ascending, slash [B,H,S] i32 descending.
    Returns (block_count [B,H,R], block_offset [B,H,R,S], column_count [B,H,R],
    column_index [B,H,R,V]) as int32 numpy arrays, zero-filled like the
    reference's torch::zeros outputs (csrc/vertical_slash_index.cu:146-149).
    """
    assert block_m == 64 and block_n == 64  # csrc/vertical_slash_index.cu:135-136
    seqlens = np.ascontiguousarray(np.asarray(seqlens, dtype=np.int32))
    vertical = np.ascontiguousarray(np.asarray(vertical, dtype=np.int32))
    slash = np.ascontiguousarray(np.asarray(slash, dtype=np.int32))
    B, H, S = slash.shape
    V = vertical.shape[2]
    R = (context_size + block_m - 1) // block_m
    bc = np.empty((B, H, R), np.int32)
    bo = np.empty((B, H, R, S), np.int32)
    cc = np.empty((B, H, R), np.int32)
    ci = np.empty((B, H, R, V), np.int32)
    rc = _lib().oracle_vs_index_build(_p(seqlens), _p(vertical), _p(slash), _p(bc), _p(bo),
                                      _p(cc), _p(ci), B, H, R, V, S)
    if rc != 0:
        raise ValueError(f"{-rc} row(s) hit a case where the reference reads out of bounds "
                         "(no slash offset below the row block's end, or empty lists)")
    return bc, bo, cc, ci


def vs_index_row_py(vertical, slash, m, seqlen):
    """Pure-Python version of one row block (small cases only); same steps as
    csrc/vertical_slash_index.cu:46-98.  Used to cross-check the C file."""
    start_m = m * 64
    if start_m >= seqlen:
        return [], []
    end_m = start_m + 64
    blocks, cols = [], []
    s = v = 0
    v_idx = vertical[v]; v += 1
    s_idx = slash[s]; s += 1
    while s_idx >= end_m:
        s_idx = slash[s]; s += 1
    s_idx = max(end_m - s_idx, 64)
    rs, re = s_idx - 64, s_idx
    while True:
        if v_idx < re:
            if v_idx < rs:
                cols.append(int(v_idx))
            if v < len(vertical):
                v_idx = vertical[v]; v += 1
            else:
                v_idx = end_m + 64
        else:
            if s < len(slash):
                s_idx = max(end_m - slash[s], 64); s += 1
            else:
                blocks.extend(range(rs, re, 64))
                break
            if s_idx > re + 64:
                blocks.extend(range(rs, re, 64))
                rs, re = s_idx - 64, s_idx
            elif s_idx > re:
                re += 64
    return blocks, cols


# --------------------------------------------------------------------------
# a-1  estimation     minference/modules/minference_forward.py:599-614, 110-116
# --------------------------------------------------------------------------
def sum_all_diagonal(p: torch.Tensor) -> torch.Tensor:
    """Diagonal sums of p [n, N] (one head): out[j] = sum_i p[i, i + j + 1 - n]
    for j in [0, n + N - 1).  Same padded-stride construction as
    minference_forward.py:110-116, restated per head."""
    n, N = p.shape
    z = torch.zeros(n, n, dtype=p.dtype)
    padded = torch.cat((z, p, z), -1).contiguous()          # [n, 2n+N]
    strided = padded.as_strided((n, n + N), (2 * n + N + 1, 1))
    return strided.sum(0)[1:]


def estimate_scores(q: torch.Tensor, k: torch.Tensor, last_q: int = 64, reference_rounding: bool = False):
    """Score vectors before forcing.  q,k [B,H,N,D] (same H) on CPU.
    Returns (vertical [B,H,N], slash [B,H,N]) fp32 where slash[..., j] is the
    probability mass on the diagonal with offset N-1-j
    (minference_forward.py:601-609).

    Default: fp32 arithmetic throughout.  ``reference_rounding=True`` rounds where the reference's
    torch code rounds for 16-bit inputs: the einsum result (fp32 accumulation, one rounding to the
    input dtype, :602), then the division by sqrt(D) in the input dtype (:602); the softmax and
    both sums run in fp32 (``dtype=torch.float32``, :604).  For fp32 inputs the two modes agree."""
    B, H, N, D = q.shape
    lq = min(last_q, N)
    qf, kf = q.float(), k.float()
    qk = torch.einsum("bhmk,bhnk->bhmn", qf[:, :, -lq:, :], kf)
    if reference_rounding and q.dtype != torch.float32:
        qk = (qk.to(q.dtype) / math.sqrt(D)).float()       # tensor / python scalar: fp32 quotient, rounded to q.dtype
    else:
        qk = qk / math.sqrt(D)
    ar = torch.arange(lq)
    corner = ar[:, None] >= ar[None, :]
    qk[:, :, :, -lq:] = torch.where(corner, qk[:, :, :, -lq:], torch.tensor(-torch.inf))
    p = torch.softmax(qk, dim=-1, dtype=torch.float32)
    vertical = p.sum(-2)
    slash = torch.empty(B, H, N, dtype=torch.float32)
    for b in range(B):
        for h in range(H):
            d = sum_all_diagonal(p[b, h])                   # [lq + N - 1]
            slash[b, h] = d[:N]                             # [..., :-last_q+1]
    return vertical, slash


def topk_lowest_index(x: torch.Tensor, k: int) -> torch.Tensor:
    """Indices of the k largest entries along the last dim; among equal values
    the lowest index wins (the reference's torch.topk leaves tie order
    unspecified).  Returned ascending by index."""
    N = x.shape[-1]
    order = torch.argsort(x, dim=-1, descending=True, stable=True)[..., :k]
    return order.sort(dim=-1).values


def estimate_vs(q, k, vertical_size, slash_size, last_q=64, force_vertical=30, force_slash=100,
                reference_rounding=False):
    """minference_forward.py:599-612: returns (v_idx [B,H,v] ascending key
    positions, s_idx [B,H,s] descending diagonal offsets, vertical scores,
    slash scores) -- scores after forcing (+inf)."""
    N = q.shape[2]
    v = min(N, max(vertical_size, 30))
    s = min(N, max(slash_size, 50))
    vertical, slash = estimate_scores(q, k, last_q, reference_rounding)
    vertical = vertical.clone(); slash = slash.clone()
    vertical[..., :force_vertical] = torch.inf
    slash[..., -force_slash:] = torch.inf
    v_idx = topk_lowest_index(vertical, v)
    s_j = topk_lowest_index(slash, s)                       # ascending j
    s_idx = (N - 1) - s_j                                    # descending offsets
    return v_idx, s_idx, vertical, slash


# --------------------------------------------------------------------------
# masks + fp32 masked dense attention (the attention oracle)
# --------------------------------------------------------------------------
def vs_mask(block_count, block_offset, column_count, column_index, n, seqlen=None):
    """Boolean [n, n] mask of one (batch, head) from the four index tensors,
    with the visiting rule of pit_sparse_flash_attention_v2.py:104-148:
    row r attends {c in union of [off, off+64) : c <= r, c < seqlen} plus the
    listed columns (no causal test on those)."""
    seqlen = n if seqlen is None else seqlen
    mask = np.zeros((n, n), dtype=bool)
    rows = (n + 63) // 64
    for m in range(rows):
        r0, r1 = m * 64, min(m * 64 + 64, n)
        if r0 >= seqlen:
            continue
        rr = np.arange(r0, r1)
        for off in block_offset[m, : block_count[m]]:
            cols = np.arange(off, off + 64)
            cols = cols[(cols < seqlen) & (cols < n)]
            mask[r0:r1, cols] |= cols[None, :] <= rr[:, None]
        cols = column_index[m, : column_count[m]]
        mask[r0:r1, cols] = True
    mask[seqlen:, :] = False
    return mask


def vs_mask_rows(block_count_m, block_offset_m, column_count_m, column_index_m, m, n, seqlen=None):
    """Rows [64m, min(64m+64, n)) of vs_mask() from the index entries of row block m alone
    (pit_sparse_flash_attention_v2.py:104-148): [rows, n] bool.  For full-size inputs where the
    [n, n] mask does not fit."""
    seqlen = n if seqlen is None else seqlen
    r0, r1 = m * 64, min(m * 64 + 64, n)
    mask = np.zeros((r1 - r0, n), dtype=bool)
    if r0 >= seqlen:
        return mask
    rr = np.arange(r0, r1)
    for off in np.asarray(block_offset_m, dtype=np.int64)[: int(block_count_m)]:
        cols = np.arange(off, off + 64)
        cols = cols[(cols < seqlen) & (cols < n)]
        mask[:, cols] |= cols[None, :] <= rr[:, None]
    mask[:, np.asarray(column_index_m, dtype=np.int64)[: int(column_count_m)]] = True
    mask[rr >= seqlen, :] = False
    return mask


def bs_block_scores(q: torch.Tensor, k: torch.Tensor, reference_rounding: bool = False):
    """Pooled block scores [B,H,R,R] (fp32 values) of block_sparse_flash_attention.py:159-164 on
    tensors already padded to a multiple of 64; non-causal pairs are -inf.  Default: fp32
    arithmetic.  ``reference_rounding=True`` rounds where the reference's torch code rounds for
    16-bit inputs: each 64-token mean (fp32 accumulation, rounded to the input dtype, :159-160)
    and each pooled dot product (fp32 accumulation, rounded to the input dtype, :163)."""
    B, H, N, D = q.shape
    qp = q.float().reshape(B, H, -1, 64, D).mean(-2)
    kp = k.float().reshape(B, H, -1, 64, D).mean(-2)
    rr = reference_rounding and q.dtype != torch.float32
    if rr:
        qp, kp = qp.to(q.dtype).float(), kp.to(q.dtype).float()
    R = qp.shape[2]
    p = torch.einsum("bhmk,bhnk->bhmn", qp, kp)
    if rr:
        p = p.to(q.dtype).float()
    ar = torch.arange(R)
    return torch.where(ar[:, None] >= ar[None, :], p, torch.tensor(-torch.inf))


def bs_block_index(q: torch.Tensor, k: torch.Tensor, top_k: int, force_diag_first: bool = False,
                   reference_rounding: bool = False):
    """block_sparse_flash_attention.py:151-166 on tensors already padded to a
    multiple of 64 (the caller pads, :178-180).  fp32 arithmetic unless
    ``reference_rounding`` (see bs_block_scores); ties -> lowest
    block id.  force_diag_first adds the benchmark rule "always keep the
    diagonal block and block 0" before the sort."""
    p = bs_block_scores(q, k, reference_rounding)
    R = p.shape[-1]
    ar = torch.arange(R)
    if force_diag_first:
        p[..., ar, ar] = torch.inf
        p[..., :, 0] = torch.inf
    top_k = min(top_k, R)
    order = torch.argsort(p, dim=-1, descending=True, stable=True)[..., :top_k]
    return order.to(torch.int32).sort(dim=-1).values


def bs_mask(block_index, n):
    """Mask of one head from block_index [R, top_k] with the kernel's visiting
    rule (block_sparse_flash_attention.py:81-96): the FIRST min(m+1, top_k)
    entries of the ascending row, element-wise causal."""
    mask = np.zeros((n, n), dtype=bool)
    R, K = block_index.shape
    for m in range((n + 63) // 64):
        r0, r1 = m * 64, min(m * 64 + 64, n)
        rr = np.arange(r0, r1)
        for j in block_index[m, : min(m + 1, K)]:
            cols = np.arange(j * 64, j * 64 + 64)
            cols = cols[cols < n]
            mask[r0:r1, cols] |= cols[None, :] <= rr[:, None]
    return mask


def ashape_mask(n, n_init, n_local):
    """streaming_kernel.py:611-646 (+ masks :66-75): row r attends
    {k : r - n_local < k <= r} plus {k < n_init : k <= r - n_local}."""
    r = np.arange(n)[:, None]
    c = np.arange(n)[None, :]
    d = r - c
    return ((d >= 0) & (d < n_local)) | ((c < n_init) & (d >= n_local))


def trishape_mask(n, n_init, n_local, n_last):
    """tri_shape_kernel (streaming_kernel.py:820-833): the A-shape mask for rows < n - n_last
    (a_shape_kernel on the truncated sequence: causality keeps those rows inside it), the full
    causal row for the last n_last rows (:826-829); n_last is clamped to n - 1 (:822)."""
    n_last = min(n_last, n - 1)
    mask = ashape_mask(n, n_init, n_local)
    if n_last > 0:
        r = np.arange(n - n_last, n)[:, None]
        mask[n - n_last:] = np.arange(n)[None, :] <= r
    return mask


def masked_attention(q, k, v, mask, scale=None):
    """Exact fp32 softmax attention of one head under a boolean mask.
    q [n,D], k,v [n,D] (any float dtype) -> [n,D] fp32.  Rows with an empty
    mask give zeros."""
    qf, kf, vf = q.float(), k.float(), v.float()
    scale = (q.shape[-1] ** -0.5) if scale is None else scale
    s = (qf @ kf.T) * scale
    m = torch.as_tensor(mask)
    s = torch.where(m, s, torch.tensor(-torch.inf))
    mx = s.max(-1, keepdim=True).values
    mx = torch.where(torch.isinf(mx), torch.zeros_like(mx), mx)
    p = torch.exp(s - mx)
    den = p.sum(-1, keepdim=True)
    out = (p @ vf) / torch.where(den == 0, torch.ones_like(den), den)
    return out


# --------------------------------------------------------------------------
# the three ops end to end on CPU (fp32), mirroring the reference wrappers
# --------------------------------------------------------------------------
def vertical_slash_sparse_attention(q, k, v, v_idx, s_idx):
    """pit_sparse_flash_attention_v2.py:195-242 on CPU in fp32 (same H for q,k,v)."""
    B, H, N, D = q.shape
    vi = v_idx.to(torch.int32).reshape(B, H, -1).sort(-1, descending=False).values.numpy()
    si = s_idx.to(torch.int32).reshape(B, H, -1).sort(-1, descending=True).values.numpy()
    seqlens = np.full((B,), N, np.int32)
    bc, bo, cc, ci = vs_index_build(seqlens, vi, si, N)
    out = torch.empty(B, H, N, D, dtype=torch.float32)
    for b in range(B):
        for h in range(H):
            m = vs_mask(bc[b, h], bo[b, h], cc[b, h], ci[b, h], N)
            out[b, h] = masked_attention(q[b, h], k[b, h], v[b, h], m)
    return out


def block_sparse_attention(q, k, v, top_k):
    """block_sparse_flash_attention.py:169-186 on CPU in fp32."""
    B, H, N, D = q.shape
    pad = 64 - (N & 63)
    qp = torch.nn.functional.pad(q, [0, 0, 0, pad])
    kp = torch.nn.functional.pad(k, [0, 0, 0, pad])
    bi = bs_block_index(qp, kp, top_k).numpy()
    out = torch.empty(B, H, N, D, dtype=torch.float32)
    for b in range(B):
        for h in range(H):
            out[b, h] = masked_attention(q[b, h], k[b, h], v[b, h], bs_mask(bi[b, h], N))
    return out


def streaming_scale(head_dim):
    """The softmax scale of the reference's streaming operator: head dims outside {16, 32, 64, 128,
    256} are zero-padded to the next power of two first (streaming_kernel.py:621-626; a_shape_kernel
    :793-797) and ``append`` then takes 1/sqrt of the PADDED size (:575)."""
    d = head_dim
    if d not in (16, 32, 64, 128, 256):
        d = 2 ** math.ceil(math.log2(d))
    return 1.0 / math.sqrt(d)


def streaming_forward(q, k, v, n_init, n_local):
    """streaming_kernel.py:611-646 on CPU in fp32 (scale: see streaming_scale)."""
    B, H, N, D = q.shape
    m = ashape_mask(N, n_init, n_local)
    out = torch.empty(B, H, N, D, dtype=torch.float32)
    for b in range(B):
        for h in range(H):
            out[b, h] = masked_attention(q[b, h], k[b, h], v[b, h], m, scale=streaming_scale(D))
    return out


def tri_shape_forward(q, k, v, n_init, n_local, n_last):
    """tri_shape_kernel (streaming_kernel.py:820-833, minference_forward.py:444-455) on CPU in fp32:
    the A-shape operator on all but the last n_last tokens (its scale: streaming_scale), dense causal
    rows scaled by 1/sqrt(head_dim) (:826) for the last n_last queries."""
    B, H, N, D = q.shape
    n_last = min(n_last, N - 1)
    if n_last <= 0:
        return streaming_forward(q, k, v, n_init, n_local)
    y1 = streaming_forward(q[:, :, :-n_last], k[:, :, :-n_last], v[:, :, :-n_last], n_init, n_local)
    dense = torch.ones(N, N, dtype=torch.bool).tril()[-n_last:]
    y2 = torch.empty(B, H, n_last, D, dtype=torch.float32)
    for b in range(B):
        for h in range(H):
            s = (q[b, h, -n_last:].float() @ k[b, h].float().T) / math.sqrt(D)
            s = torch.where(dense, s, torch.tensor(-torch.inf))
            y2[b, h] = torch.softmax(s, dim=-1) @ v[b, h].float()
    return torch.cat([y1, y2], dim=2)


# --------------------------------------------------------------------------
# f-4  offline pattern search   minference/modules/minference_forward.py:129-227
# --------------------------------------------------------------------------
SEARCH_ROW_BEGIN = 2500                                     # :161,:172,:194  [..., 2500:]
SEARCH_CANDIDATES = (                                       # :209-215
    ("stream_llm", 100, 800),
    ("vertical_and_slash", 30, 800), ("vertical_and_slash", 100, 750),
    ("vertical_and_slash", 500, 700), ("vertical_and_slash", 3500, 100),
    ("block_sparse", 8, 1),
)


def search_candidate_mask(q, k, ty, v_size, s_size):
    """Element mask [N,N] (bool, already causal) that search_pattern scores for one candidate of
    one head; q,k [N,D].  fp32 arithmetic, ties -> lowest index.
    stream_llm (:164-173): offsets 0..s_size plus the first v_size columns.
    vertical_and_slash (:133-162): the v_size best columns of the last-64-query estimate (first
    30 forced) plus the s_size best single diagonals (offsets 0..29 forced).
    block_sparse (:175-195): 32x32 blocks, zero-padded mean pooling, unscaled pooled scores,
    the block_num // v_size best key blocks of every query block row."""
    n, d = q.shape
    r = torch.arange(n)[:, None]
    c = torch.arange(n)[None, :]
    off = r - c
    causal = off >= 0
    if ty == "stream_llm":
        return (causal & (off <= s_size)) | (causal & (c < v_size))
    if ty == "vertical_and_slash":
        vertical, slash = estimate_scores(q[None, None], k[None, None], 64)
        vertical, slash = vertical[0, 0].clone(), slash[0, 0].clone()
        vertical[:30] = torch.inf
        slash[-30:] = torch.inf
        cols = topk_lowest_index(vertical, min(v_size, n))
        offs = (n - 1) - topk_lowest_index(slash, min(s_size, n))
        colkeep = torch.zeros(n, dtype=torch.bool); colkeep[cols] = True
        offkeep = torch.zeros(n, dtype=torch.bool); offkeep[offs] = True
        return causal & (colkeep[None, :] | offkeep[off.clamp(min=0)])
    if ty == "block_sparse":
        nb = (n - 1) // 32 + 1
        pad = nb * 32 - n
        bq = torch.nn.functional.pad(q.float(), [0, 0, 0, pad]).reshape(nb, 32, d).mean(1)
        bk = torch.nn.functional.pad(k.float(), [0, 0, 0, pad]).reshape(nb, 32, d).mean(1)
        sc = bq @ bk.T
        ar = torch.arange(nb)
        sc = torch.where(ar[:, None] >= ar[None, :], sc, torch.tensor(-torch.inf))
        keep = nb // v_size
        bm = torch.zeros(nb, nb, dtype=torch.bool)
        if keep > 0:
            idx = topk_lowest_index(sc, keep)
            bm[ar[:, None].expand_as(idx), idx] = True
        full = bm.repeat_interleave(32, 0).repeat_interleave(32, 1)[:n, :n]
        return causal & full
    raise ValueError(ty)


def search_pattern_scores(q, k, candidates=SEARCH_CANDIDATES, row_begin=SEARCH_ROW_BEGIN):
    """:197-219: for every candidate, the mean over query rows >= row_begin of the softmax mass
    that falls inside the candidate's mask.  q,k [N,D] of one head -> list of floats (nan when
    N <= row_begin, like the mean of an empty slice)."""
    n, d = q.shape
    s = (q.float() @ k.float().T) / math.sqrt(d)
    s = torch.where(torch.arange(n)[:, None] >= torch.arange(n)[None, :], s, torch.tensor(-torch.inf))
    attn = torch.softmax(s, dim=-1, dtype=torch.float32)
    out = []
    for ty, v_size, s_size in candidates:
        m = search_candidate_mask(q, k, ty, v_size, s_size)
        out.append((attn * m)[row_begin:].sum(-1).mean().item())
    return out


def search_pattern(q, k, candidates=SEARCH_CANDIDATES, row_begin=SEARCH_ROW_BEGIN):
    """:205-227: best candidate by score (first wins ties, score must exceed 0), relabelled like
    the reference: stream_llm -> vertical_and_slash with its own sizes, block_sparse ->
    vertical_and_slash (1000, 6096).  -> (type, v, s, score)."""
    scores = search_pattern_scores(q, k, candidates, row_begin)
    best_ty, best_v, best_s, best = "", 0, 0, 0.0
    for (ty, v_size, s_size), sc in zip(candidates, scores):
        if sc > best:
            best_ty, best_v, best_s, best = ty, v_size, s_size, sc
    if best_ty == "stream_llm":
        best_ty = "vertical_and_slash"
    if best_ty == "block_sparse":
        best_ty, best_v, best_s = "vertical_and_slash", 1000, 6096
    return best_ty, best_v, best_s, best
