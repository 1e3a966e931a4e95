"""Online vertical/slash pattern estimation and top-k -- host side.

Counterpart of ``vertical_and_slash_kernel`` inside ``minference_prefill_kernel``
(reference minference/modules/minference_forward.py:599-614): the last 64
queries score all keys; column sums ("vertical") and diagonal sums ("slash") of
the softmax are forced/top-k'ed into ``v_idx`` / ``s_idx``.  Here it is batched
over all heads of a layer (the reference loops over heads in Python) and runs
in libminf_hip.so; K/V may have fewer heads than Q.
"""
from __future__ import annotations

import torch

from . import _lib
from .ops import _NATIVE_D, _check_qkv, _narrow_fp32, _prep

LAST_Q = 64            # minference_forward.py:41
FORCE_VERTICAL = 30    # :606
FORCE_SLASH = 100      # :610


def _prep16(q, k):
    if q.dtype == torch.float32:
        q, k = _narrow_fp32(q, k)          # fp16 when the values fit, else bf16
    elif q.dtype not in (torch.bfloat16, torch.float16):
        raise ValueError(f"unsupported dtype {q.dtype}")
    d = q.shape[-1]
    if d > max(_NATIVE_D):
        raise ValueError(f"head_dim > {max(_NATIVE_D)} is not supported")
    dk = min(x for x in _NATIVE_D if x >= d)          # the kernels are built for head_dim 64 and 128
    if d != dk:
        q = torch.nn.functional.pad(q, [0, dk - d])
        k = torch.nn.functional.pad(k, [0, dk - d])
    return _prep(q), _prep(k)


def reference_rounding_for(dtype, reference_rounding=None):
    """The rounding mode of the two index selectors: by default (None) the reference's own -- its
    torch code holds the scaled q.k scores and the pooled block means / products in the INPUT dtype
    (minference_forward.py:602, block_sparse_flash_attention.py:159-163), so bf16/fp16 inputs are
    rounded at those points and fp32 inputs are not."""
    if reference_rounding is None:
        reference_rounding = dtype in (torch.bfloat16, torch.float16)
    return bool(reference_rounding) and dtype != torch.float32


def vertical_slash_scores(q, k, last_q=LAST_Q, force_vertical=FORCE_VERTICAL, force_slash=FORCE_SLASH,
                          reference_rounding=None):
    """-> (vertical [B,H,N], slash [B,H,N]) fp32 score vectors.  ``slash[..., j]`` is the
    probability mass on the diagonal with offset ``N-1-j`` (same indexing as the reference's
    ``sum_all_diagonal_matrix(qk)[..., :-last_q+1]``).  Forced entries are +inf.
    ``reference_rounding``: None = like the reference (bf16/fp16 inputs: scores rounded to the input
    dtype after the dot product and after the scaling; fp32 inputs: not), False = fp32 arithmetic."""
    _check_qkv(q, k, k)
    rounding = _lib.MINF_ROUND_INPUT_DTYPE if reference_rounding_for(q.dtype, reference_rounding) else _lib.MINF_ROUND_NONE
    head_dim = q.shape[-1]
    q16, k16 = _prep16(q, k)
    B, H, N, _ = q16.shape
    Hk = k16.shape[1]
    lib = _lib.load()
    dev = q16.device
    vertical = torch.empty((B, H, N), dtype=torch.float32, device=dev)
    slash = torch.empty((B, H, N), dtype=torch.float32, device=dev)
    ws_bytes = lib.minf_vs_estimate_workspace_bytes(B, H, N)
    ws = torch.empty((ws_bytes + 15) // 16 * 16, dtype=torch.uint8, device=dev)
    i64x3 = _lib.c_i64 * 3
    with torch.cuda.device(dev):
        st = lib.minf_vs_estimate(
            q16.data_ptr(), k16.data_ptr(), i64x3(*q16.stride()[:3]), i64x3(*k16.stride()[:3]),
            B, H, Hk, N, q16.shape[-1], _lib.MINF_BF16 if q16.dtype == torch.bfloat16 else _lib.MINF_F16,
            float(head_dim) ** -0.5, int(last_q), int(force_vertical), int(force_slash), rounding,
            vertical.data_ptr(), slash.data_ptr(), ws.data_ptr(), ws_bytes, _lib.stream_ptr(dev))
    _lib.check(st, "minf_vs_estimate")
    return vertical, slash


def topk_indices(scores, k, reverse_base=-1):
    """Indices of the k largest entries of each row of ``scores`` [..., N] (fp32, contiguous),
    int32, ascending by index; ties go to the lowest index.  ``reverse_base >= 0`` returns
    ``reverse_base - index`` instead."""
    if scores.dtype != torch.float32 or not scores.is_contiguous():
        raise ValueError("scores must be contiguous fp32")
    n = scores.shape[-1]
    rows = scores.numel() // n
    kk = min(int(k), n)
    out = torch.empty(scores.shape[:-1] + (kk,), dtype=torch.int32, device=scores.device)
    lib = _lib.load()
    with torch.cuda.device(scores.device):
        st = lib.minf_topk_indices(scores.data_ptr(), rows, n, n, kk, out.data_ptr(), kk,
                                   int(reverse_base), _lib.stream_ptr(scores.device))
    _lib.check(st, "minf_topk_indices")
    return out


def estimate_vertical_slash(q, k, vertical_size, slash_size, last_q=LAST_Q,
                            force_vertical=FORCE_VERTICAL, force_slash=FORCE_SLASH, reference_rounding=None):
    """-> (v_idx [B,H,v] int32 ascending key positions, s_idx [B,H,s] int32 descending diagonal
    offsets), already in the order the index builder wants.  Sizes are clamped like the
    reference (:600): v = min(N, max(vertical_size, 30)), s = min(N, max(slash_size, 50))."""
    N = q.shape[2]
    v = min(N, max(int(vertical_size), 30))
    s = min(N, max(int(slash_size), 50))
    vertical, slash = vertical_slash_scores(q, k, last_q, force_vertical, force_slash, reference_rounding)
    return topk_vertical_slash(vertical, slash, v, s)


def topk_vertical_slash(vertical, slash, v, s):
    """Both selections in one launch: -> (v_idx ascending positions, s_idx descending offsets)."""
    B, H, N = vertical.shape
    v, s = min(int(v), N), min(int(s), N)
    v_idx = torch.empty((B, H, v), dtype=torch.int32, device=vertical.device)
    s_idx = torch.empty((B, H, s), dtype=torch.int32, device=vertical.device)
    lib = _lib.load()
    with torch.cuda.device(vertical.device):
        st = lib.minf_topk_indices_pair(vertical.data_ptr(), v, v_idx.data_ptr(), v, -1,
                                        slash.data_ptr(), s, s_idx.data_ptr(), s, N - 1,
                                        B * H, N, N, _lib.stream_ptr(vertical.device))
    _lib.check(st, "minf_topk_indices_pair")
    return v_idx, s_idx
