"""The three sparse prefill attention operators, host side.

Same callables, argument names and defaults as the reference package
(minference/__init__.py:9-11):

* ``vertical_slash_sparse_attention``  minference/ops/pit_sparse_flash_attention_v2.py:195-242
* ``block_sparse_attention``           minference/ops/block_sparse_flash_attention.py:169-186
* ``streaming_forward``                minference/ops/streaming_kernel.py:611-646

Inputs are ``[batch, heads, n, head_dim]`` GPU tensors (any strides); the
result is a new tensor of the query's shape and dtype.  In addition to the
reference, K/V may have fewer heads than Q (grouped-query attention) and are
then read in place instead of being expanded.  All arithmetic runs in
libminf_hip.so on the caller's current stream; torch is only used for memory,
and the index sort of the vertical-slash wrapper.
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib
from .index import convert_vertical_slash_indexes

_NATIVE_D = (64, 128)         # head_dims every kernel is instantiated for; others are zero-padded up
_NATIVE_D_STREAMING = (64, 128, 256)   # ... and the A-shape / tri-shape / dense kernels also for 256


def _prep(t: torch.Tensor) -> torch.Tensor:
    """16-byte aligned rows with unit head_dim stride (copies only if needed)."""
    if t.stride(-1) != 1 or any(s % 8 for s in t.stride()[:-1]) or t.data_ptr() % 16:
        t = t.contiguous()
    return t


_F16_SAFE_ABS = 32768.0
_F16_TINY_ABS = 2.0 ** -10


def _narrow_fp32(*tensors):
    """16-bit operands for fp32 inputs.  The reference picks fp16 operands for every input that is
    not bf16 (pit_sparse_flash_attention_v2.py:175: ``tl.float16``; :99 and :123 cast q and p to
    it), with fp32 accumulation.  Here fp32 tensors are narrowed to fp16 as well, unless the values
    do not fit that format: when some |value| exceeds 32768 (fp16 would overflow) or the largest
    |value| is below 2^-10 (fp16 would flush most of the tensor to zero or to subnormals) they are
    narrowed to bf16 instead, which has fp32's exponent range and 8 mantissa bits.  The decision
    costs one max-abs reduction and ONE HOST READ (a stream synchronisation) per call: the fp32 path
    is the reference's CPU-checkable case, not the serving path.  Accumulation, softmax statistics
    and the scale stay fp32 either way."""
    amax = torch.stack([torch.linalg.vector_norm(t.reshape(-1).float(), float("inf")) if t.numel() else
                        torch.ones((), device=t.device) for t in tensors]).max().item()
    fits = _F16_TINY_ABS <= amax <= _F16_SAFE_ABS                        # (NaN / inf -> bf16)
    dt = torch.float16 if fits else torch.bfloat16
    return tuple(t.to(dt) for t in tensors)


def _check_qkv(q, k, v):
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be [batch, heads, n, head_dim]")
    if k.shape != v.shape or q.shape[0] != k.shape[0] or q.shape[2:] != k.shape[2:]:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    if q.shape[1] % k.shape[1] != 0:
        raise ValueError("query heads must be a multiple of key/value heads")
    if not (q.dtype == k.dtype == v.dtype):
        raise ValueError("q, k, v must share a dtype")
    if not q.is_cuda:
        raise RuntimeError("sparse attention operators need GPU tensors (there is no CPU path)")


class _Call:
    """Holds the (possibly cast/padded) tensors of one operator call and the
    filled ``minf_qkvo`` struct."""

    def __init__(self, q, k, v, seqlens=None, need_out=True, native_dims=_NATIVE_D, sm_scale=None):
        _check_qkv(q, k, v)
        self.out_dtype = q.dtype
        self.head_dim = q.shape[-1]
        if q.dtype == torch.float32:
            # the tile engine computes on 16-bit operands with fp32 accumulation
            q, k, v = _narrow_fp32(q, k, v)
        elif q.dtype not in (torch.bfloat16, torch.float16):
            raise ValueError(f"unsupported dtype {q.dtype}")
        D = q.shape[-1]
        if D > max(native_dims):
            # the reference's vertical-slash and block-sparse kernels assert head_dim <= 128
            # (pit_sparse_flash_attention_v2.py:172, block_sparse_flash_attention.py:128), its streaming
            # kernel head_dim <= 256 (streaming_kernel.py:429)
            raise ValueError(f"head_dim {D} > {max(native_dims)} is not supported by this operator")
        # the reference runs head_dim 16, 32, 64, 128 (pit_sparse_flash_attention_v2.py:172); here 64 and
        # 128 (and 256 for the streaming operators) are native, anything else is zero-padded to the next
        Dk = min(d for d in native_dims if d >= D)
        if D < Dk:
            # zero columns change neither q.k nor the first D output columns
            pad = Dk - D
            q = torch.nn.functional.pad(q, [0, pad])
            k = torch.nn.functional.pad(k, [0, pad])
            v = torch.nn.functional.pad(v, [0, pad])
        self.kernel_dim = Dk
        self.q, self.k, self.v = _prep(q), _prep(k), _prep(v)
        B, H, N, _ = self.q.shape
        self.B, self.H, self.N, self.Hk = B, H, N, self.k.shape[1]
        self.o = torch.empty((B, H, N, Dk) if need_out else (1, 1, 1, Dk),
                             dtype=self.q.dtype, device=q.device)
        s = _lib.QKVO()
        s.q, s.k, s.v, s.o = self.q.data_ptr(), self.k.data_ptr(), self.v.data_ptr(), self.o.data_ptr()
        for name, t in (("q_stride", self.q), ("k_stride", self.k), ("v_stride", self.v), ("o_stride", self.o)):
            getattr(s, name)[:] = list(t.stride()[:3])
        s.batch, s.heads_q, s.heads_kv, s.n = B, H, self.Hk, N
        s.head_dim = Dk
        s.dtype = _lib.MINF_BF16 if self.q.dtype == torch.bfloat16 else _lib.MINF_F16
        self.seqlens = seqlens
        s.seqlens = seqlens.data_ptr() if seqlens is not None else None
        s.sm_scale = float(self.head_dim) ** -0.5 if sm_scale is None else float(sm_scale)
        self.struct = s

    @property
    def ref(self):
        return ctypes.byref(self.struct)

    def select_heads(self, head_list=None):
        """Restrict the following launches to the query heads in head_list (int32 device tensor of
        distinct head numbers; head_list[i] reads head position i of the index tensors).  None = all
        heads again.  The output buffer is shared, so one launch per pattern type fills its heads in
        place."""
        self._head_list = head_list                       # keeps the tensor alive
        self.struct.head_list = head_list.data_ptr() if head_list is not None else None
        self.struct.index_heads = int(head_list.numel()) if head_list is not None else 0

    def result(self):
        o = self.o
        if self.head_dim != self.kernel_dim:
            o = o[..., : self.head_dim]
        if o.dtype != self.out_dtype:
            o = o.to(self.out_dtype)
        return o


def vertical_slash_attention_from_index(query, key, value, block_count, block_offset,
                                        column_count, column_index, seqlens=None):
    """Mixed block + column sparse attention over prebuilt index tensors
    (counterpart of _triton_mixed_sparse_attention, pit_sparse_flash_attention_v2.py:156-192)."""
    c = _Call(query, key, value, seqlens)
    rows = (c.N + 63) // 64
    for t in (block_count, block_offset, column_count, column_index):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise ValueError("index tensors must be contiguous int32")
    if tuple(block_count.shape) != (c.B, c.H, rows) or tuple(block_offset.shape[:3]) != (c.B, c.H, rows) \
            or tuple(column_index.shape[:3]) != (c.B, c.H, rows):
        raise ValueError("index tensors must be [batch, heads_q, ceil(n/64), ...]")
    lib = _lib.load()
    with torch.cuda.device(c.q.device):
        st = lib.minf_vs_attn_fwd(c.ref, block_count.data_ptr(), block_offset.data_ptr(),
                                  column_count.data_ptr(), column_index.data_ptr(), rows,
                                  block_offset.shape[-1], column_index.shape[-1],
                                  _lib.stream_ptr(c.q.device))
    _lib.check(st, "minf_vs_attn_fwd")
    return c.result()


def vertical_slash_sparse_attention(query, key, value, v_idx, s_idx, block_size_M: int = 64,
                                    block_size_N: int = 64):
    """Vertical-slash sparse attention (pit_sparse_flash_attention_v2.py:195-242).

    v_idx: key positions kept for every query, s_idx: diagonal offsets
    (q_pos - k_pos) kept; any integer dtype, unsorted, shapes that reshape to
    [batch, heads, nnz]."""
    if block_size_M != 64 or block_size_N != 64:
        raise ValueError("only 64x64 blocks are supported")
    _check_qkv(query, key, value)
    B, H, N, _ = query.shape
    v_idx = v_idx.to(torch.int32).reshape((B, H, -1)).sort(dim=-1, descending=False)[0]
    s_idx = s_idx.to(torch.int32).reshape((B, H, -1)).sort(dim=-1, descending=True)[0]
    seqlens = torch.full((B,), N, dtype=torch.int32, device=query.device)
    bc, bo, cc, ci = convert_vertical_slash_indexes(seqlens, v_idx, s_idx, N, block_size_M,
                                                    block_size_N, zero_fill=False)
    return vertical_slash_attention_from_index(query, key, value, bc, bo, cc, ci, seqlens)


def block_sparse_attention_from_index(query, key, value, block_index):
    """Block-sparse attention over a prebuilt [batch, heads, rows, max_blocks] int32 block
    list (counterpart of _triton_block_sparse_attention, block_sparse_flash_attention.py:115-148)."""
    c = _Call(query, key, value)
    if block_index.dtype != torch.int32 or not block_index.is_contiguous() or block_index.dim() != 4:
        raise ValueError("block_index must be a contiguous int32 [batch, heads, rows, max_blocks] tensor")
    if block_index.shape[0] != c.B or block_index.shape[1] != c.H or block_index.shape[2] < (c.N + 63) // 64:
        raise ValueError("block_index has the wrong batch/head/row sizes")
    lib = _lib.load()
    with torch.cuda.device(c.q.device):
        st = lib.minf_bs_attn_fwd(c.ref, block_index.data_ptr(), block_index.shape[2],
                                  block_index.shape[3], _lib.stream_ptr(c.q.device))
    _lib.check(st, "minf_bs_attn_fwd")
    return c.result()


def _build_block_index(query, key, top_k, block_size_M=64, block_size_N=64, force_diag_first=False,
                       reference_rounding=None):
    """Top-k key blocks per query block from mean-pooled Q/K
    (block_sparse_flash_attention.py:151-166, including the zero padding its caller applies at
    :178-180).  Pooling, block scores (fp32 matrix cores) and the top-k all run in libminf_hip.so;
    K may have fewer heads than Q.  Returns int32 [batch, heads_q, rows, min(top_k, rows)] with
    rows = (n + 64 - n % 64) / 64, every row ascending.  ``reference_rounding``: None = like the
    reference (bf16/fp16 inputs: pooled means and pooled products rounded to the input dtype, the
    dtype its ``mean`` and ``einsum`` return; fp32 inputs: not), False = fp32 arithmetic."""
    if block_size_M != 64 or block_size_N != 64:
        raise ValueError("only 64x64 blocks are supported")
    from .estimate import reference_rounding_for
    flags = (_lib.MINF_BS_FORCE_DIAG_FIRST if force_diag_first else 0) | \
            (_lib.MINF_BS_ROUND_INPUT_DTYPE if reference_rounding_for(query.dtype, reference_rounding) else 0)
    c = _Call(query, key, key, need_out=False)
    lib = _lib.load()
    rows = lib.minf_bs_block_index_rows(c.N)
    kk = min(int(top_k), rows)
    if kk <= 0:
        raise ValueError("top_k must be positive")
    ws_bytes = lib.minf_bs_block_index_workspace_bytes(c.B, c.H, c.Hk, c.N)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=c.q.device)
    out = torch.empty((c.B, c.H, rows, kk), dtype=torch.int32, device=c.q.device)
    qs = (ctypes.c_int64 * 3)(*c.q.stride()[:3])
    ks = (ctypes.c_int64 * 3)(*c.k.stride()[:3])
    with torch.cuda.device(c.q.device):
        st = lib.minf_bs_block_index(c.q.data_ptr(), c.k.data_ptr(), qs, ks, c.B, c.H, c.Hk, c.N,
                                     c.kernel_dim, c.struct.dtype, int(top_k), flags,
                                     out.data_ptr(), ws.data_ptr(), ws_bytes, _lib.stream_ptr(c.q.device))
    _lib.check(st, "minf_bs_block_index")
    return out


def block_sparse_attention(query, key, value, top_k: int, block_size_M: int = 64, block_size_N: int = 64):
    """Top-k block-sparse attention (block_sparse_flash_attention.py:169-186)."""
    if block_size_M != 64 or block_size_N != 64:
        raise ValueError("only 64x64 blocks are supported")
    _check_qkv(query, key, value)
    block_index = _build_block_index(query, key, top_k, block_size_M, block_size_N)
    return block_sparse_attention_from_index(query, key, value, block_index)


def _streaming_scale(head_dim: int) -> float:
    """Softmax scale of the reference's streaming operator: it zero-pads a head_dim outside
    {16, 32, 64, 128, 256} to the next power of two FIRST (streaming_kernel.py:621-626, :793-797) and
    then scales by 1/sqrt of the padded size (:575) -- e.g. head_dim 96 is scaled by 128^-0.5."""
    d = int(head_dim)
    if d not in (16, 32, 64, 128, 256):
        d = 1 << (d - 1).bit_length()
    return float(d) ** -0.5


def streaming_forward(q, k, v, n_init: int, n_local: int):
    """A-shape attention: n_init sink tokens + a sliding window of n_local
    (streaming_kernel.py:611-646), in one pass.  head_dim up to 256 like the reference (:429); the
    scale follows the reference's padded head_dim (see _streaming_scale)."""
    c = _Call(q, k, v, native_dims=_NATIVE_D_STREAMING, sm_scale=_streaming_scale(q.shape[-1]))
    lib = _lib.load()
    with torch.cuda.device(c.q.device):
        st = lib.minf_ashape_attn_fwd(c.ref, int(n_init), int(n_local), _lib.stream_ptr(c.q.device))
    _lib.check(st, "minf_ashape_attn_fwd")
    return c.result()


def tri_shape_forward(q, k, v, n_init: int, n_local: int, n_last: int = 100):
    """Tri-shape attention: A-shape (n_init sink tokens + window of n_local) for all but the last
    n_last query rows, dense causal attention for those (streaming_kernel.py:820-833,
    minference_forward.py:444-455), in one launch.  Like the reference, the A-shape rows are scaled
    by the padded head_dim (see _streaming_scale) and the last rows by head_dim^-0.5 (:826)."""
    c = _Call(q, k, v, native_dims=_NATIVE_D_STREAMING, sm_scale=_streaming_scale(q.shape[-1]))
    n_last = min(int(n_last), c.N - 1)                   # reference: min(n_last, q.size(2) - 1)
    lib = _lib.load()
    with torch.cuda.device(c.q.device):
        st = lib.minf_trishape_attn_fwd(c.ref, int(n_init), int(n_local), max(n_last, 0),
                                        float(c.head_dim) ** -0.5, _lib.stream_ptr(c.q.device))
    _lib.check(st, "minf_trishape_attn_fwd")
    return c.result()


def dense_causal_attention(q, k, v):
    """Dense causal attention on the same tile engine (comparator for speed-up figures)."""
    c = _Call(q, k, v, native_dims=_NATIVE_D_STREAMING)
    lib = _lib.load()
    with torch.cuda.device(c.q.device):
        st = lib.minf_dense_attn_fwd(c.ref, _lib.stream_ptr(c.q.device))
    _lib.check(st, "minf_dense_attn_fwd")
    return c.result()
