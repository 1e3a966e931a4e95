"""Per-head pattern dispatch for one attention layer -- host side.

Counterpart of ``minference_prefill_kernel`` / ``minference_prefill_forward``
(reference minference/modules/minference_forward.py:594-674) with the same
``prefill_kwargs`` dictionary: ``layer_idx`` and ``attn_forward_config`` with
``best_pattern`` (list over layers of ``{"<head>": [type, vertical_size,
slash_size, score]}``), ``starting_layer``, ``minference_ratio`` and the search mode
(``is_search``, ``config_path``, with ``num_hidden_layers`` in ``prefill_kwargs``).  Heads are
grouped by pattern TYPE and every type is one batched launch chain over the original tensors
(per-head sizes are ragged inside the chain; nothing is gathered or scattered) instead of the
reference's Python loop over heads.  K/V may have fewer heads than Q (no repeat_kv needed).
"""
from __future__ import annotations

import json
import os
from collections import OrderedDict

import torch

from .estimate import estimate_vertical_slash
from .index import convert_vertical_slash_indexes
from .ops import (block_sparse_attention, dense_causal_attention, streaming_forward, tri_shape_forward,
                  vertical_slash_attention_from_index, vertical_slash_sparse_attention)

DEFAULT_PATTERN = ("vertical_and_slash", 1000, 6096, 1)   # minference_forward.py:621


def vertical_slash_prefill(q, k, v, vertical_size=1000, slash_size=6096):
    """estimate -> top-k -> index build -> mixed sparse attention for all heads of ``q``
    (``vertical_and_slash_kernel``, minference_forward.py:599-614)."""
    B, H, N, _ = q.shape
    v_idx, s_idx = estimate_vertical_slash(q, k, vertical_size, slash_size)
    seqlens = torch.full((B,), N, dtype=torch.int32, device=q.device)
    bc, bo, cc, ci = convert_vertical_slash_indexes(seqlens, v_idx, s_idx, N, 64, 64, zero_fill=False)
    return vertical_slash_attention_from_index(q, k, v, bc, bo, cc, ci, seqlens)


def load_best_pattern(path):
    """Read a per-model pattern file (same JSON format as minference/configs/*.json)."""
    with open(path) as f:
        return json.load(f)


def _head_plan(config, layer_idx, num_heads):
    """-> {(type, vertical_size, slash_size): [head ids]} following :621-625."""
    best = config.get("best_pattern")
    layer = best[layer_idx] if best is not None else {}
    plan = {}
    for h in range(num_heads):
        ty, vs, ss, _ = layer.get(str(h), DEFAULT_PATTERN)
        if "minference_ratio" in config:
            ratio = config.get("minference_ratio", 1)
            vs, ss = int(vs * ratio), int(ss * ratio)
        plan.setdefault((ty, int(vs), int(ss)), []).append(h)
    return plan


VERTICAL_PAD = 0x3FFFFFFF      # a vertical index no range ever reaches: never emitted by the index builder


class _LayerPlan:
    """What a layer's pattern table fixes once and for all: the parsed plan and, per (batch, tokens,
    device), the small device tensors its launch chains read (head lists, per-head top-k sizes).
    The reference parses the table and copies ``[context_size]`` to the device on every call of
    every head (minference_forward.py:621-625, pit_sparse_flash_attention_v2.py:220); here a layer's
    second call issues no host-to-device copy at all."""

    def __init__(self, config, layer_idx, num_heads):
        self.pattern = config.get("best_pattern")          # pins the object whose id() is the cache key
        self.plan = _head_plan(config, layer_idx, num_heads)
        self.num_heads = num_heads
        ok = ("vertical_and_slash", "block_sparse", "stream_llm")
        for (ty, _, _) in self.plan:
            if ty not in ok:
                raise KeyError(ty)
        self.vs = sorted((h, v, s) for (ty, v, s), hs in self.plan.items() if ty == "vertical_and_slash" for h in hs)
        self.bs = sorted(h for (ty, _, _), hs in self.plan.items() if ty == "block_sparse" for h in hs)
        self.stream = {}
        for (ty, v, s), hs in self.plan.items():
            if ty == "stream_llm":
                self.stream.setdefault((v, s), []).extend(hs)
        covered = len(self.vs) + len(self.bs) + sum(len(hs) for hs in self.stream.values())
        if covered != num_heads:
            # the shared output buffer is torch.empty: a head without a launch would return garbage
            raise ValueError(f"pattern table covers {covered} of {num_heads} heads")
        self._dev = {}

    def device_tensors(self, B, N, dev):
        """-> dict of int32 device tensors for this (batch, tokens, device), built on first use."""
        key = (B, N, str(dev))
        d = self._dev.get(key)
        if d is None:
            d = {}
            if self.vs:
                # sizes clamped like the reference (:600)
                kv = [min(N, max(int(v), 30)) for _, v, _ in self.vs]
                ksl = [min(N, max(int(s), 50)) for _, _, s in self.vs]
                d["vs_heads"] = _head_list([h for h, _, _ in self.vs], dev)
                d["vs_kv"] = torch.tensor(kv * B, dtype=torch.int32).to(dev)
                d["vs_ks"] = torch.tensor(ksl * B, dtype=torch.int32).to(dev)
                d["vs_max"] = (max(kv), max(ksl))
            if self.bs:
                d["bs_heads"] = _head_list(self.bs, dev)
            d["stream_heads"] = {key2: _head_list(hs, dev) for key2, hs in self.stream.items()}
            if len(self._dev) >= 8:                        # a few prompt lengths per layer at most
                self._dev.pop(next(iter(self._dev)))
            self._dev[key] = d
        return d


_PLAN_CACHE = OrderedDict()
_PLAN_CACHE_MAX = 512          # layers x tables held; the least recently used entry goes first


def _layer_plan(config, layer_idx, num_heads):
    """The cached _LayerPlan of (pattern table object, layer, head count, ratio)."""
    best = config.get("best_pattern")
    key = (id(best), layer_idx, num_heads, config.get("minference_ratio") if "minference_ratio" in config else None)
    lp = _PLAN_CACHE.get(key)
    if lp is not None and lp.pattern is best:
        _PLAN_CACHE.move_to_end(key)
        return lp
    lp = _LayerPlan(config, layer_idx, num_heads)
    _PLAN_CACHE[key] = lp
    while len(_PLAN_CACHE) > _PLAN_CACHE_MAX:
        _PLAN_CACHE.popitem(last=False)
    return lp


def clear_plan_cache():
    """Forget every cached layer plan.  A pattern table is treated as immutable once a layer has
    used it; call this after editing a ``best_pattern`` list in place."""
    _PLAN_CACHE.clear()


def _head_list(heads, device):
    """int32 device tensor of the (ascending) query head numbers of one pattern group."""
    return torch.tensor(sorted(heads), dtype=torch.int32).to(device)


def _mixed_layer(query_states, key_states, value_states, lp):
    """All heads of a layer whose pattern table mixes types and sizes (``lp``: its _LayerPlan): q/k/v
    are prepared once, the output is one shared buffer, and every pattern type is ONE launch chain
    over the original tensors with a head selection -- no gathered copies of Q, no scattered writes
    of O:

    * vertical_and_slash heads with any mix of (vertical_size, slash_size): one estimation over those
      heads, one ragged top-k (every head keeps its own sizes; shorter lists are padded with entries
      that are no-ops of the index builder's merge), one index build, one attention launch;
    * block_sparse heads: one block index + one attention launch;
    * stream_llm heads: one launch per distinct (n_init, n_local).

    The reference runs one operator call per head here (minference_forward.py:657-667)."""
    from . import _lib
    from .estimate import FORCE_SLASH, FORCE_VERTICAL, LAST_Q, reference_rounding_for
    from .ops import _Call, _streaming_scale
    B, H, N, D = query_states.shape
    rounded = reference_rounding_for(query_states.dtype)     # the reference's rounding points on 16-bit inputs
    dev = query_states.device
    c = _Call(query_states, key_states, value_states)
    lib = _lib.load()
    stream = _lib.stream_ptr(dev)
    i64x3 = _lib.c_i64 * 3
    qs, ks = i64x3(*c.q.stride()[:3]), i64x3(*c.k.stride()[:3])
    rows = (N + 63) // 64
    keep = []                                             # tensors the enqueued kernels still read
    dt = lp.device_tensors(B, N, dev)

    try:
        with torch.cuda.device(dev):
            if lp.vs:
                nh = len(lp.vs)
                vmax, smax = dt["vs_max"]
                slot, kv_t, ks_t = dt["vs_heads"], dt["vs_kv"], dt["vs_ks"]
                vertical = torch.empty((B, nh, N), dtype=torch.float32, device=dev)
                slash = torch.empty((B, nh, N), dtype=torch.float32, device=dev)
                ws_bytes = lib.minf_vs_estimate_workspace_bytes(B, nh, N)
                ws = torch.empty((ws_bytes + 15) // 16 * 16, dtype=torch.uint8, device=dev)
                st = lib.minf_vs_estimate_heads(c.q.data_ptr(), c.k.data_ptr(), qs, ks, B, H, c.Hk, N, c.kernel_dim,
                                                c.struct.dtype, float(D) ** -0.5, LAST_Q, FORCE_VERTICAL, FORCE_SLASH,
                                                _lib.MINF_ROUND_INPUT_DTYPE if rounded else _lib.MINF_ROUND_NONE,
                                                slot.data_ptr(), nh, vertical.data_ptr(), slash.data_ptr(),
                                                ws.data_ptr(), ws_bytes, stream)
                _lib.check(st, "minf_vs_estimate_heads")
                v_idx = torch.empty((B, nh, vmax), dtype=torch.int32, device=dev)
                s_idx = torch.empty((B, nh, smax), dtype=torch.int32, device=dev)
                st = lib.minf_topk_indices_pair_ragged(vertical.data_ptr(), kv_t.data_ptr(), vmax, v_idx.data_ptr(), vmax, -1, 1, VERTICAL_PAD,
                                                       slash.data_ptr(), ks_t.data_ptr(), smax, s_idx.data_ptr(), smax, N - 1, 2, 0,
                                                       B * nh, N, N, stream)
                _lib.check(st, "minf_topk_indices_pair_ragged")
                seqlens = torch.full((B,), N, dtype=torch.int32, device=dev)
                bc, bo, cc, ci = convert_vertical_slash_indexes(seqlens, v_idx, s_idx, N, 64, 64, zero_fill=False)
                c.struct.seqlens = seqlens.data_ptr()
                c.select_heads(slot)
                st = lib.minf_vs_attn_fwd(c.ref, bc.data_ptr(), bo.data_ptr(), cc.data_ptr(), ci.data_ptr(), rows,
                                          smax, vmax, stream)
                c.struct.seqlens = None
                _lib.check(st, "minf_vs_attn_fwd")
                keep += [vertical, slash, ws, v_idx, s_idx, seqlens, bc, bo, cc, ci]
            if lp.bs:
                nh = len(lp.bs)
                slot = dt["bs_heads"]
                brows = lib.minf_bs_block_index_rows(N)
                kk = min(100, brows)                          # top_k fixed at 100 (:616-618)
                ws_bytes = lib.minf_bs_block_index_workspace_bytes(B, nh, c.Hk, N)
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
                bi = torch.empty((B, nh, brows, kk), dtype=torch.int32, device=dev)
                st = lib.minf_bs_block_index_heads(c.q.data_ptr(), c.k.data_ptr(), qs, ks, B, H, c.Hk, N, c.kernel_dim,
                                                   c.struct.dtype, 100, _lib.MINF_BS_ROUND_INPUT_DTYPE if rounded else 0,
                                                   slot.data_ptr(), nh, bi.data_ptr(),
                                                   ws.data_ptr(), ws_bytes, stream)
                _lib.check(st, "minf_bs_block_index_heads")
                c.select_heads(slot)
                st = lib.minf_bs_attn_fwd(c.ref, bi.data_ptr(), brows, kk, stream)
                _lib.check(st, "minf_bs_attn_fwd")
                keep += [ws, bi]
            # (the reference's streaming operator scales by the power-of-two padded head_dim)
            c.struct.sm_scale = _streaming_scale(D)
            for (n_init, n_local), slot in dt["stream_heads"].items():
                c.select_heads(slot)
                if N > 0:
                    st = lib.minf_ashape_attn_fwd(c.ref, int(n_init), int(n_local), stream)
                    _lib.check(st, "minf_ashape_attn_fwd")
    finally:
        c.struct.seqlens = None
        c.struct.sm_scale = float(D) ** -0.5
        c.select_heads(None)
    out = c.result()
    # torch's caching allocator hands a freed block only to work enqueued later on the same stream, so
    # dropping `keep` here is safe for kernels that are still running
    del keep
    return out


def minference_prefill_kernel(q, k, v, pattern, vertical_size, slash_size):
    """One pattern for all heads of q (minference_forward.py:626-631; for ``stream_llm`` the
    two sizes are n_init and n_local, as in the reference)."""
    if pattern == "stream_llm":
        return streaming_forward(q, k, v, vertical_size, slash_size)
    if pattern == "vertical_and_slash":
        return vertical_slash_prefill(q, k, v, vertical_size, slash_size)
    if pattern == "block_sparse":
        return block_sparse_attention(q, k, v, 100)     # top_k fixed at 100 (:616-618)
    raise KeyError(pattern)


def _search_layer(query_states, key_states, value_states, prefill_kwargs):
    """Search mode (minference_forward.py:644-673): the layer's per-head patterns are searched
    and appended to the JSON list at ``config_path`` (one ``{head: [type, v, s, score]}`` object
    per layer, in layer order), and the layer's output is dense causal attention.  A file that
    already holds ``num_hidden_layers`` layers raises, like the reference; layers the file
    already holds are not searched again."""
    from .search import search_patterns
    config = prefill_kwargs["attn_forward_config"]
    layer_idx = prefill_kwargs["layer_idx"]
    config_path = config.get("config_path", None)
    config_list = []
    if config_path and os.path.isfile(config_path):
        with open(config_path) as f:
            config_list = json.load(f)
        if len(config_list) == prefill_kwargs.get("num_hidden_layers", -1):
            raise RuntimeError(f"Search already completed; see {config_path}.")
    if layer_idx >= len(config_list):
        new_config = search_patterns(query_states, key_states)
        if config_path:
            config_list.append(new_config)
            with open(config_path, "w") as f:
                json.dump(config_list, f, indent=2)
    return dense_causal_attention(query_states, key_states, value_states)


def minference_prefill_forward(query_states, key_states, value_states, prefill_kwargs):
    """Sparse prefill attention of one layer: [B,Hq,N,D] x [B,Hk,N,D] -> [B,Hq,N,D]."""
    config = prefill_kwargs["attn_forward_config"]
    layer_idx = prefill_kwargs["layer_idx"]
    starting_layer = config.get("starting_layer", 0)
    B, H, N, D = query_states.shape
    group = H // key_states.shape[1]
    if config.get("is_search", False):
        return _search_layer(query_states, key_states, value_states, prefill_kwargs)
    if layer_idx < starting_layer:
        return dense_causal_attention(query_states, key_states, value_states)
    lp = _layer_plan(config, layer_idx, H)
    if len(lp.plan) == 1:
        (ty, vs, ss), _ = next(iter(lp.plan.items()))
        return minference_prefill_kernel(query_states, key_states, value_states, ty, vs, ss)
    return _mixed_layer(query_states, key_states, value_states, lp)


def a_shape_kernel(query_states, key_states, value_states, prefill_kwargs):
    """A-shape (sink + sliding window) attention with n_init (128) / n_local (3968) taken from
    ``attn_forward_config`` (reference minference/ops/streaming_kernel.py:781-818)."""
    cfg = prefill_kwargs["attn_forward_config"]
    return streaming_forward(query_states, key_states, value_states, cfg.get("n_init", 128),
                             cfg.get("n_local", 3968))


def tri_shape_kernel(query_states, key_states, value_states, prefill_kwargs):
    """Tri-shape attention with n_init / n_local / n_last taken from ``attn_forward_config``
    (the dispatcher-level wrapper the reference's tri_mix module calls, modules/tri_mix.py:35-37)."""
    cfg = prefill_kwargs["attn_forward_config"]
    return tri_shape_forward(query_states, key_states, value_states, cfg.get("n_init", 128),
                             cfg.get("n_local", 3968), cfg.get("n_last", 100))


def tri_mix_forward(query_states, key_states, value_states, prefill_kwargs):
    """modules/tri_mix.py:19-39: dense causal attention below ``starting_layer``, tri-shape from there on."""
    if prefill_kwargs["layer_idx"] < prefill_kwargs["attn_forward_config"].get("starting_layer", 0):
        return dense_causal_attention(query_states, key_states, value_states)
    return tri_shape_kernel(query_states, key_states, value_states, prefill_kwargs)


def tri_mix_minference_forward(query_states, key_states, value_states, prefill_kwargs):
    """modules/tri_mix.py:42-53: the per-head sparse patterns below ``starting_layer``, tri-shape from
    there on."""
    cfg = prefill_kwargs["attn_forward_config"]
    if prefill_kwargs["layer_idx"] < cfg.get("starting_layer", 0):
        inner = dict(prefill_kwargs)
        inner["attn_forward_config"] = dict(cfg, starting_layer=0)
        return minference_prefill_forward(query_states, key_states, value_states, inner)
    return tri_shape_kernel(query_states, key_states, value_states, prefill_kwargs)


def dilated_forward(q, k, v, kind):
    """The fixed "dilated" baselines of the reference (minference_forward.py:365-379): the first
    min(1024, N) columns plus, for ``dilated1``, every second diagonal of the last 8192 offsets'
    worth of positions, for ``dilated2`` the last 2048 diagonals and every second one of the 4096
    before them -- expressed, as in the reference, through the vertical-slash operator."""
    n = q.shape[2]
    dev = q.device
    vertical = torch.arange(0, min(1024, n), device=dev, dtype=torch.int32)[None, None, :]
    pos = torch.arange(0, n, device=dev, dtype=torch.int32)
    if kind == "dilated1":
        pos = pos[-8192::2]
    elif kind == "dilated2":
        pos = torch.cat([pos[-2048:], pos[-6144:-2048:2]], 0)
    else:
        raise KeyError(kind)
    slash = (n - 1) - pos[None, None, :]
    B, H = q.shape[:2]
    return vertical_slash_sparse_attention(q, k, v, vertical.expand(B, H, -1), slash.expand(B, H, -1))


def static_vertical_slash_forward(q, k, v, vertical_size, slash_size, cache):
    """The "static pattern" baseline (minference_forward.py:418-434, 476-477): the vertical and
    slash indices are estimated on the first prompt a layer sees (forcing the first 30 columns and
    the 30 nearest diagonals) and reused for every later one; ``cache`` is that layer's dictionary."""
    from .estimate import topk_vertical_slash, vertical_slash_scores
    if "vs" not in cache:
        n = q.shape[2]
        vsz, ssz = min(n, max(int(vertical_size), 30)), min(n, max(int(slash_size), 50))
        vertical, slash = vertical_slash_scores(q, k, 64, 30, 30)
        cache["vs"] = topk_vertical_slash(vertical, slash, vsz, ssz)
    v_idx, s_idx = cache["vs"]
    return vertical_slash_sparse_attention(q, k, v, v_idx, s_idx)
