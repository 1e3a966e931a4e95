"""Seeded synthetic inputs shared by the tests and bench.py (generated on the
CPU so that every box sees identical bits)."""
from __future__ import annotations

import numpy as np
import torch


def vs_index_inputs(heads, n, nnz_v, nnz_s, seed, batch=1, force_v=4, force_s=64):
    """Sorted random vertical (ascending, always containing 0..force_v-1) and
    slash (descending, always containing 0..force_s-1) index lists, int32."""
    v = np.empty((batch, heads, nnz_v), np.int32)
    s = np.empty((batch, heads, nnz_s), np.int32)
    for b in range(batch):
        for h in range(heads):
            rng = np.random.default_rng(seed + 1000 * b + h)
            fv = min(force_v, nnz_v, n)
            fs = min(force_s, nnz_s, n)
            rv = rng.choice(np.arange(fv, n), size=nnz_v - fv, replace=False) if nnz_v > fv else np.empty(0, np.int64)
            rs = rng.choice(np.arange(fs, n), size=nnz_s - fs, replace=False) if nnz_s > fs else np.empty(0, np.int64)
            v[b, h] = np.sort(np.concatenate([np.arange(fv), rv]))
            s[b, h] = np.sort(np.concatenate([np.arange(fs), rs]))[::-1]
    return v, s


def qkv(batch, hq, hk, n, d, seed, dtype=torch.float32, scale=None):
    g = torch.Generator().manual_seed(seed)
    sc = (d ** -0.5) if scale is None else scale
    q = (torch.randn(batch, hq, n, d, generator=g) * sc).to(dtype)
    k = (torch.randn(batch, hk, n, d, generator=g) * sc).to(dtype)
    v = (torch.randn(batch, hk, n, d, generator=g) * sc).to(dtype)
    return q, k, v
