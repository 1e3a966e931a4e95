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


# ---------------------------------------------------------------------------
# BASELINE config 2/4: Llama-3-8B-1M attention layer with planted structure
# ---------------------------------------------------------------------------
def _moving_average(x, w):
    """Causal moving average of width w along dim 0 (x [N, D]), unit variance per entry."""
    n = x.shape[0]
    c = torch.cumsum(x.double(), 0)
    out = c.clone()
    out[w:] = c[w:] - c[:-w]
    return (out / (min(w, n) ** 0.5)).float()


def planted_layer(n, hq=32, hk=8, d=128, seed=100, dtype=torch.bfloat16, device="cpu",
                  sink_logit=7.5, heavy_logit=4.0, n_heavy=32, band_logit=2.0, band_width=512,
                  decay_per_token=2.0 ** -7 / 128 ** 0.5):
    """Synthetic q [1,hq,n,d], k/v [1,hk,n,d] for BASELINE configs 2 and 4.

    * base: N(0,1) entries (q.k/sqrt(d) has std ~1);
    * local band: a smooth vector process z_t (causal moving average of white noise, width
      band_width) is added to Q and K of a kv group, so q_t.k_s/sqrt(d) gains about
      band_logit * max(0, 1 - |t-s|/band_width);
    * long-range decay: three dims of every q/k row are replaced by an exact positional code
      (key position in base-128 digits, query side constants, all powers of two, exact in
      bf16) that adds  +decay_per_token * s  to the logit of key s -- attention mass falls
      off as exp(-decay * distance) (6.9e-4/token: a factor 2 per 1000 tokens), as it does in
      trained long-context heads.  Without such a decay the far diagonals differ only by
      noise and the top-6096 of them scatter over the whole context (~98% of the causal area
      covered at 128K), so nothing would be sparse;
    * per kv head, along a unit direction u shared by its query heads: the first 4 keys get
      +sink_logit (attention sink) and n_heavy random keys get +heavy_logit;
    * V is N(0,1).
    Returns (q, k, v, meta)."""
    assert d == 128 and n <= 128 ** 3
    group = hq // hk
    sd = d ** 0.5
    q = torch.empty(1, hq, n, d, dtype=dtype, device=device)
    k = torch.empty(1, hk, n, d, dtype=dtype, device=device)
    v = torch.empty(1, hk, n, d, dtype=dtype, device=device)
    meta = {"seed": seed, "sink_logit": sink_logit, "heavy_logit": heavy_logit,
            "band_logit": band_logit, "band_width": band_width,
            "decay_per_token": decay_per_token, "heavy": []}
    pos = torch.arange(n)
    digits = torch.stack([pos // 16384, (pos // 128) % 128, pos % 128], 1).float()   # [n, 3]
    c0 = decay_per_token * sd                      # query-side constant of the lowest digit
    qconst = torch.tensor([c0 * 16384, c0 * 128, c0])
    for j in range(hk):
        g = torch.Generator().manual_seed(seed + j)
        u = torch.randn(d, generator=g)
        u[-3:] = 0
        u = u / u.norm()
        heavy = torch.randperm(n - 4, generator=g)[:n_heavy] + 4
        meta["heavy"].append(sorted(heavy.tolist()))
        z = _moving_average(torch.randn(n, d, generator=g), band_width) / sd   # |z_t|^2 ~ 1
        gl = (band_logit * sd) ** 0.5
        a = sd ** 0.5                              # q gets a*u; keys get (logit * sd / a) * u
        kk = torch.randn(n, d, generator=g) + gl * z
        kk[:4] += (sink_logit * sd / a) * u
        kk[heavy] += (heavy_logit * sd / a) * u
        kk[:, -3:] = digits
        k[0, j] = kk.to(dtype).to(device)
        v[0, j] = torch.randn(n, d, generator=g).to(dtype).to(device)
        for i in range(group):
            qq = torch.randn(n, d, generator=g) + gl * z + a * u
            qq[:, -3:] = qconst
            q[0, j * group + i] = qq.to(dtype).to(device)
    return q, k, v, meta
