"""Score profiles chosen against the softmax bookkeeping of the tile engine, every operator, EVERY row.

The engine looks at a row's maximum only now and then and walks a workgroup again when its sums
leave the fp32 range, so what can go wrong depends on how the scores move along the keys: steep
ramps, saw teeth, random walks, sudden steps, isolated spikes, oscillations of changing frequency,
with rows that see the mirror image or a growing gain, and values of any size.  One input dimension
carries the profile (scores of hundreds to thousands of natural-log units); the rest is noise.

Every row of two heads per case is recomputed as an fp32 masked-dense softmax by torch on the GPU
from the index tensors the HIP kernels produced (vertical-slash: listed blocks up to the causal limit
plus listed columns, pit_sparse_flash_attention_v2.py:104-148; block-sparse: the first min(m + 1, k)
listed blocks, block_sparse_flash_attention.py:81-96; A-shape / tri-shape: the closed form of
streaming_kernel.py:35-75).  Tolerance: max-abs 2e-2, mean-abs 1.5e-3 per row block, times
max(1, max|V| / 4)."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import gen

pytestmark = pytest.mark.gpu


def profile_inputs(kind, n, hq, hk, d, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    r = np.random.default_rng(seed)
    q = torch.randn(1, hq, n, d, generator=g) * 0.5
    k = torch.randn(1, hk, n, d, generator=g) * 0.5
    v = torch.randn(1, hk, n, d, generator=g)
    pos = torch.arange(n).float()
    if kind == "steps":
        nj = max(1, n // int(r.integers(40, 600)))
        jumps = torch.zeros(n)
        jumps[torch.from_numpy(r.integers(0, n, nj))] = torch.from_numpy(r.uniform(-200, 200, nj)).float()
        f = torch.cumsum(jumps, 0).clamp(-2000, 2000)
    elif kind == "saw":
        f = (pos % float(r.integers(100, 5000))) / float(r.integers(100, 5000)) * float(r.uniform(50, 600))
    elif kind == "walk":
        f = torch.cumsum(torch.randn(n, generator=g) * float(r.uniform(0.5, 5.0)), 0).clamp(-2500, 2500)
    elif kind == "chirp":
        f = torch.sin(pos * pos / float(r.uniform(2e4, 2e6))) * float(r.uniform(30, 400))
    elif kind == "spikes":
        f = torch.zeros(n)
        cnt = max(1, n // int(r.integers(50, 2000)))
        f[torch.from_numpy(r.integers(0, n, cnt))] = torch.from_numpy(r.uniform(50, 1000, cnt)).float()
    elif kind == "ramp":
        f = (pos * float(r.uniform(0.01, 0.6)) * (1 if r.random() < 0.7 else -1)).clamp(-2500, 2500)
    elif kind == "wave":
        f = torch.sin(2 * math.pi * pos / float(r.choice([200, 512, 2048, 8192]))) * float(r.uniform(40, 300))
    else:
        raise ValueError(kind)
    k[..., 0] = (f * d ** 0.5 / 8.0)[None, None, :]
    q[..., 0] = 8.0
    mode = int(r.integers(0, 3))
    if mode == 1:          # odd rows see the mirror image
        q[:, :, 1::2, 0] = -8.0
    elif mode == 2:        # the gain grows with the row
        q[..., 0] = (4.0 + 8.0 * pos / n)[None, None, :]
    v = v * float(r.choice([1.0, 1.0, 30.0, 1000.0]))
    return q.to(dtype), k.to(dtype), v.to(dtype), r


def _check_head(tag, out_h, q_h, k32, v32, n, mask_of, tol):
    dev = out_h.device
    assert torch.isfinite(out_h.float()).all(), tag
    pos = torch.arange(n, device=dev)
    ar64 = torch.arange(64, device=dev)
    scale = q_h.shape[-1] ** -0.5
    worst = 0.0
    for m in range((n + 63) // 64):
        rows = (m * 64 + ar64)[: min(64, n - m * 64)]
        s = (q_h[rows].float() @ k32.T) * scale
        s = s.masked_fill(~mask_of(m, rows, pos), float("-inf"))
        err = (out_h[rows].float() - torch.softmax(s, dim=-1) @ v32).abs()
        mx, mean = err.max().item(), err.mean().item()
        worst = max(worst, mx)
        assert mx <= 2e-2 * tol and mean <= 1.5e-3 * tol, (tag, m, mx, mean, tol)
    return worst


def _vs_mask(bc, bo, cc, ci, h, n):
    nb, nc = bc[0, h].tolist(), cc[0, h].tolist()
    dev = bo.device
    ar64 = torch.arange(64, device=dev)

    def f(m, rows, pos):
        allowed = torch.zeros(n, dtype=torch.bool, device=dev)
        idx = (bo[0, h, m, :nb[m]].long()[:, None] + ar64[None, :]).reshape(-1)
        allowed[idx[(idx >= 0) & (idx < n)]] = True
        mask = allowed[None, :] & (pos[None, :] <= rows[:, None])
        if nc[m]:
            col = torch.zeros(n, dtype=torch.bool, device=dev)
            col[ci[0, h, m, :nc[m]].long()] = True
            mask = mask | col[None, :]
        return mask
    return f


def _bs_mask(bi, h, n):
    dev = bi.device
    ar64 = torch.arange(64, device=dev)

    def f(m, rows, pos):
        allowed = torch.zeros(n, dtype=torch.bool, device=dev)
        idx = (bi[0, h, m, :min(m + 1, bi.shape[-1])].long()[:, None] * 64 + ar64[None, :]).reshape(-1)
        allowed[idx[(idx >= 0) & (idx < n)]] = True
        return allowed[None, :] & (pos[None, :] <= rows[:, None])
    return f


def _streaming_mask(n_init, n_local, dense_from):
    def f(m, rows, pos):
        i, j = rows[:, None], pos[None, :]
        return (j <= i) & (((i - j) < n_local) | (j < n_init) | (i >= dense_from))
    return f


CASES = [
    ("steps", 9000, 4, 1, 128, torch.bfloat16, 1), ("steps", 23000, 2, 2, 64, torch.bfloat16, 2),
    ("saw", 12345, 2, 1, 128, torch.bfloat16, 3), ("saw", 4000, 8, 2, 64, torch.float16, 4),
    ("walk", 20000, 2, 1, 128, torch.bfloat16, 5), ("walk", 51000, 1, 1, 128, torch.bfloat16, 6),
    ("chirp", 16000, 2, 1, 64, torch.bfloat16, 7), ("chirp", 7000, 4, 2, 128, torch.float16, 8),
    ("spikes", 10000, 2, 1, 128, torch.bfloat16, 9), ("spikes", 30011, 2, 2, 64, torch.bfloat16, 10),
    ("ramp", 14000, 4, 1, 128, torch.bfloat16, 11), ("ramp", 2254, 1, 1, 64, torch.bfloat16, 12),
    ("wave", 18000, 2, 1, 128, torch.bfloat16, 13), ("wave", 6000, 2, 1, 64, torch.bfloat16, 14),
]


@pytest.mark.parametrize("kind,n,hq,hk,d,dtype,seed", CASES)
def test_score_profiles_every_operator_every_row(gpu, kind, n, hq, hk, d, dtype, seed):
    import minference_amd as M
    from minference_amd.ops import _build_block_index
    q, k, v, r = profile_inputs(kind, n, hq, hk, d, dtype, seed)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    tol = max(1.0, vg.float().abs().max().item() / 4.0)
    group = hq // hk
    heads = sorted({0, hq - 1})
    seqlens = torch.full((1,), n, dtype=torch.int32, device=gpu)
    print(f"case {kind} n={n} hq={hq} hk={hk} d={d} {dtype} seed={seed} tol x{tol:.1f}", flush=True)

    def sweep(tag, out, mask_for_head):
        for h in heads:
            w = _check_head(f"{tag} h={h}", out[0, h], qg[0, h], kg[0, h // group].float(), vg[0, h // group].float(), n,
                            mask_for_head(h), tol)
            print(f"  {tag} head {h}: worst max-abs {w:.3e}", flush=True)

    # vertical-slash on random lists, and on the lists the estimate selects
    nv, ns = int(min(n, r.integers(1, 400))), int(min(n, r.integers(1, 700)))
    vi, si = gen.vs_index_inputs(hq, n, nv, ns, seed, force_v=min(4, nv), force_s=min(int(r.integers(1, 80)), ns))
    for tag, (v_idx, s_idx) in (("vs-random", (torch.from_numpy(vi).to(gpu), torch.from_numpy(si.copy()).to(gpu))),
                                ("vs-estimate", M.estimate_vertical_slash(qg, kg, int(r.integers(30, 500)), int(r.integers(50, 1500))))):
        bc, bo, cc, ci = M.convert_vertical_slash_indexes(seqlens, v_idx, s_idx, n, 64, 64, zero_fill=False)
        out = M.vertical_slash_attention_from_index(qg, kg, vg, bc, bo, cc, ci, seqlens)
        assert torch.equal(out, M.vertical_slash_sparse_attention(qg, kg, vg, v_idx, s_idx))
        sweep(tag, out, lambda h: _vs_mask(bc, bo, cc, ci, h, n))
    bi = _build_block_index(qg, kg, int(r.integers(1, 120)), force_diag_first=bool(r.random() < 0.7))
    sweep("block-sparse", M.block_sparse_attention_from_index(qg, kg, vg, bi), lambda h: _bs_mask(bi, h, n))
    n_init, n_local = int(r.choice([0, 4, 64, 128, 200])), int(r.choice([1, 64, 100, 512, 1024, 4096]))
    n_last = int(r.choice([1, 64, 100, 333]))
    sweep(f"a-shape {n_init}+{n_local}", M.streaming_forward(qg, kg, vg, n_init, n_local),
          lambda h: _streaming_mask(n_init, n_local, 1 << 40))
    sweep(f"tri-shape {n_init}+{n_local}+{n_last}", M.tri_shape_forward(qg, kg, vg, n_init, n_local, n_last),
          lambda h: _streaming_mask(n_init, n_local, n - n_last))
    if n <= 24000:
        sweep("dense", M.dense_causal_attention(qg, kg, vg), lambda h: _streaming_mask(0, 1 << 40, 0))


@pytest.mark.parametrize("kind,n,d,dtype,seed", [("steps", 9000, 128, torch.bfloat16, 1), ("walk", 20000, 128, torch.bfloat16, 5),
                                                 ("ramp", 14000, 64, torch.bfloat16, 11), ("spikes", 10000, 128, torch.float16, 9),
                                                 ("wave", 18000, 64, torch.bfloat16, 13)])
def test_score_profiles_estimation_against_the_oracle(gpu, kind, n, d, dtype, seed):
    """The last-64-query estimate on the same profiles (logits of hundreds to thousands of units: the
    softmax of a row is close to one-hot), fp32 arithmetic, against the oracle."""
    import minference_amd as M
    hq, hk = 2, 1
    q, k, _, _ = profile_inputs(kind, n, hq, hk, d, dtype, seed)
    ke = k.repeat_interleave(hq // hk, dim=1)
    vert, slash = M.vertical_slash_scores(q.to(gpu), k.to(gpu), force_vertical=0, force_slash=0, reference_rounding=False)
    rv, rs = O.estimate_scores(q, ke)
    for name, got, ref in (("vertical", vert, rv), ("slash", slash, rs)):
        got = got.cpu()
        assert torch.isfinite(got).all(), name
        err = (got - ref).abs()
        print(f"  {kind} {name}: max-abs {err.max().item():.3e}, sum {got.sum(-1).tolist()}", flush=True)
        # (a probability moves by about 1e-3 of itself with the summation order of a logit of a few
        # thousand units: fp32 has 24 bits)
        assert (err <= 2e-3 * (1.0 + ref)).all(), name
        assert torch.allclose(got.sum(-1), torch.full((1, hq), 64.0), atol=2e-2), name
