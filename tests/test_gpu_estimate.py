"""GPU parity of the estimation kernels and the top-k selection against the oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import gen

pytestmark = pytest.mark.gpu


def expand(x, hq):
    return x.repeat_interleave(hq // x.shape[1], dim=1)


@pytest.mark.parametrize("rounded", [False, True])
@pytest.mark.parametrize("n,hq,hk,dtype,d", [
    (64, 1, 1, torch.bfloat16, 128), (100, 2, 1, torch.bfloat16, 128), (1024, 4, 2, torch.bfloat16, 128),
    (3000, 2, 2, torch.float16, 128), (5000, 4, 1, torch.bfloat16, 128), (40, 1, 1, torch.bfloat16, 128),
    (100, 2, 1, torch.bfloat16, 64), (3000, 4, 2, torch.float16, 64), (5000, 4, 1, torch.bfloat16, 64),
    (700, 2, 2, torch.bfloat16, 32),
])
def test_scores_vs_oracle(gpu, monkeypatch, n, hq, hk, dtype, d, rounded):
    """Score vectors against the oracle in both rounding modes: fp32 arithmetic, and the reference's
    rounding points on 16-bit inputs (minference_forward.py:602: scores held in the input dtype
    after the dot product and after the division by sqrt(head_dim))."""
    from minference_amd.estimate import vertical_slash_scores
    print(f"case est n={n} hq={hq} hk={hk} {dtype} d={d} rounded={rounded}", flush=True)
    q, k, _ = gen.qkv(1, hq, hk, n, d, seed=n, scale=1.0)
    q, k = q.to(dtype), k.to(dtype)
    if d in (64, 128):          # both are native instantiations: no zero-padded copies of q / k
        def no_pad(*a, **kw):
            raise AssertionError("native head_dim must not be zero-padded")
        monkeypatch.setattr(torch.nn.functional, "pad", no_pad)
    vert, slash = vertical_slash_scores(q.to(gpu), k.to(gpu), force_vertical=0, force_slash=0,
                                        reference_rounding=rounded)
    monkeypatch.undo()
    rv, rs = O.estimate_scores(q, expand(k, hq), reference_rounding=rounded)
    vert, slash = vert.cpu(), slash.cpu()
    lq = min(64, n)
    assert torch.allclose(vert.sum(-1), torch.full((1, hq), float(lq)), atol=1e-3)
    assert torch.allclose(slash.sum(-1), torch.full((1, hq), float(lq)), atol=1e-3)
    if not rounded:
        # fp32 arithmetic on identical 16-bit inputs: relative 1e-3 on the score vectors
        assert torch.allclose(vert, rv, rtol=1e-3, atol=1e-6), (vert - rv).abs().max()
        assert torch.allclose(slash, rs, rtol=1e-3, atol=1e-6), (slash - rs).abs().max()
    else:
        # the matrix cores add the 128 products in another order than the CPU, so a dot product that
        # lies within an fp32 rounding error of a 16-bit rounding boundary may land on the other side
        # (about one score in 10^4): that moves one logit by one unit of the 16-bit format, i.e. one
        # probability by up to a few per cent.  Nearly all entries agree to 1e-3, every entry to 5e-2.
        for got, want, name in ((vert, rv, "vertical"), (slash, rs, "slash")):
            rel = (got - want).abs() / want.abs().clamp_min(1e-6)
            off = (rel > 1e-3).float().mean().item()
            print(f"  {name}: {off:.2e} of the entries off by more than 1e-3, worst {rel.max().item():.2e}", flush=True)
            assert off <= 5e-3 and rel.max() <= 5e-2, (name, off, rel.max())
        # and the mode is not a no-op on random inputs of this size (bf16: 8 mantissa bits)
        if n >= 1000 and dtype == torch.bfloat16:
            r32, _ = O.estimate_scores(q, expand(k, hq))
            assert ((vert - r32).abs() / r32.abs().clamp_min(1e-6) > 1e-3).float().mean() > 0.05


def test_forcing(gpu):
    from minference_amd.estimate import vertical_slash_scores
    q, k, _ = gen.qkv(1, 2, 2, 500, 128, seed=9, scale=1.0)
    vert, slash = vertical_slash_scores(q.bfloat16().to(gpu), k.bfloat16().to(gpu))
    assert torch.isinf(vert[..., :30]).all() and torch.isfinite(vert[..., 30:]).all()
    assert torch.isinf(slash[..., -100:]).all() and torch.isfinite(slash[..., :-100]).all()


@pytest.mark.parametrize("n,k", [(1000, 10), (5000, 1000), (131072, 6096), (70001, 1000), (300, 300), (64, 100),
                                 (200, 7), (256, 255), (2049, 100), (4096, 4000), (4097, 100), (65, 1)])
def test_topk_exact_vs_oracle(gpu, n, k):
    from minference_amd.estimate import topk_indices
    g = torch.Generator().manual_seed(n + k)
    x = torch.rand(3, n, generator=g)
    x[0, : min(30, n)] = torch.inf
    x[1, -min(100, n):] = torch.inf
    x[2] = (x[2] * 50).floor() / 50             # many ties
    x[2, n // 2:] = -torch.inf                   # masked tail, as in block-causal score rows
    got = topk_indices(x.to(gpu), k).cpu()
    ref = O.topk_lowest_index(x, min(k, n)).to(torch.int32)
    assert torch.equal(got, ref)
    got_r = topk_indices(x.to(gpu), k, reverse_base=n - 1).cpu()
    assert torch.equal(got_r, (n - 1) - ref)


def test_estimate_sets_vs_oracle(gpu):
    from minference_amd.estimate import estimate_vertical_slash
    n = 4096
    q, k, _ = gen.qkv(1, 4, 2, n, 128, seed=77, scale=1.0)
    q, k = q.bfloat16(), k.bfloat16()
    # (default mode for bf16 inputs: the reference's rounding points)
    v_idx, s_idx = estimate_vertical_slash(q.to(gpu), k.to(gpu), 200, 600)
    rv, rs, vs, ss = O.estimate_vs(q, expand(k, 4), 200, 600, reference_rounding=True)
    v_idx, s_idx = v_idx.cpu(), s_idx.cpu()
    assert v_idx.dtype == torch.int32 and v_idx.shape == (1, 4, 200) and s_idx.shape == (1, 4, 600)
    for h in range(4):
        a, b = set(v_idx[0, h].tolist()), set(rv[0, h].tolist())
        c, d = set(s_idx[0, h].tolist()), set(rs[0, h].tolist())
        # identical up to near-ties at the k-th score: recall >= 0.99
        assert len(a & b) >= 0.99 * 200 and len(c & d) >= 0.99 * 600
        assert set(range(30)) <= a and set(range(100)) <= c
        assert (np.diff(v_idx[0, h].numpy()) > 0).all() and (np.diff(s_idx[0, h].numpy()) < 0).all()


@pytest.mark.parametrize("n", [3000, 20000])
def test_ragged_topk_pads_with_noop_entries(gpu, n):
    """minf_topk_indices_pair_ragged: every row keeps its own k; the first k entries equal the plain
    selection with that k, the rest of the row is the padding (a constant for the first problem, the
    last selected value repeated for the second).  n = 3000 runs the one-wave-per-row kernel,
    n = 20000 the wide one."""
    from minference_amd import _lib
    from minference_amd.estimate import topk_indices
    lib = _lib.load()
    rows = 5
    g = torch.Generator().manual_seed(n)
    a = torch.randn(rows, n, generator=g).to(gpu)
    b = torch.randn(rows, n, generator=g).to(gpu)
    ka = [30, 1000, 1, 577, 1000]
    kb = [2048, 50, 2048, 1, 999]
    kam, kbm = max(ka), max(kb)
    out_a = torch.full((rows, kam), -5, dtype=torch.int32, device=gpu)
    out_b = torch.full((rows, kbm), -5, dtype=torch.int32, device=gpu)
    ka_t = torch.tensor(ka, dtype=torch.int32, device=gpu)
    kb_t = torch.tensor(kb, dtype=torch.int32, device=gpu)
    st = lib.minf_topk_indices_pair_ragged(a.data_ptr(), ka_t.data_ptr(), kam, out_a.data_ptr(), kam, -1, 1, 0x3FFFFFFF,
                                           b.data_ptr(), kb_t.data_ptr(), kbm, out_b.data_ptr(), kbm, n - 1, 2, 0,
                                           rows, n, n, _lib.stream_ptr(gpu))
    torch.cuda.synchronize()
    assert st == 0
    for r in range(rows):
        want_a = topk_indices(a[r:r + 1].contiguous(), ka[r])[0]
        assert torch.equal(out_a[r, :ka[r]], want_a)
        assert (out_a[r, ka[r]:] == 0x3FFFFFFF).all()
        want_b = topk_indices(b[r:r + 1].contiguous(), kb[r], reverse_base=n - 1)[0]
        assert torch.equal(out_b[r, :kb[r]], want_b)
        assert (out_b[r, kb[r]:] == want_b[-1]).all()


@pytest.mark.parametrize("hq,hk,n,dtype,d", [(4, 1, 20000 + 37, torch.bfloat16, 128), (8, 2, 9000, torch.float16, 64),
                                              (2, 1, 5000, torch.bfloat16, 128), (6, 2, 2048 * 3, torch.bfloat16, 64)])
def test_a_heads_scores_do_not_depend_on_the_heads_it_is_launched_with(gpu, hq, hk, n, dtype, d):
    """Grouped-query launches score four (or two) heads per workgroup, one wave per head over a whole
    2048-key chunk; a head on its own is scored by four waves of 512 keys.  Both sum a chunk as the same
    four pieces in the same order, so the score vectors -- and with them the selected sets and the
    attention output of the per-head dispatcher -- are identical bit for bit however the heads are
    grouped into launches."""
    from minference_amd.estimate import vertical_slash_scores
    q, k, _ = gen.qkv(1, hq, hk, n, d, seed=n + hq, scale=1.0)
    qg, kg = q.to(dtype).to(gpu), k.to(dtype).to(gpu)
    group = hq // hk
    for rounded in (True, False):
        vert, slash = vertical_slash_scores(qg, kg, reference_rounding=rounded)
        for h in range(hq):
            v1, s1 = vertical_slash_scores(qg[:, h:h + 1], kg[:, h // group:h // group + 1], reference_rounding=rounded)
            assert torch.equal(v1[0, 0], vert[0, h]) and torch.equal(s1[0, 0], slash[0, h]), (h, rounded)
        if group > 1:      # ... and two heads of a group launched as a pair
            v2, s2 = vertical_slash_scores(qg[:, :2], kg[:, :1], reference_rounding=rounded)
            assert torch.equal(v2[0], vert[0, :2]) and torch.equal(s2[0], slash[0, :2]), rounded
