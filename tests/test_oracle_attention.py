"""Pins the attention side of the oracle (masks + fp32 masked-dense softmax) through special
cases that reduce to torch's scaled_dot_product_attention and per-element brute force."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import gen


def sdpa(q, k, v, mask=None, causal=False):
    return torch.nn.functional.scaled_dot_product_attention(
        q[None, None].float(), k[None, None].float(), v[None, None].float(),
        attn_mask=None if mask is None else torch.as_tensor(mask)[None, None], is_causal=causal)[0, 0]


def test_masked_attention_equals_sdpa_with_mask():
    q, k, v = gen.qkv(1, 1, 1, 200, 32, seed=1, scale=1.0)
    rng = np.random.default_rng(0)
    mask = np.tril(rng.random((200, 200)) < 0.3) | np.eye(200, dtype=bool)
    out = O.masked_attention(q[0, 0], k[0, 0], v[0, 0], mask)
    assert torch.allclose(out, sdpa(q[0, 0], k[0, 0], v[0, 0], mask), atol=1e-5)


def test_vs_mask_all_offsets_is_causal():
    n = 300
    vi = np.zeros((1, 1, 1), np.int32)
    si = np.arange(n, dtype=np.int32)[::-1][None, None]
    bc, bo, cc, ci = O.vs_index_build([n], vi, si, n)
    m = O.vs_mask(bc[0, 0], bo[0, 0], cc[0, 0], ci[0, 0], n)
    assert np.array_equal(m, np.tril(np.ones((n, n), bool)))


def test_vs_mask_matches_definition_bruteforce():
    # the mask must be exactly {(r, c): c <= r, (r - c in S) up to 64-block granularity} U verticals:
    # check the two guarantees that matter: every selected diagonal/vertical element is kept, and
    # nothing above the diagonal is kept except listed columns (which are < row-block start)
    n = 1000
    vi, si = gen.vs_index_inputs(1, n, 20, 40, seed=2, force_v=2, force_s=3)
    bc, bo, cc, ci = O.vs_index_build([n], vi, si, n)
    m = O.vs_mask(bc[0, 0], bo[0, 0], cc[0, 0], ci[0, 0], n)
    r, c = np.nonzero(m)
    assert (c <= r).all()
    S, V = set(si[0, 0].tolist()), set(vi[0, 0].tolist())
    for rr in range(0, n, 37):
        for cc_ in range(rr + 1):
            if (rr - cc_) in S or cc_ in V:
                assert m[rr, cc_], (rr, cc_)


def test_vs_mask_rows_is_a_slice_of_vs_mask():
    for n, seqlen in ((1000, None), (777, 700)):
        vi, si = gen.vs_index_inputs(1, n, 20, 40, seed=3, force_v=2, force_s=3)
        bc, bo, cc, ci = O.vs_index_build([seqlen or n], vi, si, n)
        full = O.vs_mask(bc[0, 0], bo[0, 0], cc[0, 0], ci[0, 0], n, seqlen)
        for m in range((n + 63) // 64):
            part = O.vs_mask_rows(bc[0, 0, m], bo[0, 0, m], cc[0, 0, m], ci[0, 0, m], m, n, seqlen)
            assert np.array_equal(part, full[m * 64: m * 64 + 64])


def test_block_sparse_index_properties_and_dense_limit():
    n = 640
    q, k, v = gen.qkv(1, 2, 2, n, 16, seed=3, scale=1.0)
    bi = O.bs_block_index(q, k, 4)
    assert bi.shape == (1, 2, 10, 4) and bi.dtype == torch.int32
    for h in range(2):
        for m in range(10):
            row = bi[0, h, m].numpy()
            assert (np.diff(row) > 0).all()
            assert (row[: min(m + 1, 4)] <= m).all()      # causal picks sort first (reference :81-85)
    # top_k >= number of blocks -> every causal block -> plain causal attention
    out = O.block_sparse_attention(q, k, v, 100)
    ref = torch.stack([sdpa(q[0, h], k[0, h], v[0, h], causal=True) for h in range(2)])[None]
    assert torch.allclose(out, ref, atol=1e-5)
    # forced diagonal + first block option
    bf = O.bs_block_index(q, k, 3, force_diag_first=True)
    for m in range(10):
        assert 0 in bf[0, 0, m].tolist() and m in bf[0, 0, m].tolist()


@pytest.mark.parametrize("n,d,top_k,force", [(128, 8, 2, False), (200, 16, 3, False), (192, 4, 2, True), (70, 8, 5, False)])
def test_block_sparse_index_against_explicit_loops(n, d, top_k, force):
    """bs_block_index restated without any vectorised pooling: per-block means by Python loops over
    tokens (block_sparse_flash_attention.py:159-160), one dot product per (query block, key block)
    pair (:163), block-causal -inf (:164), then the k best by an explicit scan.  The caller's padding
    (:178: 64 - n % 64 zero rows, a WHOLE extra block when n % 64 == 0) is applied here with loops as
    well, so a wrong pooling axis, a mean over the wrong count or a missing extra block would show."""
    q, k, _ = gen.qkv(1, 2, 2, n, d, seed=40 + n, scale=1.0)
    pad = 64 - (n & 63)
    assert pad == 64 if n % 64 == 0 else pad == 64 - n % 64
    qp = torch.nn.functional.pad(q, [0, 0, 0, pad])
    kp = torch.nn.functional.pad(k, [0, 0, 0, pad])
    got = O.bs_block_index(qp, kp, top_k, force_diag_first=force)
    R = (n + pad) // 64
    assert R == n // 64 + 1
    kk = min(top_k, R)
    assert tuple(got.shape) == (1, 2, R, kk)
    for h in range(2):
        qbar = [[0.0] * d for _ in range(R)]
        kbar = [[0.0] * d for _ in range(R)]
        for blk in range(R):
            for t in range(64):                       # padded rows are zeros and still count in the mean
                tok = blk * 64 + t
                for e in range(d):
                    if tok < n:
                        qbar[blk][e] += float(q[0, h, tok, e])
                        kbar[blk][e] += float(k[0, h, tok, e])
            for e in range(d):
                qbar[blk][e] /= 64.0
                kbar[blk][e] /= 64.0
        for m in range(R):
            score = []
            for j in range(R):
                if j > m:
                    score.append(-math.inf)
                    continue
                sc = sum(qbar[m][e] * kbar[j][e] for e in range(d))
                if force and (j == m or j == 0):
                    sc = math.inf
                score.append(sc)
            order = sorted(range(R), key=lambda j: (-score[j], j))[:kk]      # ties: lowest block id
            want = sorted(order)
            row = got[0, h, m].tolist()
            if row != want:
                # only a near-tie at the k-th score may differ (float32 einsum vs Python doubles)
                kth = score[order[-1]]
                assert all(abs(score[j] - kth) < 1e-5 for j in set(row) ^ set(want)), (h, m, row, want)


def test_ashape_mask_closed_form():
    n, n_init, n_local = 257, 10, 40
    m = O.ashape_mask(n, n_init, n_local)
    for r in range(n):
        for c in range(n):
            exp = (c <= r) and ((r - c) < n_local or c < n_init)
            assert m[r, c] == exp
    assert np.array_equal(O.ashape_mask(100, 0, 100), np.tril(np.ones((100, 100), bool)))
    q, k, v = gen.qkv(1, 1, 1, 100, 16, seed=4, scale=1.0)
    out = O.streaming_forward(q, k, v, 4, 1000)
    assert torch.allclose(out[0, 0], sdpa(q[0, 0], k[0, 0], v[0, 0], causal=True), atol=1e-5)


def test_golden_fixtures_reproduce():
    import os
    path = os.path.join(os.path.dirname(__file__), "golden", "small_cases.npz")
    z = np.load(path)
    bc, bo, cc, ci = O.vs_index_build(z["seqlens"], z["vertical"], z["slash"], int(z["n"]))
    assert np.array_equal(bc, z["block_count"]) and np.array_equal(bo, z["block_offset"])
    assert np.array_equal(cc, z["column_count"]) and np.array_equal(ci, z["column_index"])
    q, k, v = (torch.from_numpy(z[x]).float() for x in ("q", "k", "v"))
    out = O.vertical_slash_sparse_attention(q, k, v, torch.from_numpy(z["vertical"]), torch.from_numpy(z["slash"]))
    assert np.allclose(out.numpy(), z["vs_out"], atol=1e-6)
    assert np.allclose(O.streaming_forward(q, k, v, 8, 48).numpy(), z["ashape_out"], atol=1e-6)
    assert np.allclose(O.block_sparse_attention(q, k, v, 2).numpy(), z["bs_out"], atol=1e-6)


def test_trishape_mask_definition_and_limits():
    n, n_init, n_local, n_last = 300, 8, 40, 100
    m = O.trishape_mask(n, n_init, n_local, n_last)
    for r in range(n):
        for c in range(n):
            if r >= n - n_last:
                want = c <= r
            else:
                want = (c <= r and c > r - n_local) or (c < n_init and c <= r - n_local)
            assert m[r, c] == want, (r, c)
    # n_last >= n clamps to n - 1: every row but the first is dense, and row 0 only sees key 0 anyway
    assert np.array_equal(O.trishape_mask(50, 2, 5, 1000), np.tril(np.ones((50, 50), bool)))
    assert np.array_equal(O.trishape_mask(50, 2, 5, 0), O.ashape_mask(50, 2, 5))


def test_streaming_scale_follows_the_padded_head_dim():
    """streaming_kernel.py:621-626 zero-pads a head_dim outside {16, ..., 256} to the next power of
    two and :575 then scales by 1/sqrt(q.shape[-1]) of the PADDED tensor.  Restated literally: pad
    physically, run the generic masked attention with its default 1/sqrt(last dim), slice."""
    n, n_init, n_local = 150, 4, 40
    for d, padded in ((96, 128), (192, 256), (48, 64), (64, 64), (128, 128), (256, 256), (16, 16)):
        assert abs(O.streaming_scale(d) - padded ** -0.5) < 1e-12
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(1, 2, n, 96, generator=g) for _ in range(3))
    got = O.streaming_forward(q, k, v, n_init, n_local)
    pad = lambda t: torch.nn.functional.pad(t, [0, 32])
    m = O.ashape_mask(n, n_init, n_local)
    for h in range(2):
        want = O.masked_attention(pad(q)[0, h], pad(k)[0, h], pad(v)[0, h], m)[:, :96]
        assert torch.allclose(got[0, h], want, atol=1e-6)
        plain = O.masked_attention(q[0, h], k[0, h], v[0, h], m)           # 1/sqrt(96): not what the reference does
        assert (plain - got[0, h]).abs().max() > 1e-3


def test_tri_shape_forward_two_scales():
    """tri_shape_kernel (streaming_kernel.py:820-833): A-shape operator on the first n - n_last tokens,
    dense rows scaled by 1/sqrt(head_dim) for the rest.  For a power-of-two head_dim both scales agree
    and the result is the masked attention under trishape_mask; for head_dim 96 the last rows equal
    torch's causal SDPA rows (scale 1/sqrt(96)) and the first rows the streaming operator's."""
    n, n_init, n_local, n_last = 130, 3, 20, 17
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(1, 1, n, 64, generator=g) for _ in range(3))
    got = O.tri_shape_forward(q, k, v, n_init, n_local, n_last)
    want = O.masked_attention(q[0, 0], k[0, 0], v[0, 0], O.trishape_mask(n, n_init, n_local, n_last))
    assert torch.allclose(got[0, 0], want, atol=1e-6)
    q, k, v = (torch.randn(1, 1, n, 96, generator=g) for _ in range(3))
    got = O.tri_shape_forward(q, k, v, n_init, n_local, n_last)
    sdpa = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert torch.allclose(got[:, :, -n_last:], sdpa[:, :, -n_last:], atol=1e-5)
    first = O.streaming_forward(q[:, :, :-n_last], k[:, :, :-n_last], v[:, :, :-n_last], n_init, n_local)
    assert torch.equal(got[:, :, :-n_last], first)
    assert torch.equal(O.tri_shape_forward(q, k, v, n_init, n_local, 0), O.streaming_forward(q, k, v, n_init, n_local))
