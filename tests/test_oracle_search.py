"""Pins the oracle's restatement of the offline pattern search (search_candidate_mask,
search_pattern_scores, search_pattern) with facts that do not reuse its formulas: closed forms
under uniform attention counted by explicit loops, candidates that keep everything, and
per-element brute force on tiny inputs."""
import math

import numpy as np
import torch

from oracle import oracle as O


def rand(n, seed, d=128):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n, d, generator=g), torch.randn(n, d, generator=g)


def test_stream_llm_under_uniform_attention_is_a_count():
    # q = 0 -> every causal row is uniform, so the kept mass of row r is (#kept columns)/(r+1)
    n, v, s, begin = 150, 7, 20, 40
    q = torch.zeros(n, 128)
    k = rand(n, 1)[1]
    want = 0.0
    for r in range(begin, n):
        kept = sum(1 for c in range(r + 1) if (r - c) <= s or c < v)
        want += kept / (r + 1)
    want /= n - begin
    got = O.search_pattern_scores(q, k, [("stream_llm", v, s)], row_begin=begin)[0]
    assert abs(got - want) < 1e-6


def test_candidates_that_keep_everything_score_one():
    n = 130
    q, k = rand(n, 2)
    sc = O.search_pattern_scores(q, k, [("stream_llm", 0, n), ("stream_llm", n, 0),
                                        ("vertical_and_slash", n, 1), ("vertical_and_slash", 1, n),
                                        ("block_sparse", 1, 1)], row_begin=10)
    assert all(abs(x - 1.0) < 1e-6 for x in sc)


def test_no_rows_to_average_gives_nan():
    q, k = rand(64, 3)
    assert all(math.isnan(x) for x in O.search_pattern_scores(q, k, [("stream_llm", 4, 8)], row_begin=64))


def test_vertical_and_slash_mask_elementwise_brute_force():
    n, v, s = 100, 35, 40
    q, k = rand(n, 4)
    q = q * 3.0
    mask = O.search_candidate_mask(q, k, "vertical_and_slash", v, s).numpy()
    # independent recomputation with double loops (last 64 queries, exact softmax)
    lq = 64
    sc = np.full((lq, n), -np.inf)
    qn, kn = q.numpy().astype(np.float64), k.numpy().astype(np.float64)
    for i in range(lq):
        r = n - lq + i
        for c in range(r + 1):
            sc[i, c] = qn[r] @ kn[c] / math.sqrt(128)
    p = np.exp(sc - sc.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    vertical = p.sum(0)
    slash = np.zeros(n)                       # by offset
    for i in range(lq):
        r = n - lq + i
        for c in range(r + 1):
            slash[r - c] += p[i, c]
    vertical[:30] = np.inf
    slash[:30] = np.inf                       # offsets 0..29
    cols = set(np.argsort(-vertical, kind="stable")[:v].tolist())
    offs = set(np.argsort(-slash, kind="stable")[:s].tolist())
    assert set(range(30)) <= cols and set(range(30)) <= offs
    for r in range(n):
        for c in range(n):
            want = c <= r and (c in cols or (r - c) in offs)
            assert mask[r, c] == want, (r, c)


def test_block_sparse_mask_brute_force():
    n, ratio = 150, 2                          # 5 blocks of 32, the last one padded; keep 2 per row
    q, k = rand(n, 5)
    mask = O.search_candidate_mask(q, k, "block_sparse", ratio, 1).numpy()
    nb = 5
    bq = np.zeros((nb, 128)); bk = np.zeros((nb, 128))
    for t in range(n):
        bq[t // 32] += q[t].numpy() / 32
        bk[t // 32] += k[t].numpy() / 32
    keep = nb // ratio
    kept = {}
    for R in range(nb):
        cand = sorted(range(R + 1), key=lambda C: (-(bq[R] @ bk[C]), C))
        kept[R] = set(cand[:keep])
    for r in range(n):
        for c in range(n):
            assert mask[r, c] == (c <= r and (c // 32) in kept[r // 32]), (r, c)


def test_scores_equal_per_element_sum_on_tiny_input():
    n, begin = 48, 9
    q, k = rand(n, 6)
    cands = [("stream_llm", 3, 5), ("vertical_and_slash", 31, 33), ("block_sparse", 2, 1)]
    got = O.search_pattern_scores(q, k, cands, row_begin=begin)
    qn, kn = q.numpy().astype(np.float64), k.numpy().astype(np.float64)
    for (ty, a, b), g in zip(cands, got):
        mask = O.search_candidate_mask(q, k, ty, a, b).numpy()
        total = 0.0
        for r in range(begin, n):
            w = np.array([math.exp(qn[r] @ kn[c] / math.sqrt(128)) for c in range(r + 1)])
            w /= w.sum()
            total += sum(w[c] for c in range(r + 1) if mask[r, c])
        assert abs(g - total / (n - begin)) < 1e-5


def test_choice_rules():
    q, k = rand(200, 7)
    # a window wide enough to hold everything wins and is relabelled vertical_and_slash
    ty, v, s, sc = O.search_pattern(q, k, [("vertical_and_slash", 30, 30), ("stream_llm", 100, 800)], row_begin=50)
    assert (ty, v, s) == ("vertical_and_slash", 100, 800) and abs(sc - 1.0) < 1e-6
    # a block_sparse winner is replaced by vertical_and_slash (1000, 6096)
    ty, v, s, sc = O.search_pattern(q, k, [("block_sparse", 1, 1), ("stream_llm", 1, 1)], row_begin=50)
    assert (ty, v, s) == ("vertical_and_slash", 1000, 6096)
    # first of equal scores wins
    ty, v, s, sc = O.search_pattern(q, k, [("stream_llm", 200, 0), ("vertical_and_slash", 200, 50)], row_begin=50)
    assert (v, s) == (200, 0)
