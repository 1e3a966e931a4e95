"""Pins oracle.estimate_* (restatement of minference_forward.py:599-614, 110-116) by brute
force, invariants and a closed form -- no reference import."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import gen


def brute_scores(q, k, last_q=64):
    """Explicit loops, float64."""
    N, D = q.shape
    lq = min(last_q, N)
    qd, kd = q.double().numpy(), k.double().numpy()
    P = np.zeros((lq, N))
    for i in range(lq):
        pos = N - lq + i
        s = (kd[: pos + 1] @ qd[pos]) / np.sqrt(D)
        e = np.exp(s - s.max())
        P[i, : pos + 1] = e / e.sum()
    vertical = P.sum(0)
    slash = np.zeros(N)
    for i in range(lq):
        for c in range(N):
            off = (N - lq + i) - c
            if off >= 0:
                slash[N - 1 - off] += P[i, c]
    return vertical, slash


@pytest.mark.parametrize("n", [64, 100, 257])
def test_scores_vs_bruteforce(n):
    q, k, _ = gen.qkv(1, 2, 2, n, 16, seed=n, scale=1.0)
    vert, slash = O.estimate_scores(q, k)
    for h in range(2):
        bv, bs = brute_scores(q[0, h], k[0, h])
        np.testing.assert_allclose(vert[0, h].numpy(), bv, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(slash[0, h].numpy(), bs, rtol=1e-5, atol=1e-6)


def test_sum_invariants_and_forcing():
    n = 300
    q, k, _ = gen.qkv(1, 3, 3, n, 32, seed=3, scale=1.0)
    vert, slash = O.estimate_scores(q, k)
    assert torch.allclose(vert.sum(-1), torch.full((1, 3), 64.0), atol=1e-4)
    assert torch.allclose(slash.sum(-1), torch.full((1, 3), 64.0), atol=1e-4)
    v_idx, s_idx, vf, sf = O.estimate_vs(q, k, 50, 120)
    assert v_idx.shape[-1] == 50 and s_idx.shape[-1] == 120
    for h in range(3):
        assert set(range(30)) <= set(v_idx[0, h].tolist())
        assert set(range(100)) <= set(s_idx[0, h].tolist())          # offsets 0..99 forced
        assert (np.diff(v_idx[0, h].numpy()) > 0).all() and (np.diff(s_idx[0, h].numpy()) < 0).all()
        assert ((s_idx[0, h] >= 0) & (s_idx[0, h] < n)).all()


def test_q_zero_closed_form():
    # Q = 0 -> row i is uniform over its N-64+i+1 visible keys
    n = 200
    q = torch.zeros(1, 1, n, 8)
    k = torch.randn(1, 1, n, 8)
    vert, slash = O.estimate_scores(q, k)
    w = 1.0 / (n - 64 + np.arange(64) + 1.0)
    exp_v = np.array([w[max(0, c - (n - 64)):].sum() for c in range(n)])
    np.testing.assert_allclose(vert[0, 0].numpy(), exp_v, rtol=1e-5)
    # diagonal with offset o gets w_i from every row i whose position >= o
    exp_s = np.array([w[max(0, (n - 1 - j) - (n - 64)):].sum() for j in range(n)])
    np.testing.assert_allclose(slash[0, 0].numpy(), exp_s, rtol=1e-5)


def test_size_clamps():
    q, k, _ = gen.qkv(1, 1, 1, 128, 8, seed=1)
    v_idx, s_idx, _, _ = O.estimate_vs(q, k, 5, 10)          # clamped up to 30 / 50
    assert v_idx.shape[-1] == 30 and s_idx.shape[-1] == 50
    v_idx, s_idx, _, _ = O.estimate_vs(q, k, 1000, 6096)      # clamped down to N
    assert v_idx.shape[-1] == 128 and s_idx.shape[-1] == 128


def test_topk_lowest_index_rule():
    x = torch.tensor([[1.0, 3.0, 3.0, 2.0, 3.0, 0.5]])
    assert O.topk_lowest_index(x, 2).tolist() == [[1, 2]]
    assert O.topk_lowest_index(x, 4).tolist() == [[1, 2, 3, 4]]
