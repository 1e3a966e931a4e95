"""Pins the oracle's ``reference_rounding`` modes: the places where the reference's torch code
rounds to the input dtype on 16-bit inputs.

* estimation (minference/modules/minference_forward.py:602-604): ``einsum`` of bf16 tensors returns
  bf16 (one rounding of the fp32-accumulated dot product), ``/ math.sqrt(head_dim)`` is a bf16
  division (fp32 quotient rounded to bf16), ``softmax(dtype=torch.float32)`` then works in fp32;
* block index (minference/ops/block_sparse_flash_attention.py:159-163): ``mean`` of bf16 returns
  bf16, the pooled ``einsum`` returns bf16.

Each is restated here element by element with explicit ``.to(torch.bfloat16)`` at those points and
compared with the vectorised oracle, which is what the GPU recall tests use at full size.
"""
import math

import pytest
import torch

from oracle import oracle as O


def _rand(shape, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * 1.5).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_estimation_rounding_points_by_element_loops(dtype):
    n, d, lq = 96, 32, 64
    q, k = _rand((1, 1, n, d), 1, dtype), _rand((1, 1, n, d), 2, dtype)
    vertical, slash = O.estimate_scores(q, k, lq, reference_rounding=True)
    qk = torch.full((lq, n), -math.inf, dtype=torch.float32)
    for i in range(lq):
        qi = n - lq + i
        for c in range(n):
            if c > qi:
                continue                                    # causal corner (:603)
            dot = torch.zeros((), dtype=torch.float32)
            for x in range(d):
                dot = dot + q[0, 0, qi, x].float() * k[0, 0, c, x].float()
            r1 = dot.to(dtype)                              # einsum result in the input dtype
            r2 = (r1.float() / torch.tensor(math.sqrt(d), dtype=torch.float32)).to(dtype)   # the division
            qk[i, c] = r2.float()
    p = torch.zeros((lq, n), dtype=torch.float64)
    for i in range(lq):
        row = qk[i].double()
        e = torch.exp(row - row.max())
        p[i] = e / e.sum()
    want_v = p.sum(0)
    want_s = torch.zeros(n, dtype=torch.float64)
    for i in range(lq):
        for c in range(n):
            off = (n - lq + i) - c
            if off >= 0:
                want_s[n - 1 - off] += p[i, c]
    assert torch.allclose(vertical[0, 0].double(), want_v, rtol=2e-5, atol=1e-7)
    assert torch.allclose(slash[0, 0].double(), want_s, rtol=2e-5, atol=1e-7)
    # the mode is not a no-op: the fp32 path differs from it on these inputs
    v32, _ = O.estimate_scores(q, k, lq)
    assert (v32[0, 0] - vertical[0, 0]).abs().max() > 1e-4
    # ... and is one for fp32 inputs
    a = O.estimate_scores(q.float(), k.float(), lq, reference_rounding=True)
    b = O.estimate_scores(q.float(), k.float(), lq)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_rounded_logits_are_representable_in_the_input_dtype():
    """Every finite logit the rounded mode feeds to the softmax is a bf16 number."""
    q, k = _rand((1, 2, 200, 64), 3, torch.bfloat16), _rand((1, 2, 200, 64), 4, torch.bfloat16)
    qk = torch.einsum("bhmk,bhnk->bhmn", q.float()[:, :, -64:], k.float())
    r = (qk.to(torch.bfloat16) / math.sqrt(64)).float()
    assert torch.equal(r, r.to(torch.bfloat16).float())
    # sqrt(64) is a power of two: the division is exact, only the einsum rounding remains
    assert torch.equal(r, qk.to(torch.bfloat16).float() / 8)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_block_score_rounding_points_by_element_loops(dtype):
    n, d = 64 * 5, 16
    q, k = _rand((1, 1, n, d), 5, dtype), _rand((1, 1, n, d), 6, dtype)
    got = O.bs_block_scores(q, k, reference_rounding=True)[0, 0]
    rows = n // 64
    qp = torch.zeros(rows, d, dtype=torch.float32)
    kp = torch.zeros(rows, d, dtype=torch.float32)
    for r in range(rows):
        for x in range(d):
            aq = torch.zeros((), dtype=torch.float32)
            ak = torch.zeros((), dtype=torch.float32)
            for t in range(64):
                aq = aq + q[0, 0, 64 * r + t, x].float()
                ak = ak + k[0, 0, 64 * r + t, x].float()
            qp[r, x] = (aq / 64).to(dtype).float()          # mean() returns the input dtype
            kp[r, x] = (ak / 64).to(dtype).float()
    for m in range(rows):
        for c in range(rows):
            if c > m:
                assert got[m, c] == -math.inf
                continue
            dot = torch.zeros((), dtype=torch.float32)
            for x in range(d):
                dot = dot + qp[m, x] * kp[c, x]
            want = dot.to(dtype).float()                    # einsum returns the input dtype
            # the vectorised sums may associate differently: allow one unit of the 16-bit format
            ulp = abs(want.item()) * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10) + 1e-12
            assert abs(got[m, c].item() - want.item()) <= ulp, (m, c, got[m, c].item(), want.item())
            assert got[m, c] == got[m, c].to(dtype).float()
    plain = O.bs_block_scores(q, k)[0, 0]
    finite = torch.isfinite(plain)
    assert (plain[finite] - got[finite]).abs().max() > 0
    idx_r = O.bs_block_index(q, k, 3, reference_rounding=True)
    assert idx_r.shape == (1, 1, rows, 3) and idx_r.dtype == torch.int32
