"""GPU parity of the offline pattern search (flag builders + minf_pattern_recall through the
C ABI) against the oracle's N x N restatement.  Tolerance: the scores are means of softmax
masses in [0, 1]; both sides compute in fp32 on identical 16-bit inputs, so they agree to 2e-3
absolute (the slack covers a top-k boundary element whose two fp32 estimates differ in the last
bits and fall on either side of the threshold)."""

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import gen

pytestmark = pytest.mark.gpu

TOL = 2e-3


def heads(n, hq, hk, seed, dtype=torch.bfloat16, planted=True):
    q, k, _ = gen.qkv(1, hq, hk, n, 128, seed, dtype=torch.float32, scale=1.0)
    if planted:          # a sink, a few heavy columns and some local structure, so that candidates differ
        g = torch.Generator().manual_seed(seed + 1)
        u = torch.randn(hk, 128, generator=g)
        u = u / u.norm(dim=-1, keepdim=True)
        q = q + 4.0 * u.repeat_interleave(hq // hk, 0)[None, :, None, :]
        k[:, :, :4] += 8.0 * u[None, :, None, :]
        cols = torch.randperm(n, generator=g)[:n // 50]
        k[:, :, cols] += 5.6 * u[None, :, None, :]
        z = torch.randn(n + 255, 128, generator=g)
        z = torch.nn.functional.avg_pool1d(z.T[None], 256, 1)[0].T * 16.0     # smooth over 256 tokens
        q = q + 0.5 * z[None, None]
        k = k + 0.5 * z[None, None]
    return q.to(dtype), k.to(dtype)


SMALL = [("stream_llm", 10, 80), ("vertical_and_slash", 30, 80), ("vertical_and_slash", 50, 75),
         ("vertical_and_slash", 100, 40), ("block_sparse", 8, 1)]


def oracle_scores(q, k, cands, begin):
    hq, hk = q.shape[1], k.shape[1]
    return [O.search_pattern_scores(q[0, h].float(), k[0, h // (hq // hk)].float(), cands, begin) for h in range(hq)]


@pytest.mark.parametrize("n,hq,hk,begin,dtype,cands", [
    (3000, 2, 1, 2500, torch.bfloat16, None), (4100, 1, 1, 2500, torch.bfloat16, None),
    (1111, 4, 2, 300, torch.float16, SMALL), (640, 1, 1, 0, torch.bfloat16, SMALL),
    (97, 2, 2, 10, torch.bfloat16, SMALL[:3] + [("block_sparse", 2, 1)]),
])
def test_candidates_vs_oracle(gpu, n, hq, hk, begin, dtype, cands):
    from minference_amd import pattern_recall
    from minference_amd.search import CANDIDATES
    cands = list(CANDIDATES) if cands is None else cands     # None: the reference's own list
    print(f"case search n={n} hq={hq} hk={hk} begin={begin} {dtype}", flush=True)
    q, k = heads(n, hq, hk, 40 + n, dtype)
    got = pattern_recall(q.to(gpu), k.to(gpu), cands, begin)[0].cpu().numpy()
    want = np.array(oracle_scores(q, k, cands, begin))
    print(np.round(got, 4), np.round(want, 4), flush=True)
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= TOL
    if n >= 600:
        assert want.min() < 0.9 and want.max() - want.min() > 0.1     # the case separates candidates


def test_eight_candidates_of_every_kind_and_their_bits_do_not_mix(gpu):
    from minference_amd import pattern_recall
    n, begin = 1500, 200
    q, k = heads(n, 2, 1, 77)
    cands = [("stream_llm", 4, 64), ("block_sparse", 4, 1), ("vertical_and_slash", 40, 60), ("stream_llm", 0, 0),
             ("block_sparse", 1, 1), ("vertical_and_slash", 1500, 30), ("stream_llm", 1, 1500), ("block_sparse", 16, 1)]
    got = pattern_recall(q.to(gpu), k.to(gpu), cands, begin)[0].cpu().numpy()
    want = np.array(oracle_scores(q, k, cands, begin))
    print(np.round(got, 4), np.round(want, 4), flush=True)
    assert np.abs(got - want).max() <= TOL
    # candidates that keep everything are exactly 1 up to fp32 rounding, in any bit position
    assert np.abs(got[:, [4, 5, 6]] - 1.0).max() < 1e-5
    # each candidate alone (in bit 0) gives the same number as in its bit of the group of eight,
    # up to the last bits (the compiler may fuse the multiply-adds of different bits differently)
    for i in (0, 1, 2, 7):
        alone = pattern_recall(q.to(gpu), k.to(gpu), [cands[i]], begin)[0, :, 0].cpu().numpy()
        assert np.abs(alone - got[:, i]).max() < 1e-6


def test_uniform_attention_closed_form(gpu):
    # q = 0: row r keeps (#kept columns)/(r+1)
    from minference_amd import pattern_recall
    n, v, s, begin = 700, 5, 33, 100
    q = torch.zeros(1, 1, n, 128, dtype=torch.bfloat16)
    k = heads(n, 1, 1, 5, planted=False)[1]
    want = np.mean([(min(r, s) + 1 + max(0, min(v, r - s))) / (r + 1) for r in range(begin, n)])
    got = pattern_recall(q.to(gpu), k.to(gpu), [("stream_llm", v, s)], begin)[0, 0, 0].item()
    assert abs(got - want) < 1e-5


def test_search_pattern_choice_and_table(gpu):
    from minference_amd import search_pattern, search_patterns
    n = 4200
    q, k = heads(n, 4, 2, 91)
    table = search_patterns(q.to(gpu), k.to(gpu))
    assert sorted(table) == ["0", "1", "2", "3"]
    for h in range(4):
        want = O.search_pattern(q[0, h].float(), k[0, h // 2].float())
        got = table[str(h)]
        assert tuple(got[:3]) == want[:3], (h, got, want)
        assert abs(got[3] - want[3]) <= TOL
        assert got[0] == "vertical_and_slash"
    one = search_pattern(q[:, 1:2].to(gpu), k[:, 0:1].to(gpu), 1)
    assert list(one) == table["1"]
    # a block_sparse winner is replaced by vertical_and_slash (1000, 6096), as in the reference
    cands = [("stream_llm", 4, 16), ("block_sparse", 2, 1)]
    want = O.search_pattern(q[0, 0].float(), k[0, 0].float(), cands)
    got = search_pattern(q[:, 0:1].to(gpu), k[:, 0:1].to(gpu), 0, cands)
    assert want[:3] == ("vertical_and_slash", 1000, 6096) and got[:3] == want[:3] and abs(got[3] - want[3]) <= TOL


def test_too_short_context_gives_nan_and_no_choice(gpu):
    from minference_amd import search_pattern
    q, k = heads(512, 1, 1, 3)
    ty, v, s, sc = search_pattern(q.to(gpu), k.to(gpu), 0)       # 512 <= 2500: mean of nothing
    assert ty == "" and sc == 0.0


def test_deterministic(gpu):
    from minference_amd import pattern_recall
    q, k = heads(2000, 2, 1, 8)
    a = pattern_recall(q.to(gpu), k.to(gpu), row_begin=500)
    b = pattern_recall(q.to(gpu), k.to(gpu), row_begin=500)
    assert torch.equal(a, b)


def test_search_mode_of_the_dispatcher_writes_the_pattern_file(gpu, tmp_path):
    """minference_forward.py:644-673: with is_search every layer's heads are searched, the result
    is appended to config_path, the layer's output is dense causal attention; the finished file
    drives the sparse dispatcher."""
    import json
    from minference_amd import dense_causal_attention, minference_prefill_forward
    n = 2900
    q, k = heads(n, 4, 2, 17)
    v = torch.randn(1, 2, n, 128, generator=torch.Generator().manual_seed(3)).bfloat16()
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    path = tmp_path / "best_pattern.json"
    cfg = {"is_search": True, "config_path": str(path)}
    dense = dense_causal_attention(qg, kg, vg)
    for layer in range(2):
        out = minference_prefill_forward(qg, kg, vg, {"layer_idx": layer, "num_hidden_layers": 2, "attn_forward_config": cfg})
        assert torch.equal(out, dense)
    table = json.loads(path.read_text())
    assert len(table) == 2 and sorted(table[0]) == ["0", "1", "2", "3"]
    for h in range(4):
        want = O.search_pattern(q[0, h].float(), k[0, h // 2].float())
        assert tuple(table[1][str(h)][:3]) == want[:3]
    with pytest.raises(RuntimeError, match="Search already completed"):
        minference_prefill_forward(qg, kg, vg, {"layer_idx": 0, "num_hidden_layers": 2, "attn_forward_config": cfg})
    sparse = minference_prefill_forward(qg, kg, vg, {"layer_idx": 1, "attn_forward_config": {"best_pattern": table}})
    assert sparse.shape == dense.shape and torch.isfinite(sparse.float()).all()
