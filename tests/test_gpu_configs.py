"""BASELINE configs at the shapes they name (head counts, GQA ratios, lengths), through the C ABI:
config 3 at 524288 tokens (index builder, bit-exact), config 2 with 32 query / 8 kv heads, config 4
with 4:1 GQA, and config 5 as a two-layer Llama-3-8B-shaped stack at 262144 tokens with the seeded
70/20/10 pattern table.  Attention rows are compared with the fp32 masked-dense oracle on the index
entries the GPU produced (max-abs 2e-2, mean-abs 1e-3); index rows with the reference algorithm."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import gen

pytestmark = pytest.mark.gpu


def _rows_reference(q_rows, k, v, mask):
    s = (q_rows.float() @ k.float().T) * (q_rows.shape[-1] ** -0.5)
    s = torch.where(torch.as_tensor(mask), s, torch.tensor(-torch.inf))
    return torch.softmax(s, dim=-1) @ v.float()


def _check_vs_row_block(tag, out_rows, q_rows, k, v, v_list, s_list, bc_m, bo_m, cc_m, ci_m, m, n):
    """One row block of a vertical-slash head: the GPU's index row equals the reference algorithm's
    row, and the attention rows agree with the fp32 masked-dense result on that row."""
    rbo, rci = O.vs_index_row_py(v_list, s_list, m, n)
    assert int(bc_m) == len(rbo) and int(cc_m) == len(rci), tag
    assert bo_m[: len(rbo)].tolist() == rbo and ci_m[: len(rci)].tolist() == rci, tag
    mask = O.vs_mask_rows(len(rbo), rbo, len(rci), rci, m, n)
    ref = _rows_reference(q_rows, k, v, mask[: q_rows.shape[0]])
    err = (out_rows.float().cpu() - ref).abs()
    scale = ref.abs().max().item()
    print(f"  {tag}: max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e} (max |ref| {scale:.3e})", flush=True)
    assert err.max() <= 2e-2 and err.mean() <= 1e-3, tag
    # and relative to the size of the outputs (rows that average over thousands of keys are small)
    assert err.max() <= 2e-2 * scale and err.mean() <= 1e-3 * scale, tag


def test_config3_index_at_524288_tokens(gpu):
    """BASELINE config 3 at its longer length: 32 heads, 524288 tokens, 1000 verticals (0..3 forced),
    6096 slashes (0..63 forced), seeded.  Both HIP builders on all 32 heads must produce identical
    full tensors (7.4 GB each, zero tails included; compared on the GPU), and heads 0, 17 and 31 are
    compared bit for bit, full tensors, with the C restatement of the reference kernel."""
    from minference_amd import convert_vertical_slash_indexes
    n, heads = 524288, 32
    v, s = gen.vs_index_inputs(heads, n, 1000, 6096, seed=300)
    seqlens = torch.tensor([n], dtype=torch.int32, device=gpu)
    vg, sg = torch.from_numpy(v).to(gpu), torch.from_numpy(np.ascontiguousarray(s)).to(gpu)
    print("case c3-524288 table-driven builder", flush=True)
    fast = convert_vertical_slash_indexes(seqlens, vg, sg, n, 64, 64)
    print("case c3-524288 plain builder", flush=True)
    plain = convert_vertical_slash_indexes(seqlens, vg, sg, n, 64, 64, use_tables=False)
    torch.cuda.synchronize()
    names = ["block_count", "block_offset", "column_count", "column_index"]
    for name, a, b in zip(names, fast, plain):
        assert a.dtype == torch.int32 and torch.equal(a, b), f"builders differ in {name}"
    del plain
    torch.cuda.empty_cache()
    for h in (0, 17, 31):
        print(f"case c3-524288 oracle head {h}", flush=True)
        ref = O.vs_index_build([n], v[:, h:h + 1], s[:, h:h + 1], n)
        for name, a, r in zip(names, fast, ref):
            got = a[:, h:h + 1].cpu().numpy()
            assert got.shape == r.shape and np.array_equal(got, r), f"head {h}: {name} differs from the oracle"


def test_config2_all_32_query_heads_8_kv_heads(gpu):
    """BASELINE config 2 at its stated geometry (131072 tokens, 32 query / 8 kv heads, bf16,
    vertical 1000, slash 6096): the launch shape the benchmark times.  Sampled (head, row block)
    pairs from four kv groups, incl. the last head and the last row block."""
    import minference_amd as M
    n, hq, hk = 131072, 32, 8
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=100, dtype=torch.bfloat16)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    v_idx, s_idx = M.estimate_vertical_slash(qg, kg, 1000, 6096)
    seqlens = torch.full((1,), n, dtype=torch.int32, device=gpu)
    bc, bo, cc, ci = M.convert_vertical_slash_indexes(seqlens, v_idx, s_idx, n, 64, 64, zero_fill=False)
    out = M.vertical_slash_attention_from_index(qg, kg, vg, bc, bo, cc, ci, seqlens)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    rows = n // 64
    vi_c, si_c = v_idx.cpu().numpy(), s_idx.cpu().numpy()
    for h, m in [(0, 0), (3, 700), (13, 1), (13, 1999), (22, 1024), (31, rows - 1), (31, 64), (26, 333)]:
        print(f"case c2-32x8 head={h} row-block={m}", flush=True)
        kv = h // (hq // hk)
        _check_vs_row_block(f"head {h} row block {m}", out[0, h, m * 64: m * 64 + 64], q[0, h, m * 64: m * 64 + 64],
                            k[0, kv], v[0, kv], vi_c[0, h].tolist(), si_c[0, h].tolist(),
                            bc[0, h, m], bo[0, h, m].cpu().numpy(), cc[0, h, m], ci[0, h, m].cpu().numpy(), m, n)


def test_config4_gqa_4_to_1(gpu):
    """BASELINE config 4 with the 4:1 GQA ratio of its 32 q / 8 kv heads (8 query heads on 2 kv
    heads at 131072 tokens): top-100 block index with diagonal and block 0 forced, sampled query
    blocks of heads from both kv groups against explicit per-block means and the masked-dense rows."""
    from minference_amd.ops import _build_block_index, block_sparse_attention_from_index
    n, hq, hk, top_k = 131072, 8, 2, 100
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=100, dtype=torch.bfloat16)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    bi = _build_block_index(qg, kg, top_k, force_diag_first=True)
    out = block_sparse_attention_from_index(qg, kg, vg, bi)
    torch.cuda.synchronize()
    R = n // 64 + 1
    assert tuple(bi.shape) == (1, hq, R, top_k)
    bic = bi[0].cpu().numpy()
    for h, m in [(0, 0), (3, 150), (4, 99), (5, 1200), (7, 2047), (2, 100)]:
        print(f"case c4-gqa head={h} query-block={m}", flush=True)
        kv = h // (hq // hk)
        # pooled scores by an explicit loop over the causal key blocks of this query block
        # (bf16 inputs: means and products are rounded to bf16 where the reference's torch code holds
        # them in bf16, block_sparse_flash_attention.py:159-163)
        qbar = q[0, h, m * 64: m * 64 + 64].float().mean(0).to(torch.bfloat16).float()
        p = np.full(R, -np.inf)
        for j in range(m + 1):
            kbar = k[0, kv, j * 64: j * 64 + 64].float().mean(0).to(torch.bfloat16).float()
            p[j] = float((qbar @ kbar).to(torch.bfloat16))
        p[m] = p[0] = np.inf
        row = bic[h, m]
        assert (np.diff(row) > 0).all()
        kth = np.sort(p)[::-1][top_k - 1]
        sel = np.zeros(R, bool)
        sel[row] = True
        if np.isfinite(kth):
            tol = 2.0 ** -7 * max(1e-3, abs(kth))       # one unit of bf16 at the k-th score
            assert sel[p > kth + tol].all() and (p[sel] >= kth - tol).all()
        else:
            assert sel[: m + 1].all()
        mask = np.zeros((64, n), bool)
        rr = np.arange(m * 64, m * 64 + 64)
        for j in row[: min(m + 1, top_k)]:
            cols = np.arange(j * 64, min(j * 64 + 64, n))
            mask[:, cols] |= cols[None, :] <= rr[:, None]
        err = (out[0, h, m * 64: m * 64 + 64].float().cpu()
               - _rows_reference(q[0, h, m * 64: m * 64 + 64], k[0, kv], v[0, kv], mask)).abs()
        print(f"  max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e}", flush=True)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3


def test_config5_two_layer_llama3_8b_shape_at_262144_tokens(gpu, monkeypatch):
    """BASELINE config 5 with two of its 32 layers: random-init Llama-3-8B shapes (hidden 4096, 32 q /
    8 kv heads, RoPE theta 500000, SwiGLU 14336, vocab 128256), 262144 random tokens, the seeded
    70 % vertical_slash / 20 % block_sparse / 10 % A-shape table through minference_prefill_forward.
    The logits must be finite; for layer 0, one head of every pattern type is checked on sampled row
    blocks against the oracle masks built from what the dispatcher's own stages produce on that
    layer's q/k (the stages are deterministic, so re-running them gives the indices it used)."""
    import minference_amd as M
    from minference_amd import llama
    from minference_amd.ops import _build_block_index
    n = 262144
    cfg = llama.LlamaConfig(num_layers=2)
    model = llama.LlamaPrefill(cfg, device=gpu, seed=0)
    ids = torch.randint(0, cfg.vocab_size, (n,), generator=torch.Generator().manual_seed(500))
    table = llama.seeded_pattern_mix(cfg.num_layers, cfg.num_heads, seed=501)
    types = {t: [h for h in range(cfg.num_heads) if table[0][str(h)][0] == t]
             for t in ("vertical_and_slash", "block_sparse", "stream_llm")}
    assert all(types.values()), types
    picks = {t: hs[-1] for t, hs in types.items()}
    blocks = [0, 70, 2500, n // 64 - 1]
    captured = {}
    real = llama.minference_prefill_forward

    def recording(q, k, v, kwargs):
        out = real(q, k, v, kwargs)
        if kwargs["layer_idx"] == 0:
            # q is overwritten by the next layer: keep the sampled rows, and K/V of the heads used
            for t, h in picks.items():
                kv = h // (cfg.num_heads // cfg.num_kv_heads)
                captured[t] = {
                    "h": h, "k": k[0, kv].float().cpu(), "v": v[0, kv].float().cpu(),
                    "q": {m: q[0, h, m * 64: m * 64 + 64].clone() for m in blocks},
                    "o": {m: out[0, h, m * 64: m * 64 + 64].clone() for m in blocks},
                    "q_full": q[:, h:h + 1].clone(), "k_full": k[:, kv:kv + 1].clone()}
        return out

    monkeypatch.setattr(llama, "minference_prefill_forward", recording)
    print("case c5 two-layer prefill", flush=True)
    logits, _ = model.prefill(ids, {"best_pattern": table})
    torch.cuda.synchronize()
    assert logits.shape == (cfg.vocab_size,) and torch.isfinite(logits).all()

    # vertical-slash head
    c = captured["vertical_and_slash"]
    v_idx, s_idx = M.estimate_vertical_slash(c["q_full"], c["k_full"], 1000, 6096)
    seqlens = torch.full((1,), n, dtype=torch.int32, device=gpu)
    bc, bo, cc, ci = M.convert_vertical_slash_indexes(seqlens, v_idx, s_idx, n, 64, 64, zero_fill=False)
    vl, sl = v_idx[0, 0].cpu().tolist(), s_idx[0, 0].cpu().tolist()
    for m in blocks:
        print(f"case c5 vertical_slash head={c['h']} row-block={m}", flush=True)
        _check_vs_row_block(f"vs head {c['h']} row block {m}", c["o"][m], c["q"][m].cpu(), c["k"], c["v"], vl, sl,
                            bc[0, 0, m], bo[0, 0, m].cpu().numpy(), cc[0, 0, m], ci[0, 0, m].cpu().numpy(), m, n)
    # block-sparse head (top-100, no forced blocks: the dispatcher's call, minference_forward.py:616-618)
    c = captured["block_sparse"]
    bi = _build_block_index(c["q_full"], c["k_full"], 100)[0, 0].cpu().numpy()
    for m in blocks:
        print(f"case c5 block_sparse head={c['h']} row-block={m}", flush=True)
        mask = np.zeros((64, n), bool)
        rr = np.arange(m * 64, m * 64 + 64)
        for j in bi[m, : min(m + 1, 100)]:
            cols = np.arange(j * 64, min(j * 64 + 64, n))
            mask[:, cols] |= cols[None, :] <= rr[:, None]
        err = (c["o"][m].float().cpu() - _rows_reference(c["q"][m].cpu(), c["k"], c["v"], mask)).abs()
        print(f"  max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e}", flush=True)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3
    # A-shape head: sink 128 + local 4096
    c = captured["stream_llm"]
    for m in blocks:
        print(f"case c5 a-shape head={c['h']} row-block={m}", flush=True)
        r = np.arange(m * 64, m * 64 + 64)[:, None]
        col = np.arange(n)[None, :]
        mask = ((col <= r) & (col > r - 4096)) | ((col < 128) & (col <= r - 4096))
        err = (c["o"][m].float().cpu() - _rows_reference(c["q"][m].cpu(), c["k"], c["v"], mask)).abs()
        print(f"  max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e}", flush=True)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3


def test_vertical_slash_walks_that_are_not_split(gpu):
    """The paired vertical-slash walk splits the two block lists of a workgroup into common entries and
    leftovers only when both are strictly ascending, at most 2048 entries long and differ in at most
    512 entries; everything else takes the walk in which each half follows its own list.  Three inputs
    that force that walk, on sampled row blocks against the fp32 masked-dense oracle:
    scattered slashes (more than 512 leftovers), one run of more than 2048 blocks, and block lists
    handed over in descending order (the reference's kernel accepts any order,
    pit_sparse_flash_attention_v2.py:84-117)."""
    import minference_amd as M

    def run(tag, n, hq, hk, nv, ns, vi, si, sample, seed):
        # logits of standard deviation 2: a few dozen keys, spread over all tiles of a row's list, carry
        # most of each row's weight, so a tile that is skipped, doubled or misplaced shows; with
        # thousands of keys per row the outputs are small, hence the bound relative to max |ref|
        q, k, v = gen.qkv(1, hq, hk, n, 128, seed=seed, scale=1.0)
        q, k, v = (2.0 * q).bfloat16(), k.bfloat16(), v.bfloat16()
        qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
        seqlens = torch.full((1,), n, dtype=torch.int32, device=gpu)
        v_idx, s_idx = torch.from_numpy(vi).to(gpu), torch.from_numpy(np.ascontiguousarray(si)).to(gpu)
        bc, bo, cc, ci = M.convert_vertical_slash_indexes(seqlens, v_idx, s_idx, n, 64, 64, zero_fill=True)
        out = M.vertical_slash_attention_from_index(qg, kg, vg, bc, bo, cc, ci, seqlens)
        torch.cuda.synchronize()
        for h, m in sample:
            print(f"case {tag} head={h} row-block={m} blocks={int(bc[0, h, m])}", flush=True)
            kv = h // (hq // hk)
            _check_vs_row_block(f"{tag} head {h} row block {m}", out[0, h, m * 64: m * 64 + 64], q[0, h, m * 64: m * 64 + 64],
                                k[0, kv], v[0, kv], vi[0, h].tolist(), si[0, h].tolist(),
                                bc[0, h, m], bo[0, h, m].cpu().numpy(), cc[0, h, m], ci[0, h, m].cpu().numpy(), m, n)
        return (qg, kg, vg, seqlens, bc, bo, cc, ci, out)

    # (a) 1100 uniformly drawn slashes over 128K tokens: mostly isolated blocks, so the lists of two
    # neighbouring row blocks (one is the other moved by 64 keys) share few entries
    n = 131072 + 64 * 3
    vi, si = gen.vs_index_inputs(2, n, 500, 1100, seed=41)
    rows = n // 64
    qg, kg, vg, seqlens, bc, bo, cc, ci, out = run("scattered", n, 2, 1, 500, 1100, vi, si,
                                                     [(0, rows - 1), (1, rows - 2), (0, 1700), (1, 1701), (1, 3)], 42)
    la = set(bo[0, 0, rows - 2, : int(bc[0, 0, rows - 2])].tolist())
    lb = set(bo[0, 0, rows - 1, : int(bc[0, 0, rows - 1])].tolist())
    assert len(la - lb) > 512 and len(lb - la) > 512, (len(la - lb), len(lb - la))
    # (c) the same lists in descending order: same mask, so the same rows within the tolerance
    cnt = bc.long().unsqueeze(-1)
    pos = torch.arange(bo.shape[-1], device=gpu).expand_as(bo)
    rev = torch.where(pos < cnt, bo.gather(-1, (cnt - 1 - pos).clamp_(min=0)), bo)
    out_rev = M.vertical_slash_attention_from_index(qg, kg, vg, bc, rev, cc, ci, seqlens)
    err = (out_rev.float() - out.float()).abs()
    scale = out.float().abs().max().item()
    print(f"case descending lists: max-abs {err.max().item():.3e} (max |out| {scale:.3e})", flush=True)
    assert err.max() <= 2e-2 * scale and err.mean() <= 1e-3 * scale
    del qg, kg, vg, bc, bo, cc, ci, out, out_rev, rev, pos, cnt
    torch.cuda.empty_cache()
    # (b) slashes 37 apart over the whole context: one run per row block, more than 2048 blocks at the end
    n = 64 * 2200
    si = np.ascontiguousarray(np.arange(0, 37 * 3900, 37, dtype=np.int32)[::-1]).reshape(1, 1, -1)
    vi = np.arange(0, 64, dtype=np.int32).reshape(1, 1, -1)
    rows = n // 64
    res = run("long run", n, 1, 1, 64, 3900, vi, si, [(0, rows - 1), (0, rows - 2), (0, 2100), (0, 5)], 43)
    assert int(res[4].max()) > 2048


def _recall(got, want):
    got, want = set(int(x) for x in got), set(int(x) for x in want)
    return len(got & want) / max(1, len(want))


def test_config2_selected_sets_follow_the_reference_rounding(gpu):
    """BASELINE config 2 (131072 tokens, 32 q / 8 kv heads, bf16): the vertical and slash sets the HIP
    estimation + top-k select, against the oracle run with the REFERENCE'S rounding points
    (minference_forward.py:602-604: bf16 einsum result, bf16 quotient, fp32 softmax) on four heads of
    four kv groups.  Rule: set recall >= 0.99.  Also reported: the recall of the fp32 arithmetic this
    build used before (it fails that rule on the vertical set), and how far the attention output moves
    when the oracle's sets replace the GPU's."""
    import minference_amd as M
    n, hq, hk = 131072, 32, 8
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=100, dtype=torch.bfloat16)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    v_idx, s_idx = M.estimate_vertical_slash(qg, kg, 1000, 6096)
    v32, s32 = M.estimate_vertical_slash(qg, kg, 1000, 6096, reference_rounding=False)
    heads = (0, 5, 13, 31)
    for h in heads:
        kv = h // (hq // hk)
        print(f"case c2 selector recall head={h}", flush=True)
        ov, os_, _, _ = O.estimate_vs(q[:, h:h + 1], k[:, kv:kv + 1], 1000, 6096, reference_rounding=True)
        rv, rs = _recall(v_idx[0, h].tolist(), ov[0, 0].tolist()), _recall(s_idx[0, h].tolist(), os_[0, 0].tolist())
        rv32, rs32 = _recall(v32[0, h].tolist(), ov[0, 0].tolist()), _recall(s32[0, h].tolist(), os_[0, 0].tolist())
        print(f"  head {h}: recall vs the reference's rounding: vertical {rv:.4f} slash {rs:.4f} "
              f"(fp32 arithmetic: vertical {rv32:.4f} slash {rs32:.4f})", flush=True)
        assert rv >= 0.99 and rs >= 0.99, (h, rv, rs)
        # end to end: one head's attention with the GPU's sets and with the oracle's sets
        o_gpu = M.vertical_slash_sparse_attention(qg[:, h:h + 1], kg[:, kv:kv + 1], vg[:, kv:kv + 1],
                                                  v_idx[:, h:h + 1], s_idx[:, h:h + 1])
        o_ref = M.vertical_slash_sparse_attention(qg[:, h:h + 1], kg[:, kv:kv + 1], vg[:, kv:kv + 1],
                                                  ov.to(gpu), os_.to(gpu))
        d = (o_gpu.float() - o_ref.float()).abs()
        print(f"  head {h}: output with the GPU's sets vs with the oracle's sets: max-abs {d.max().item():.3e} "
              f"mean-abs {d.mean().item():.3e}", flush=True)
        assert d.mean() <= 1e-3


def test_config4_block_sets_follow_the_reference_rounding(gpu):
    """BASELINE config 4 shape (131072 tokens, top-100 blocks, 4:1 GQA): the block sets of the HIP
    block index against the oracle run with the reference's rounding points
    (block_sparse_flash_attention.py:159-163: bf16 means, bf16 pooled products) on two heads.
    bf16 scores tie often and torch.topk's tie order is unspecified, so a row is compared as the rule
    allows: every block strictly above the k-th score must be selected and nothing strictly below it;
    the recall of the oracle's lowest-index choice is reported and must be >= 0.99 on average."""
    from minference_amd.ops import _build_block_index
    n, hq, hk, top_k = 131072, 8, 2, 100
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=100, dtype=torch.bfloat16)
    qg, kg = q.to(gpu), k.to(gpu)
    bi = _build_block_index(qg, kg, top_k).cpu().numpy()
    bi32 = _build_block_index(qg, kg, top_k, reference_rounding=False).cpu().numpy()
    pad = 64
    for h in (0, 6):
        kv = h // (hq // hk)
        print(f"case c4 selector recall head={h}", flush=True)
        qp = torch.nn.functional.pad(q[:, h:h + 1], [0, 0, 0, pad])
        kp = torch.nn.functional.pad(k[:, kv:kv + 1], [0, 0, 0, pad])
        p = O.bs_block_scores(qp, kp, reference_rounding=True)[0, 0].numpy()
        ob = O.bs_block_index(qp, kp, top_k, reference_rounding=True)[0, 0].numpy()
        R = p.shape[0]
        rec, rec32, bad = [], [], 0
        for m in range(100, R - 1):
            rec.append(_recall(bi[0, h, m], ob[m]))
            rec32.append(_recall(bi32[0, h, m], ob[m]))
            kth = np.sort(p[m])[::-1][top_k - 1]
            sel = np.zeros(R, bool)
            sel[bi[0, h, m]] = True
            tol = 2.0 ** -7 * abs(kth)                  # one unit of bf16: sums in another order may round the other way
            if not (sel[p[m] > kth + tol].all() and (p[m][sel] >= kth - tol).all()):
                bad += 1
        print(f"  head {h}: mean recall {np.mean(rec):.4f} min {np.min(rec):.4f} "
              f"(fp32 arithmetic: mean {np.mean(rec32):.4f} min {np.min(rec32):.4f}); rows breaking the rule: {bad}", flush=True)
        assert bad == 0
        assert np.mean(rec) >= 0.99


def test_full_size_rows_are_normalised_and_linear_in_v(gpu):
    """Size-independent properties on EVERY row of every head at BASELINE's full shapes (the oracle
    comparisons above sample row blocks): with V = 1 every output row is a weighted mean of ones, i.e.
    exactly 1 wherever a row attends to anything -- numerator and denominator are sums of the same
    rounded probabilities -- for the vertical-slash path (config 2: 131072 tokens, 32 q / 8 kv heads),
    the block-sparse path (config 4) and the A-shape path (config 5's 128 + 4096); and the output is
    linear in V: out(V1 + V2) = out(V1) + out(V2) within the 16-bit rounding of the three outputs."""
    import minference_amd as M
    from minference_amd.ops import _build_block_index, block_sparse_attention_from_index
    n, hq, hk = 131072, 32, 8
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=100, dtype=torch.bfloat16)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    ones = torch.ones_like(vg)
    seqlens = torch.full((1,), n, dtype=torch.int32, device=gpu)
    v_idx, s_idx = M.estimate_vertical_slash(qg, kg, 1000, 6096)
    idx = M.convert_vertical_slash_indexes(seqlens, v_idx, s_idx, n, 64, 64, zero_fill=False)
    bi = _build_block_index(qg, kg, 100, force_diag_first=True)
    runs = {
        "vertical-slash": lambda vv: M.vertical_slash_attention_from_index(qg, kg, vv, *idx, seqlens),
        "block-sparse": lambda vv: block_sparse_attention_from_index(qg, kg, vv, bi),
        "a-shape": lambda vv: M.streaming_forward(qg, kg, vv, 128, 4096),
    }
    g = torch.Generator().manual_seed(7)
    v2 = torch.randn(v.shape, generator=g).to(torch.bfloat16).to(gpu)
    for name, f in runs.items():
        print(f"case full-size properties: {name}", flush=True)
        o1 = f(ones)
        dev = (o1.float() - 1.0).abs().max().item()
        print(f"  V = 1: max |out - 1| = {dev:.3e}", flush=True)
        assert dev <= 2.0 ** -8, name                      # half a unit of bf16 at 1.0
        del o1
        oa, ob, oab = f(vg), f(v2), f(vg + v2)
        d = (oab.float() - oa.float() - ob.float()).abs()
        scale = oab.float().abs().max().item()
        print(f"  linearity: max {d.max().item():.3e} mean {d.mean().item():.3e} (max |out| {scale:.3e})", flush=True)
        # three bf16 roundings of outputs of size <= scale, plus the rounding of V1 + V2 itself
        assert d.max().item() <= 3e-2 * max(scale, 1.0) and d.mean().item() <= 2e-3 * max(scale, 1.0), name
        del oa, ob, oab


def test_full_size_estimation_and_selection_invariants(gpu):
    """BASELINE config 2's shape, all 32 heads: the score vectors of the estimation are two
    decompositions of the same 64 softmax rows, so each sums to 64 before forcing (both rounding modes);
    the selected lists are strictly ordered, inside the context and contain the forced entries
    (first 30 columns, offsets 0..99: minference_forward.py:606, :610)."""
    import minference_amd as M
    from minference_amd.estimate import vertical_slash_scores
    n, hq, hk = 131072, 32, 8
    q, k, _, _ = gen.planted_layer(n, hq, hk, seed=100, dtype=torch.bfloat16)
    qg, kg = q.to(gpu), k.to(gpu)
    for rounded in (True, False):
        vert, slash = vertical_slash_scores(qg, kg, force_vertical=0, force_slash=0, reference_rounding=rounded)
        sv, ss = vert.double().sum(-1), slash.double().sum(-1)
        print(f"case c2 estimation sums rounded={rounded}: vertical {sv.min().item():.4f}..{sv.max().item():.4f} "
              f"slash {ss.min().item():.4f}..{ss.max().item():.4f}", flush=True)
        assert torch.isfinite(vert).all() and torch.isfinite(slash).all()
        assert (sv - 64).abs().max() <= 2e-2 and (ss - 64).abs().max() <= 2e-2
        assert (vert >= 0).all() and (slash >= 0).all()
    v_idx, s_idx = M.estimate_vertical_slash(qg, kg, 1000, 6096)
    vi, si = v_idx[0].cpu().numpy(), s_idx[0].cpu().numpy()
    assert vi.shape == (hq, 1000) and si.shape == (hq, 6096)
    assert (np.diff(vi, axis=-1) > 0).all() and (np.diff(si, axis=-1) < 0).all()
    assert vi.min() >= 0 and vi.max() < n and si.min() >= 0 and si.max() < n
    assert (vi[:, :30] == np.arange(30)).all() and (si[:, -100:] == np.arange(99, -1, -1)).all()


def test_config5_layer_slice_every_row_is_normalised(gpu):
    """BASELINE config 5's attention layer (262144 tokens, 32 q / 8 kv heads, the seeded 70/20/10
    table of layer 0: vertical_and_slash, block_sparse and stream_llm heads) through the per-head
    dispatcher with V = 1: every output row of every head must be exactly 1, whichever kernel and
    list its head took -- the planted inputs' scores span 260 powers of two between the sink keys and
    the latest keys at this length, more than fp32's exponent range."""
    import minference_amd as M
    from minference_amd.llama import seeded_pattern_mix
    n, hq, hk = 262144, 32, 8
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=100, dtype=torch.bfloat16)
    qg, kg = q.to(gpu), k.to(gpu)
    del q, v
    ones = torch.ones_like(kg)
    table = seeded_pattern_mix(1, hq, seed=501)
    print("case c5 layer slice, V = 1", flush=True)
    out = M.minference_prefill_forward(qg, kg, ones, {"layer_idx": 0, "attn_forward_config": {"best_pattern": table}})
    torch.cuda.synchronize()
    dev = (out.float() - 1.0).abs().amax(dim=(0, 2, 3))
    for h in range(hq):
        assert dev[h].item() <= 2.0 ** -8, f"head {h} ({table[0][str(h)][0]}): max |out - 1| = {dev[h].item()}"


def test_full_size_every_operator_reduces_to_dense_on_all_rows(gpu):
    """Library special cases at 131072 tokens, compared on EVERY row: dense causal attention of this
    engine against torch's own flash attention (an independent implementation; 16-bit tolerance), and
    every sparse operator in the setting where its index keeps the whole causal triangle -- every
    diagonal kept (block lists of 2048 entries: the walk that is not split in LDS), window wider than
    the sequence, top_k >= number of blocks, n_last = n - 1 -- against this engine's dense output."""
    import minference_amd as M
    n, hq, hk = 131072, 2, 1
    q, k, v = gen.qkv(1, hq, hk, n, 128, seed=21, scale=1.0)
    qg, kg, vg = q.bfloat16().to(gpu), k.bfloat16().to(gpu), v.bfloat16().to(gpu)
    print("case full-size dense vs torch SDPA", flush=True)
    dense = M.dense_causal_attention(qg, kg, vg)
    ref = torch.nn.functional.scaled_dot_product_attention(qg, kg, vg, is_causal=True, enable_gqa=True)
    d = (dense.float() - ref.float()).abs()
    print(f"  dense vs SDPA: max-abs {d.max().item():.3e} mean-abs {d.mean().item():.3e}", flush=True)
    assert d.max().item() <= 2e-2 and d.mean().item() <= 1e-3
    del ref, d

    def same_as_dense(name, out, tol=4e-3):
        dd = (out.float() - dense.float()).abs()
        print(f"  {name} vs dense: max-abs {dd.max().item():.3e} mean-abs {dd.mean().item():.3e}", flush=True)
        assert dd.max().item() <= tol, name

    print("case full-size a-shape / tri-shape / block-sparse / vertical-slash in their dense limits", flush=True)
    same_as_dense("a-shape, window > n", M.streaming_forward(qg, kg, vg, 4, n + 5))
    same_as_dense("tri-shape, n_last = n - 1", M.tri_shape_forward(qg, kg, vg, 4, 64, n - 1))
    same_as_dense("block-sparse, top_k >= blocks", M.block_sparse_attention(qg, kg, vg, n // 64 + 1))
    s_idx = torch.arange(n, dtype=torch.int32, device=gpu)[None, None].expand(1, 1, n).contiguous()
    v_idx = torch.zeros((1, 1, 1), dtype=torch.int32, device=gpu)
    out = M.vertical_slash_sparse_attention(qg[:, :1], kg, vg, v_idx, s_idx)        # one head: 1 GiB of block lists
    dd = (out.float() - dense[:, :1].float()).abs()
    print(f"  vertical-slash, every diagonal vs dense: max-abs {dd.max().item():.3e} mean-abs {dd.mean().item():.3e}", flush=True)
    assert dd.max().item() <= 4e-3


def _fp32_rows_on_gpu(q_rows, k32, v32, mask):
    s_ = (q_rows.float() @ k32.T) * (q_rows.shape[-1] ** -0.5)
    s_ = s_.masked_fill(~mask, float("-inf"))
    return torch.softmax(s_, dim=-1) @ v32


def test_config2_whole_heads_against_fp32_masked_dense_on_the_gpu(gpu):
    """BASELINE config 2 at full size, EVERY row block of two heads (one of the first and one of the last
    kv group): the mask of each row block is expanded on the GPU from the index tensors the HIP builder
    wrote -- keys of every listed block up to the causal limit, plus the listed columns
    (pit_sparse_flash_attention_v2.py:104-148) -- and the rows are recomputed as an fp32 masked-dense
    softmax in torch.  Tolerance as everywhere: max-abs 2e-2, mean-abs 1e-3 per row block.  (The
    sampled tests above check the index rows against the reference algorithm and a few row blocks
    against the CPU oracle; this one leaves no row of a head unchecked.)"""
    import minference_amd as M
    n, hq, hk = 131072, 32, 8
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=100, dtype=torch.bfloat16)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    v_idx, s_idx = M.estimate_vertical_slash(qg, kg, 1000, 6096)
    seqlens = torch.full((1,), n, dtype=torch.int32, device=gpu)
    bc, bo, cc, ci = M.convert_vertical_slash_indexes(seqlens, v_idx, s_idx, n, 64, 64, zero_fill=False)
    out = M.vertical_slash_attention_from_index(qg, kg, vg, bc, bo, cc, ci, seqlens)
    torch.cuda.synchronize()
    ar64 = torch.arange(64, device=gpu)
    pos = torch.arange(n, device=gpu)
    for h in (2, 29):
        kv = h // (hq // hk)
        k32, v32 = kg[0, kv].float(), vg[0, kv].float()
        nb, nc = bc[0, h].tolist(), cc[0, h].tolist()
        worst_max = worst_mean = 0.0
        print(f"case c2 whole head {h}", flush=True)
        for m in range(n // 64):
            allowed = torch.zeros(n + 64, dtype=torch.bool, device=gpu)
            starts = bo[0, h, m, :nb[m]].long()
            allowed[(starts[:, None] + ar64[None, :]).reshape(-1).clamp_(0, n + 63)] = True
            rows = m * 64 + ar64
            mask = allowed[None, :n] & (pos[None, :] <= rows[:, None])
            if nc[m]:
                colmask = torch.zeros(n, dtype=torch.bool, device=gpu)
                colmask[ci[0, h, m, :nc[m]].long()] = True
                mask |= colmask[None, :]
            ref = _fp32_rows_on_gpu(qg[0, h, m * 64:m * 64 + 64], k32, v32, mask)
            err = (out[0, h, m * 64:m * 64 + 64].float() - ref).abs()
            worst_max, worst_mean = max(worst_max, err.max().item()), max(worst_mean, err.mean().item())
            assert err.max().item() <= 2e-2 and err.mean().item() <= 1e-3, (h, m, err.max().item(), err.mean().item())
        print(f"  head {h}: worst row block max-abs {worst_max:.3e} mean-abs {worst_mean:.3e}", flush=True)


def test_config4_and_config5_whole_heads_against_fp32_masked_dense_on_the_gpu(gpu):
    """Every row block of one head, fp32 masked-dense softmax recomputed in torch on the GPU: the
    block-sparse operator at BASELINE config 4's shape (131072 tokens, top-100 with diagonal and first
    block; mask = the first min(m + 1, top_k) listed blocks up to the causal limit,
    block_sparse_flash_attention.py:81-96) and the A-shape operator at config 5's (262144 tokens, sink 128
    + window 4096; mask = the closed form of streaming_kernel.py:35-75)."""
    import minference_amd as M
    from minference_amd.ops import _build_block_index, block_sparse_attention_from_index
    n5, hq, hk = 262144, 4, 1
    q, k, v, _ = gen.planted_layer(n5, hq, hk, seed=100, dtype=torch.bfloat16)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    ar64 = torch.arange(64, device=gpu)

    def sweep(tag, out, n, h, mask_of):
        k32, v32 = kg[0, 0, :n].float(), vg[0, 0, :n].float()
        worst_max = worst_mean = 0.0
        for m in range(n // 64):
            rows = m * 64 + ar64
            ref = _fp32_rows_on_gpu(qg[0, h, m * 64:m * 64 + 64], k32, v32, mask_of(m, rows))
            err = (out[0, h, m * 64:m * 64 + 64].float() - ref).abs()
            worst_max, worst_mean = max(worst_max, err.max().item()), max(worst_mean, err.mean().item())
            assert err.max().item() <= 2e-2 and err.mean().item() <= 1e-3, (tag, m, err.max().item(), err.mean().item())
        print(f"  {tag}: worst row block max-abs {worst_max:.3e} mean-abs {worst_mean:.3e}", flush=True)

    n4 = 131072
    print("case c4 whole head", flush=True)
    q4, k4, v4 = qg[:, :, :n4], kg[:, :, :n4], vg[:, :, :n4]
    bi = _build_block_index(q4, k4, 100, force_diag_first=True)
    out4 = block_sparse_attention_from_index(q4, k4, v4, bi)
    pos4 = torch.arange(n4, device=gpu)

    def bs_mask(m, rows, h=1):
        allowed = torch.zeros(n4 + 64, dtype=torch.bool, device=gpu)
        blocks = bi[0, h, m, :min(m + 1, 100)].long() * 64
        allowed[(blocks[:, None] + ar64[None, :]).reshape(-1)] = True
        return allowed[None, :n4] & (pos4[None, :] <= rows[:, None])
    sweep("block-sparse head 1 at 131072", out4, n4, 1, bs_mask)
    del out4, bi

    print("case c5 a-shape whole head", flush=True)
    out5 = M.streaming_forward(qg, kg, vg, 128, 4096)
    pos5 = torch.arange(n5, device=gpu)

    def ashape_mask(m, rows):
        d = rows[:, None] - pos5[None, :]
        return (d >= 0) & ((d < 4096) | (pos5[None, :] < 128))
    sweep("a-shape head 3 at 262144", out5, n5, 3, ashape_mask)


@pytest.mark.parametrize("d,dtype,n", [(64, torch.bfloat16, 65536), (128, torch.float16, 32768), (64, torch.float16, 20000 + 37)])
def test_whole_head_of_the_other_instantiations(gpu, d, dtype, n):
    """The head_dim 64 and the fp16 instantiations of the vertical-slash path (estimate -> top-k ->
    index -> attention), every row block of one head against the fp32 masked-dense softmax in torch
    on the GPU, incl. a length that is not a multiple of 64."""
    import minference_amd as M
    hq, hk = 2, 1
    q, k, v = gen.qkv(1, hq, hk, n, d, seed=d + n, scale=1.0)
    qg, kg, vg = q.to(dtype).to(gpu), k.to(dtype).to(gpu), v.to(dtype).to(gpu)
    v_idx, s_idx = M.estimate_vertical_slash(qg, kg, 300, 2000)
    seqlens = torch.full((1,), n, dtype=torch.int32, device=gpu)
    bc, bo, cc, ci = M.convert_vertical_slash_indexes(seqlens, v_idx, s_idx, n, 64, 64, zero_fill=False)
    out = M.vertical_slash_attention_from_index(qg, kg, vg, bc, bo, cc, ci, seqlens)
    assert torch.isfinite(out.float()).all()
    h = 1
    ar64 = torch.arange(64, device=gpu)
    pos = torch.arange(n, device=gpu)
    k32, v32 = kg[0, 0].float(), vg[0, 0].float()
    nb, nc = bc[0, h].tolist(), cc[0, h].tolist()
    worst_max = worst_mean = 0.0
    print(f"case whole head d={d} {dtype} n={n}", flush=True)
    for m in range((n + 63) // 64):
        rows = (m * 64 + ar64)[: min(64, n - m * 64)]
        allowed = torch.zeros(n + 128, dtype=torch.bool, device=gpu)
        starts = bo[0, h, m, :nb[m]].long()
        allowed[(starts[:, None] + ar64[None, :]).reshape(-1).clamp_(0, n + 127)] = True
        mask = allowed[None, :n] & (pos[None, :] <= rows[:, None])
        if nc[m]:
            colmask = torch.zeros(n, dtype=torch.bool, device=gpu)
            colmask[ci[0, h, m, :nc[m]].long()] = True
            mask |= colmask[None, :]
        ref = _fp32_rows_on_gpu(qg[0, h, rows], k32, v32, mask)
        err = (out[0, h, rows].float() - ref).abs()
        worst_max, worst_mean = max(worst_max, err.max().item()), max(worst_mean, err.mean().item())
        assert err.max().item() <= 2e-2 and err.mean().item() <= 1e-3, (m, err.max().item(), err.mean().item())
    print(f"  worst row block max-abs {worst_max:.3e} mean-abs {worst_mean:.3e}", flush=True)


def test_index_tensors_of_more_than_2_to_31_elements(gpu):
    """32 heads x 16384 row blocks x 6096 slash slots at 1 048 576 tokens: block_offset holds 1.49 x 2^31
    elements (12.8 GB), so every offset into it -- in the index builder and in the attention kernel's
    list walk -- has to be 64-bit (the reference's int offsets overflow here,
    csrc/vertical_slash_index.cu:55-59).  The lists keep the attention cheap (a window of 64..192
    diagonals, twenty far ones, the rest beyond the context, i.e. skipped; 1000 verticals); sampled
    (head, row block) pairs from the first and the last heads: index rows against the reference
    algorithm, attention rows against an fp32 masked-dense softmax in torch on the GPU."""
    import minference_amd as M
    n, hq, hk, S, V = 1048576, 32, 8, 6096, 1000
    g = torch.Generator(device=gpu).manual_seed(5)
    q = torch.randn(1, hq, n, 128, generator=g, device=gpu, dtype=torch.bfloat16)
    k = torch.randn(1, hk, n, 128, generator=g, device=gpu, dtype=torch.bfloat16)
    v = torch.randn(1, hk, n, 128, generator=g, device=gpu, dtype=torch.bfloat16)
    rng = np.random.default_rng(7)
    s_np, v_np = np.zeros((1, hq, S), np.int64), np.zeros((1, hq, V), np.int64)
    for h in range(hq):
        near = np.arange(int(rng.integers(64, 193)))
        far = rng.choice(np.arange(1000, n), size=20, replace=False)
        beyond = n + np.arange(S - len(near) - len(far)) * 3 + int(rng.integers(0, 1000))
        s_np[0, h] = np.sort(np.concatenate([near, far, beyond]))[::-1]
        v_np[0, h] = np.sort(np.concatenate([np.arange(4), rng.choice(np.arange(4, n), size=V - 4, replace=False)]))
    s_idx, v_idx = torch.from_numpy(s_np.astype(np.int32)).to(gpu), torch.from_numpy(v_np.astype(np.int32)).to(gpu)
    seqlens = torch.full((1,), n, dtype=torch.int32, device=gpu)
    print("case index tensors beyond 2^31 elements", flush=True)
    bc, bo, cc, ci = M.convert_vertical_slash_indexes(seqlens, v_idx, s_idx, n, 64, 64, zero_fill=False)
    assert bo.numel() > 2 ** 31
    out = M.vertical_slash_attention_from_index(q, k, v, bc, bo, cc, ci, seqlens)
    torch.cuda.synchronize()
    rows = n // 64
    pos = torch.arange(n, device=gpu)
    for h, m in [(0, 0), (0, rows - 1), (20, 5), (21, 8000), (22, rows - 1), (31, 0), (31, 12345), (31, rows - 1), (30, rows - 2)]:
        rbo, rci = O.vs_index_row_py(v_np[0, h].tolist(), s_np[0, h].tolist(), m, n)
        assert int(bc[0, h, m]) == len(rbo) and int(cc[0, h, m]) == len(rci), (h, m)
        assert bo[0, h, m, :len(rbo)].cpu().tolist() == rbo and ci[0, h, m, :len(rci)].cpu().tolist() == rci, (h, m)
        allowed = torch.zeros(n + 128, dtype=torch.bool, device=gpu)
        for st in rbo:
            allowed[st:st + 64] = True
        rows_m = m * 64 + torch.arange(64, device=gpu)
        mask = allowed[None, :n] & (pos[None, :] <= rows_m[:, None])
        if rci:
            col = torch.zeros(n, dtype=torch.bool, device=gpu)
            col[torch.tensor(rci, device=gpu)] = True
            mask |= col[None, :]
        ref = _fp32_rows_on_gpu(q[0, h, rows_m], k[0, h // 4].float(), v[0, h // 4].float(), mask)
        err = (out[0, h, rows_m].float() - ref).abs()
        print(f"  head {h} row block {m}: blocks {len(rbo)} cols {len(rci)} max-abs {err.max().item():.3e}", flush=True)
        assert err.max().item() <= 2e-2 and err.mean().item() <= 1e-3, (h, m)


def test_block_index_at_one_million_tokens(gpu):
    """The block index of 32 heads at 1 048 576 tokens: 16385 block rows, so the pooled score matrix in
    the workspace has 8.6e9 elements (more than 2^31; 34 GB) and the general top-k runs on 524 320 rows
    of 16388 scores.  Sampled rows of the first, a middle and the last head against the reference's
    arithmetic restated with torch on the GPU (bf16 means, bf16 pooled products,
    block_sparse_flash_attention.py:159-163; an entry the restatement lacks must lie within one bf16
    unit of its k-th score)."""
    from minference_amd.ops import _build_block_index
    n, hq, hk = 1048576, 32, 8
    g = torch.Generator(device=gpu).manual_seed(5)
    q = torch.randn(1, hq, n, 128, generator=g, device=gpu, dtype=torch.bfloat16)
    k = torch.randn(1, hk, n, 128, generator=g, device=gpu, dtype=torch.bfloat16)
    # a slow drift shared by q and k, so that the pooled scores separate
    drift = torch.cumsum(torch.randn(n // 64 + 1, 128, generator=g, device=gpu) * 0.3, 0).repeat_interleave(64, 0)[:n]
    q, k = (q.float() + drift[None, None]).bfloat16(), (k.float() + drift[None, None]).bfloat16()
    del drift
    print("case block index at 1M tokens", flush=True)
    bi = _build_block_index(q, k, 100, force_diag_first=True)
    R = bi.shape[2]
    assert bi.shape == (1, hq, n // 64 + 1, 100)
    for h in (0, 13, 31):
        qp = torch.nn.functional.pad(q[0, h].float(), [0, 0, 0, 64]).reshape(R, 64, 128).mean(1).bfloat16().float()
        kp = torch.nn.functional.pad(k[0, h // 4].float(), [0, 0, 0, 64]).reshape(R, 64, 128).mean(1).bfloat16().float()
        for m in (0, 1, 99, 100, 5000, 12000, R - 2, R - 1):
            sc = (kp[: m + 1] @ qp[m]).bfloat16().float()
            sc[m] = sc[0] = float("inf")
            kk = min(100, m + 1)
            want = torch.argsort(sc, descending=True, stable=True)[:kk]
            got = bi[0, h, m, :kk].long()
            assert bool((got[1:] > got[:-1]).all()), (h, m)
            kth = sc[want].min().item()
            extra = set(got.tolist()) - set(want.tolist())
            assert all(x <= m and sc[x].item() >= kth - abs(kth) * 2.0 ** -6 - 1e-6 for x in extra), (h, m, sorted(extra)[:5])
