"""GPU tests of the per-head dispatcher and the fused vertical-slash layer path."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import gen

pytestmark = pytest.mark.gpu


def expand(x, hq):
    return x.repeat_interleave(hq // x.shape[1], dim=1)


def test_mixed_patterns_route_to_the_right_kernels(gpu):
    import minference_amd as M
    n, hq, hk = 1024, 8, 2
    q, k, v = gen.qkv(1, hq, hk, n, 128, seed=3, scale=1.0)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    layer = {"0": ["stream_llm", 64, 256, 1.0], "1": ["stream_llm", 64, 256, 1.0],
             "2": ["block_sparse", 100, 6096, 1.0], "5": ["vertical_and_slash", 100, 300, 1.0]}
    kwargs = {"layer_idx": 1, "attn_forward_config": {"best_pattern": [{}, layer], "starting_layer": 1}}
    out = M.minference_prefill_forward(q.to(gpu), k.to(gpu), v.to(gpu), kwargs).float().cpu()
    ke, ve = expand(k, hq), expand(v, hq)
    ref_stream = O.streaming_forward(q[:, :2], ke[:, :2], ve[:, :2], 64, 256)
    assert (out[:, :2] - ref_stream).abs().max() <= 2e-2
    ref_dense = torch.nn.functional.scaled_dot_product_attention(q[:, 2:3].float(), ke[:, 2:3].float(), ve[:, 2:3].float(), is_causal=True)
    assert (out[:, 2:3] - ref_dense).abs().max() <= 2e-2          # top-100 of 16 blocks = dense causal
    # vertical_and_slash heads: same result as the explicit estimate -> op chain on those heads
    v_idx, s_idx = M.estimate_vertical_slash(q[:, 5:6].to(gpu), k[:, 1:2].to(gpu), 100, 300)
    ref_vs = O.vertical_slash_sparse_attention(q[:, 5:6], ke[:, 5:6], ve[:, 5:6], v_idx.cpu(), s_idx.cpu())
    assert (out[:, 5:6] - ref_vs).abs().max() <= 2e-2
    # default pattern heads (3, 4, 6, 7): vertical 1000 / slash 6096 clamp to n -> dense causal
    ref_def = torch.nn.functional.scaled_dot_product_attention(q[:, 3:5].float(), ke[:, 3:5].float(), ve[:, 3:5].float(), is_causal=True)
    assert (out[:, 3:5] - ref_def).abs().max() <= 2e-2


def test_mixed_patterns_at_head_dim_96(gpu):
    """A Phi-3-shaped head_dim (96, zero-padded to 128 by the operators): every head of a mixed layer
    equals its own operator call bit for bit -- in particular the stream_llm heads, which the
    reference scales by the PADDED head_dim (streaming_kernel.py:575), the others by head_dim^-0.5
    (pit_sparse_flash_attention_v2.py:221)."""
    import minference_amd as M
    n, hq, hk, d = 1500, 4, 2, 96
    q, k, v = gen.qkv(1, hq, hk, n, d, seed=5, scale=1.0)
    q, k, v = q.bfloat16().to(gpu), k.bfloat16().to(gpu), v.bfloat16().to(gpu)
    layer = {"0": ["stream_llm", 16, 200, 1.0], "1": ["vertical_and_slash", 100, 300, 1.0],
             "2": ["block_sparse", 100, 0, 1.0], "3": ["stream_llm", 16, 200, 1.0]}
    out = M.minference_prefill_forward(q, k, v, {"layer_idx": 0, "attn_forward_config": {"best_pattern": [layer]}})
    assert out.shape == q.shape
    for h in range(hq):
        qh, kh, vh = q[:, h:h + 1], k[:, h // 2:h // 2 + 1], v[:, h // 2:h // 2 + 1]
        ty = layer[str(h)][0]
        ref = (M.streaming_forward(qh, kh, vh, 16, 200) if ty == "stream_llm" else
               M.vertical_slash_prefill(qh, kh, vh, 100, 300) if ty == "vertical_and_slash" else
               M.block_sparse_attention(qh, kh, vh, 100))
        assert torch.equal(out[:, h:h + 1], ref), (h, ty)
    want = O.streaming_forward(q[:, :1].cpu(), k[:, :1].cpu(), v[:, :1].cpu(), 16, 200)
    assert (out[:, :1].float().cpu() - want).abs().max() <= 2e-2


def _ragged_table(hq):
    """Per-head patterns in the shape of the shipped Llama-3-8B table: vertical_and_slash heads with
    five distinct (vertical, slash) sizes, block_sparse heads, stream_llm heads with two settings."""
    sizes = [(1000, 6096), (500, 3000), (30, 800), (100, 750), (3500, 100)]
    layer = {}
    for h in range(hq):
        if h % 8 == 3:
            layer[str(h)] = ["block_sparse", 100, 0, 1.0]
        elif h % 8 == 6:
            layer[str(h)] = ["stream_llm", 100, 800, 1.0] if h < hq // 2 else ["stream_llm", 64, 1500, 1.0]
        else:
            v, s = sizes[(h * 7) % 5]
            layer[str(h)] = ["vertical_and_slash", v, s, 1.0]
    return layer


def test_ragged_per_head_sizes_one_launch_chain_per_type(gpu, monkeypatch):
    """A 32-head layer (8 kv heads) whose table mixes five (vertical, slash) sizes, block_sparse and
    two stream_llm settings: the dispatcher must issue ONE estimation, ONE top-k, ONE index build and
    ONE attention launch for all vertical_and_slash heads (ragged sizes), one block index + one
    attention launch for the block_sparse heads, one launch per stream_llm setting -- and the result
    must be bit-identical to running every head on its own through the public operators (what the
    reference's per-head loop does, minference_forward.py:657-667)."""
    import minference_amd as M
    from minference_amd import _lib
    n, hq, hk = 8192 + 40, 32, 8
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=7, dtype=torch.bfloat16)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    layer = _ragged_table(hq)
    kwargs = {"layer_idx": 0, "attn_forward_config": {"best_pattern": [layer]}}
    lib = _lib.load()
    counts = {}
    for name in ("minf_vs_estimate_heads", "minf_topk_indices_pair_ragged", "minf_vs_index_build_ws", "minf_vs_attn_fwd",
                 "minf_bs_block_index_heads", "minf_bs_attn_fwd", "minf_ashape_attn_fwd", "minf_vs_estimate"):
        real = getattr(lib, name)

        def counting(*a, _real=real, _name=name):
            counts[_name] = counts.get(_name, 0) + 1
            return _real(*a)
        monkeypatch.setattr(lib, name, counting)
    print("case ragged dispatcher, one chain per type", flush=True)
    out = M.minference_prefill_forward(qg, kg, vg, kwargs)
    torch.cuda.synchronize()
    assert counts == {"minf_vs_estimate_heads": 1, "minf_topk_indices_pair_ragged": 1, "minf_vs_index_build_ws": 1,
                      "minf_vs_attn_fwd": 1, "minf_bs_block_index_heads": 1, "minf_bs_attn_fwd": 1,
                      "minf_ashape_attn_fwd": 2}, counts
    monkeypatch.undo()
    assert out.shape == q.shape and out.dtype == torch.bfloat16 and torch.isfinite(out.float()).all()
    group = hq // hk
    for h in range(hq):
        ty, a, b, _ = layer[str(h)]
        qh, kh, vh = qg[:, h:h + 1], kg[:, h // group:h // group + 1], vg[:, h // group:h // group + 1]
        if ty == "vertical_and_slash":
            ref = M.vertical_slash_prefill(qh, kh, vh, a, b)
        elif ty == "block_sparse":
            ref = M.block_sparse_attention(qh, kh, vh, 100)
        else:
            ref = M.streaming_forward(qh, kh, vh, a, b)
        assert torch.equal(out[:, h:h + 1], ref), f"head {h} ({ty} {a} {b}) differs from its own per-head run"
    # and against the oracle for one head of each kind (same indices as the GPU produced)
    for h in (0, 3, 6):
        ty, a, b, _ = layer[str(h)]
        kv = h // group
        if ty == "vertical_and_slash":
            v_idx, s_idx = M.estimate_vertical_slash(qg[:, h:h + 1], kg[:, kv:kv + 1], a, b)
            ref = O.vertical_slash_sparse_attention(q[:, h:h + 1], k[:, kv:kv + 1], v[:, kv:kv + 1], v_idx.cpu(), s_idx.cpu())
        elif ty == "block_sparse":
            from minference_amd.ops import _build_block_index
            bi = _build_block_index(qg[:, h:h + 1], kg[:, kv:kv + 1], 100)[0, 0].cpu().numpy()
            ref = O.masked_attention(q[0, h], k[0, kv], v[0, kv], O.bs_mask(bi, n))[None, None]
        else:
            ref = O.streaming_forward(q[:, h:h + 1], k[:, kv:kv + 1], v[:, kv:kv + 1], a, b)
        err = (out[:, h:h + 1].float().cpu() - ref).abs()
        print(f"  head {h} {ty}: max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e}", flush=True)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3


def test_second_call_of_a_layer_issues_no_host_to_device_copy(gpu, monkeypatch):
    """The per-layer plan (parsed table, head lists, per-head top-k sizes) is built on a layer's
    first call and reused: the second call with the same table builds no tensor from host data and
    copies nothing from the host (the reference does one H2D copy per head and call,
    pit_sparse_flash_attention_v2.py:220), and returns the same bits."""
    import minference_amd as M
    from minference_amd import prefill
    n, hq, hk = 4096 + 17, 32, 8
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=11, dtype=torch.bfloat16)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    kwargs = {"layer_idx": 0, "attn_forward_config": {"best_pattern": [_ragged_table(hq)]}}
    prefill.clear_plan_cache()
    print("case plan cache: first call", flush=True)
    first = M.minference_prefill_forward(qg, kg, vg, kwargs)
    torch.cuda.synchronize()
    made, copied = [], []
    real_tensor, real_to = torch.tensor, torch.Tensor.to

    def counting_tensor(*a, **kw):
        made.append(a)
        return real_tensor(*a, **kw)

    def counting_to(self, *a, **kw):
        if not self.is_cuda and any(isinstance(x, (torch.device, str)) and "cuda" in str(x) for x in list(a) + list(kw.values())):
            copied.append(tuple(self.shape))
        return real_to(self, *a, **kw)
    monkeypatch.setattr(torch, "tensor", counting_tensor)
    monkeypatch.setattr(torch.Tensor, "to", counting_to)
    monkeypatch.setattr(torch.Tensor, "cuda", lambda self, *a, **kw: (_ for _ in ()).throw(AssertionError("Tensor.cuda called")))
    print("case plan cache: second call", flush=True)
    second = M.minference_prefill_forward(qg, kg, vg, kwargs)
    monkeypatch.undo()
    torch.cuda.synchronize()
    assert made == [] and copied == [], (made, copied)
    assert torch.equal(first, second)
    # another prompt length with the same table: new device tensors once, then none again
    q2, k2, v2 = qg[:, :, :2048], kg[:, :, :2048], vg[:, :, :2048]
    a = M.minference_prefill_forward(q2, k2, v2, kwargs)
    monkeypatch.setattr(torch, "tensor", counting_tensor)
    b = M.minference_prefill_forward(q2, k2, v2, kwargs)
    monkeypatch.undo()
    assert made == [] and torch.equal(a, b)


def test_head_selection_leaves_other_heads_untouched(gpu):
    """minf_qkvo.head_list through the C ABI: a dense launch restricted to heads {1, 4, 5} of 6 writes
    exactly those heads of the output buffer and reproduces the unrestricted launch on them."""
    import ctypes
    from minference_amd import _lib
    from minference_amd.ops import _Call
    n, hq, hk = 700, 6, 2
    q, k, v = gen.qkv(1, hq, hk, n, 128, seed=12, scale=1.0)
    q, k, v = q.bfloat16().to(gpu), k.bfloat16().to(gpu), v.bfloat16().to(gpu)
    lib = _lib.load()
    full = _Call(q, k, v)
    assert lib.minf_dense_attn_fwd(full.ref, _lib.stream_ptr(gpu)) == 0
    part = _Call(q, k, v)
    part.o.fill_(-3.0)
    part.select_heads(torch.tensor([1, 4, 5], dtype=torch.int32, device=gpu))
    assert lib.minf_dense_attn_fwd(part.ref, _lib.stream_ptr(gpu)) == 0
    torch.cuda.synchronize()
    for h in range(hq):
        if h in (1, 4, 5):
            assert torch.equal(part.o[:, h], full.o[:, h])
        else:
            assert (part.o[:, h] == -3.0).all()
    # a list without a length is refused
    part.struct.index_heads = 0
    assert lib.minf_dense_attn_fwd(part.ref, _lib.stream_ptr(gpu)) == -1


def test_starting_layer_falls_back_to_dense(gpu):
    import minference_amd as M
    q, k, v = gen.qkv(1, 4, 4, 512, 128, seed=4, scale=1.0)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    kwargs = {"layer_idx": 0, "attn_forward_config": {"best_pattern": [{"0": ["stream_llm", 4, 16, 1]}], "starting_layer": 2}}
    out = M.minference_prefill_forward(q.to(gpu), k.to(gpu), v.to(gpu), kwargs).float().cpu()
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True)
    assert (out - ref).abs().max() <= 2e-2


def test_a_shape_and_tri_shape_kernels_take_the_reference_config(gpu):
    """``a_shape_kernel(q, k, v, config)`` / ``tri_shape_kernel(q, k, v, config)`` with the
    reference's config dictionary and its defaults (streaming_kernel.py:781-833: n_init 128,
    n_local 3968, n_last 100) against the masked-dense oracle."""
    import minference_amd as M
    n = 5000                                                        # longer than n_init + n_local
    q, k, v = gen.qkv(1, 2, 2, n, 128, seed=21, scale=1.0)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    dq, dk, dv = q.to(gpu), k.to(gpu), v.to(gpu)
    for cfg, (ni, nl, nlast) in (({}, (128, 3968, 100)), ({"n_init": 16, "n_local": 700, "n_last": 33}, (16, 700, 33))):
        kwargs = {"attn_forward_config": cfg}
        a = M.a_shape_kernel(dq, dk, dv, kwargs).float().cpu()
        t = M.tri_shape_kernel(dq, dk, dv, kwargs).float().cpu()
        for h in range(2):
            for got, mask in ((a, O.ashape_mask(n, ni, nl)), (t, O.trishape_mask(n, ni, nl, nlast))):
                err = (got[0, h] - O.masked_attention(q[0, h], k[0, h], v[0, h], mask)).abs()
                assert err.max() <= 2e-2 and err.mean() <= 1e-3, (cfg, h, float(err.max()))


def test_config1_shape_fp32_full(gpu):
    """BASELINE config 1 at full size (batch 1, 4 heads, seq 8192, head_dim 128, fp32, vertical 1000,
    slash 2048): op output vs fp32 masked-dense on identical indices, sampled row blocks."""
    import minference_amd as M
    n = 8192
    q, k, v = gen.qkv(1, 4, 4, n, 128, seed=0, dtype=torch.float32)
    v_idx, s_idx = M.estimate_vertical_slash(q.to(gpu), k.to(gpu), 1000, 2048)
    out = M.vertical_slash_sparse_attention(q.to(gpu), k.to(gpu), v.to(gpu), v_idx, s_idx).cpu()
    assert out.dtype == torch.float32 and out.shape == q.shape
    ref = O.vertical_slash_sparse_attention(q[:, :1], k[:, :1], v[:, :1], v_idx[:, :1].cpu(), s_idx[:, :1].cpu())
    err = (out[:, :1] - ref).abs()
    assert err.max() <= 2e-2 and err.mean() <= 1e-3
    # the inputs are N(0,1)/sqrt(128): outputs are of order 1e-2, so the bound that means something
    # is the one relative to the output magnitude
    scale = ref.abs().max()
    print(f"config 1: max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e} max|ref| {scale.item():.3e}", flush=True)
    assert err.max() <= 2e-2 * scale and err.mean() <= 1e-3 * scale


def test_config2_full_size_sampled_row_blocks(gpu):
    """BASELINE config 2 at full length (131072 tokens, GQA 4:1, bf16, vertical 1000, slash 6096,
    planted structure; 4 query heads to keep the host work small) with a ragged tail (n % 64 != 0):
    the whole GPU path (estimate -> top-k -> index -> attention), then for sampled (head, row block)
    pairs, incl. the first, the last partial one and the forced-diagonal region, the fp32
    masked-dense oracle on the index entries the GPU produced."""
    import minference_amd as M
    n, hq, hk = 131072 - 37, 4, 1
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=100, dtype=torch.bfloat16)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    v_idx, s_idx = M.estimate_vertical_slash(qg, kg, 1000, 6096)
    seqlens = torch.full((1,), n, dtype=torch.int32, device=gpu)
    bc, bo, cc, ci = M.convert_vertical_slash_indexes(seqlens, v_idx, s_idx, n, 64, 64)
    out = M.vertical_slash_attention_from_index(qg, kg, vg, bc, bo, cc, ci, seqlens)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    # the index rows the GPU built are the reference algorithm's rows (C restatement, bit-exact)
    rows = (n + 63) // 64
    vi_c, si_c = v_idx.cpu().numpy(), s_idx.cpu().numpy()
    for h, m in [(0, 0), (1, 1), (2, 777), (3, rows - 1), (0, rows - 2), (1, 1024)]:
        print(f"case c2-full head={h} row-block={m}", flush=True)
        rbo, rci = O.vs_index_row_py(vi_c[0, h].tolist(), si_c[0, h].tolist(), m, n)
        rbc, rcc = len(rbo), len(rci)
        assert int(bc[0, h, m]) == rbc and int(cc[0, h, m]) == rcc
        assert bo[0, h, m, :rbc].cpu().tolist() == rbo and ci[0, h, m, :rcc].cpu().tolist() == rci
        mask = O.vs_mask_rows(rbc, rbo, rcc, rci, m, n)
        r0, r1 = m * 64, min(m * 64 + 64, n)
        s = (q[0, h, r0:r1].float() @ k[0, 0].float().T) * (128 ** -0.5)
        s = torch.where(torch.as_tensor(mask), s, torch.tensor(-torch.inf))
        ref = torch.softmax(s, dim=-1) @ v[0, 0].float()
        err = (out[0, h, r0:r1].float().cpu() - ref).abs()
        scale = ref.abs().max().item()
        print(f"  max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e} (max |ref| {scale:.3e})", flush=True)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3
        # and relative to the size of the outputs (rows that average over thousands of keys are small)
        assert err.max() <= 2e-2 * scale and err.mean() <= 1e-3 * scale


def test_one_million_tokens_sampled_row_blocks(gpu):
    """The longest context the reference advertises (Llama-3-8B-1M): 1 048 576 tokens minus a ragged
    tail, 2 query heads on one kv head, the whole GPU path with zero-filled index tensors; sampled
    row blocks are checked like in the 131072-token test (index rows bit-exact against the reference
    algorithm, attention rows against the fp32 masked-dense result)."""
    import minference_amd as M
    n, hq, hk = 1048576 - 11, 2, 1
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=101, dtype=torch.bfloat16)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    v_idx, s_idx = M.estimate_vertical_slash(qg, kg, 1000, 6096)
    seqlens = torch.full((1,), n, dtype=torch.int32, device=gpu)
    bc, bo, cc, ci = M.convert_vertical_slash_indexes(seqlens, v_idx, s_idx, n, 64, 64)
    out = M.vertical_slash_attention_from_index(qg, kg, vg, bc, bo, cc, ci, seqlens)
    torch.cuda.synchronize()
    rows = (n + 63) // 64
    assert bc.shape == (1, hq, rows) and int(bc.max()) <= 6096 and int(cc.max()) <= 1000
    vi_c, si_c = v_idx.cpu().numpy(), s_idx.cpu().numpy()
    kf, vf = k[0, 0].float(), v[0, 0].float()
    for h, m in [(0, 0), (1, rows - 1), (0, 9000), (1, 16000)]:
        print(f"case 1M head={h} row-block={m}", flush=True)
        rbo, rci = O.vs_index_row_py(vi_c[0, h].tolist(), si_c[0, h].tolist(), m, n)
        rbc, rcc = len(rbo), len(rci)
        assert int(bc[0, h, m]) == rbc and int(cc[0, h, m]) == rcc
        assert bo[0, h, m, :rbc].cpu().tolist() == rbo and ci[0, h, m, :rcc].cpu().tolist() == rci
        assert int(bo[0, h, m, rbc:].abs().max() if rbc < 6096 else 0) == 0          # zero tail
        mask = O.vs_mask_rows(rbc, rbo, rcc, rci, m, n)
        r0, r1 = m * 64, min(m * 64 + 64, n)
        s = (q[0, h, r0:r1].float() @ kf.T) * (128 ** -0.5)
        s = torch.where(torch.as_tensor(mask), s, torch.tensor(-torch.inf))
        ref = torch.softmax(s, dim=-1) @ vf
        err = (out[0, h, r0:r1].float().cpu() - ref).abs()
        scale = ref.abs().max().item()
        print(f"  max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e} (max |ref| {scale:.3e})", flush=True)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3
        # and relative to the size of the outputs (rows that average over thousands of keys are small)
        assert err.max() <= 2e-2 * scale and err.mean() <= 1e-3 * scale


def _rows_reference(q_rows, k, v, mask):
    s = (q_rows.float() @ k.float().T) * (q_rows.shape[-1] ** -0.5)
    s = torch.where(torch.as_tensor(mask), s, torch.tensor(-torch.inf))
    return torch.softmax(s, dim=-1) @ v.float()


def test_config4_full_size_sampled_row_blocks(gpu):
    """BASELINE config 4 at full length (131072 tokens, top-100 key blocks incl. diagonal and block
    0, GQA, bf16; 2 query heads): block index from the HIP kernels checked against fp32 pooled
    scores for sampled query blocks, attention checked on the same row blocks."""
    from minference_amd.ops import _build_block_index, block_sparse_attention_from_index
    n, hq, hk, top_k = 131072, 2, 1, 100
    q, k, v, _ = gen.planted_layer(n, hq, hk, seed=101, dtype=torch.bfloat16)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    bi = _build_block_index(qg, kg, top_k, force_diag_first=True)
    out = block_sparse_attention_from_index(qg, kg, vg, bi)
    torch.cuda.synchronize()
    R = n // 64 + 1
    assert tuple(bi.shape) == (1, hq, R, top_k)
    # bf16 inputs: pooled means and pooled products are held in bf16 by the reference's torch code
    # (block_sparse_flash_attention.py:159-163) and rounded there by the HIP kernels' default mode
    kp = torch.nn.functional.pad(k[0, 0].float(), [0, 0, 0, 64]).reshape(R, 64, 128).mean(1).to(torch.bfloat16).float()
    bic = bi[0].cpu().numpy()
    for h, m in [(0, 0), (1, 5), (0, 99), (1, 100), (0, 1500), (1, 2047)]:
        print(f"case c4-full head={h} query-block={m}", flush=True)
        row = bic[h, m]
        assert (np.diff(row) > 0).all()
        p = (q[0, h, m * 64: m * 64 + 64].float().mean(0).to(torch.bfloat16).float() @ kp.T).to(torch.bfloat16).float().numpy()
        p[m + 1:] = -np.inf
        p[m] = p[0] = np.inf
        kth = np.sort(p)[::-1][top_k - 1]
        sel = np.zeros(R, bool); sel[row] = True
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
        ref = _rows_reference(q[0, h, m * 64: m * 64 + 64], k[0, 0], v[0, 0], mask)
        err = (out[0, h, m * 64: m * 64 + 64].float().cpu() - ref).abs()
        scale = ref.abs().max().item()
        print(f"  max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e} (max |ref| {scale:.3e})", flush=True)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3
        # and relative to the size of the outputs (rows that average over thousands of keys are small)
        assert err.max() <= 2e-2 * scale and err.mean() <= 1e-3 * scale


def test_config5_ashape_heads_full_size_sampled_row_blocks(gpu):
    """BASELINE config 5's A-shape heads at full length (262144 tokens, sink 128 + local 4096, GQA,
    bf16; 2 query heads), sampled row blocks against the closed-form mask
    {k : r - n_local < k <= r} U {k < n_init : k <= r - n_local}."""
    import minference_amd as M
    n, hq, hk, n_init, n_local = 262144 - 5, 2, 1, 128, 4096
    q, k, v = gen.qkv(1, hq, hk, n, 128, seed=55, dtype=torch.bfloat16, scale=1.0)
    out = M.streaming_forward(q.to(gpu), k.to(gpu), v.to(gpu), n_init, n_local)
    torch.cuda.synchronize()
    rows = (n + 63) // 64
    for h, m in [(0, 0), (1, 1), (0, 63), (1, 64), (0, 65), (1, 2000), (0, rows - 1)]:
        print(f"case c5-ashape head={h} row-block={m}", flush=True)
        r0, r1 = m * 64, min(m * 64 + 64, n)
        r = np.arange(r0, r1)[:, None]
        c = np.arange(n)[None, :]
        mask = ((c <= r) & (c > r - n_local)) | ((c < n_init) & (c <= r - n_local))
        ref = _rows_reference(q[0, h, r0:r1], k[0, 0], v[0, 0], mask)
        err = (out[0, h, r0:r1].float().cpu() - ref).abs()
        scale = ref.abs().max().item()
        print(f"  max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e} (max |ref| {scale:.3e})", flush=True)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3
        # and relative to the size of the outputs (rows that average over thousands of keys are small)
        assert err.max() <= 2e-2 * scale and err.mean() <= 1e-3 * scale


def test_mixed_layer_replays_from_a_hip_graph(gpu):
    """Every launch chain of a mixed layer (estimate -> ragged top-k -> index build -> vertical-slash
    attention; block index -> block-sparse attention; A-shape) recorded once into a HIP graph through
    torch.cuda.graph and replayed on new inputs written into the captured buffers: each replay must be
    bit-identical to the eager call on the same inputs.  Between the replays the process does eager
    work and synchronises, and the layer's host-side plan (head lists, per-head sizes) is already on
    the device, so the capture contains no host-to-device copy and no allocation outside torch's
    graph pool."""
    import minference_amd as M
    n, hq, hk = 8192 + 64, 8, 2
    layer = {"0": ["vertical_and_slash", 1000, 6096, 1.0], "1": ["vertical_and_slash", 100, 800, 1.0],
             "2": ["block_sparse", 100, 0, 1.0], "3": ["stream_llm", 64, 1024, 1.0],
             "4": ["vertical_and_slash", 500, 3000, 1.0], "5": ["block_sparse", 100, 0, 1.0],
             "6": ["stream_llm", 128, 512, 1.0]}                      # head 7: the default pattern
    kwargs = {"layer_idx": 0, "attn_forward_config": {"best_pattern": [layer]}}
    inputs = [tuple(t.to(gpu) for t in gen.planted_layer(n, hq, hk, seed=s, dtype=torch.bfloat16)[:3]) for s in (1, 2, 3)]
    qs, ks, vs = (t.clone() for t in inputs[0])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            M.minference_prefill_forward(qs, ks, vs, kwargs)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    print("case graph capture of a mixed layer", flush=True)
    with torch.cuda.graph(graph):
        out_static = M.minference_prefill_forward(qs, ks, vs, kwargs)
    for rep, (q, k, v) in enumerate(inputs + inputs[:1]):
        qs.copy_(q); ks.copy_(k); vs.copy_(v)
        graph.replay()
        torch.cuda.synchronize()
        got = out_static.clone()
        eager = M.minference_prefill_forward(q, k, v, kwargs)          # eager work between the replays
        torch.cuda.synchronize()
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, eager), f"replay {rep} differs from the eager call"
