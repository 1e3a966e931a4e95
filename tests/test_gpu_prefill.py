"""GPU tests of the per-head dispatcher and the fused vertical-slash layer path."""
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


def test_starting_layer_falls_back_to_dense(gpu):
    import minference_amd as M
    q, k, v = gen.qkv(1, 4, 4, 512, 128, seed=4, scale=1.0)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    kwargs = {"layer_idx": 0, "attn_forward_config": {"best_pattern": [{"0": ["stream_llm", 4, 16, 1]}], "starting_layer": 2}}
    out = M.minference_prefill_forward(q.to(gpu), k.to(gpu), v.to(gpu), kwargs).float().cpu()
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True)
    assert (out - ref).abs().max() <= 2e-2


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
