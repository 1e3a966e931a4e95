"""The Llama block stack around the sparse attention path (minference_amd/llama.py): conventions
(RMSNorm, RoPE, GQA, SwiGLU, weight names) pinned against transformers' LlamaForCausalLM on the CPU
in fp32, per-head pattern dispatch pinned against an fp32 restatement with the oracle's masks."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

TINY = dict(vocab_size=500, hidden_size=256, intermediate_size=512, num_layers=2, num_heads=2,
            num_kv_heads=1, head_dim=128, rope_theta=500000.0, rms_eps=1e-5)


def _hf_model(seed):
    tr = pytest.importorskip("transformers")
    kw = dict(vocab_size=500, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
              num_attention_heads=2, num_key_value_heads=1, head_dim=128, rms_norm_eps=1e-5,
              max_position_embeddings=4096, attention_bias=False, mlp_bias=False, tie_word_embeddings=False)
    try:
        cfg = tr.LlamaConfig(rope_theta=500000.0, **kw)
    except TypeError:
        cfg = tr.LlamaConfig(rope_parameters={"rope_type": "default", "rope_theta": 500000.0}, **kw)
    torch.manual_seed(seed)
    model = tr.LlamaForCausalLM(cfg).float().eval()
    theta = getattr(cfg, "rope_theta", None)
    if theta is None:
        theta = cfg.rope_parameters["rope_theta"]
    assert float(theta) == 500000.0
    return model


def test_dense_equivalent_patterns_match_transformers_llama(gpu):
    from minference_amd.llama import LlamaConfig, LlamaPrefill
    hf = _hf_model(0)
    n = 700
    ids = torch.randint(0, 500, (n,), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        ref = hf(input_ids=ids[None]).logits[0, -1].float()
    m = LlamaPrefill(LlamaConfig(**TINY), device=gpu)
    m.load_state_dict(hf.state_dict())
    # every head's pattern covers the whole causal triangle, each through a different kernel
    pat = [{"0": ["stream_llm", 4, 4096, 1], "1": ["vertical_and_slash", 4096, 4096, 1]},
           {"0": ["block_sparse", 100, 0, 1], "1": ["stream_llm", 0, 1000, 1]}]
    logits, _ = m.prefill(ids, {"best_pattern": pat}, chunk=256)
    err = (logits.cpu() - ref).abs().max().item()
    scale = ref.abs().max().item()
    print(f"llama dense-equivalent: max-abs {err:.3e} of logit scale {scale:.3e}", flush=True)
    assert err <= 3e-2 * scale


def _reference_stack(hf, ids, masks):
    """fp32 block stack with one boolean mask per (layer, head); weights from the HF model."""
    sd = {k: v.float() for k, v in hf.state_dict().items()}
    n = ids.numel()
    h = sd["model.embed_tokens.weight"][ids]
    inv = 1.0 / (500000.0 ** (torch.arange(0, 128, 2).float() / 128))
    ang = torch.arange(n).float()[:, None] * inv[None]
    ang = torch.cat([ang, ang], -1)
    cos, sin = ang.cos()[:, None], ang.sin()[:, None]

    def rms(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * w

    def rot(x):
        return x * cos + torch.cat([-x[..., 64:], x[..., :64]], -1) * sin

    for li in range(2):
        p = f"model.layers.{li}."
        x = rms(h, sd[p + "input_layernorm.weight"])
        q = rot((x @ sd[p + "self_attn.q_proj.weight"].T).view(n, 2, 128))
        k = rot((x @ sd[p + "self_attn.k_proj.weight"].T).view(n, 1, 128))
        v = (x @ sd[p + "self_attn.v_proj.weight"].T).view(n, 1, 128)
        a = torch.stack([O.masked_attention(q[:, hd], k[:, 0], v[:, 0], masks[li][hd]) for hd in range(2)], 1)
        h = h + a.reshape(n, 256) @ sd[p + "self_attn.o_proj.weight"].T
        x = rms(h, sd[p + "post_attention_layernorm.weight"])
        h = h + (torch.nn.functional.silu(x @ sd[p + "mlp.gate_proj.weight"].T) * (x @ sd[p + "mlp.up_proj.weight"].T)) \
            @ sd[p + "mlp.down_proj.weight"].T
    return rms(h[-1:], sd["model.norm.weight"]) @ sd["lm_head.weight"].T


def test_sparse_patterns_match_fp32_stack_with_oracle_masks(gpu):
    from minference_amd.llama import LlamaConfig, LlamaPrefill
    hf = _hf_model(2)
    n = 900
    ids = torch.randint(0, 500, (n,), generator=torch.Generator().manual_seed(3))
    pat = [{"0": ["stream_llm", 8, 64, 1], "1": ["stream_llm", 128, 200, 1]},
           {"0": ["stream_llm", 0, 33, 1], "1": ["block_sparse", 100, 0, 1]}]
    causal = np.tril(np.ones((n, n), bool))
    masks = [[O.ashape_mask(n, 8, 64), O.ashape_mask(n, 128, 200)], [O.ashape_mask(n, 0, 33), causal]]
    ref = _reference_stack(hf, ids, masks)[0]
    m = LlamaPrefill(LlamaConfig(**TINY), device=gpu)
    m.load_state_dict(hf.state_dict())
    logits, kv = m.prefill(ids, {"best_pattern": pat}, chunk=300, keep_kv=True)
    assert len(kv) == 2 and tuple(kv[0][0].shape) == (n, 1, 128)
    err = (logits.cpu() - ref).abs().max().item()
    scale = ref.abs().max().item()
    print(f"llama sparse heads: max-abs {err:.3e} of logit scale {scale:.3e}", flush=True)
    assert err <= 3e-2 * scale


def test_seeded_pattern_mix_matches_config5_description():
    from minference_amd.llama import seeded_pattern_mix
    t = seeded_pattern_mix(32, 32, seed=501)
    assert len(t) == 32 and all(len(l) == 32 for l in t)
    kinds = [p[0] for l in t for p in l.values()]
    frac = {k: kinds.count(k) / len(kinds) for k in set(kinds)}
    assert abs(frac["vertical_and_slash"] - 0.7) < 0.05 and abs(frac["block_sparse"] - 0.2) < 0.05
    assert abs(frac["stream_llm"] - 0.1) < 0.05
    assert t == seeded_pattern_mix(32, 32, seed=501)
