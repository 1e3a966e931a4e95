"""Long-context prefill of a Llama-architecture decoder around the sparse attention path.

A caller of the path, not part of it: the counterpart of the reference's Llama patch
(minference/patch.py:688-693 chunked MLP, :500-558 chunked norms, :787-790 last-token lm_head;
minference/modules/forward.py:22-234 attention forward that hands [B,H,N,D] q/k/v to
``prefill_forwards["minference"]``) as a self-contained block stack instead of a monkey patch of
a particular transformers version.  Linear layers are plain library GEMMs (torch matmul ->
hipBLASLt); everything between the q/k/v projections and o_proj is
``minference_prefill_forward``.  K/V keep their own (fewer) heads: no repeat_kv copy.

Memory layout for 262144 tokens of Llama-3-8B on one 288 GB GPU: weights 16 GB, hidden state
2 GiB, q 2 GiB, k/v 0.5 GiB each per layer; norms, projections, RoPE and the MLP are applied over
token chunks so no intermediate is larger than ``chunk x intermediate_size``.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .prefill import minference_prefill_forward


@dataclass
class LlamaConfig:
    """Defaults are Llama-3-8B (BASELINE config 5)."""
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5


class LlamaPrefill:
    """Random-init (or caller-filled) decoder weights + a chunked prefill that returns the
    last token's logits.  Weight names follow the Hugging Face Llama state dict."""

    def __init__(self, config: LlamaConfig, device="cuda", dtype=torch.bfloat16, seed=0, std=0.02):
        self.cfg, self.device, self.dtype = config, torch.device(device), dtype
        c = config
        g = torch.Generator(device=self.device).manual_seed(seed)

        def w(*shape):
            return (torch.randn(*shape, device=self.device, dtype=torch.float32, generator=g) * std).to(dtype)

        qd, kd = c.num_heads * c.head_dim, c.num_kv_heads * c.head_dim
        self.embed_tokens = w(c.vocab_size, c.hidden_size)
        self.layers = []
        for _ in range(c.num_layers):
            self.layers.append({
                "input_layernorm": torch.ones(c.hidden_size, device=self.device, dtype=dtype),
                "q_proj": w(qd, c.hidden_size), "k_proj": w(kd, c.hidden_size), "v_proj": w(kd, c.hidden_size),
                "o_proj": w(c.hidden_size, qd),
                "post_attention_layernorm": torch.ones(c.hidden_size, device=self.device, dtype=dtype),
                "gate_proj": w(c.intermediate_size, c.hidden_size), "up_proj": w(c.intermediate_size, c.hidden_size),
                "down_proj": w(c.hidden_size, c.intermediate_size),
            })
        self.norm = torch.ones(c.hidden_size, device=self.device, dtype=dtype)
        self.lm_head = w(c.vocab_size, c.hidden_size)

    def load_state_dict(self, sd):
        """Fill the weights from a Hugging Face Llama state dict (tensors are cast and moved)."""
        def get(name):
            return sd[name].to(self.device, self.dtype)
        self.embed_tokens = get("model.embed_tokens.weight")
        for i, layer in enumerate(self.layers):
            pre = f"model.layers.{i}."
            for k in ("input_layernorm", "post_attention_layernorm"):
                layer[k] = get(pre + k + ".weight")
            for k in ("q_proj", "k_proj", "v_proj", "o_proj"):
                layer[k] = get(pre + "self_attn." + k + ".weight")
            for k in ("gate_proj", "up_proj", "down_proj"):
                layer[k] = get(pre + "mlp." + k + ".weight")
        self.norm = get("model.norm.weight")
        self.lm_head = get("lm_head.weight") if "lm_head.weight" in sd else self.embed_tokens

    # ---- pieces ---------------------------------------------------------------------------
    def _rms(self, x, weight):
        xf = x.float()
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.cfg.rms_eps)
        return (xf.to(self.dtype)) * weight

    def _rope_tables(self, start, stop):
        c = self.cfg
        inv = 1.0 / (c.rope_theta ** (torch.arange(0, c.head_dim, 2, device=self.device, dtype=torch.float32) / c.head_dim))
        ang = torch.arange(start, stop, device=self.device, dtype=torch.float32)[:, None] * inv[None, :]
        ang = torch.cat([ang, ang], dim=-1)              # rotate_half convention: pairs (i, i + D/2)
        return ang.cos()[:, None, :], ang.sin()[:, None, :]

    @staticmethod
    def _rotate(x, cos, sin):
        half = x.shape[-1] // 2
        xr = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
        return (x.float() * cos + xr.float() * sin).to(x.dtype)

    # ---- prefill --------------------------------------------------------------------------
    @torch.no_grad()
    def prefill(self, input_ids, attn_forward_config=None, chunk=32768, keep_kv=False):
        """input_ids [N] (one sequence).  ``attn_forward_config`` is the reference's dictionary
        (best_pattern per layer/head, starting_layer, minference_ratio); None = every head
        vertical_and_slash (1000, 6096).  Returns (last-token logits [vocab] fp32, kv list or None)."""
        c = self.cfg
        ids = input_ids.to(self.device).reshape(-1)
        n = ids.numel()
        cfg = attn_forward_config if attn_forward_config is not None else {"best_pattern": None}
        hidden = self.embed_tokens[ids]                                    # [N, hidden]
        q = torch.empty((n, c.num_heads, c.head_dim), device=self.device, dtype=self.dtype)
        kv_cache = [] if keep_kv else None
        k = v = None
        for li, L in enumerate(self.layers):
            if k is None or keep_kv:
                k = torch.empty((n, c.num_kv_heads, c.head_dim), device=self.device, dtype=self.dtype)
                v = torch.empty((n, c.num_kv_heads, c.head_dim), device=self.device, dtype=self.dtype)
            for s in range(0, n, chunk):
                e = min(s + chunk, n)
                x = self._rms(hidden[s:e], L["input_layernorm"])
                cos, sin = self._rope_tables(s, e)
                q[s:e] = self._rotate((x @ L["q_proj"].T).view(e - s, c.num_heads, c.head_dim), cos, sin)
                k[s:e] = self._rotate((x @ L["k_proj"].T).view(e - s, c.num_kv_heads, c.head_dim), cos, sin)
                v[s:e] = (x @ L["v_proj"].T).view(e - s, c.num_kv_heads, c.head_dim)
            # [N, H, D] storage viewed as [1, H, N, D]: the kernels take strides, nothing is copied
            attn = minference_prefill_forward(q.permute(1, 0, 2)[None], k.permute(1, 0, 2)[None],
                                              v.permute(1, 0, 2)[None],
                                              {"layer_idx": li, "attn_forward_config": cfg})
            attn = attn[0].permute(1, 0, 2)                                 # [N, H, D] view
            for s in range(0, n, chunk):
                e = min(s + chunk, n)
                a = attn[s:e].reshape(e - s, c.num_heads * c.head_dim)
                h = hidden[s:e] + a @ L["o_proj"].T
                x = self._rms(h, L["post_attention_layernorm"])
                mlp = (torch.nn.functional.silu(x @ L["gate_proj"].T) * (x @ L["up_proj"].T)) @ L["down_proj"].T
                hidden[s:e] = h + mlp
            del attn
            if keep_kv:
                kv_cache.append((k, v))
        last = self._rms(hidden[-1:], self.norm)
        logits = (last @ self.lm_head.T).float()[0]
        return logits, kv_cache

    def flops_linear(self, n):
        """FLOPs of the GEMMs of one prefill of n tokens (attention excluded, lm_head on one token)."""
        c = self.cfg
        per_tok = 2 * (c.hidden_size * (c.num_heads + 2 * c.num_kv_heads) * c.head_dim
                       + c.num_heads * c.head_dim * c.hidden_size + 3 * c.hidden_size * c.intermediate_size)
        return c.num_layers * n * per_tok + 2 * c.hidden_size * c.vocab_size


def seeded_pattern_mix(num_layers, num_heads, seed=501, p_vs=0.7, p_bs=0.2,
                       vs=(1000, 6096), ashape=(128, 4096)):
    """BASELINE config 5's per-head pattern table: a seeded mix of vertical_and_slash, block_sparse
    and A-shape heads in the best_pattern format (list over layers of {head: [type, a, b, score]})."""
    import numpy as np
    rng = np.random.default_rng(seed)
    table = []
    for _ in range(num_layers):
        layer = {}
        for h in range(num_heads):
            u = rng.random()
            if u < p_vs:
                layer[str(h)] = ["vertical_and_slash", vs[0], vs[1], 1.0]
            elif u < p_vs + p_bs:
                layer[str(h)] = ["block_sparse", 100, 0, 1.0]
            else:
                layer[str(h)] = ["stream_llm", ashape[0], ashape[1], 1.0]
        table.append(layer)
    return table
