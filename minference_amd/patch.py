"""``MInference(attn_type, model_name, ...)(model)`` -- the reference's patch entry point for
Hugging Face models, on this package's kernels.

Counterpart of ``MInference`` / ``MInferenceConfig`` (reference minference/models_patch.py:18-160,
minference/minference_configuration.py:7-100) and of the attention forward the patch installs
(minference/modules/forward.py:22-234, which hands ``[B, H, N, D]`` q/k/v to
``prefill_forwards[attn_type]``).  The reference replaces ``forward`` methods of a particular
transformers release; here the hook is transformers' own attention-function registry
(``AttentionInterface``): an attention function named ``"minference_amd"`` is registered and the
model is switched to it, so every decoder architecture whose attention module goes through that
registry (Llama, Qwen2, Mistral, ...) is covered without touching its code.  The function
receives K/V with their own (fewer) heads -- no ``repeat_kv`` copy is ever made.

Scope: the prefill of one unpadded sequence (what the reference's prefill path assumes as well).
Decode steps, chunks that attend to a longer cache (``key length != query length``) and calls that
carry an explicit attention mask (padding, packing) are passed to transformers' SDPA function unchanged.  KV-cache compression (``kv_type``), CPU KV offload and
the reference's other attention types belong to other paths of the reference and raise.
"""
from __future__ import annotations

import json

from .configs import resolve_config_path

SUPPORTED_ATTN_TYPES = ("minference", "tri_mix_minference", "tri_mix", "static", "dilated1", "dilated2", "dense",
                        "a_shape", "tri_shape", "hf")
INTERFACE_NAME = "minference_amd"
_registered = False


class MInferenceConfig:
    """Same constructor arguments as the reference's configuration object
    (minference_configuration.py:43-55); unsupported choices raise instead of being ignored."""

    def __init__(self, attn_type="minference", model_name=None, config_path=None, starting_layer=-1,
                 kv_cache_cpu=False, kv_type="dense", is_search=False, attn_kwargs=None, **kwargs):
        if attn_type not in SUPPORTED_ATTN_TYPES:
            raise NotImplementedError(
                f"attn_type {attn_type!r}: this package implements {SUPPORTED_ATTN_TYPES} "
                "(the dynamic sparse prefill path and its dense / A-shape / tri-shape relatives)")
        if kv_type != "dense" or kv_cache_cpu:
            raise NotImplementedError("KV-cache compression and CPU offload are not part of the prefill path")
        if kwargs:
            raise TypeError(f"unknown arguments {sorted(kwargs)}")
        self.attn_type = attn_type
        self.model_name = model_name
        # minference_configuration.py:85-93: only the types that read a best_pattern table look one
        # up by model name; a search writes its table and therefore needs an explicit path
        if attn_type in ("minference", "tri_mix_minference", "static") and not is_search:
            config_path = resolve_config_path(config_path, model_name)
        self.config_path = config_path
        self.starting_layer = starting_layer
        self.is_search = is_search
        self.attn_kwargs = dict(attn_kwargs or {})


def _attention(module, query, key, value, attention_mask, dropout=0.0, scaling=None, **kwargs):
    """The registered attention function: [B,H,N,D] q, [B,Hk,N,D] k/v -> ([B,N,H,D], None)."""
    from .ops import dense_causal_attention, streaming_forward, tri_shape_forward
    from .prefill import (DEFAULT_PATTERN, dilated_forward, minference_prefill_forward,
                          static_vertical_slash_forward, tri_mix_forward, tri_mix_minference_forward)
    state = getattr(module.config, "minference_amd", None)
    n = query.shape[2]
    # an explicit mask means padding or packing: not the single-sequence prefill this path covers
    if state is None or n == 1 or key.shape[2] != n or attention_mask is not None or not query.is_cuda:
        from transformers.integrations.sdpa_attention import sdpa_attention_forward
        return sdpa_attention_forward(module, query, key, value, attention_mask, dropout=dropout,
                                      scaling=scaling, **kwargs)
    d = query.shape[-1]
    if scaling is not None and abs(scaling * d ** 0.5 - 1.0) > 1e-6:
        query = query * (scaling * d ** 0.5)              # the kernels scale by 1/sqrt(head_dim)
    ty = state["attn_type"]
    kw = state["attn_kwargs"]
    if ty in ("minference", "tri_mix_minference", "tri_mix"):
        fn = {"minference": minference_prefill_forward, "tri_mix_minference": tri_mix_minference_forward,
              "tri_mix": tri_mix_forward}[ty]
        out = fn(query, key, value, {
            "layer_idx": module.layer_idx, "num_hidden_layers": module.config.num_hidden_layers,
            "attn_forward_config": kw})
    elif ty in ("dilated1", "dilated2"):
        out = dilated_forward(query, key, value, ty)
    elif ty == "static":
        # one (vertical_size, slash_size) per layer: the sizes of head 0 of the table, like a layer
        # whose heads share a pattern (the reference estimates per head inside its head loop)
        best = kw.get("best_pattern")
        _, vs, ss, _ = (best[module.layer_idx].get("0", DEFAULT_PATTERN) if best else DEFAULT_PATTERN)
        cache = state.setdefault("static_cache", {}).setdefault(module.layer_idx, {})
        out = static_vertical_slash_forward(query, key, value, vs, ss, cache)
    elif ty == "dense":
        out = dense_causal_attention(query, key, value)
    elif ty == "a_shape":
        out = streaming_forward(query, key, value, kw["n_init"], kw["n_local"])
    else:
        out = tri_shape_forward(query, key, value, kw["n_init"], kw["n_local"], kw["n_last"])
    return out.transpose(1, 2), None


def _register():
    global _registered
    if not _registered:
        from transformers import AttentionInterface
        from transformers.masking_utils import AttentionMaskInterface, sdpa_mask
        AttentionInterface.register(INTERFACE_NAME, _attention)
        # masks are built as for SDPA: none at all for one unpadded causal sequence, a boolean 4-D
        # mask when there is padding (without this registration transformers would build no mask
        # for an attention function it does not know, padding or not)
        AttentionMaskInterface.register(INTERFACE_NAME, sdpa_mask)
        _registered = True


class MInference:
    """``MInference("minference", model_name, config_path=...)(model)`` returns the model with its
    attention switched to this package (models_patch.py:18-52).

    * ``"minference"``: per-head patterns from the ``best_pattern`` JSON at ``config_path``
      (``is_search=True``: search them instead, layer by layer, and write the file;
      ``attn_kwargs`` may carry ``minference_ratio``); layers below ``starting_layer`` run dense.
      Without a file every head uses vertical_and_slash (1000, 6096).
    * ``"tri_mix_minference"`` / ``"tri_mix"``: the per-head patterns (resp. dense attention) below
      ``attn_kwargs["starting_layer"]`` (16), tri-shape (n_init 8, n_local 512, n_last 128) from there on.
    * ``"static"``: vertical-slash indices estimated on the first prompt and reused afterwards;
      ``"dilated1"`` / ``"dilated2"``: the fixed dilated-window baselines (minference_forward.py:365-379).
    * ``"dense"``: dense causal attention on the same tile engine.
    * ``"a_shape"`` / ``"tri_shape"``: ``n_init`` (128), ``n_local`` (3968) and ``n_last`` (100)
      from ``attn_kwargs`` (defaults of models_patch.py:134-143).
    * ``"hf"``: the model is returned unchanged.
    """

    def __init__(self, attn_type="minference", model_name=None, config_path=None, starting_layer=-1,
                 kv_cache_cpu=False, kv_type="dense", is_search=False, attn_kwargs=None, **kwargs):
        self.config = MInferenceConfig(attn_type=attn_type, model_name=model_name, config_path=config_path,
                                       starting_layer=starting_layer, kv_cache_cpu=kv_cache_cpu,
                                       kv_type=kv_type, is_search=is_search, attn_kwargs=attn_kwargs, **kwargs)

    @classmethod
    def from_config(cls, config):
        """A patcher around an existing ``MInferenceConfig``."""
        if not isinstance(config, MInferenceConfig):
            raise TypeError("config must be a MInferenceConfig")
        self = cls.__new__(cls)
        self.config = config
        return self

    def __call__(self, model):
        return self.patch_model(model)

    def patch_model(self, model):
        c = self.config
        if c.attn_type == "hf":
            return model
        kw = dict(c.attn_kwargs)
        if c.attn_type == "static" and "best_pattern" not in kw and c.config_path:
            with open(c.config_path) as f:
                kw["best_pattern"] = json.load(f)
        if c.attn_type == "minference":
            kw.setdefault("starting_layer", c.starting_layer)
            kw["is_search"] = bool(c.is_search)
            kw["config_path"] = c.config_path
            if not c.is_search and "best_pattern" not in kw:
                if c.config_path:
                    with open(c.config_path) as f:
                        kw["best_pattern"] = json.load(f)
                else:
                    kw["best_pattern"] = None            # every head: vertical_and_slash (1000, 6096)
            if c.is_search and not c.config_path:
                raise ValueError("is_search needs a config_path to write the patterns to")
        elif c.attn_type in ("tri_mix_minference", "tri_mix"):
            # models_patch.py:116-127: tri-shape (8 + 512, last 128 rows dense) from layer 16 on
            if c.attn_type == "tri_mix_minference" and "best_pattern" not in kw:
                if c.config_path:
                    with open(c.config_path) as f:
                        kw["best_pattern"] = json.load(f)
                else:
                    kw["best_pattern"] = None
            kw.setdefault("n_local", 512)
            kw.setdefault("n_init", 8)
            kw.setdefault("n_last", 128)
            kw.setdefault("starting_layer", 16)
        elif c.attn_type in ("a_shape", "tri_shape"):
            kw.setdefault("n_local", 3968)
            kw.setdefault("n_init", 128)
            kw.setdefault("n_last", 100)
        _register()
        model.config.starting_layer = c.starting_layer       # models_patch.py:112-114
        model.config.config_path = c.config_path
        model.config.minference_amd = {"attn_type": c.attn_type, "attn_kwargs": kw}
        model.set_attn_implementation(INTERFACE_NAME)
        return model


def minference_patch(model, config):
    """``minference_patch(model, MInferenceConfig(...))`` (reference minference/patch.py:895-903)."""
    return MInference.from_config(config).patch_model(model)


def patch_hf(model, attn_type="a_shape", attn_kwargs=None, **kwargs):
    """``patch_hf(model, attn_type, attn_kwargs)`` (reference minference/patch.py:1313-1321, the call
    the reference makes for its streaming types, models_patch.py:128-143): extra keyword arguments
    are merged into ``attn_kwargs``.  The reference's default type of this function, InfLLM, is a
    KV-cache method and not part of this package, hence the different default."""
    kw = dict(attn_kwargs or {})
    kw.update(kwargs)
    return MInference(attn_type, attn_kwargs=kw)(model)
