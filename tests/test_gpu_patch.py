"""``MInference(...)(model)`` on a Hugging Face Llama (random init, transformers' own modelling
code): the patch routes the prefill attention of every layer through this package.  Patterns that
keep every causal key must reproduce the unpatched model (bf16 tolerance on the logits), sparse
patterns must change them, generation (prefill + decode steps) must still work, and the search
mode must write a pattern file the patch can load again."""
import json

import pytest
import torch

pytestmark = pytest.mark.gpu


def tiny_llama(gpu, layers=2):
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=320, hidden_size=512, intermediate_size=1024, num_hidden_layers=layers,
                      num_attention_heads=4, num_key_value_heads=2, head_dim=128, max_position_embeddings=8192,
                      rope_theta=500000.0)
    return LlamaForCausalLM(cfg).to(gpu).to(torch.bfloat16).eval()


def logits_of(model, ids):
    with torch.no_grad():
        return model(ids).logits.float()


def close(a, b, what):
    err = (a - b).abs()
    scale = b.abs().max().item()
    print(f"{what}: max-abs {err.max().item():.3e} of scale {scale:.3e}", flush=True)
    assert err.max().item() <= 3e-2 * scale + 1e-2, what       # bf16 model, two layers


def test_patterns_that_keep_everything_reproduce_the_unpatched_model(gpu, tmp_path):
    from minference_amd import MInference
    n = 700
    ids = torch.randint(0, 320, (1, n), generator=torch.Generator().manual_seed(1)).to(gpu)
    model = tiny_llama(gpu)
    base = logits_of(model, ids)

    dense = MInference("dense")(model)
    assert dense.config._attn_implementation == "minference_amd"
    close(logits_of(dense, ids), base, "dense")

    # per-head table: a window wider than the sequence for some heads, vertical-slash with every
    # diagonal for the others; layer 0 below starting_layer runs dense
    table = [{str(h): (["stream_llm", 4, 4096, 1.0] if h % 2 else ["vertical_and_slash", 30, 100000, 1.0])
              for h in range(4)} for _ in range(2)]
    path = tmp_path / "patterns.json"
    path.write_text(json.dumps(table))
    mi = MInference("minference", "tiny-llama", config_path=str(path), starting_layer=1)(model)
    close(logits_of(mi, ids), base, "minference (all-keeping patterns)")

    tri = MInference("tri_shape", attn_kwargs={"n_init": 8, "n_local": 4096, "n_last": 64})(model)
    close(logits_of(tri, ids), base, "tri_shape (window wider than the sequence)")


def test_tri_mix_switches_method_at_the_starting_layer(gpu):
    from minference_amd import MInference, dense_causal_attention, tri_mix_forward, tri_mix_minference_forward, tri_shape_forward
    from minference_amd import minference_prefill_forward
    n = 1300
    g = torch.Generator().manual_seed(9)
    q = torch.randn(1, 4, n, 128, generator=g).bfloat16().to(gpu)
    k = torch.randn(1, 2, n, 128, generator=g).bfloat16().to(gpu)
    v = torch.randn(1, 2, n, 128, generator=g).bfloat16().to(gpu)
    cfg = {"starting_layer": 1, "n_init": 8, "n_local": 128, "n_last": 64,
           "best_pattern": [{str(h): ["stream_llm", 16, 200, 1.0] for h in range(4)}] * 2}
    tri = tri_shape_forward(q, k, v, 8, 128, 64)
    assert torch.equal(tri_mix_forward(q, k, v, {"layer_idx": 0, "attn_forward_config": cfg}), dense_causal_attention(q, k, v))
    assert torch.equal(tri_mix_forward(q, k, v, {"layer_idx": 1, "attn_forward_config": cfg}), tri)
    sparse0 = minference_prefill_forward(q, k, v, {"layer_idx": 0, "attn_forward_config": dict(cfg, starting_layer=0)})
    assert torch.equal(tri_mix_minference_forward(q, k, v, {"layer_idx": 0, "attn_forward_config": cfg}), sparse0)
    assert torch.equal(tri_mix_minference_forward(q, k, v, {"layer_idx": 1, "attn_forward_config": cfg}), tri)
    # through the patch: everything wide enough to keep all keys -> the unpatched model
    ids = torch.randint(0, 320, (1, 500), generator=torch.Generator().manual_seed(5)).to(gpu)
    model = tiny_llama(gpu)
    base = logits_of(model, ids)
    mixed = MInference("tri_mix", attn_kwargs={"starting_layer": 1, "n_local": 4096})(model)
    close(logits_of(mixed, ids), base, "tri_mix (window wider than the sequence)")


def test_dilated_and_static_baselines(gpu):
    from oracle import oracle as O
    from minference_amd import MInference, dilated_forward, static_vertical_slash_forward
    n = 3000
    g = torch.Generator().manual_seed(11)
    q = torch.randn(1, 2, n, 128, generator=g).bfloat16()
    k = torch.randn(1, 2, n, 128, generator=g).bfloat16()
    v = torch.randn(1, 2, n, 128, generator=g).bfloat16()
    for kind in ("dilated1", "dilated2"):
        out = dilated_forward(q.to(gpu), k.to(gpu), v.to(gpu), kind).float().cpu()
        pos = torch.arange(n)
        pos = pos[-8192::2] if kind == "dilated1" else torch.cat([pos[-2048:], pos[-6144:-2048:2]])
        v_idx = torch.arange(min(1024, n)).expand(1, 2, -1)
        s_idx = ((n - 1) - pos).expand(1, 2, -1)
        ref = O.vertical_slash_sparse_attention(q, k, v, v_idx, s_idx)
        err = (out - ref).abs()
        print(kind, err.max().item(), err.mean().item(), flush=True)
        assert err.max() <= 2e-2 and err.mean() <= 1e-3
    cache = {}
    a = static_vertical_slash_forward(q.to(gpu), k.to(gpu), v.to(gpu), 100, 200, cache)
    q2 = torch.randn(1, 2, n, 128, generator=g).bfloat16()
    b = static_vertical_slash_forward(q2.to(gpu), k.to(gpu), v.to(gpu), 100, 200, cache)      # reuses the indices
    v_idx, s_idx = cache["vs"]
    ref = O.vertical_slash_sparse_attention(q2, k, v, v_idx.cpu(), s_idx.cpu())
    assert (b.float().cpu() - ref).abs().max() <= 2e-2 and a.shape == b.shape
    # through the patch (short prompt: the dilated patterns keep every key)
    ids = torch.randint(0, 320, (1, 400), generator=torch.Generator().manual_seed(6)).to(gpu)
    model = tiny_llama(gpu)
    base = logits_of(model, ids)
    close(logits_of(MInference("dilated2")(model), ids), base, "dilated2 on a short prompt")
    assert torch.isfinite(logits_of(MInference("static")(model), ids)).all()


def test_sparse_patterns_are_really_applied(gpu):
    from minference_amd import MInference
    n = 1500
    ids = torch.randint(0, 320, (1, n), generator=torch.Generator().manual_seed(2)).to(gpu)
    model = tiny_llama(gpu)
    base = logits_of(model, ids)
    a = MInference("a_shape", attn_kwargs={"n_init": 4, "n_local": 64})(model)
    out = logits_of(a, ids)
    assert torch.isfinite(out).all()
    # rows inside the first window see every key: identical there, different far behind it
    close(out[:, :60], base[:, :60], "a_shape, first rows")
    assert (out[:, -200:] - base[:, -200:]).abs().max() > 5e-2


def test_generate_runs_prefill_sparse_and_decode_through_transformers(gpu):
    from minference_amd import MInference
    n = 300
    ids = torch.randint(0, 320, (1, n), generator=torch.Generator().manual_seed(3)).to(gpu)
    model = tiny_llama(gpu)
    want = model.generate(ids, max_new_tokens=4, do_sample=False)
    got = MInference("dense")(model).generate(ids, max_new_tokens=4, do_sample=False)
    assert got.shape == want.shape == (1, n + 4)
    assert torch.equal(got[:, :n], ids)


def test_padded_batches_fall_through_to_transformers(gpu):
    from minference_amd import MInference
    ids = torch.randint(0, 320, (2, 200), generator=torch.Generator().manual_seed(8)).to(gpu)
    mask = torch.ones_like(ids)
    mask[1, :37] = 0                                       # left padding in the second sequence
    model = tiny_llama(gpu)
    with torch.no_grad():
        want = model(ids, attention_mask=mask).logits.float()
        got = MInference("a_shape", attn_kwargs={"n_init": 1, "n_local": 8})(model)(ids, attention_mask=mask).logits.float()
    close(got[:, 40:], want[:, 40:], "padded batch")      # identical path: the sparse pattern was not applied


def test_search_mode_writes_a_table_the_patch_loads(gpu, tmp_path):
    from minference_amd import MInference
    n = 2900                                  # the search averages over rows >= 2500
    ids = torch.randint(0, 320, (1, n), generator=torch.Generator().manual_seed(4)).to(gpu)
    model = tiny_llama(gpu)
    base = logits_of(model, ids)
    path = tmp_path / "found.json"
    searching = MInference("minference", config_path=str(path), is_search=True)(model)
    close(logits_of(searching, ids), base, "search mode output is dense")
    table = json.loads(path.read_text())
    assert len(table) == 2 and all(sorted(layer) == ["0", "1", "2", "3"] for layer in table)
    assert all(entry[0] == "vertical_and_slash" for layer in table for entry in layer.values())
    sparse = MInference("minference", config_path=str(path))(model)
    assert torch.isfinite(logits_of(sparse, ids)).all()
