"""Host-side logic that needs no GPU: per-head pattern planning of the dispatcher
(reference minference/modules/minference_forward.py:594-674), argument checks of the
operators, generators."""
import os

import numpy as np
import pytest
import torch

from minference_amd import prefill
from tests import gen


def cfg(best_pattern, **kw):
    return {"best_pattern": best_pattern, **kw}


def test_default_pattern_and_grouping():
    layer = {"0": ["vertical_and_slash", 30, 800, 0.9], "1": ["stream_llm", 128, 4096, 0.8],
             "3": ["block_sparse", 100, 6096, 0.7], "2": ["vertical_and_slash", 30, 800, 0.5]}
    plan = prefill._head_plan(cfg([layer]), 0, 6)
    assert plan[("vertical_and_slash", 30, 800)] == [0, 2]
    assert plan[("stream_llm", 128, 4096)] == [1]
    assert plan[("block_sparse", 100, 6096)] == [3]
    assert plan[("vertical_and_slash", 1000, 6096)] == [4, 5]      # default entry (:621)


def test_minference_ratio_truncates_like_the_reference():
    layer = {"0": ["vertical_and_slash", 1000, 6096, 1]}
    plan = prefill._head_plan(cfg([layer], minference_ratio=0.33), 0, 1)
    assert list(plan) == [("vertical_and_slash", int(1000 * 0.33), int(6096 * 0.33))]


def test_head_list_of_a_pattern_group():
    # the ascending head numbers of a group: entry i is the head that owns index position i
    hl = prefill._head_list([5, 1, 4], "cpu")
    assert hl.dtype == torch.int32 and hl.tolist() == [1, 4, 5]
    assert prefill._head_list([], "cpu").numel() == 0


def test_search_mode_has_no_cpu_path_and_respects_a_finished_file(tmp_path):
    cfg_path = tmp_path / "patterns.json"
    kw = {"layer_idx": 0, "num_hidden_layers": 2,
          "attn_forward_config": {"is_search": True, "config_path": str(cfg_path)}}
    z = torch.zeros(1, 1, 64, 128)
    with pytest.raises(RuntimeError):                     # CPU tensors: the search kernels need the GPU
        prefill.minference_prefill_forward(z, z, z, kw)
    cfg_path.write_text('[{"0": ["vertical_and_slash", 30, 800, 0.9]}, {"0": ["vertical_and_slash", 30, 800, 0.9]}]')
    with pytest.raises(RuntimeError, match="Search already completed"):
        prefill.minference_prefill_forward(z, z, z, kw)


def test_shipped_pattern_files_have_the_expected_format():
    path = "/root/reference/minference/configs/Llama_3_8B_Instruct_262k_kv_out_v32_fit_o_best_pattern.json"
    if not os.path.exists(path):
        pytest.skip("reference configs not present on this box")
    pat = prefill.load_best_pattern(path)
    assert len(pat) == 32 and len(pat[0]) == 32
    plan = prefill._head_plan(cfg(pat), 5, 32)
    assert sum(len(v) for v in plan.values()) == 32
    for (ty, vs, ss) in plan:
        assert ty in ("vertical_and_slash", "stream_llm", "block_sparse") and vs > 0 and ss > 0


def test_operators_reject_cpu_tensors_and_bad_shapes():
    import minference_amd as M
    q = torch.zeros(1, 2, 64, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        M.streaming_forward(q, q, q, 4, 16)
    with pytest.raises(ValueError):
        M.vertical_slash_sparse_attention(q, q, q, torch.zeros(1, 2, 4), torch.zeros(1, 2, 4), block_size_M=128)
    with pytest.raises(ValueError):
        M.block_sparse_attention(q, q, q, 10, block_size_N=32)
    with pytest.raises(ValueError):
        M.ops._check_qkv(q, q[:, :1], q)            # k/v shape mismatch
    with pytest.raises(ValueError):
        M.ops._check_qkv(torch.zeros(1, 3, 64, 128), torch.zeros(1, 2, 64, 128), torch.zeros(1, 2, 64, 128))


def test_index_generator_matches_config3_description():
    v, s = gen.vs_index_inputs(2, 4096, 100, 600, seed=300)
    assert v.dtype == np.int32 and s.dtype == np.int32
    for h in range(2):
        assert (np.diff(v[0, h]) > 0).all() and (np.diff(s[0, h]) < 0).all()
        assert set(range(4)) <= set(v[0, h].tolist()) and set(range(64)) <= set(s[0, h].tolist())


def test_planted_layer_is_deterministic_and_structured():
    q, k, v, meta = gen.planted_layer(2048, hq=4, hk=2, seed=7)
    q2, k2, _, _ = gen.planted_layer(2048, hq=4, hk=2, seed=7)
    assert torch.equal(q, q2) and torch.equal(k, k2)
    assert q.shape == (1, 4, 2048, 128) and k.shape == (1, 2, 2048, 128) and q.dtype == torch.bfloat16
    # positional code: last three dims of K are the base-128 digits of the position
    pos = (k[0, 0, :, -3].float() * 16384 + k[0, 0, :, -2].float() * 128 + k[0, 0, :, -1].float())
    assert torch.equal(pos, torch.arange(2048).float())
    assert len(meta["heavy"]) == 2 and len(meta["heavy"][0]) == 32


def test_patch_configuration_rejects_what_is_not_built():
    from minference_amd import MInference
    for bad in ("inf_llm", "flexprefill", "vllm_minference", "xattention"):
        with pytest.raises(NotImplementedError):
            MInference(bad)
    with pytest.raises(NotImplementedError):
        MInference("minference", kv_type="snapkv")
    with pytest.raises(NotImplementedError):
        MInference("minference", kv_cache_cpu=True)
    with pytest.raises(TypeError):
        MInference("minference", not_an_argument=1)
    m = MInference("a_shape", attn_kwargs={"n_local": 100})
    assert m.config.attn_type == "a_shape" and m.config.attn_kwargs == {"n_local": 100}
    sentinel = object()
    assert MInference("hf")(sentinel) is sentinel                     # "hf": model unchanged


def test_model_name_resolves_to_a_pattern_file(tmp_path, monkeypatch):
    """minference_configuration.py:85-93: explicit path wins, unknown model is an error; here the
    files live in a user-filled directory, and a missing file is reported with its path."""
    from minference_amd import MInference, get_support_models
    from minference_amd.configs import PATTERN_FILES, resolve_config_path
    names = get_support_models()
    assert "meta-llama/Llama-3.1-8B-Instruct" in names and len(names) == len(set(names)) == 18
    monkeypatch.setenv("MINFERENCE_CONFIG_DIR", str(tmp_path))
    assert resolve_config_path("x.json", "no/such-model") == "x.json"
    assert resolve_config_path(None, None) is None
    with pytest.raises(ValueError):
        MInference("minference", "no/such-model")
    with pytest.raises(FileNotFoundError) as err:
        MInference("minference", "Qwen/Qwen2-7B-Instruct")
    assert str(tmp_path) in str(err.value)
    path = tmp_path / PATTERN_FILES["Qwen/Qwen2-7B-Instruct"]
    path.write_text("[]")
    assert MInference("minference", "Qwen/Qwen2-7B-Instruct").config.config_path == str(path)
    # types that read no table never look one up; a search needs its own output path
    assert MInference("a_shape", "no/such-model").config.config_path is None
    assert MInference("minference", "no/such-model", config_path="out.json", is_search=True).config.config_path == "out.json"


def test_reference_patch_function_names():
    from minference_amd import MInferenceConfig, minference_patch, patch_hf
    sentinel = object()
    assert minference_patch(sentinel, MInferenceConfig("hf")) is sentinel
    assert patch_hf(sentinel, "hf", {"n_init": 1}, n_local=2) is sentinel
    with pytest.raises(NotImplementedError):
        patch_hf(sentinel, "inf_llm")


def test_layer_plan_is_cached_per_table_object_and_checks_head_coverage():
    """The dispatcher parses a layer's table once (minference_forward.py:621-625 does it per call)."""
    layer = {"0": ["vertical_and_slash", 100, 200, 0.9], "1": ["block_sparse", 100, 6096, 0.9],
             "2": ["stream_llm", 128, 512, 0.9]}
    config = cfg([layer])
    prefill.clear_plan_cache()
    a = prefill._layer_plan(config, 0, 3)
    assert prefill._layer_plan(config, 0, 3) is a
    assert [h for h, _, _ in a.vs] == [0] and a.bs == [1] and a.stream == {(128, 512): [2]}
    # an equal table in another object is another entry; a ratio is part of the key
    assert prefill._layer_plan(cfg([dict(layer)]), 0, 3) is not a
    assert prefill._layer_plan(dict(config, minference_ratio=0.5), 0, 3) is not a
    # heads without an entry take the default pattern, so 5 heads are covered as well
    assert len(prefill._layer_plan(config, 0, 5).vs) == 3
    with pytest.raises(KeyError):
        prefill._layer_plan(cfg([{"0": ["no_such_pattern", 1, 1, 0.5]}]), 0, 1)
    prefill.clear_plan_cache()
    assert prefill._layer_plan(config, 0, 3) is not a
