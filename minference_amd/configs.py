"""Model name -> ``best_pattern`` file, the lookup behind ``MInference("minference", model_name)``.

Counterpart of ``MODEL2PATH`` / ``get_support_models`` (reference minference/configs/model2path.py:7-76)
and of ``MInferenceConfig.update_config_path`` (minference/minference_configuration.py:85-93).
The reference ships one searched JSON per model beside that table.  This package ships none of
them: the table below only records which file name belongs to which model, and the files are
looked up in a directory the user fills -- with the reference's files (the format is identical,
see ``load_best_pattern``) or with files written by this package's own search mode
(``MInference("minference", is_search=True, config_path=...)``).

The directory is ``$MINFERENCE_CONFIG_DIR`` when set, else ``configs/`` beside this file.
"""
from __future__ import annotations

import os

_LLAMA3_8B = "Llama_3_8B_Instruct_262k_kv_out_v32_fit_o_best_pattern.json"
_LLAMA3_70B = "Llama_3_70B_Instruct_262k_kv_out_v32_fit_o_best_pattern.json"
_LLAMA31_8B = "Llama_3.1_8B_Instruct_128k_kv_out_v32_fit_o_best_pattern_v2.json"
_LLAMA31_70B = "Llama_3.1_70B_Instruct_128k_kv_out_v32_fit_o_best_pattern_v2.json"

PATTERN_FILES = {
    "gradientai/Llama-3-8B-Instruct-262k": _LLAMA3_8B,
    "gradientai/Llama-3-8B-Instruct-Gradient-1048k": _LLAMA3_8B,
    "gradientai/Llama-3-8B-Instruct-Gradient-4194k": _LLAMA3_8B,
    "gradientai/Llama-3-70B-Instruct-Gradient-262k": _LLAMA3_70B,
    "gradientai/Llama-3-70B-Instruct-Gradient-1048k": _LLAMA3_70B,
    "meta-llama/Meta-Llama-3.1-8B-Instruct": _LLAMA31_8B,
    "meta-llama/Llama-3.1-8B-Instruct": _LLAMA31_8B,
    "meta-llama/Meta-Llama-3.1-70B-Instruct": _LLAMA31_70B,
    "meta-llama/Llama-3.1-70B-Instruct": _LLAMA31_70B,
    "01-ai/Yi-9B-200K": "Yi_9B_200k_kv_out_v32_fit_o_best_pattern.json",
    "microsoft/Phi-3-mini-128k-instruct": "Phi_3_mini_128k_instruct_kv_out_v32_fit_o_best_pattern.json",
    "Qwen/Qwen2-7B-Instruct": "Qwen2_7B_Instruct_128k_instruct_kv_out_v32_fit_o_best_pattern.json",
    "Qwen/Qwen2.5-7B-Instruct": "Qwen2.5_7B_Instruct_128k_instruct_kv_out_v32_fit_o_best_pattern.json",
    "Qwen/Qwen2.5-32B-Instruct": "Qwen2.5_32B_Instruct_128k_kv_out_v32_fit_o_best_pattern.json",
    "Qwen/Qwen2.5-72B-Instruct": "Qwen2.5_72B_Instruct_128k_kv_out_v32_fit_o_best_pattern.json",
    "Qwen/Qwen2.5-7B-Instruct-1M": "Qwen2.5_7B_Instruct_1M.json",
    "Qwen/Qwen2.5-14B-Instruct-1M": "Qwen2.5_14B_Instruct_1M.json",
    "THUDM/glm-4-9b-chat-1m": "GLM_4_9B_1M_instruct_kv_out_v32_fit_o_best_pattern.json",
}


def pattern_dir():
    return os.environ.get("MINFERENCE_CONFIG_DIR") or os.path.join(os.path.dirname(os.path.abspath(__file__)),
                                                                   "configs")


def get_support_models():
    """The model names the table knows (model2path.py:75-76)."""
    return list(PATTERN_FILES)


def resolve_config_path(config_path=None, model_name=None):
    """An explicit ``config_path`` wins; otherwise the model's file in ``pattern_dir()``.

    Like the reference, a model name outside the table is an error when no path is given
    (minference_configuration.py:90-92).  A known model whose file has not been placed in the
    directory is an error too, naming the path that was tried: silently running every head on the
    default pattern would not be what ``model_name`` asked for."""
    if config_path is not None:
        return config_path
    if model_name is None:
        return None
    if model_name not in PATTERN_FILES:
        raise ValueError(f"model {model_name!r} has no best_pattern file on record "
                         f"(known: {get_support_models()}); pass config_path, or search one with is_search=True")
    path = os.path.join(pattern_dir(), PATTERN_FILES[model_name])
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{path}: best_pattern file of {model_name!r} not found; put it there "
                                "(or point MINFERENCE_CONFIG_DIR at its directory), or pass config_path")
    return path
