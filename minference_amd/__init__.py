"""minference_amd -- MI355X (gfx950) dynamic sparse prefill attention.

Same operator surface as microsoft/MInference (minference/__init__.py:9-11):
``vertical_slash_sparse_attention``, ``block_sparse_attention`` and
``streaming_forward``, backed by hand-written HIP kernels in
``libminf_hip.so`` (C ABI in include/minf_hip.h) instead of Triton/CUDA.
Importing the package needs neither a GPU nor the built library; calling an
operator without them raises.
"""
from .index import convert_vertical_slash_indexes
from .ops import (block_sparse_attention, block_sparse_attention_from_index, dense_causal_attention,
                  streaming_forward, tri_shape_forward, vertical_slash_attention_from_index,
                  vertical_slash_sparse_attention)

from .estimate import estimate_vertical_slash, topk_indices, vertical_slash_scores
from .configs import get_support_models
from .prefill import (a_shape_kernel, tri_shape_kernel, load_best_pattern, minference_prefill_forward, minference_prefill_kernel,
                      dilated_forward, static_vertical_slash_forward, tri_mix_forward,
                      tri_mix_minference_forward, vertical_slash_prefill)
from .search import pattern_recall, search_pattern, search_patterns
from .patch import MInference, MInferenceConfig, minference_patch, patch_hf

__all__ = [
    "estimate_vertical_slash", "vertical_slash_scores", "topk_indices", "vertical_slash_prefill",
    "minference_prefill_forward", "minference_prefill_kernel", "load_best_pattern",
    "vertical_slash_sparse_attention", "block_sparse_attention", "streaming_forward",
    "convert_vertical_slash_indexes", "vertical_slash_attention_from_index",
    "block_sparse_attention_from_index", "dense_causal_attention", "tri_shape_forward",
    "pattern_recall", "search_pattern", "search_patterns", "MInference", "MInferenceConfig",
    "tri_mix_forward", "tri_mix_minference_forward", "dilated_forward", "static_vertical_slash_forward",
    "a_shape_kernel", "tri_shape_kernel", "minference_patch", "patch_hf", "get_support_models",
]
__version__ = "0.3.0"
