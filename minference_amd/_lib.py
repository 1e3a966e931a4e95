"""ctypes binding of libminf_hip.so (the C ABI declared in include/minf_hip.h).

The library is never built implicitly and there is no fallback: if it is
missing, or a call returns a non-zero status, a RuntimeError is raised.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("MINF_HIP_LIB", os.path.join(_HERE, "libminf_hip.so"))
_lib = None

c_int = ctypes.c_int
c_i64 = ctypes.c_int64
c_f32 = ctypes.c_float
c_ptr = ctypes.c_void_p

# name -> (restype, argtypes); must list every symbol of include/minf_hip.h
SIGNATURES = {
    "minf_version": (c_int, []),
    "minf_status_string": (ctypes.c_char_p, [c_int]),
    "minf_qkvo_size": (ctypes.c_size_t, []),
    "minf_vs_index_build": (c_int, [c_ptr] * 7 + [c_int] * 6 + [c_ptr, c_ptr]),
    "minf_vs_index_workspace_bytes": (ctypes.c_size_t, [c_int] * 4),
    "minf_vs_index_build_ws": (c_int, [c_ptr] * 7 + [c_int] * 6 + [c_ptr, c_ptr, ctypes.c_size_t, c_ptr]),
    "minf_vs_index_build_static": (c_int, [c_ptr] * 7 + [c_int] * 6 + [c_ptr, c_ptr]),
    "minf_vs_attn_fwd": (c_int, [c_ptr] * 5 + [c_int] * 3 + [c_ptr]),
    "minf_bs_attn_fwd": (c_int, [c_ptr, c_ptr, c_int, c_int, c_ptr]),
    "minf_ashape_attn_fwd": (c_int, [c_ptr, c_int, c_int, c_ptr]),
    "minf_trishape_attn_fwd": (c_int, [c_ptr, c_int, c_int, c_int, c_f32, c_ptr]),
    "minf_dense_attn_fwd": (c_int, [c_ptr, c_ptr]),
    "minf_vs_estimate_workspace_bytes": (ctypes.c_size_t, [c_int, c_int, c_int]),
    "minf_vs_estimate": (c_int, [c_ptr, c_ptr, c_ptr, c_ptr] + [c_int] * 6 + [c_f32] + [c_int] * 4
                         + [c_ptr, c_ptr, c_ptr, ctypes.c_size_t, c_ptr]),
    "minf_vs_estimate_heads": (c_int, [c_ptr, c_ptr, c_ptr, c_ptr] + [c_int] * 6 + [c_f32] + [c_int] * 4 + [c_ptr, c_int]
                               + [c_ptr, c_ptr, c_ptr, ctypes.c_size_t, c_ptr]),
    "minf_topk_indices_pair_ragged": (c_int, [c_ptr, c_ptr, c_int, c_ptr, c_i64, c_int, c_int, c_int] * 2
                                      + [c_int, c_int, c_i64, c_ptr]),
    "minf_bs_block_index_heads": (c_int, [c_ptr, c_ptr, c_ptr, c_ptr] + [c_int] * 8 + [c_ptr, c_int]
                                  + [c_ptr, c_ptr, ctypes.c_size_t, c_ptr]),
    "minf_topk_indices": (c_int, [c_ptr, c_int, c_int, c_i64, c_int, c_ptr, c_i64, c_int, c_ptr]),
    "minf_topk_indices_block_causal": (c_int, [c_ptr, c_int, c_int, c_i64, c_int, c_ptr, c_i64, c_int, c_ptr]),
    "minf_topk_indices_pair": (c_int, [c_ptr, c_int, c_ptr, c_i64, c_int] * 2 + [c_int, c_int, c_i64, c_ptr]),
    "minf_bs_block_index_rows": (c_int, [c_int]),
    "minf_bs_block_index_workspace_bytes": (ctypes.c_size_t, [c_int] * 4),
    "minf_bs_block_index": (c_int, [c_ptr, c_ptr, c_ptr, c_ptr] + [c_int] * 8 + [c_ptr, c_ptr, ctypes.c_size_t, c_ptr]),
    "minf_pattern_recall_workspace_bytes": (ctypes.c_size_t, [c_int] * 3),
    "minf_pattern_recall": (c_int, [c_ptr, c_ptr, c_ptr, c_ptr] + [c_int] * 6 + [c_f32, c_ptr, c_ptr, c_i64, c_ptr, c_i64,
                                                                                   c_int, c_ptr, c_ptr, ctypes.c_size_t, c_ptr]),
    "minf_flags_set_indices": (c_int, [c_ptr, c_int, c_int, c_i64, c_int, c_ptr, c_i64, c_int, c_ptr]),
    "minf_flags_set_range": (c_int, [c_int, c_int, c_int, c_int, c_ptr, c_i64, c_ptr]),
    "minf_search_block_index_workspace_bytes": (ctypes.c_size_t, [c_int] * 4),
    "minf_search_block_index": (c_int, [c_ptr, c_ptr, c_ptr, c_ptr] + [c_int] * 7 + [c_ptr, c_ptr, ctypes.c_size_t, c_ptr]),
}


class QKVO(ctypes.Structure):
    """struct minf_qkvo of include/minf_hip.h."""
    _fields_ = [
        ("q", c_ptr), ("k", c_ptr), ("v", c_ptr), ("o", c_ptr),
        ("q_stride", c_i64 * 3), ("k_stride", c_i64 * 3), ("v_stride", c_i64 * 3), ("o_stride", c_i64 * 3),
        ("batch", c_int), ("heads_q", c_int), ("heads_kv", c_int), ("n", c_int),
        ("head_dim", c_int), ("dtype", c_int),
        ("seqlens", c_ptr),
        ("sm_scale", c_f32),
        ("head_list", c_ptr),
        ("index_heads", c_int),
    ]


MINF_BF16, MINF_F16 = 0, 1
MINF_ROUND_NONE, MINF_ROUND_INPUT_DTYPE = 0, 1
MINF_BS_FORCE_DIAG_FIRST, MINF_BS_ROUND_INPUT_DTYPE = 1, 2


class MinfError(RuntimeError):
    pass


def load():
    """Load libminf_hip.so once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MinfError(
                f"{LIB_PATH} not found: build it with `python -m minference_amd.build` "
                "(there is no fallback path)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        if lib.minf_qkvo_size() != ctypes.sizeof(QKVO):
            raise MinfError(f"{LIB_PATH} was built from another revision of include/minf_hip.h "
                            f"(struct minf_qkvo: {lib.minf_qkvo_size()} bytes there, {ctypes.sizeof(QKVO)} here); rebuild it")
        _lib = lib
    return _lib


def check(status: int, what: str):
    if status != 0:
        msg = load().minf_status_string(status)
        raise MinfError(f"{what} failed: {msg.decode() if msg else status} ({status})")


def stream_ptr(device=None):
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
