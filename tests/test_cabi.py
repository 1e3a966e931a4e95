"""CPU-side checks of the C ABI: the library loads, exports every symbol that
include/minf_hip.h declares, and validates arguments before touching a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "minf_hip.h")


@pytest.fixture(scope="module")
def lib():
    from minference_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH):
        build.build()
    return _lib.load()


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(minf_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_exported_and_bound(lib):
    from minference_amd import _lib
    names = declared_symbols()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/minf_hip.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature in minference_amd/_lib.py"
    assert sorted(_lib.SIGNATURES) == names


def test_version_and_status_strings(lib):
    assert lib.minf_version() >= 100
    assert lib.minf_status_string(0) == b"ok"
    for code in (-1, -2, -3, -4):
        assert lib.minf_status_string(code) not in (b"ok", b"unknown status")


def test_argument_validation_needs_no_gpu(lib):
    from minference_amd import _lib
    # null pointers / bad sizes are rejected before any HIP call
    assert lib.minf_vs_index_build(None, None, None, None, None, None, None, 1, 1, 1, 1, 1, 1, None, None) == -1
    assert lib.minf_topk_indices(None, 1, 10, 10, 5, None, 5, -1, None) == -1
    # the entry point without a workspace argument: null pointers, then a problem larger than its
    # fixed array (refused by size alone, before any HIP call)
    assert lib.minf_vs_index_build_static(None, None, None, None, None, None, None, 1, 1, 1, 1, 1, 1, None, None) == -1
    assert lib.minf_vs_index_workspace_bytes(1, 64, 6096, 16384) > (8 << 20)
    assert lib.minf_vs_index_build_static(16, 16, 16, 16, 16, 16, 16, 1, 64, 16384, 1000, 6096, 1, None, None) == -4
    t = _lib.QKVO()
    assert lib.minf_dense_attn_fwd(ctypes.byref(t), None) == -1          # null tensors
    t.q = t.k = t.v = t.o = 16
    t.batch, t.heads_q, t.heads_kv, t.n, t.head_dim, t.dtype = 1, 4, 3, 64, 128, 0
    assert lib.minf_dense_attn_fwd(ctypes.byref(t), None) == -1          # 4 % 3 != 0
    t.heads_kv = 2
    t.head_dim = 96
    assert lib.minf_dense_attn_fwd(ctypes.byref(t), None) == -2          # unsupported head_dim
    t.head_dim = 128
    t.q = 8
    assert lib.minf_dense_attn_fwd(ctypes.byref(t), None) == -3          # misaligned pointer
    t.q = 16
    t.q_stride[2] = 100
    assert lib.minf_dense_attn_fwd(ctypes.byref(t), None) == -3          # row pitch not 16-byte aligned
    assert lib.minf_vs_estimate_workspace_bytes(1, 32, 131072) > 0
    assert lib.minf_vs_estimate_workspace_bytes(0, 32, 131072) == 0


def test_argument_validation_of_the_index_estimate_and_search_entry_points(lib):
    from minference_amd import _lib
    i3 = (_lib.c_i64 * 3)(128 * 64 * 4, 128 * 64, 128)
    bad = (_lib.c_i64 * 3)(128 * 64 * 4, 128 * 64, 100)
    P = 4096                                                     # any 16-byte aligned non-null address; never dereferenced
    # estimate: workspace too small / misaligned strides / last_q out of range
    assert lib.minf_vs_estimate(P, P, i3, i3, 1, 4, 4, 64, 128, 0, 0.1, 64, 30, 100, 0, P, P, P, 16, None) == -4
    assert lib.minf_vs_estimate(P, P, bad, i3, 1, 4, 4, 64, 128, 0, 0.1, 64, 30, 100, 0, P, P, P, 1 << 30, None) == -3
    assert lib.minf_vs_estimate(P, P, i3, i3, 1, 4, 4, 64, 128, 0, 0.1, 65, 30, 100, 0, P, P, P, 1 << 30, None) == -1
    assert lib.minf_vs_estimate(P, P, i3, i3, 1, 4, 4, 64, 96, 0, 0.1, 64, 30, 100, 1, P, P, P, 1 << 30, None) == -2
    assert lib.minf_vs_estimate(P, P, i3, i3, 1, 4, 4, 64, 128, 0, 0.1, 64, 30, 100, 7, P, P, P, 1 << 30, None) == -1   # no such rounding mode
    assert lib.minf_bs_block_index(P, P, i3, i3, 1, 4, 4, 64, 128, 0, 10, 4, P, P, 1 << 30, None) == -1      # unknown flag bit
    # block index: head counts, head_dim, workspace
    assert lib.minf_bs_block_index(P, P, i3, i3, 1, 4, 3, 64, 128, 0, 10, 0, P, P, 1 << 30, None) == -1
    assert lib.minf_bs_block_index(P, P, i3, i3, 1, 4, 4, 64, 256, 0, 10, 0, P, P, 1 << 30, None) == -2
    assert lib.minf_bs_block_index(P, P, i3, i3, 1, 4, 4, 64, 128, 0, 10, 0, P, P, 8, None) == -4
    assert lib.minf_search_block_index(P, P, i3, i3, 1, 4, 4, 64, 128, 0, 0, P, P, 1 << 30, None) == -1   # top_k 0
    assert lib.minf_bs_block_index_rows(64) == 2 and lib.minf_bs_block_index_rows(65) == 2
    # vertical-slash attention: row count must be ceil(n/64), list widths positive
    t = _lib.QKVO()
    t.q = t.k = t.v = t.o = P
    t.batch, t.heads_q, t.heads_kv, t.n, t.head_dim, t.dtype = 1, 4, 4, 130, 128, 0
    for name in ("q_stride", "k_stride", "v_stride", "o_stride"):
        getattr(t, name)[:] = [128 * 130 * 4, 128 * 130, 128]
    assert lib.minf_vs_attn_fwd(ctypes.byref(t), P, P, P, P, 2, 8, 8, None) == -1         # rows must be 3
    assert lib.minf_vs_attn_fwd(ctypes.byref(t), P, P, P, P, 3, 0, 8, None) == -1         # nnz_s < 1
    assert lib.minf_vs_attn_fwd(ctypes.byref(t), None, P, P, P, 3, 8, 8, None) == -1
    assert lib.minf_bs_attn_fwd(ctypes.byref(t), P, 2, 4, None) == -1                     # too few rows
    assert lib.minf_ashape_attn_fwd(ctypes.byref(t), 4, 0, None) == -1                    # n_local < 1
    assert lib.minf_trishape_attn_fwd(ctypes.byref(t), 4, 8, -1, 0.0, None) == -1
    # pattern search: flag pitch rules, candidate bit range, workspace
    assert lib.minf_pattern_recall(P, P, i3, i3, 1, 4, 4, 130, 128, 0, 0.1, P, P, 128, None, 0, 0, P, P, 1 << 20, None) == -1   # pitch < 192
    assert lib.minf_pattern_recall(P, P, i3, i3, 1, 4, 4, 130, 128, 0, 0.1, P, P, 192, None, 0, 0, P, P, 8, None) == -4
    assert lib.minf_pattern_recall(P, P, i3, i3, 1, 4, 4, 130, 128, 0, 0.1, P, P, 192, P, 2, 0, P, P, 1 << 20, None) == -1      # block pitch < 5
    assert lib.minf_pattern_recall_workspace_bytes(1, 4, 130) == 4 * 3 * 8 * 4
    assert lib.minf_flags_set_indices(P, 4, 10, 10, 8, P, 192, 130, None) == -1           # bit 8
    assert lib.minf_flags_set_indices(P, 4, 10, 10, 0, P, 190, 130, None) == -1           # pitch % 4
    assert lib.minf_flags_set_range(0, 200, 4, 0, P, 192, None) == -1                     # end > pitch
    assert lib.minf_flags_set_range(10, 10, 4, 0, P, 192, None) == 0                      # empty range: nothing to do


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from minference_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.MinfError):
        _lib.load()
