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


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from minference_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.MinfError):
        _lib.load()
