"""minf_vs_index_build_static (the entry point that allocates nothing: its tables live in a
device array inside the library) against minf_vs_index_build_ws, through the C ABI: identical
tensors, bit for bit, on two calls in a row -- the second on a smaller problem, so that whatever
the first call left in the shared array must not leak into it -- and a size beyond the array is
refused.  The C oracle checks the second (small) case as well."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import gen

pytestmark = pytest.mark.gpu

NAMES = ["block_count", "block_offset", "column_count", "column_index"]


def _build(entry, n, v, s, dev, sentinel):
    """Calls `entry` ('static' or 'ws') directly through ctypes; outputs start as `sentinel`."""
    from minference_amd import _lib
    lib = _lib.load()
    B, H, V = v.shape
    S = s.shape[2]
    rows = (n + 63) // 64
    seqlens = torch.tensor([n] * B, dtype=torch.int32, device=dev)
    vg = torch.from_numpy(v).to(dev)
    sg = torch.from_numpy(np.ascontiguousarray(s)).to(dev)
    outs = [torch.full(shape, sentinel, dtype=torch.int32, device=dev)
            for shape in [(B, H, rows), (B, H, rows, S), (B, H, rows), (B, H, rows, V)]]
    args = [seqlens.data_ptr(), vg.data_ptr(), sg.data_ptr()] + [o.data_ptr() for o in outs] + \
           [B, H, rows, V, S, 1, None]
    stream = _lib.stream_ptr(dev)
    if entry == "static":
        st = lib.minf_vs_index_build_static(*args, stream)
    else:
        nbytes = lib.minf_vs_index_workspace_bytes(B, H, S, rows)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        st = lib.minf_vs_index_build_ws(*args, ws.data_ptr(), nbytes, stream)
    torch.cuda.synchronize()
    assert st == 0, (entry, st)
    return [o.cpu().numpy() for o in outs]


def test_static_entry_matches_workspace_entry_twice(gpu):
    big = dict(heads=8, n=65536, nv=1000, ns=6096, seed=11)
    small = dict(heads=3, n=5000, nv=33, ns=65, seed=12)
    with torch.cuda.device(gpu):
        for case, sentinel in ((big, -7), (small, -9)):
            print(f"case {case}", flush=True)
            v, s = gen.vs_index_inputs(case["heads"], case["n"], case["nv"], case["ns"], seed=case["seed"])
            got = _build("static", case["n"], v, s, gpu, sentinel)
            ref = _build("ws", case["n"], v, s, gpu, sentinel)
            for name, a, b in zip(NAMES, got, ref):
                assert np.array_equal(a, b), f"{name} differs between the static and the workspace entry ({case})"
            if case is small:
                for name, a, b in zip(NAMES, got, O.vs_index_build([case["n"]], v, s, case["n"])):
                    assert np.array_equal(a, b), f"{name} differs from the oracle"


def test_static_entry_refuses_sizes_beyond_its_array(gpu):
    from minference_amd import _lib
    lib = _lib.load()
    limit = 8 << 20
    assert lib.minf_vs_index_workspace_bytes(1, 64, 6096, 16384) > limit
    one = torch.zeros(1, dtype=torch.int32, device=gpu)
    p = one.data_ptr()
    with torch.cuda.device(gpu):
        st = lib.minf_vs_index_build_static(p, p, p, p, p, p, p, 1, 64, 16384, 1000, 6096, 1, None, None)
    assert st == -4
    assert lib.minf_status_string(st) not in (b"ok", b"unknown status")
    assert isinstance(ctypes.c_int(st).value, int)
