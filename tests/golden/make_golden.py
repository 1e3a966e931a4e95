"""Writes tests/golden/small_cases.npz: seeded inputs plus the CPU oracle's outputs for the index
builder and the three attention operators (n = 256, 1 head, head_dim 128; q/k/v are stored as fp16, outputs as fp32).  The reference itself is never imported: its own tests hold no
vectors for this path, so these fixtures pin the oracle (and, through the GPU tests, the HIP
kernels) against regressions, not against the reference.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as O      # noqa: E402
from tests import gen               # noqa: E402

n, H = 256, 1
q, k, v = gen.qkv(1, H, H, n, 128, seed=42, dtype=torch.float32, scale=1.0)
q, k, v = q.half().float(), k.half().float(), v.half().float()
vi, si = gen.vs_index_inputs(H, n, 12, 24, seed=42, force_v=2, force_s=4)
si = np.ascontiguousarray(si)
seqlens = np.array([n], np.int32)
bc, bo, cc, ci = O.vs_index_build(seqlens, vi, si, n)
np.savez_compressed(
    os.path.join(os.path.dirname(os.path.abspath(__file__)), "small_cases.npz"),
    n=n, seqlens=seqlens, vertical=vi, slash=si, block_count=bc, block_offset=bo, column_count=cc,
    column_index=ci, q=q.half().numpy(), k=k.half().numpy(), v=v.half().numpy(),
    vs_out=O.vertical_slash_sparse_attention(q, k, v, torch.from_numpy(vi), torch.from_numpy(si)).numpy(),
    ashape_out=O.streaming_forward(q, k, v, 8, 48).numpy(),
    bs_out=O.block_sparse_attention(q, k, v, 2).numpy())
print("wrote small_cases.npz")
