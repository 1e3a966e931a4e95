"""GPU parity of minf_vs_index_build (through the C ABI) against the C oracle:
bit-exact on the full tensors, zero tails included."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests import gen

pytestmark = pytest.mark.gpu


def run_gpu(seqlens, v, s, n, dev, zero_fill=True):
    """Table-driven builder (minf_vs_index_build_ws); with zero_fill the plain wave-per-row
    builder (minf_vs_index_build) is run on the same inputs and must give the same tensors."""
    from minference_amd import convert_vertical_slash_indexes
    args = (torch.tensor(seqlens, dtype=torch.int32, device=dev), torch.from_numpy(v).to(dev),
            torch.from_numpy(np.ascontiguousarray(s)).to(dev), n, 64, 64)
    out = convert_vertical_slash_indexes(*args, zero_fill=zero_fill)
    torch.cuda.synchronize()
    out = [o.cpu().numpy() for o in out]
    if zero_fill:
        plain = convert_vertical_slash_indexes(*args, zero_fill=True, use_tables=False)
        torch.cuda.synchronize()
        for name, a, b in zip(["block_count", "block_offset", "column_count", "column_index"], out, plain):
            assert np.array_equal(a, b.cpu().numpy()), f"table-driven and plain builders differ in {name}"
    return out


def assert_same(got, ref):
    for name, g, r in zip(["block_count", "block_offset", "column_count", "column_index"], got, ref):
        assert g.dtype == np.int32 and g.shape == r.shape, name
        assert np.array_equal(g, r), f"{name}: {np.argwhere(g != r)[:5]}"


@pytest.mark.parametrize("heads,n,nv,ns,seed", [
    (1, 1024, 7, 5, 0), (3, 4096, 100, 300, 1), (4, 8192, 1000, 2048, 2),
    (2, 16384, 1000, 6096, 3), (2, 5000, 33, 65, 4), (1, 200, 1, 1, 5),
    (2, 70000, 257, 129, 6),
])
def test_random_lists(gpu, heads, n, nv, ns, seed):
    print(f"case heads={heads} n={n} nv={nv} ns={ns} seed={seed}", flush=True)
    v, s = gen.vs_index_inputs(heads, n, nv, ns, seed=seed, force_v=min(4, nv), force_s=min(64, ns))
    ref = O.vs_index_build([n], v, s, n)
    assert_same(run_gpu([n], v, s, n, gpu), ref)


@pytest.mark.parametrize("n,smax,ns,nv", [(1024, 9000, 300, 60), (4096, 4160, 129, 500), (2000, 200000, 64, 1000)])
def test_offsets_beyond_the_context(gpu, n, smax, ns, nv):
    """Slash offsets far larger than the context (every row block skips most of the list): the
    per-head table then spans more positions than the coverage bitmap holds, and the row blocks
    fall back to searching the tabulated ranges.  Same tensors as the oracle either way."""
    rng = np.random.default_rng(n + ns)
    for h_seed in range(3):
        big = rng.choice(np.arange(64, smax), size=ns - 40, replace=False)
        sl = np.sort(np.concatenate([np.arange(40), big]))[::-1].astype(np.int32)
        vl = np.sort(rng.choice(n, size=min(nv, n), replace=False)).astype(np.int32)
        v, s = vl[None, None, :].copy(), sl[None, None, :].copy()
        ref = O.vs_index_build([n], v, s, n)
        assert_same(run_gpu([n], v, s, n, gpu), ref)


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
def test_structured_lists_all_rows(gpu, mode):
    """Slash lists that stress the table-driven path: clusters with gaps just below / above the
    64-token merge distance, duplicates, offsets up to n-1 (so most rows skip or clip entries and
    join the tabulated ranges late), dense runs whose 64-phase depends on the first valid entry;
    mode 4: runs of hundreds to thousands of consecutive or nearly consecutive offsets (what the
    estimated slashes of a real head look like), which the row blocks cross in one step."""
    rng = np.random.default_rng(100 + mode)
    for trial in range(6):
        n = int(rng.choice([1500, 4096, 9000, 20000]))
        S = int(rng.integers(2, 400)); V = int(rng.integers(1, 200))
        if mode == 0:
            sl = np.sort(rng.choice(n, size=min(S, n), replace=False))[::-1]
        elif mode == 1:
            sl = np.unique(np.concatenate([np.arange(min(S, 300)), rng.integers(0, n, 7)]))[::-1]
        elif mode == 2:
            c = rng.integers(0, n, 6)
            sl = np.sort(np.clip(np.concatenate([cc + rng.integers(-150, 150, S // 6 + 1) for cc in c]), 0, n - 1))[::-1]
        elif mode == 4:
            parts, pos = [], int(rng.integers(0, 3))
            while pos < n and sum(len(x) for x in parts) < 3000:
                run = int(rng.choice([70, 130, 500, 2000]))
                step = rng.choice([1, 1, 1, 2, 30, 64], size=run, p=[0.5, 0.2, 0.1, 0.1, 0.05, 0.05])
                seg = pos + np.cumsum(step)
                parts.append(seg[seg < n])
                pos = int(seg[-1]) + int(rng.choice([65, 66, 100, 127, 128, 129, 191, 192, 193, 1000]))
            sl = np.unique(np.concatenate(parts + [np.arange(3)]))[::-1]
        else:
            steps = rng.choice([1, 1, 2, 63, 64, 65, 127, 128, 129, 500], size=S)
            sl = np.cumsum(steps); sl = sl[sl < n][::-1]
            if sl.size == 0: sl = np.array([0])
        vt = np.sort(rng.choice(n, size=min(V, n), replace=False))
        if sl[-1] >= 64:
            sl = np.concatenate([sl, [int(rng.integers(0, 64))]])   # every row block needs a valid entry
        s = np.ascontiguousarray(sl[None, None].astype(np.int32))
        v = np.ascontiguousarray(vt[None, None].astype(np.int32))
        seqlen = n if trial % 3 else n - 77
        print(f"case structured mode={mode} trial={trial} n={n} S={s.shape[-1]} V={v.shape[-1]} seqlen={seqlen}", flush=True)
        ref = O.vs_index_build([seqlen], v, s, n)
        assert_same(run_gpu([seqlen], v, s, n, gpu), ref)


@pytest.mark.parametrize("kind", ["maybe chains", "two or three chunks", "more chunks than the marks hold"])
def test_table_pass_shares_of_the_list(gpu, kind):
    """The table pass cuts a head's list into shares for 16 wavefronts; a wavefront finds the state at
    the head of its share by replaying the "maybe" entries (65..127 above their predecessor) since
    the last "sure" start (more than 127 above).  Lists built to stress that: hundreds of entries in
    a row whose gaps are all 65..127 (no sure start for whole shares, so the replay crosses several
    of them), lists of two chunks (walked by one wavefront) and three (shared), and a list of more
    chunks than the mark arrays hold (walked by one wavefront).  Bit-exact against the C oracle and
    against the plain wave-per-row builder."""
    rng = np.random.default_rng(len(kind))
    cases = []
    if kind == "maybe chains":
        for trial in range(3):
            steps = rng.choice([65, 66, 100, 126, 127, 128, 1, 64], size=5000,
                               p=[0.25, 0.1, 0.3, 0.1, 0.15, 0.02 * trial, 0.05, 0.05 - 0.02 * trial])
            sl = np.concatenate([[0], np.cumsum(steps)])
            n = int(sl[-1]) + 100
            cases.append((n, sl[::-1], np.sort(rng.choice(n, size=300, replace=False))))
    elif kind == "two or three chunks":
        for S in (65, 127, 128, 129, 191, 192, 193):
            steps = rng.choice([1, 2, 64, 65, 127, 128, 300], size=S - 1)
            sl = np.concatenate([[0], np.cumsum(steps)])
            n = int(sl[-1]) + 70
            cases.append((n, sl[::-1], np.sort(rng.choice(n, size=min(n, 90), replace=False))))
    else:
        S = 2049 * 64 + 5
        steps = rng.choice([1, 66, 130], size=S - 1, p=[0.999, 0.0005, 0.0005])
        sl = np.concatenate([[0], np.cumsum(steps)])
        n = int(sl[-1]) + 200
        sl = sl[sl < n]
        assert sl.size > 2048 * 64
        cases.append((n, sl[::-1], np.sort(rng.choice(n, size=500, replace=False))))
    for n, sl, vt in cases:
        s = np.ascontiguousarray(sl[None, None].astype(np.int32))
        v = np.ascontiguousarray(vt[None, None].astype(np.int32))
        print(f"case table pass: {kind} n={n} S={s.shape[-1]} V={v.shape[-1]}", flush=True)
        ref = O.vs_index_build([n], v, s, n)
        assert_same(run_gpu([n], v, s, n, gpu), ref)


def test_hand_kat(gpu):
    V = np.array([[[0, 1, 2, 3, 100, 130, 700]]], np.int32)
    S = np.array([[[500, 70, 64, 3, 0]]], np.int32)
    bc, bo, cc, ci = run_gpu([1024], V, S, 1024, gpu)
    assert bo[0, 0, 10, : bc[0, 0, 10]].tolist() == [140, 570, 634, 698]
    assert ci[0, 0, 10, : cc[0, 0, 10]].tolist() == [0, 1, 2, 3, 100, 130]


def test_clustered_slashes_and_duplicates(gpu):
    # contiguous offsets near the diagonal (what real heads look like) + repeated entries
    n = 20000
    s = np.sort(np.concatenate([np.arange(3000), np.array([5000, 5000, 5064, 5100, 9000, 9127, 9128, 19999])]))[::-1]
    s = np.ascontiguousarray(s[None, None].astype(np.int32))
    v = np.sort(np.random.default_rng(1).choice(n, 500, replace=False)).astype(np.int32)[None, None]
    v[0, 0, 0] = 0
    ref = O.vs_index_build([n], v, s, n)
    assert_same(run_gpu([n], v, s, n, gpu), ref)


def test_seqlen_shorter_than_context_and_batch(gpu):
    v, s = gen.vs_index_inputs(2, 3000, 50, 200, seed=11, batch=2)
    ref = O.vs_index_build([3000, 1700], v, s, 3000)
    assert_same(run_gpu([3000, 1700], v, s, 3000, gpu), ref)


@pytest.mark.parametrize("lists", ["uniform", "dense runs"])
def test_payload_only_mode(gpu, lists):
    """The form without zero tails (its row-block kernel is an instantiation of its own): counts and
    payload prefixes as in the oracle, on uniform lists and on lists made of long runs of
    consecutive offsets."""
    n = 4096
    if lists == "uniform":
        v, s = gen.vs_index_inputs(2, n, 64, 256, seed=12)
    else:
        rng = np.random.default_rng(12)
        sl = [np.unique(np.concatenate([np.arange(700), 900 + np.arange(0, 400, int(st)), 1500 + np.arange(1200),
                                        rng.integers(2800, n, 40)]))[::-1] for st in (1, 2)]
        m = min(len(x) for x in sl)
        s = np.ascontiguousarray(np.stack([x[-m:] for x in sl])[None].astype(np.int32))
        v = np.sort(np.stack([rng.choice(n, size=200, replace=False) for _ in range(2)]), axis=-1)[None].astype(np.int32)
    ref = O.vs_index_build([n], v, s, n)
    bc, bo, cc, ci = run_gpu([n], v, s, n, gpu, zero_fill=False)
    assert np.array_equal(bc, ref[0]) and np.array_equal(cc, ref[2])
    for h in range(2):
        for m in range(64):
            assert np.array_equal(bo[0, h, m, : bc[0, h, m]], ref[1][0, h, m, : bc[0, h, m]])
            assert np.array_equal(ci[0, h, m, : cc[0, h, m]], ref[3][0, h, m, : cc[0, h, m]])


def test_out_of_bounds_row_sets_flag(gpu):
    from minference_amd import convert_vertical_slash_indexes
    V = torch.tensor([[[0, 5]]], dtype=torch.int32, device=gpu)
    S = torch.tensor([[[500, 400]]], dtype=torch.int32, device=gpu)
    flag = torch.zeros(1, dtype=torch.int32, device=gpu)
    bc, bo, cc, ci = convert_vertical_slash_indexes(
        torch.tensor([1024], dtype=torch.int32, device=gpu), V, S, 1024, error_flag=flag)
    torch.cuda.synchronize()
    assert flag.item() == 1
    assert bc[0, 0, 0].item() == 0 and bc[0, 0, 8].item() > 0


def test_config3_shape_bit_exact(gpu):
    # BASELINE config 3: 32 heads, 1000 verticals, 6096 slashes, seq 262144 -- checked on
    # 2 of the 32 heads against the oracle (full tensors), all heads for invariants
    n, H = 262144, 32
    v, s = gen.vs_index_inputs(H, n, 1000, 6096, seed=300)
    got = run_gpu([n], v, s, n, gpu)
    ref = O.vs_index_build([n], v[:, :2], s[:, :2], n)
    for g, r in zip(got, ref):
        assert np.array_equal(g[:, :2], r)
    bc, bo, cc, ci = got
    assert (bc >= 1).all() and (bc <= 6096).all() and (cc <= 1000).all()
