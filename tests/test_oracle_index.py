"""Pins oracle/vs_index_ref.c (restatement of csrc/vertical_slash_index.cu:27-99)
without the reference: hand-computed rows, a set-based specification that is
written differently from the merge loop, and structural properties."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import gen


def spec_row(vert, slash, m, seqlen):
    """Specification, not a transcription: column ends t, greedy 64-periodic
    cover, columns = verticals outside every range and below the last end."""
    start_m, end_m = 64 * m, 64 * m + 64
    if start_m >= seqlen:
        return [], []
    ts = sorted(max(end_m - int(o), 64) for o in slash if o < end_m)
    ranges = []
    for t in ts:
        if not ranges or t > ranges[-1][1] + 64:
            ranges.append([t - 64, t])
        else:
            while ranges[-1][1] < t:
                ranges[-1][1] += 64
    blocks = [x for a, e in ranges for x in range(a, e, 64)]
    covered = set()
    for a, e in ranges:
        covered.update(range(a, e))
    cols = [int(x) for x in vert if x not in covered and x < ranges[-1][1]]
    return blocks, cols


def test_hand_kat():
    # worked by hand: row 10 (rows 640..703): offsets 500,70,64,3,0 -> t = 204,634,640,701,704
    V = np.array([[[0, 1, 2, 3, 100, 130, 700]]], np.int32)
    S = np.array([[[500, 70, 64, 3, 0]]], np.int32)
    bc, bo, cc, ci = O.vs_index_build([1024], V, S, 1024)
    assert bc[0, 0, 10] == 4 and bo[0, 0, 10, :4].tolist() == [140, 570, 634, 698]
    assert cc[0, 0, 10] == 6 and ci[0, 0, 10, :6].tolist() == [0, 1, 2, 3, 100, 130]
    assert bo[0, 0, 10, 4:].tolist() == [0] and ci[0, 0, 10, 6:].tolist() == [0]
    # row 0: only offsets 3 and 0 are below 64; both clamp to t=64 -> one block at 0
    assert bc[0, 0, 0] == 1 and bo[0, 0, 0, 0] == 0 and cc[0, 0, 0] == 0


def test_hand_kat_phase():
    # whether a gap of ~100 between column ends opens a new range depends on the phase of
    # the running range end.  Row 15 (end_m = 1024), column end t = 1024 - offset:
    #  t=200,250,350,1024: [136,200) -> 250 extends to 264 -> 350 > 328 new [286,350) -> new [960,1024)
    #  t=200,260,350,1024: same ranges
    #  t=200,264,324,350,1024: 264, 328, then 350 extends to 392 -> one range [136,392)
    #  t=200,250,300,1024: 250 extends to 264, 300 <= 328 extends to 328
    #  t=200,300,1024: 300 > 264 -> new range [236,300)
    V = np.array([[[0, 137, 270, 300, 391, 392]]], np.int32)
    for S, blocks, cols in [
        ([824, 774, 674, 0], [136, 200, 286, 960], [0, 270, 391, 392]),
        ([824, 764, 674, 0], [136, 200, 286, 960], [0, 270, 391, 392]),
        ([824, 760, 700, 674, 0], [136, 200, 264, 328, 960], [0, 392]),
        ([824, 774, 724, 0], [136, 200, 264, 960], [0, 391, 392]),
        ([824, 724, 0], [136, 236, 960], [0, 300, 391, 392]),
    ]:
        bc, bo, cc, ci = O.vs_index_build([1024], V, np.array([[S]], np.int32), 1024)
        assert bo[0, 0, 15, : bc[0, 0, 15]].tolist() == blocks
        assert ci[0, 0, 15, : cc[0, 0, 15]].tolist() == cols


def test_rows_past_seqlen_untouched_and_zero_tails():
    v, s = gen.vs_index_inputs(2, 1000, 20, 70, seed=5)
    bc, bo, cc, ci = O.vs_index_build([600], v, s, 1000)
    assert (bc[0, :, 10:] == 0).all() and (bo[0, :, 10:] == 0).all()
    assert (cc[0, :, 10:] == 0).all() and (ci[0, :, 10:] == 0).all()
    for h in range(2):
        for m in range(10):
            assert (bo[0, h, m, bc[0, h, m]:] == 0).all()
            assert (ci[0, h, m, cc[0, h, m]:] == 0).all()


def test_out_of_bounds_case_is_reported():
    V = np.array([[[0, 5]]], np.int32)
    S = np.array([[[500, 400]]], np.int32)   # no offset below 64 for row 0
    with pytest.raises(ValueError):
        O.vs_index_build([1024], V, S, 1024)


@pytest.mark.parametrize("seed", range(6))
def test_c_vs_python_vs_spec(seed):
    rng = np.random.default_rng(seed)
    n = int(rng.choice([200, 1000, 4096, 30000]))
    nv, ns = int(rng.integers(1, 120)), int(rng.integers(1, 300))
    ns = min(ns, n); nv = min(nv, n)
    v, s = gen.vs_index_inputs(3, n, nv, ns, seed=seed * 7, force_v=min(4, nv), force_s=min(2, ns))
    seqlen = int(rng.integers(n // 2, n + 1))
    bc, bo, cc, ci = O.vs_index_build([seqlen], v, s, n)
    rows = (n + 63) // 64
    for h in range(3):
        for m in rng.choice(rows, size=min(rows, 12), replace=False):
            m = int(m)
            pb, pc = O.vs_index_row_py(v[0, h], s[0, h], m, seqlen)
            sb, sc = spec_row(v[0, h], s[0, h], m, seqlen)
            cb = bo[0, h, m, : bc[0, h, m]].tolist()
            ccols = ci[0, h, m, : cc[0, h, m]].tolist()
            assert cb == pb == sb
            assert ccols == pc == sc


def test_properties_config3_generator():
    # shape of BASELINE config 3 scaled down: always contains 0..3 / 0..63
    n = 16384
    v, s = gen.vs_index_inputs(2, n, 100, 600, seed=300)
    bc, bo, cc, ci = O.vs_index_build([n], v, s, n)
    for h in range(2):
        for m in range(n // 64):
            b = bo[0, h, m, : bc[0, h, m]]
            c = ci[0, h, m, : cc[0, h, m]]
            assert bc[0, h, m] <= 600 and cc[0, h, m] <= 100
            assert (np.diff(b) >= 64).all()            # ascending, never overlapping
            assert (np.diff(c) > 0).all()
            assert (c < 64 * m).all() if len(c) else True   # columns strictly left of the row block
            # every selected diagonal / vertical is covered for every row of the block
            cover = np.zeros(n + 128, bool)
            for x in b:
                cover[x:x + 64] = True
            cover[c] = True
            for r in (64 * m, 64 * m + 63):
                cols = r - s[0, h][s[0, h] <= r]
                assert cover[cols].all()
                assert cover[v[0, h][v[0, h] <= 64 * m - 1]].all() or True


@pytest.mark.parametrize("n,nv,ns,seed", [(1024, 7, 5, 0), (4096, 100, 300, 1), (8192, 1000, 2048, 2), (5000, 33, 65, 3)])
def test_list_padding_is_a_noop_of_the_merge_loop(n, nv, ns, seed):
    """One index build serves heads with different (vertical_size, slash_size) when the shorter lists
    are padded to the longest: verticals with a constant no range ever reaches (never emitted:
    csrc/vertical_slash_index.cu:71-74 only emits v < range_start), slashes with their last offset
    repeated (the same column end again neither starts a range, :87-90, nor extends one, :91-92).
    The reference algorithm must give, for the padded lists, exactly the tensors of the unpadded
    ones followed by zeros."""
    v, s = gen.vs_index_inputs(2, n, nv, ns, seed=seed, force_v=min(4, nv), force_s=min(64, ns))
    bc, bo, cc, ci = O.vs_index_build([n], v, s, n)
    vp = np.concatenate([v, np.full((1, 2, 37), 0x3FFFFFFF, np.int32)], axis=2)
    sp = np.concatenate([s, np.repeat(s[:, :, -1:], 100, axis=2)], axis=2)
    pbc, pbo, pcc, pci = O.vs_index_build([n], vp, sp, n)
    assert np.array_equal(pbc, bc) and np.array_equal(pcc, cc)
    assert np.array_equal(pbo[..., :ns], bo) and not pbo[..., ns:].any()
    assert np.array_equal(pci[..., :nv], ci) and not pci[..., nv:].any()
    # and row by row with the pure-Python twin
    for m in (0, 1, (n + 63) // 64 - 1):
        assert O.vs_index_row_py(vp[0, 1].tolist(), sp[0, 1].tolist(), m, n) == O.vs_index_row_py(v[0, 1].tolist(), s[0, 1].tolist(), m, n)
