"""Host planning of a step, checked without a GPU through the C ABI (rd_plan_attention, rd_plan_gemm).

What the plans must guarantee: every (row, kv head) has its blocks covered once, in order, by items of a sixteenth of the
sequence but at most eight blocks (so a sequence of up to 128 blocks has at most 16 items, a longer one more); a row's cut
depends on its own length only (the partial results are merged in item order, so this is what keeps a row in a batch
bit-identical to the row alone, goinfer's StepBatch contract, decoder/resident/subsystems.go:102-110); rows share items only
when they are consecutive positions of one sequence with the same number of blocks."""
import numpy as np
import pytest

from goinfer_amd import capi

PIECES, MAX_CHUNK = 16, 8


def rows_of(item):
    return max(1, int(item[1]) >> 16)


def cuts(items, ranges, r, h):
    i0, i1, _ = ranges[r, h]
    return [(int(b0), int(b1)) for _, _, b0, b1 in items[i0:i1]]


def check_cover(items, ranges, lens, n_kv):
    for r, n in enumerate(lens):
        nb = (n + 63) // 64
        for h in range(n_kv):
            c = cuts(items, ranges, r, h)
            chunk = min(-(-nb // PIECES), MAX_CHUNK)
            assert len(c) == -(-nb // chunk) and all(b1 - b0 <= chunk for b0, b1 in c)
            assert len(c) <= PIECES or nb > PIECES * MAX_CHUNK
            assert c[0][0] == 0 and c[-1][1] == nb
            assert all(a[1] == b[0] for a, b in zip(c, c[1:])) and all(b0 < b1 for b0, b1 in c)
            i0, i1, sub = ranges[r, h]
            for it in items[i0:i1]:
                assert (int(it[1]) & 0xffff) == h
                assert int(it[0]) + sub == r and sub < rows_of(it)


@pytest.mark.parametrize("n_kv,G", [(8, 4), (2, 7), (4, 8), (1, 1), (1, 16)])
def test_one_row_per_sequence(n_kv, G):
    rng = np.random.default_rng(3)
    lens = [1, 63, 64, 65, 1024, 1025, 8192, 8193, 40000] + list(rng.integers(1, 9000, 23))
    items, ranges, grouped = capi.plan_attention(lens, None, G, n_kv)
    assert not grouped and all(int(it[1]) >> 16 == 0 for it in items)
    check_cover(items, ranges, lens, n_kv)
    # the longest sequences come first (the grid is dispatched in index order, the short items fill the tail)
    first = [lens[int(it[0])] for it in items]
    assert first == sorted(first, reverse=True)
    # a row's cut is the cut of the row alone
    for r in (0, 3, 6, 20):
        solo_items, solo_ranges, _ = capi.plan_attention([lens[r]], None, G, n_kv)
        for h in range(n_kv):
            assert cuts(items, ranges, r, h) == cuts(solo_items, solo_ranges, 0, h)


@pytest.mark.parametrize("n_kv,G", [(8, 4), (2, 7), (4, 8), (2, 2)])
def test_rows_of_one_sequence_share_items(n_kv, G):
    # slot 0: positions 60..70 (cross a block boundary at 64), slot 1: one row, slot 2: 130..134, slot 0 again later is a new run
    lens = list(range(60, 71)) + [500] + list(range(130, 135)) + [71]
    slots = [0] * 11 + [1] + [2] * 5 + [0]
    items, ranges, grouped = capi.plan_attention(lens, slots, G, n_kv)
    assert grouped == (16 // G > 1)
    check_cover(items, ranges, lens, n_kv)
    cap = max(1, 16 // G)
    for it in items:
        n, r0 = rows_of(it), int(it[0])
        assert n <= cap
        grp = range(r0, r0 + n)
        assert len({slots[r] for r in grp}) == 1
        assert [lens[r] for r in grp] == list(range(lens[r0], lens[r0] + n))
        assert len({(lens[r] + 63) // 64 for r in grp}) == 1  # same blocks, hence the same cut for every row of the item
    # every row's cut is still the cut of the row alone
    for r in range(len(lens)):
        solo_items, solo_ranges, _ = capi.plan_attention([lens[r]], None, G, n_kv)
        assert cuts(items, ranges, r, 0) == cuts(solo_items, solo_ranges, 0, 0)
    # fewer items than one per row
    single, _, _ = capi.plan_attention(lens, None, G, n_kv)
    assert len(items) < len(single) or cap == 1


def test_rows_that_do_not_ascend_by_one_stay_apart():
    items, ranges, grouped = capi.plan_attention([10, 12, 13, 13], [0, 0, 0, 0], 4, 2)
    assert grouped
    sizes = sorted(rows_of(it) for it in items if (int(it[1]) & 0xffff) == 0)
    assert sizes == [1, 1, 2]  # only 12,13 are consecutive positions


def test_plan_rejects_bad_input():
    with pytest.raises(capi.RocmError):
        capi.plan_attention([5, 0], None, 4, 2)
    with pytest.raises(capi.RocmError):
        capi.plan_attention([100000] * 4, None, 4, 8, max_items=16)


@pytest.mark.parametrize("N,nkb", [(6144, 16), (4096, 16), (28672, 16), (4096, 56), (128256, 32), (896, 7), (32, 1), (512, 3)])
def test_gemm_plan_covers_k(N, nkb):
    splits, per = capi.plan_gemm(N, nkb)
    assert splits >= 1 and per >= 1
    assert (splits - 1) * per < nkb <= splits * per  # no empty split, nothing left over
    assert per >= 2 or nkb == 1 or splits == nkb  # a split keeps at least two K-blocks unless K is that short
