"""Host logic of the LDS-staging kernels' own copy of the matrix: adjacent windows
merged into units of up to four windows that carry the union of their column lists
(hspmm_panel_units_preview; no GPU needed).  The rewritten matrix must be the same
matrix, bit for bit, with zeros added; the choice of what to merge follows the
step-count rule stated in include/hspmm.h."""
import numpy as np
import pytest

from util import IDX_MAX, btcf_to_csr, encode, random_csr

PANEL, STEP = 256, 32


def convert(hs, A):
    return hs.csr_to_btcf(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], A["dtype"])


def real_ids(b, ro, a2b, w):
    cw = b["cw"]
    ids = a2b[ro[w] * cw:ro[w + 1] * cw]
    n = ids.size
    while n and ids[n - 1] == IDX_MAX:
        n -= 1
    assert not (ids[:n] == IDX_MAX).any(), "padding inside a list"
    return ids[:n]


def panel_steps(ids):
    """Steps of 32 columns a list needs when no step straddles a panel of 256 columns."""
    if ids.size == 0:
        return 0
    per_panel = np.bincount(ids // PANEL)
    return int(((per_panel + STEP - 1) // STEP).sum())


def check_grouping(b, g, max_windows):
    W = b["eff_row_windows"]
    first, count = g["group_first"], g["group_count"]
    # the groups tile the windows in order, and their windows are adjacent in the matrix
    assert first[0] == 0 and int(count.sum()) == W
    assert np.array_equal(first[1:], (first + count)[:-1])
    assert count.min() >= 1 and count.max() <= max_windows
    ro, a2b = g["rowOffset"], g["tcA2B"]
    assert ro[0] == 0 and ro[W] == g["total_tiles"]
    for f, c in zip(first, count):
        rows = b["rowIdx"][f:f + c]
        assert np.array_equal(rows, rows[0] + 8 * np.arange(c)), "windows of a unit must be adjacent"
        lists = [real_ids(b, b["rowOffset"], b["tcA2B"], w) for w in range(f, f + c)]
        want = lists[0] if c == 1 else np.unique(np.concatenate(lists))
        for w in range(f, f + c):
            assert np.array_equal(real_ids(b, ro, a2b, w), want), "every window of a unit carries the union"
            assert ro[w + 1] - ro[w] == (want.size + b["cw"] - 1) // b["cw"]
    # the same matrix: identical (row, column, value) triples, everything added is zero
    rewritten = dict(b, rowOffset=ro, tcA2B=a2b, data=g["data"], total_tiles=g["total_tiles"])
    assert btcf_to_csr(rewritten) == btcf_to_csr(b)
    return lists


@pytest.mark.parametrize("dtype", [0, 1, 2])
@pytest.mark.parametrize("density", [0.01, 0.08, 0.3])
def test_grouped_matrix_is_the_same_matrix(hs, dtype, density):
    rng = np.random.default_rng(int(density * 1000) + dtype)
    A = random_csr(rng, 211, 700, density, dtype, empty_row_prob=0.1)
    A["row_ptr"] = A["row_ptr"].copy()
    b = convert(hs, A)
    for max_windows in (1, 2, 4):
        g = hs.panel_units_preview(b, max_windows)
        check_grouping(b, g, max_windows)
        if max_windows == 1:
            assert g["total_tiles"] == b["total_tiles"] and np.array_equal(g["tcA2B"], b["tcA2B"])
            assert np.array_equal(g["data"], b["data"].reshape(-1))


def windows_matrix(column_lists, row_starts, cols, dtype=0):
    """One entry per (window, column) in the window's first row."""
    rows = max(row_starts) + 8
    rp = np.zeros(rows + 1, np.uint32)
    ci = []
    by_row = dict(zip(row_starts, column_lists))
    for r in range(rows):
        ci += sorted(by_row.get(r, []))
        rp[r + 1] = len(ci)
    vals = encode(np.arange(1, len(ci) + 1, dtype=np.float32) % 7 + 1, dtype)
    return dict(rows=rows, cols=cols, dtype=dtype, row_ptr=rp, col_idx=np.array(ci, np.uint32), values=vals)


def groups_of(hs, A, max_windows):
    b = convert(hs, A)
    g = hs.panel_units_preview(b, max_windows)
    check_grouping(b, g, max_windows)
    return list(zip(g["group_first"].tolist(), g["group_count"].tolist()))


def test_merge_rule_on_hand_made_windows(hs):
    # overlapping lists inside one panel: 16 + 16 columns -> 24, one step instead of two
    A = windows_matrix([range(0, 16), range(8, 24)], [0, 8], 600)
    assert groups_of(hs, A, 2) == [(0, 2)]
    # lists in different panels: the union needs both steps, nothing is saved
    A = windows_matrix([range(0, 32), range(256, 288)], [0, 8], 600)
    assert groups_of(hs, A, 2) == [(0, 1), (1, 1)]
    # the same list twice is a pair whatever its length; a window with a gap in front of it is not adjacent
    A = windows_matrix([range(0, 40), range(0, 40), range(0, 40)], [0, 8, 24], 600)
    assert groups_of(hs, A, 4) == [(0, 2), (2, 1)]
    # four windows with one list: two pairs, or one unit of four
    A = windows_matrix([range(3, 90)] * 4, [0, 8, 16, 24], 600)
    assert groups_of(hs, A, 2) == [(0, 2), (2, 2)]
    assert groups_of(hs, A, 4) == [(0, 4)]
    assert groups_of(hs, A, 1) == [(0, 1), (1, 1), (2, 1), (3, 1)]
    # seven adjacent windows with heavily overlapping lists: 4 + 3
    A = windows_matrix([range(k, 200 + k) for k in range(7)], [8 * k for k in range(7)], 600)
    assert groups_of(hs, A, 4) == [(0, 4), (4, 3)]
    # a unit of four is counted as 1.25 steps per step: pairs whose union doubles the steps stay pairs
    A = windows_matrix([range(0, 32), range(0, 32), range(32, 64), range(32, 64)], [0, 8, 16, 24], 600)
    assert groups_of(hs, A, 4) == [(0, 2), (2, 2)]


def test_pairs_follow_the_step_count(hs):
    """With max_windows = 2: a merged pair has fewer steps than its windows apart (or one list),
    and two adjacent windows left alone would not have saved a step."""
    rng = np.random.default_rng(9)
    A = random_csr(rng, 1600, 20000, 2e-5, 0)           # a few entries per window, 79 panels
    b = convert(hs, A)
    g = hs.panel_units_preview(b, 2)
    first, count = g["group_first"], g["group_count"]
    merged = alone = 0
    for i, (f, c) in enumerate(zip(first, count)):
        a = real_ids(b, b["rowOffset"], b["tcA2B"], f)
        if c == 2:
            o = real_ids(b, b["rowOffset"], b["tcA2B"], f + 1)
            u = np.union1d(a, o)
            assert np.array_equal(a, o) or panel_steps(u) < panel_steps(a) + panel_steps(o)
            merged += 1
        elif i + 1 < first.size and count[i + 1] == 1 and b["rowIdx"][f + 1] == b["rowIdx"][f] + 8:
            o = real_ids(b, b["rowOffset"], b["tcA2B"], f + 1)
            assert panel_steps(np.union1d(a, o)) >= panel_steps(a) + panel_steps(o)
            alone += 1
    assert merged > 0 and alone > 0, (merged, alone)


def test_preview_rejects_bad_arguments(hs):
    A = windows_matrix([range(0, 16), range(8, 24)], [0, 8], 600)
    b = convert(hs, A)
    with pytest.raises(hs.HspmmError):
        hs.panel_units_preview(b, 3)
    bad = dict(b, rowIdx=b["rowIdx"][::-1].copy())
    with pytest.raises(hs.HspmmError):
        hs.panel_units_preview(bad, 2)


def test_lists_that_do_not_ascend_or_repeat_an_id_are_never_merged(hs):
    """The gather and all-shapes kernels take any column order; merging windows and the LDS-staging
    stream need strictly ascending lists with padding only behind a window's last column.  A matrix
    that breaks that rule anywhere comes back from the preview unmerged and unchanged."""
    def matrix(lists, cols=400):
        W = len(lists)
        a2b = np.full((W, 16), IDX_MAX, np.uint32)
        data = np.zeros((W, 8, 16), np.uint16)
        for w, ids in enumerate(lists):
            a2b[w, :len(ids)] = ids
            for k in range(len(ids)):
                data[w, (w + k) % 8, k] = encode(np.array([1.0 + k]), 0)[0]
        return dict(rows=8 * W, cols=cols, dtype=0, cw=16, eff_row_windows=W, total_tiles=W,
                    rowOffset=np.arange(W + 1, dtype=np.uint32), rowIdx=8 * np.arange(W, dtype=np.uint32),
                    tcA2B=a2b.ravel(), data=data.ravel())
    for lists in ([[5, 5, 9, 300], [5, 5, 9, 300]],          # a repeated id, both windows alike
                  [[9, 5, 300], [5, 9, 300]],                # descending
                  [[5, 9, 300], [5, 9, 300], [7, 7]]):       # one bad window spoils the plan's merging altogether
        b = matrix(lists)
        g = hs.panel_units_preview(b, 4)
        assert np.array_equal(g["group_count"], np.ones(len(lists), np.uint32)), lists
        assert g["total_tiles"] == b["total_tiles"]
        assert np.array_equal(g["tcA2B"], b["tcA2B"]) and np.array_equal(g["data"], b["data"])
    # the same lists in canonical form do merge
    g = hs.panel_units_preview(matrix([[5, 9, 300], [5, 9, 300]]), 4)
    assert np.array_equal(g["group_count"], [2])
    # padding inside a window (a tile that is not the window's last ends in padding) also keeps it unmerged
    b = matrix([[1, 2, 3], [1, 2, 3]])
    two = dict(b, eff_row_windows=1, total_tiles=2, rowOffset=np.array([0, 2], np.uint32), rowIdx=np.array([0], np.uint32),
               rows=8)
    g = hs.panel_units_preview(two, 4)
    assert np.array_equal(g["group_count"], [1]) and g["total_tiles"] == 2
