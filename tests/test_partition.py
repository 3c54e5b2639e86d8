"""The host-side work partition (hspmm_partition_preview): every tile belongs to
exactly one range, partial-sum slots are consistent with the rule the kernel
applies, and split windows are exactly the windows cut by a range boundary."""
import numpy as np
import pytest

NO = 0xFFFFFFFF


def simulate(ranges, ro):
    """Walk each range the way the kernel does; returns {window: [slots in range order]}
    and the set of windows stored directly."""
    partial, direct = {}, []
    for t0, t1, w, head, tail in ranges.tolist():
        assert ro[w] <= t0 < ro[w + 1]
        t = t0
        while t < t1:
            ws, we = int(ro[w]), int(ro[w + 1])
            se = min(we, t1)
            if t == ws and se == we:
                direct.append(w)
            else:
                slot = head if t == t0 else tail
                assert slot != NO
                partial.setdefault(w, []).append(slot)
            t = se
            if se == we:
                w += 1
    return partial, direct


def check(hs, ro, target, group_offset=None):
    ro = np.asarray(ro, np.uint32)
    p = hs.partition_preview(ro, target, group_offset=group_offset)
    r = p["ranges"]
    W, T = ro.size - 1, int(ro[-1])
    assert r[0, 0] == 0 and r[-1, 1] == T
    assert np.array_equal(r[1:, 0], r[:-1, 1]) and np.all(r[:, 1] > r[:, 0])     # exact cover, no empty range
    assert len(r) <= max(1, target)
    partial, direct = simulate(r, ro)
    slots = [s for w in sorted(partial) for s in partial[w]]
    assert sorted(slots) == list(range(p["n_partial_slots"]))                     # each slot used once
    assert p["n_split_windows"] == len(partial)
    assert sorted(direct + list(partial)) == list(range(W))                       # every window finished once
    assert all(len(v) >= 2 for v in partial.values())
    used = set(r[:, 3].tolist()) | set(r[:, 4].tolist())
    used.discard(NO)
    assert used == set(slots)
    return p


def test_partition_small_cases(hs):
    check(hs, [0, 1], 1)
    check(hs, [0, 1], 8)
    check(hs, [0, 100], 7)                      # one window cut into pieces
    check(hs, [0, 1, 2, 40, 41], 4)
    check(hs, np.arange(0, 1001), 16)           # 1000 one-tile windows: cuts snap, nothing split
    p = check(hs, np.arange(0, 1001), 16)
    assert p["n_split_windows"] == 0


def test_partition_random(hs):
    rng = np.random.default_rng(0)
    for _ in range(60):
        W = int(rng.integers(1, 400))
        tiles = np.maximum(1, rng.pareto(1.2, W) * rng.integers(1, 8)).astype(np.int64)
        ro = np.concatenate([[0], np.cumsum(tiles)])
        check(hs, ro, int(rng.integers(1, 300)))


def test_partition_that_keeps_the_cuts_of_the_callers_groups(hs):
    """hspmm_set_group_cuts(1): a window is cut only where one of the caller's groups ends (groupOffset of
    GBTCF_MTX, reference src/utils/convert.h:245-259); windows given as one group are never cut."""
    rng = np.random.default_rng(3)
    for trial in range(40):
        W = int(rng.integers(1, 200))
        tiles = np.maximum(1, rng.pareto(1.0, W) * rng.integers(1, 30)).astype(np.int64)
        ro = np.concatenate([[0], np.cumsum(tiles)]).astype(np.uint32)
        tgl = int(rng.integers(1, 40))
        # the reference's grouping: every window in pieces of tgl tiles
        go = np.unique(np.concatenate([np.arange(a, b, tgl) for a, b in zip(ro[:-1], ro[1:])] + [ro[-1:]]))
        target = int(rng.integers(1, 300))
        p = check(hs, ro, target, group_offset=go)
        starts = p["ranges"][:, 0]
        assert np.isin(starts, go).all()
        # no further from the balanced cut than half a group: ranges stay balanced to within one group
        free = hs.partition_preview(ro, target)["ranges"]
        ln = (p["ranges"][:, 1] - p["ranges"][:, 0]).astype(np.int64)
        assert ln.max() <= (free[:, 1] - free[:, 0]).max() + tgl
    # groups = windows: nothing is cut, however heavy the window
    ro = np.array([0, 1000, 1001, 1002], np.uint32)
    p = check(hs, ro, 64, group_offset=ro)
    assert p["n_split_windows"] == 0 and len(p["ranges"]) <= 3
    assert check(hs, ro, 64)["n_split_windows"] == 1
    # a window boundary that is not the end of a group is refused
    with pytest.raises(hs.HspmmError):
        hs.partition_preview(ro, 4, group_offset=np.array([0, 500, 1002], np.uint32))
    with pytest.raises(hs.HspmmError):
        hs.partition_preview(ro, 4, group_offset=np.array([0, 1000, 1000, 1001, 1002], np.uint32))


def test_partition_balance_on_power_law(hs):
    from hopper_spmm_amd import generators as G
    A = G.rmat(16, 16, seed=5)
    b = hs.csr_to_btcf(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], 0)
    p = check(hs, b["rowOffset"], 1024)
    ln = (p["ranges"][:, 1] - p["ranges"][:, 0]).astype(np.int64)
    assert ln.max() <= 2.0 * ln.mean()          # no range is more than twice the mean
    assert p["n_partial_slots"] <= 2 * len(ln)


def test_partition_rejects_bad_offsets(hs):
    with pytest.raises(hs.HspmmError):
        hs.partition_preview(np.array([0, 5, 5], np.uint32), 4)
    with pytest.raises(hs.HspmmError):
        hs.partition_preview(np.array([1, 5], np.uint32), 4)


def simulate_grouped(ranges, ro, group):
    """The kernel's rule with workgroups of `group` waves: a wave whose range has the combine
    mark keeps its sums; wave 0 of the workgroup stores the workgroup's total in its head slot."""
    partial, direct = {}, []
    for i, (t0, t1, w, head, tail, combine) in enumerate(ranges.tolist()):
        assert ro[w] <= t0 < ro[w + 1]
        if combine:
            mates = ranges[i - i % group: i - i % group + group]
            assert len(mates) == group and np.all(mates[:, 5] == 1) and np.all(mates[:, 2] == w)
            assert ro[w] <= t0 and t1 <= ro[w + 1] and (t0, t1) != (ro[w], ro[w + 1])   # one piece of one window
            assert tail == NO
            if i % group == 0:
                assert head != NO
                partial.setdefault(w, []).append(head)
            else:
                assert head == NO
            continue
        t = t0
        while t < t1:
            ws, we = int(ro[w]), int(ro[w + 1])
            se = min(we, t1)
            if t == ws and se == we:
                direct.append(w)
            else:
                slot = head if t == t0 else tail
                assert slot != NO
                partial.setdefault(w, []).append(slot)
            t = se
            if se == we:
                w += 1
    return partial, direct


@pytest.mark.parametrize("group", [2, 3, 4])
def test_partition_with_sums_added_per_workgroup(hs, group):
    rng = np.random.default_rng(group)
    cases = [np.array([0, 100]), np.array([0, 1, 2, 400, 401]), np.arange(0, 1001),
             np.concatenate([[0], np.cumsum(rng.integers(1, 600, 64))]),
             np.concatenate([[0], np.cumsum(np.minimum(5000, np.floor(rng.pareto(1.2, 300)) + 1).astype(np.int64))])]
    for ro in cases:
        ro = np.asarray(ro, np.uint32)
        for target in (1, 5, 16, 64, 255):
            plain = hs.partition_preview(ro, target)
            p = hs.partition_preview(ro, target, group=group)
            r = p["ranges"]
            assert np.array_equal(r[:, :3], plain["ranges"][:, :3])                   # the same cuts
            partial, direct = simulate_grouped(r, ro, group)
            slots = [s for w in sorted(partial) for s in partial[w]]
            assert sorted(slots) == list(range(p["n_partial_slots"]))
            assert p["n_split_windows"] == len(partial)
            assert sorted(direct + list(partial)) == list(range(ro.size - 1))
            assert p["n_partial_slots"] <= plain["n_partial_slots"]
            # slots of a window appear in range order
            for w, sl in partial.items():
                assert sl == sorted(sl)
    # a long window cut into many pieces: whole workgroups inside it share one slot each
    p = hs.partition_preview(np.array([0, 4096], np.uint32), 64, group=4)
    assert p["n_partial_slots"] == 16 and np.all(p["ranges"][:, 5] == 1)


def test_aligned_partition_cuts_every_window_into_the_ranges_of_one_workgroup(hs):
    """Every window becomes `group` contiguous ranges of nearly equal length that cover it exactly; no
    range has a slot (the workgroup stores the window itself); windows too short for it are refused."""
    rng = np.random.default_rng(4)
    for group in (4, 8):
        tiles = rng.integers(group, 700, 300)
        ro = np.concatenate([[0], np.cumsum(tiles)]).astype(np.uint32)
        r = hs.partition_preview_aligned(ro, group)
        assert r.shape == (300 * group, 6)
        assert (r[:, 5] == 2).all() and (r[:, 3] == 0xFFFFFFFF).all() and (r[:, 4] == 0xFFFFFFFF).all()
        assert r[0, 0] == 0 and r[-1, 1] == ro[-1]
        assert np.array_equal(r[1:, 0], r[:-1, 1])                      # contiguous, nothing skipped
        per = r.reshape(300, group, 6)
        assert np.array_equal(per[:, 0, 0], ro[:-1]) and np.array_equal(per[:, -1, 1], ro[1:])
        assert (per[:, :, 2] == np.arange(300)[:, None]).all()
        lengths = (per[:, :, 1] - per[:, :, 0]).astype(np.int64)
        assert lengths.min() >= 1 and (lengths.max(axis=1) - lengths.min(axis=1) <= 1).all()
    with pytest.raises(hs.HspmmError):
        hs.partition_preview_aligned(np.array([0, 3, 40], np.uint32), 4)    # a window of three tiles
    with pytest.raises(hs.HspmmError):
        hs.partition_preview_aligned(np.array([0, 30, 60], np.uint32), 3)
