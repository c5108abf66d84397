import numpy as np
import pytest

from halite_amd.kernels.attention import plan_items


def check_plan(plan, q_len, kv_len, group, window):
    """Every 16-row tile belongs to exactly one item group; the pieces of a group are
    contiguous, meet on block edges and cover every key that any of its tiles may see;
    a cut group has one merge entry per tile whose partial slots are its own."""
    per_item = max(1, plan.rows_big // 16)
    groups = {}
    # the long segments' items come in runs of four (a workgroup's waves): one segment per
    # run, padded with items that have no rows and no keys
    assert plan.n_big % 4 == 0
    for r in range(0, plan.n_big, 4):
        run = plan.big_items[r : r + 4]
        assert len(set(run[:, 0].tolist())) == 1 and run[0, 1] >= 0
    # the long segments' items are 16 wide: after the eight, the segment's first token, tokens
    # and keys, and the first and end key that the run of four walks together
    for r in range(0, plan.n_big, 4):
        run = plan.big_items[r : r + 4]
        seg = int(run[0, 0])
        live = run[run[:, 3] > run[:, 2]]
        assert (run[:, 8:11] == [int(sum(q_len[:seg])), int(q_len[seg]), int(kv_len[seg])]).all()
        assert (run[:, 11] == live[:, 2].min()).all() and (run[:, 12] == live[:, 3].max()).all()
        assert (run[:, 13:] == 0).all()
    for arr, is_big in ((plan.items, False), (plan.big_items[:, :8], True)):
        for seg, rho0, b, e, partial, *more in arr.tolist():
            if is_big and rho0 < 0:
                assert (b, e, partial, more) == (0, 0, -1, [-1, -1, -1])
                continue
            rows = q_len[seg] * group
            assert (rows > 16 and per_item > 1) == is_big
            assert 0 <= b < e <= kv_len[seg]
            tiles = tuple([rho0] + [m for m in more[: per_item - 1] if m >= 0]) if is_big else (rho0,)
            if not is_big:  # the segment's first token, tokens and keys ride along
                assert more == [int(sum(q_len[:seg])), int(q_len[seg]), int(kv_len[seg])]
            assert all(t % 16 == 0 and 0 <= t < rows for t in tiles)
            groups.setdefault((seg, tiles), []).append((b, e, partial))
    for s in range(len(q_len)):
        rows = q_len[s] * group
        tiles = sorted(t for (seg, ts) in groups for t in ts if seg == s)
        assert tiles == list(range(0, rows, 16))
    used_slots = set()
    n_merges = 0
    for (seg, tiles), pieces in groups.items():
        rows = q_len[seg] * group
        pos0 = kv_len[seg] - q_len[seg]
        lo = hi = None
        for t in tiles:
            first_q, last_q = t // group, min(rows - 1, t + 15) // group
            t_lo = max(0, pos0 + first_q - window + 1) if window else 0
            t_hi = pos0 + last_q + 1
            lo = t_lo if lo is None else min(lo, t_lo)
            hi = t_hi if hi is None else max(hi, t_hi)
        pieces.sort()
        assert pieces[0][0] == lo and pieces[-1][1] == hi
        for (b0, e0, _), (b1, e1, _) in zip(pieces, pieces[1:]):
            assert e0 == b1 and e0 % 32 == 0
        if len(pieces) == 1:
            assert pieces[0][2] == -1
            continue
        stride = per_item if len(tiles) > 1 or rows > 16 and per_item > 1 else 1
        slots = [p for _, _, p in pieces]
        assert slots == list(range(slots[0], slots[0] + stride * len(slots), stride))
        for sub, t in enumerate(tiles):
            match = [m for m in plan.merges.tolist() if m[0] == seg and m[1] == t]
            assert match == [[seg, t, slots[0] + sub, len(slots), stride,
                              int(sum(q_len[:seg])), int(q_len[seg]), 0]]
            n_merges += 1
        for s0 in slots:
            for sub in range(stride):
                assert s0 + sub not in used_slots
                used_slots.add(s0 + sub)
    assert n_merges == plan.n_merges
    assert not used_slots or max(used_slots) < plan.n_partials


@pytest.mark.parametrize("rows_big", [64, 32, 16])
@pytest.mark.parametrize("window", [0, 7, 100])
@pytest.mark.parametrize("group", [1, 3, 4, 20])
def test_every_row_and_key_is_covered_once(group, window, rows_big):
    q_len = np.array([1, 1, 37, 2, 300, 1], dtype=np.int32)
    kv_len = q_len + np.array([0, 5000, 0, 91, 470, 63], dtype=np.int32)
    plan = plan_items(q_len, kv_len, group, 2, window, rows_big)
    check_plan(plan, q_len, kv_len, group, window)


def test_long_decode_is_split_and_prefill_is_not():
    plan = plan_items(np.array([1] * 8), np.array([8192] * 8), 4, 8, 0)
    assert plan.n_merges == 8 and plan.n_items > 8 * 4 and plan.n_big == 0
    plan = plan_items(np.array([2048]), np.array([2048]), 4, 8, 0)
    assert plan.n_merges == 0 and plan.n_big == 2048 * 4 // 64 and plan.n_items == 0
    # neighbouring tiles ride together
    pair = plan_items(np.array([2048]), np.array([2048]), 4, 8, 0, 32)
    assert pair.n_big == 256 and (pair.big_items[:, 5] == pair.big_items[:, 1] + 16).all()
    assert sorted(pair.big_items[:, 1].tolist() + pair.big_items[:, 5].tolist()) == list(range(0, 8192, 16))
    # a short portion of a prompt against a long context: few big tiles, so they are cut
    q_len, kv_len = np.array([64]), np.array([20000])
    plan = plan_items(q_len, kv_len, 4, 8, 0)
    assert plan.n_big > 4 and plan.n_merges == 16
    check_plan(plan, q_len, kv_len, 4, 0)
    empty = plan_items(np.array([], dtype=np.int32), np.array([], dtype=np.int32), 4, 8, 0)
    assert empty.n_items == 0 and empty.n_big == 0
