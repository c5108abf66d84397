import numpy as np
import pytest

from halite_amd.kernels.attention import plan_items


def check_plan(plan, q_len, kv_len, group, window):
    """Every (row tile, key) pair is covered exactly once; pieces meet on block edges;
    a cut tile has one merge entry per 16 rows whose partial slots are its own."""
    seen = {}
    for rows_per_tile, arr in ((16, plan.items), (plan.rows_big, plan.big_items)):
        for seg, rho0, b, e, partial, *_ in arr.tolist():
            rows = q_len[seg] * group
            assert (rows <= 16 or plan.rows_big == 16) == (rows_per_tile == 16 and arr is plan.items)
            assert 0 <= b < e <= kv_len[seg] and rho0 % rows_per_tile == 0 and rho0 < rows
            seen.setdefault((seg, rho0, rows_per_tile), []).append((b, e, partial))
    for s in range(len(q_len)):
        rows = q_len[s] * group
        per = 16 if rows <= 16 or plan.rows_big == 16 else plan.rows_big
        assert sorted(r for (seg, r, _) in seen if seg == s) == list(range(0, rows, per))
    used_slots = set()
    n_merges = 0
    for (seg, rho0, per), pieces in seen.items():
        rows = q_len[seg] * group
        pos0 = kv_len[seg] - q_len[seg]
        first_q = rho0 // group
        last_q = min(rows - 1, rho0 + per - 1) // group
        lo = max(0, pos0 + first_q - window + 1) if window else 0
        hi = pos0 + last_q + 1
        pieces.sort()
        assert pieces[0][0] == lo and pieces[-1][1] == hi
        for (b0, e0, _), (b1, e1, _) in zip(pieces, pieces[1:]):
            assert e0 == b1 and e0 % 32 == 0
        if len(pieces) == 1:
            assert pieces[0][2] == -1
            continue
        stride = per // 16
        slots = [p for _, _, p in pieces]
        assert slots == list(range(slots[0], slots[0] + stride * len(slots), stride))
        sub_tiles = min(stride, -(-(rows - rho0) // 16))
        for sub in range(sub_tiles):
            match = [m for m in plan.merges.tolist() if m[0] == seg and m[1] == rho0 + 16 * sub]
            assert match == [[seg, rho0 + 16 * sub, slots[0] + sub, len(slots), stride, 0, 0, 0]]
            n_merges += 1
        for s0 in slots:
            for sub in range(stride):
                assert s0 + sub not in used_slots
                used_slots.add(s0 + sub)
    assert n_merges == plan.n_merges
    assert not used_slots or max(used_slots) < plan.n_partials


@pytest.mark.parametrize("rows_big", [64, 16])
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
    # a short portion of a prompt against a long context: few big tiles, so they are cut
    q_len, kv_len = np.array([64]), np.array([20000])
    plan = plan_items(q_len, kv_len, 4, 8, 0)
    assert plan.n_big > 4 and plan.n_merges == 16
    check_plan(plan, q_len, kv_len, 4, 0)
    empty = plan_items(np.array([], dtype=np.int32), np.array([], dtype=np.int32), 4, 8, 0)
    assert empty.n_items == 0 and empty.n_big == 0
