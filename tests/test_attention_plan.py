import numpy as np
import pytest

from halite_amd.kernels.attention import plan_items


@pytest.mark.parametrize("window", [0, 7, 100])
@pytest.mark.parametrize("group", [1, 3, 4, 20])
def test_every_row_and_key_is_covered_once(group, window):
    rng = np.random.default_rng(group * 100 + window)
    q_len = np.array([1, 1, 37, 2, 300, 1], dtype=np.int32)
    kv_len = q_len + np.array([0, 5000, 0, 91, 470, 63], dtype=np.int32)
    plan = plan_items(q_len, kv_len, group, 2, window)
    assert plan.items.shape == (plan.n_items, 8) and plan.merges.shape == (plan.n_merges, 4)
    seen = {}
    for seg, rho0, b, e, partial, *_ in plan.items.tolist():
        assert 0 <= b < e <= kv_len[seg] and rho0 % 16 == 0 and rho0 < q_len[seg] * group
        seen.setdefault((seg, rho0), []).append((b, e, partial))
    for s in range(len(q_len)):
        rows = q_len[s] * group
        assert sorted(r for (seg, r) in seen if seg == s) == list(range(0, rows, 16))
    n_partials = 0
    for (seg, rho0), pieces in seen.items():
        pos0 = kv_len[seg] - q_len[seg]
        first_q = rho0 // group
        last_q = min(q_len[seg] * group - 1, rho0 + 15) // group
        lo = max(0, pos0 + first_q - window + 1) if window else 0
        hi = pos0 + last_q + 1
        pieces.sort()
        assert pieces[0][0] == lo and pieces[-1][1] == hi
        for (b0, e0, _), (b1, e1, _) in zip(pieces, pieces[1:]):
            assert e0 == b1 and e0 % 32 == 0  # pieces meet on block edges
        if len(pieces) == 1:
            assert pieces[0][2] == -1
        else:
            ids = [p for _, _, p in pieces]
            assert ids == list(range(ids[0], ids[0] + len(ids)))
            n_partials += len(ids)
            match = [m for m in plan.merges.tolist() if m[0] == seg and m[1] == rho0]
            assert match == [[seg, rho0, ids[0], len(ids)]]
    assert n_partials == plan.n_partials
    assert plan.n_merges == sum(1 for p in seen.values() if len(p) > 1)


def test_long_decode_is_split_and_prefill_is_not():
    plan = plan_items(np.array([1] * 8), np.array([8192] * 8), 4, 8, 0)
    assert plan.n_merges == 8 and plan.n_items > 8 * 4
    plan = plan_items(np.array([2048]), np.array([2048]), 4, 8, 0)
    assert plan.n_merges == 0 and plan.n_items == 2048 * 4 // 16
    assert plan_items(np.array([], dtype=np.int32), np.array([], dtype=np.int32), 4, 8, 0).n_items == 0
