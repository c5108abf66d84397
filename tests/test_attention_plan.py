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
    # the one-tile items come in runs of four too: a piece of one tile's key range cut in four
    # (some may be empty, the first never is), which the kernel joins into one result
    assert plan.n_items % 4 == 0
    for r in range(0, plan.n_items, 4):
        run = plan.items[r : r + 4]
        assert len(set(map(tuple, run[:, [0, 1, 4, 5, 6, 7, 8, 9]].tolist()))) == 1 and (run[:, 10:] == 0).all()
        live = run[run[:, 3] > run[:, 2]]
        assert run[0, 3] > run[0, 2] and (live[1:, 2] == live[:-1, 3]).all() and (live[:-1, 3] % 32 == 0).all()
        # an empty quarter names the piece's first key twice: a key whose page is held
        assert (run[run[:, 3] <= run[:, 2], 2:4] == run[0, 2]).all()
        blocks = -(-(live[:, 3] - live[:, 2] // 32 * 32) // 32)
        assert blocks.max() - blocks.min() <= 1 or len(live) < 4
    in_kernel = {}  # (segment, tile) -> (first partial slot, pieces) that the items themselves name
    for seg, rho0, first, n in plan.items[:, [0, 1, 8, 9]].tolist():
        assert n != 1 and (n > 1 or first == 0)
        if n > 1:
            assert in_kernel.setdefault((seg, (rho0,)), (first, n)) == (first, n)
    for arr, is_big in ((plan.items[:, :8], False), (plan.big_items[:, :8], True)):
        for seg, rho0, b, e, partial, *more in arr.tolist():
            if is_big and rho0 < 0:
                assert (b, e, partial, more) == (0, 0, -1, [-1, -1, -1])
                continue
            if not is_big and b == e:  # an empty quarter of a short piece
                pos0 = kv_len[seg] - q_len[seg]
                first_seen = 0 if window <= 0 else max(0, pos0 + rho0 // group - window + 1)
                assert first_seen <= b < kv_len[seg]  # inside the window: its page is held
                continue
            rows = q_len[seg] * group
            assert (rows > 16 and q_len[seg] > 1 and per_item > 1) == is_big
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
        if len(tiles) == 1 and (rows <= 16 or q_len[seg] == 1 or per_item == 1):  # the quarters of a piece share its slot
            whole = []
            for b, e, p in pieces:
                if whole and whole[-1][2] == p and (p >= 0 or whole[-1][1] == b):
                    whole[-1] = (whole[-1][0], e, p)
                else:
                    whole.append((b, e, p))
            pieces = whole
            assert all(e - b >= 352 for b, e, _ in pieces) or len(pieces) == 1
        assert pieces[0][0] == lo and pieces[-1][1] == hi
        for (b0, e0, _), (b1, e1, _) in zip(pieces, pieces[1:]):
            assert e0 == b1 and e0 % 32 == 0
        if len(pieces) == 1:
            assert pieces[0][2] == -1
            continue
        stride = per_item if len(tiles) > 1 or rows > 16 and q_len[seg] > 1 and per_item > 1 else 1
        slots = [p for _, _, p in pieces]
        assert slots == list(range(slots[0], slots[0] + stride * len(slots), stride))
        if (seg, tiles) in in_kernel:  # merged by the attention kernel: no merge entry
            assert in_kernel.pop((seg, tiles)) == (slots[0], len(slots)) and len(slots) <= 8
            assert not [m for m in plan.merges.tolist() if m[0] == seg and m[1] == tiles[0]]
            assert not used_slots & set(slots)
            used_slots.update(slots)
            continue
        for sub, t in enumerate(tiles):
            match = [m for m in plan.merges.tolist() if m[0] == seg and m[1] == t]
            assert match == [[seg, t, slots[0] + sub, len(slots), stride,
                              int(sum(q_len[:seg])), int(q_len[seg]), 0]]
            n_merges += 1
        for s0 in slots:
            for sub in range(stride):
                assert s0 + sub not in used_slots
                used_slots.add(s0 + sub)
    assert n_merges == plan.n_merges and not in_kernel
    assert plan.merged_in_kernel == bool((plan.items[:, 9] > 1).any())
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
    # eight requests, eight key/value heads: four pieces each fill the 256 compute units
    plan = plan_items(np.array([1] * 8), np.array([8192] * 8), 4, 8, 0)
    assert plan.n_merges == 0 and plan.n_items == 8 * 4 * 4 and plan.n_partials == 32 and plan.n_big == 0
    assert plan.merged_in_kernel and (plan.items[:, 9] == 4).all()  # the kernel merges a tile's four itself
    assert plan.items[:4, [2, 3, 4, 8]].tolist() == [[0, 512, 0, 0], [512, 1024, 0, 0], [1024, 1536, 0, 0], [1536, 2048, 0, 0]]
    assert sorted(set(plan.items[:, 8].tolist())) == [0, 4, 8, 12, 16, 20, 24, 28]
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


def test_the_pieces_of_decode_tokens_key_ranges():
    from halite_amd.kernels.attention import pieces_per_tile

    # short ranges stay whole: one workgroup, its four waves a quarter each, nothing to merge
    plan = plan_items(np.array([1] * 8), np.array([570] * 8), 4, 8, 0)
    assert plan.n_items == 32 and plan.n_merges == 0 and plan.n_partials == 0
    assert plan.items[:4, 2:5].tolist() == [[0, 160, -1], [160, 288, -1], [288, 448, -1], [448, 570, -1]]
    # few keys: some quarters are empty
    plan = plan_items(np.array([1]), np.array([40]), 4, 8, 0)
    assert plan.items[:, 2:4].tolist() == [[0, 32], [0, 0], [32, 40], [0, 0]]
    # no piece under 384 keys, whatever room there is
    assert plan_items(np.array([1]), np.array([767]), 4, 8, 0).n_items == 4
    plan = plan_items(np.array([1]), np.array([1200]), 4, 8, 0)
    assert plan.n_items == 12 and plan.items[:, 4].tolist() == [0] * 4 + [1] * 4 + [2] * 4
    assert plan.merges.tolist() == [[0, 0, 0, 3, 1, 0, 1, 0]] and (plan.items[:, 8:10] == 0).all()  # (one tile could have 32 pieces)
    plan = plan_items(np.array([1] * 4), np.array([1200, 50, 50, 50]), 4, 8, 0)
    assert plan.n_items == 12 + 3 * 4 and plan.n_merges == 0 and (plan.items[:12, 8:10] == [0, 3]).all()
    # as many pieces as fill the compute units once, and none where the tiles alone do
    assert [pieces_per_tile(n, 8) for n in (1, 2, 3, 8, 12, 16, 24, 32, 64)] == [32, 16, 10, 4, 2, 2, 1, 1, 1]
    assert pieces_per_tile(1, 1) == 256 and pieces_per_tile(0, 8) == 256
    plan = plan_items(np.array([1] * 64), np.array([30000] * 64), 4, 8, 0)
    assert plan.n_items == 256 and plan.n_merges == 0
    plan = plan_items(np.array([1] * 4), np.array([131072] * 4), 4, 8, 0)
    assert plan.n_items == 128 and (plan.items[:, 9] == 8).all() and plan.n_merges == 0
    # more pieces than the attention kernel merges itself: they are the merge kernel's
    plan = plan_items(np.array([1]), np.array([131072]), 4, 2, 0)
    assert plan.n_items == 4 * 128 and not plan.merged_in_kernel and (plan.items[:, 8:] == 0).all()
    assert plan.merges.tolist() == [[0, 0, 0, 128, 1, 0, 1, 0]]
    for kv_heads in (1, 2, 8):
        q_len, kv_len = np.array([1, 2, 1]), np.array([40000, 9000, 300])
        check_plan(plan_items(q_len, kv_len, 4, kv_heads, 0), q_len, kv_len, 4, 0)
        check_plan(plan_items(q_len, kv_len, 4, kv_heads, 5000), q_len, kv_len, 4, 5000)
        q_len, kv_len = np.array([1, 2, 1, 1, 1]), np.array([40000, 9000, 300, 2000, 767])
        plan = plan_items(q_len, kv_len, 4, kv_heads, 0)
        assert plan.merged_in_kernel == (kv_heads == 8) and (plan.n_merges == 0) == (kv_heads == 8)
        check_plan(plan, q_len, kv_len, 4, 0)
        check_plan(plan_items(q_len, kv_len, 4, kv_heads, 5000), q_len, kv_len, 4, 5000)
    # a mixed step: the decode tokens' pieces do not depend on the prompt portion beside them
    mixed = plan_items(np.array([1, 700, 1]), np.array([5000, 700, 5000]), 4, 8, 0)
    alone = plan_items(np.array([1, 1]), np.array([5000, 5000]), 4, 8, 0)
    assert (mixed.items[:, 2:5] == alone.items[:, 2:5]).all() and mixed.n_big > 0


def test_random_steps_are_covered():
    """Random mixes of decode tokens and prompt portions, contexts from nothing to 200,000
    keys, any head grouping and window: every plan passes the same checks."""
    rng = np.random.default_rng(7)
    for case in range(300):
        n_seg = int(rng.integers(1, 40))
        kinds = rng.integers(0, 4, n_seg)
        q_len = np.where(kinds == 0, rng.integers(1, 4, n_seg), np.where(kinds == 1, 1, rng.integers(1, 600, n_seg)))
        q_len = np.where(kinds == 3, 1, q_len).astype(np.int32)
        before = np.where(rng.random(n_seg) < 0.3, 0, rng.integers(0, int(rng.choice([50, 900, 5000, 200000])), n_seg))
        kv_len = (q_len + before).astype(np.int32)
        group = int(rng.choice([1, 2, 3, 4, 8, 20]))
        kv_heads = int(rng.choice([1, 2, 8]))
        window = int(rng.choice([0, 0, 1, 37, 1000, 5000]))
        rows_big = int(rng.choice([16, 32, 64]))
        plan = plan_items(q_len, kv_len, group, kv_heads, window, rows_big)
        try:
            check_plan(plan, q_len, kv_len, group, window)
        except AssertionError as e:
            raise AssertionError(f"case {case}: q {q_len.tolist()} kv {kv_len.tolist()} group {group} kv heads {kv_heads} "
                                 f"window {window} rows {rows_big}") from e


def test_recorded_decode_steps_have_room_for_any_lengths():
    """A decode step that is replayed from a graph has the launches and the room of the step
    it was recorded with; whatever the requests' lengths later are, the plan fits that room
    and merges its pieces the same way."""
    from halite_amd.kernels.attention import fix_room_for_decode

    rng = np.random.default_rng(3)
    for case in range(400):
        n = int(rng.integers(1, 70))
        group, kv_heads = int(rng.choice([1, 2, 4, 8, 16, 20, 40])), int(rng.choice([1, 2, 8]))
        window = int(rng.choice([0, 0, 500]))
        first = plan_items(np.ones(n, dtype=np.int32), np.ones(n, dtype=np.int32), group, kv_heads, window)
        fix_room_for_decode(first, n, group, kv_heads)
        kv_len = rng.integers(1, int(rng.choice([40, 2000, 200000])), n).astype(np.int32)
        plan = plan_items(np.ones(n, dtype=np.int32), kv_len, group, kv_heads, window)
        assert plan.n_big == 0 and plan.n_items <= first.cap_items and plan.n_items % 4 == 0
        assert plan.n_merges <= first.cap_merges and plan.n_partials <= first.cap_partials
        assert plan.max_parts <= first.max_parts
        if plan.n_partials:  # some range is cut: by the kernel itself or by the merge kernel, as recorded
            assert plan.merged_in_kernel == first.merged_in_kernel and (plan.n_merges > 0) == (first.cap_merges > 0)
