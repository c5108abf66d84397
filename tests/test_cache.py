import random
from dataclasses import dataclass

import numpy as np
import pytest
import torch

from halite_amd.cache import CacheManager, NoSlot, NoSpace, PagePool
from halite_amd.parts.base import PagedKVNeed, PagedNeed, StateNeed

FULL = PagedKVNeed(2, 16)
WIN = PagedKVNeed(2, 16, window=10)


def manager(needs=None, **kw):
    kw.setdefault("page_size", 4)
    kw.setdefault("num_pages", 17)
    kw.setdefault("n_slots", 4)
    return CacheManager(needs or {0: FULL, 1: FULL}, allocate=False, **kw)


def test_page_pool():
    pool = PagePool(5)
    assert pool.capacity == 4 and pool.available == 4
    pages = pool.alloc(3)
    assert 0 not in pages and len(set(pages)) == 3
    with pytest.raises(NoSpace):
        pool.alloc(2)
    assert pool.available == 1  # a failed request takes nothing
    pool.free(pages[:1])
    with pytest.raises(RuntimeError, match="not held"):
        pool.free(pages[:1])  # freed twice
    with pytest.raises(RuntimeError, match="not held"):
        pool.free([0])
    assert set(pool.alloc(2)) & set(pages[1:]) == set()  # held pages are not handed out again


def test_groups_by_need():
    m = manager({0: FULL, 1: WIN, 2: FULL, 3: WIN}, borrowed={4: 1})
    assert len(m.groups) == 2
    assert m.groups[0].runs == [0, 2] and m.groups[1].runs == [1, 3]
    assert m.group_of_run[4] == 1
    with pytest.raises(ValueError, match="owns none"):
        manager({0: FULL}, borrowed={1: 5})


@dataclass(frozen=True)
class OneVectorNeed(PagedNeed):
    """A need that is defined here: one vector a token and a count a page."""

    width: int
    window: int | None = None

    def page_tensors(self, page_size):
        return {"vector": (page_size, self.width), "count": (1,)}

    def bind(self, group_id, tensors, page_size, dtype):
        return {"group": group_id, **tensors}


def test_a_need_says_what_a_page_holds():
    needs = {0: OneVectorNeed(6), 1: FULL, 2: OneVectorNeed(6), 3: OneVectorNeed(6, window=8)}
    m = CacheManager(needs, page_size=4, num_pages=9, n_slots=2, dtype=torch.bfloat16)
    assert [g.runs for g in m.groups] == [[0, 2], [1], [3]]
    assert [tuple(g.storage.shape) for g in m.groups] == [(2, 9 * 25), (1, 9 * 2 * 2 * 4 * 16), (1, 9 * 25)]
    assert CacheManager.bytes_per_page(needs, 4, torch.bfloat16) == (3 * 25 + 2 * 2 * 4 * 16) * 2
    a, b = m.layer_pages(0), m.layer_pages(2)
    assert a["group"] == b["group"] == 0 and m.layer_pages(3)["group"] == 2
    assert tuple(a["vector"].shape) == (9, 4, 6) and tuple(a["count"].shape) == (9, 1)
    # every tensor of every run has memory of its own, inside the group's storage
    a["vector"].fill_(1), a["count"].fill_(2), b["vector"].fill_(3), b["count"].fill_(4)
    assert m.groups[0].storage[0].float().sum() == 9 * 24 * 1 + 9 * 2 and m.groups[0].storage[1].float().sum() == 9 * 24 * 3 + 9 * 4
    kv = m.layer_pages(1)
    assert tuple(kv.k.shape) == (9, 2, 4, 16) and tuple(kv.v.shape) == (9, 2, 16, 4)
    # the books are the same for every kind of page
    s = m.admit()
    m.reserve([(s, 14)])
    m.advance(s, 14)
    assert [sum(p >= 0 for p in g.tables[s]) for g in m.groups] == [4, 4, 3]
    m.check()
    m.free(s)
    assert m.idle()
    m.release_storage()
    assert m.layer_pages(0) is None and m.groups[0].storage is None


def test_reserve_advance_free():
    m = manager()
    s = m.admit()
    assert m.length(s) == 0
    m.reserve([(s, 6)])
    assert m.groups[0].pool.available == 14  # two pages of four tokens
    bt = m.block_table(0, [s])
    assert bt.shape == (1, 2) and (bt > 0).all()
    m.advance(s, 6)
    m.reserve([(s, 8)])  # still inside the second page
    assert m.groups[0].pool.available == 14
    m.advance(s, 8)
    m.reserve([(s, 9)])
    assert m.groups[0].pool.available == 13
    with pytest.raises(ValueError, match="does not extend"):
        m.reserve([(s, 8)])
    m.check()
    m.free(s)
    assert m.idle()
    m.check()


def test_pages_taken_for_tokens_that_did_not_come_are_given_back():
    m = manager({0: FULL, 1: WIN}, num_pages=9)
    a, b = m.admit(), m.admit()
    m.reserve([(a, 6)])
    m.advance(a, 6)
    m.reserve([(a, 9)])  # a step ahead: three more tokens, a page more in each group
    assert [len(g.tables[a]) for g in m.groups] == [3, 3] and m.free_pages() == 5
    with pytest.raises(NoSpace):
        m.reserve([(b, 21)])
    version = m.version
    assert m.release_unused(a) == 1 and m.version > version
    assert [len(g.tables[a]) for g in m.groups] == [2, 2] and m.free_pages() == 6
    assert m.release_unused(a) == 0  # nothing beyond the length is left
    m.reserve([(b, 21)])
    m.check()
    m.reserve([(a, 7)])  # the page that holds token 6 is still there
    m.advance(a, 7)
    m.check()
    m.free(a), m.free(b)
    assert m.idle()


def test_all_or_nothing():
    m = manager(num_pages=5)  # 4 pages of 4 tokens
    a, b = m.admit(), m.admit()
    m.reserve([(a, 8)])
    m.advance(a, 8)
    assert not m.can_reserve([(a, 12), (b, 8)])
    with pytest.raises(NoSpace):
        m.reserve([(a, 12), (b, 8)])
    assert m.groups[0].pool.available == 2 and m.block_table(0, [b]).max() == -1
    m.check()
    m.reserve([(a, 12), (b, 4)])
    assert m.free_pages() == 0


def test_window_pages_come_back():
    m = manager({0: FULL, 1: WIN}, num_pages=33)
    s = m.admit()
    full, win = m.groups
    pos = 0
    for n in [7, 2, 13, 3, 1, 1, 1, 20, 1, 1]:
        m.reserve([(s, pos + n)])
        # every key a query of this portion may read is on a held page
        for q in range(pos, pos + n):
            for j in range(max(0, q - 10 + 1), q + 1):
                assert win.tables[s][j // 4] > 0
        pos += n
        m.advance(s, pos)
        m.check()
        held = [p for p in win.tables[s] if p >= 0]
        assert len(held) <= 10 // 4 + 2  # only the window's pages stay
        assert len([p for p in full.tables[s] if p >= 0]) == -(-pos // 4)
        first = max(0, pos - 10 + 1) // 4
        assert all(p < 0 for p in win.tables[s][:first]) and all(p > 0 for p in win.tables[s][first:])
    m.free(s)
    assert m.idle()


def test_slots_and_state():
    m = CacheManager({0: FULL}, None, {0: {"acc": StateNeed((3,))}}, page_size=4, num_pages=9, n_slots=2, device="cpu")
    a, b = m.admit(), m.admit()
    with pytest.raises(NoSlot):
        m.admit()
    st = m.state_of_run(0)["acc"]
    assert st.shape == (2, 3)
    st[a] += 5
    m.free(a)
    with pytest.raises(RuntimeError, match="not live"):
        m.slots.free(a)
    a2 = m.admit()
    assert a2 == a and float(st[a2].abs().sum()) == 0  # a slot starts from zero
    assert m.layer_pages(0).k.shape == (9, 2, 4, 16) and m.layer_pages(0).v.shape == (9, 2, 16, 4)
    assert m.layer_pages(0).k.data_ptr() != m.layer_pages(0).v.data_ptr()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders(seed):
    """No page lost, held twice or freed twice under random admissions, growth and
    endings, with and without a window, with a pool that keeps running dry."""
    rng = random.Random(seed)
    m = manager({0: FULL, 1: WIN, 2: FULL}, num_pages=rng.choice([9, 13, 21]), n_slots=5)
    live = {}
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.slots.available:
            live[m.admit()] = 0
        elif op < 0.85 and live:
            k = rng.randint(1, min(3, len(live)))
            chosen = rng.sample(sorted(live), k)
            spans = [(s, live[s] + rng.choice([1, 1, 1, 2, 5, 11])) for s in chosen]
            before = [g.pool.available for g in m.groups]
            if m.can_reserve(spans):
                m.reserve(spans)
                for s, n in spans:
                    m.advance(s, n)
                    live[s] = n
            else:
                with pytest.raises(NoSpace):
                    m.reserve(spans)
                assert [g.pool.available for g in m.groups] == before
        elif live:
            s = rng.choice(sorted(live))
            m.free(s)
            del live[s]
        m.check()
        for g in m.groups:
            rows = m.block_table(g.group_id, sorted(live))
            held = rows[rows >= 0]
            assert len(np.unique(held)) == len(held) and (held > 0).all()
    for s in list(live):
        m.free(s)
    assert m.idle()
    m.check()
