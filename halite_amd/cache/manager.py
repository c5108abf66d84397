"""The cache manager: groups of pages, block tables, slots and per-request state.

Everything here is host bookkeeping except the page storage and the state rows.  A
step asks for room for its tokens first (all groups or none), runs, then advances
the requests' lengths, at which point windowed groups give back the pages that have
been passed.  When a request ends, all its pages and its slot return.  The idle
invariant is the reference's ``check_memory``
(src/halite/transformers/infer/engine/scheduler.py:109-123): every page but the
reserved one is free and every slot is free.
"""

from __future__ import annotations

import sys

import numpy as np
import torch

from ..parts.base import PagedNeed, StateNeed
from .pages import CacheGroup, NoSpace, PagePool
from .slots import SlotAllocator, StateStore


class CacheManager:
    def __init__(
        self,
        needs: dict[int, PagedNeed],
        borrowed: dict[int, int] | None = None,
        state_needs: dict[int, dict[str, StateNeed]] | None = None,
        *,
        page_size: int,
        num_pages: int,
        n_slots: int,
        dtype: torch.dtype = torch.float32,
        device="cpu",
        allocate: bool = True,
    ):
        """``needs[run]`` for every run that owns a cache; ``borrowed[run] = owner``
        for runs that read another run's cache; ``num_pages`` counts the reserved
        page 0 of each group."""
        self.page_size = page_size
        self.num_pages = num_pages
        self.dtype = dtype
        self.device = torch.device(device)
        self.groups: list[CacheGroup] = []
        self.group_of_run: dict[int, int] = {}
        by_need: dict[PagedNeed, CacheGroup] = {}
        for run in sorted(needs):
            need = needs[run]
            if need not in by_need:
                g = CacheGroup(len(self.groups), need, [], page_size, PagePool(num_pages))
                by_need[need] = g
                self.groups.append(g)
            by_need[need].runs.append(run)
            self.group_of_run[run] = by_need[need].group_id
        self.borrowed = dict(borrowed or {})
        for run, owner in self.borrowed.items():
            if owner not in self.group_of_run:
                raise ValueError(f"run {run} borrows the cache of run {owner}, which owns none")
            self.group_of_run[run] = self.group_of_run[owner]
        # what a run's mixer finds in ``run.kv``: the need says which tensors a page number
        # stands for and binds them; a run's tensors lie one after the other in the group's
        # storage, each ``[pages, *shape]``
        self._pages: dict[int, object] = {}
        for g in self.groups:
            shapes = g.need.page_tensors(page_size)
            sizes = {name: int(np.prod(shape)) for name, shape in shapes.items()}
            if allocate:
                g.storage = torch.zeros((len(g.runs), num_pages * sum(sizes.values())), dtype=dtype, device=self.device)
            for i, run in enumerate(g.runs):
                tensors, at = {}, 0
                for name, shape in shapes.items():
                    n = num_pages * sizes[name]
                    tensors[name] = g.storage[i, at : at + n].view(num_pages, *shape) if allocate else None
                    at += n
                self._pages[run] = g.need.bind(g.group_id, tensors, page_size, dtype)
        for run, owner in self.borrowed.items():
            self._pages[run] = self._pages[owner]
        self.slots = SlotAllocator(n_slots)
        self.state = StateStore(n_slots, state_needs or {}, self.device if allocate else "cpu")
        self.lengths: dict[int, int] = {}
        self.version = 0  # counts every change of slots, lengths and pages

    # -- sizes ------------------------------------------------------------------
    @staticmethod
    def bytes_per_page(needs: dict[int, PagedNeed], page_size: int, dtype: torch.dtype) -> int:
        """Bytes that one page number costs over all groups and runs."""
        return sum(int(np.prod(shape)) * dtype.itemsize for n in needs.values() for shape in n.page_tensors(page_size).values())

    @property
    def token_capacity(self) -> int:
        return (self.num_pages - 1) * self.page_size

    def free_pages(self) -> int:
        """Free pages of the tightest group; a model without paged layers has no page to
        run out of, which the largest integer stands for."""
        return min((g.pool.available for g in self.groups), default=sys.maxsize)

    def layer_pages(self, run: int):
        return self._pages.get(run)

    def state_of_run(self, run: int) -> dict[str, torch.Tensor]:
        return self.state.tensors.get(run, {})

    def release_storage(self) -> None:
        """Drops the device memory of pages and state rows (the bookkeeping stays); the
        manager serves no step afterwards."""
        for g in self.groups:
            g.storage = None
        self._pages = {}  # (whoever took a run's pages from ``layer_pages`` lets go of them too)
        self.state.tensors = {}

    # -- requests -----------------------------------------------------------------
    def admit(self) -> int:
        self.version += 1
        slot = self.slots.alloc()
        self.lengths[slot] = 0
        self.state.reset(slot)
        return slot

    def length(self, slot: int) -> int:
        return self.lengths[slot]

    def pages_missing(self, spans: list[tuple[int, int]]) -> list[int]:
        """Per group, the pages that ``reserve`` would take for ``(slot, new
        length)`` spans (each span starts at the slot's current length)."""
        return [
            sum(g.pages_missing(slot, self.lengths[slot], new_len) for slot, new_len in spans)
            for g in self.groups
        ]

    def can_reserve(self, spans: list[tuple[int, int]]) -> bool:
        return all(m <= g.pool.available for m, g in zip(self.pages_missing(spans), self.groups))

    def reserve(self, spans: list[tuple[int, int]]) -> None:
        """Room for every span in every group, or ``NoSpace`` and nothing taken."""
        for slot, new_len in spans:
            if new_len <= self.lengths[slot]:
                raise ValueError(f"slot {slot}: new length {new_len} does not extend {self.lengths[slot]}")
        missing = self.pages_missing(spans)
        for m, g in zip(missing, self.groups):
            if m > g.pool.available:
                raise NoSpace(f"group {g.group_id}: {m} pages wanted, {g.pool.available} free")
        self.version += 1
        for g in self.groups:
            for slot, new_len in spans:
                g.reserve(slot, self.lengths[slot], new_len)

    def advance(self, slot: int, new_len: int) -> None:
        """The tokens up to ``new_len`` are in the cache now."""
        self.version += 1
        self.lengths[slot] = new_len
        for g in self.groups:
            g.release_passed(slot, new_len)

    def release_unused(self, slot: int) -> int:
        """Gives back what ``reserve`` took for ``slot`` beyond its length (a step that was
        prepared and did not come); returns the pages of the tightest group that this freed."""
        freed = [g.release_beyond(slot, self.lengths[slot]) for g in self.groups]
        if any(freed):
            self.version += 1
        return min(freed, default=0)

    def free(self, slot: int) -> None:
        self.version += 1
        for g in self.groups:
            g.release_all(slot)
        del self.lengths[slot]
        self.slots.free(slot)

    # -- what a step reads ----------------------------------------------------------
    def block_table(self, group_id: int, slots: list[int], width: int | None = None) -> np.ndarray:
        """``[len(slots), P]`` int32, row i the page list of ``slots[i]``, -1 where
        the request holds no page.  ``P`` is the longest list unless ``width`` fixes it."""
        g = self.groups[group_id]
        if width is None:
            width = max((len(g.tables.get(s, ())) for s in slots), default=0)
        out = np.full((len(slots), max(width, 1)), -1, dtype=np.int32)
        for i, s in enumerate(slots):
            t = g.tables.get(s, ())
            out[i, : len(t)] = t
        return out

    # -- invariants -------------------------------------------------------------------
    def check(self) -> None:
        """No page lost, none held twice; tables only of live slots."""
        live = self.slots.live()
        if set(self.lengths) != live:
            raise AssertionError(f"lengths of {sorted(self.lengths)} but live slots {sorted(live)}")
        for g in self.groups:
            seen: dict[int, int] = {}
            for slot, table in g.tables.items():
                if slot not in live:
                    raise AssertionError(f"group {g.group_id}: table of dead slot {slot}")
                done = g.released.get(slot, 0)
                if any(p >= 0 for p in table[:done]) or any(p < 0 for p in table[done:]):
                    raise AssertionError(
                        f"group {g.group_id}: slot {slot} has a hole behind its first held page "
                        f"(released {done}, table {table})"
                    )
                for p in table:
                    if p < 0:
                        continue
                    if p == 0 or p >= g.pool.num_pages:
                        raise AssertionError(f"group {g.group_id}: slot {slot} holds page {p}")
                    if p in seen:
                        raise AssertionError(f"group {g.group_id}: page {p} held by slots {seen[p]} and {slot}")
                    seen[p] = slot
            if set(seen) != g.pool.held_pages():
                raise AssertionError(f"group {g.group_id}: tables and pool disagree on held pages")
            if len(seen) + g.pool.available != g.pool.capacity:
                raise AssertionError(f"group {g.group_id}: {len(seen)} held + {g.pool.available} free != {g.pool.capacity}")

    def idle(self) -> bool:
        return self.slots.available == self.slots.n_slots and all(
            g.pool.available == g.pool.capacity for g in self.groups
        )
