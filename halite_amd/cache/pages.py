"""Pages of keys and values, and the tables that say which pages a request holds.

The reference's two engines keep a token-granular pool with one block-table row per
request (src/halite/transformers/infer/engine/memory_pool.py:4-158) and real pages of
16 tokens with per-sequence page lists
(src/halite/transformers/tokainfer/kv_cache.py:7-54; tokainfer/engine/allocator.py:
11-126).  Here a *group* is a set of layer runs with the same need (heads, head size,
window): it has its own pool of pages, its own page list per request, and gives pages
back when a request ends or, for a window, when every later query has passed them.
Page 0 of every group is never handed out: padded rows may write there
(memory_pool.py:85-105 reserves slot 0 for the same reason).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..parts.base import PagedNeed


class NoSpace(Exception):
    """Not enough free pages (src/halite/transformers/tokainfer/engine/allocator.py:
    ``NoSpaceException``)."""


class PagePool:
    """Free pages of one group: a stack of page numbers, page 0 excluded."""

    def __init__(self, num_pages: int):
        if num_pages < 2:
            raise ValueError("a pool needs the reserved page 0 and at least one more")
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, 0, -1))  # pop() hands out 1, 2, ...
        self._held = [False] * num_pages

    @property
    def available(self) -> int:
        return len(self._free)

    @property
    def capacity(self) -> int:
        return self.num_pages - 1

    def alloc(self, n: int) -> list[int]:
        if n > len(self._free):
            raise NoSpace(f"{n} pages wanted, {len(self._free)} free")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._held[p] = True
        return out

    def free(self, pages) -> None:
        for p in pages:
            if p <= 0 or p >= self.num_pages or not self._held[p]:
                raise RuntimeError(f"page {p} is freed but not held")
            self._held[p] = False
            self._free.append(p)

    def held_pages(self) -> set[int]:
        return {p for p, h in enumerate(self._held) if h}


def tiled_layout(dtype: torch.dtype, head_dim: int, page_size: int) -> bool:
    """Whether pages of this shape are kept in the order in which the matrix-core
    attention kernel loads them (contiguous KB per MFMA operand) instead of row by row:
    bf16, heads of a multiple of 32 (up to 256), pages of a power of two of at least 32
    tokens.  The kernel that appends and the kernel that reads are told by
    ``LayerPages.tiled``."""
    return (
        dtype == torch.bfloat16
        and head_dim % 32 == 0
        and head_dim <= 256
        and page_size >= 32
        and page_size & (page_size - 1) == 0
    )


@dataclass
class LayerPages:
    """The device pages of one run: keys ``[pages, K, page_size, D]`` and values,
    transposed, ``[pages, K, D, page_size]``.  With ``tiled`` the bytes of one
    (page, kv head) are the same in number but lie in blocks of 32 tokens, keys as
    ``[block][16-key tile][32-dim step][dim quad][key][8 dims]`` and values as
    ``[block][16-dim tile][8-key group][dim][8 keys]``."""

    group_id: int
    k: torch.Tensor | None
    v: torch.Tensor | None
    tiled: bool = False


@dataclass
class CacheGroup:
    group_id: int
    need: PagedNeed  # (its ``window`` is all that the bookkeeping below reads)
    runs: list[int]  # indices of the runs that own a cache in this group
    page_size: int
    pool: PagePool
    # per live slot: page number for every logical page, -1 where none is held
    tables: dict[int, list[int]] = field(default_factory=dict)
    released: dict[int, int] = field(default_factory=dict)
    storage: torch.Tensor | None = None  # [runs, pages * elements of a page]: a run's tensors one after the other

    def first_needed_page(self, next_position: int) -> int:
        """Logical pages before this one are out of reach of every query at
        ``next_position`` or later."""
        if self.need.window is None:
            return 0
        oldest_key = next_position - self.need.window + 1
        return max(0, oldest_key // self.page_size)

    # A request's table has no holes behind its first held page: ``released[slot]``
    # leading entries were given back (they are -1), every later entry holds a page.
    def pages_missing(self, slot: int, start: int, new_len: int) -> int:
        """Pages to allocate so that the tokens ``[start, new_len)`` can be run:
        their own positions, and nothing that the window has passed."""
        return len(self._wanted(slot, start, new_len))

    def _wanted(self, slot: int, start: int, new_len: int) -> range | list[int]:
        table = self.tables.get(slot, ())
        first = self.first_needed_page(start)
        last = (new_len - 1) // self.page_size
        if first >= self.released.get(slot, 0):  # nothing that was given back is asked for again
            return range(max(first, len(table)), last + 1)
        return [i for i in range(first, last + 1) if i >= len(table) or table[i] < 0]

    def reserve(self, slot: int, start: int, new_len: int) -> None:
        want = self._wanted(slot, start, new_len)
        table = self.tables.setdefault(slot, [])
        last = (new_len - 1) // self.page_size
        pages = self.pool.alloc(len(want))
        while len(table) <= last:
            table.append(-1)
        for i, p in zip(want, pages):
            table[i] = p

    def release_passed(self, slot: int, next_position: int) -> int:
        """Gives back the pages that no query at ``next_position`` or later reads."""
        if self.need.window is None:
            return 0
        table = self.tables.get(slot)
        if not table:
            return 0
        first = min(self.first_needed_page(next_position), len(table))
        done = self.released.get(slot, 0)
        if first <= done:
            return 0
        dead = [p for p in table[done:first] if p >= 0]
        for i in range(done, first):
            table[i] = -1
        self.released[slot] = first
        self.pool.free(dead)
        return len(dead)

    def release_beyond(self, slot: int, length: int) -> int:
        """Gives back the pages behind the one that holds token ``length - 1`` (pages that
        were taken for tokens that did not come)."""
        table = self.tables.get(slot)
        keep = -(-length // self.page_size)
        if not table or len(table) <= keep:
            return 0
        dead = [p for p in table[keep:] if p >= 0]
        del table[keep:]
        self.pool.free(dead)
        return len(dead)

    def release_all(self, slot: int) -> int:
        table = self.tables.pop(slot, [])
        self.released.pop(slot, None)
        held = [p for p in table if p >= 0]
        self.pool.free(held)
        return len(held)

    def tokens_held_at_most(self, n_tokens: float) -> float:
        """Cache tokens of this group that ``n_tokens`` tokens of one request take at
        most: all of them, or what a window spans (whole pages, and the one being left)."""
        if self.need.window is None:
            return n_tokens
        return min(n_tokens, (-(-self.need.window // self.page_size) + 1) * self.page_size)

    def pages_per_token_span(self, n_tokens: int) -> int:
        """Upper bound of the pages a request of ``n_tokens`` holds at once."""
        if self.need.window is None:
            return -(-n_tokens // self.page_size)
        return min(-(-n_tokens // self.page_size), -(-self.need.window // self.page_size) + 1)
