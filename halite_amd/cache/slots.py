"""Slots: the fixed-size part of what a live request owns.

A request gets a slot for life at admission, as the reference's ``tokainfer`` engine
gives each sequence a ``batch_index`` (src/halite/transformers/tokainfer/engine/
allocator.py:428-445) and its ``infer`` engine a row of the request-to-token table
(src/halite/transformers/infer/engine/memory_pool.py:38-49).  The slot indexes the
per-request state tensors that parts declare (``StateNeed``): one row each, zeroed at
admission.  Llama's attention declares none; the rows exist all the same for mixers
that carry state from step to step.
"""

from __future__ import annotations

import torch

from ..parts.base import StateNeed


class NoSlot(Exception):
    pass


class SlotAllocator:
    def __init__(self, n_slots: int):
        self.n_slots = n_slots
        self._free = list(range(n_slots - 1, -1, -1))
        self._live = [False] * n_slots

    @property
    def available(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise NoSlot(f"all {self.n_slots} slots are taken")
        s = self._free.pop()
        self._live[s] = True
        return s

    def free(self, slot: int) -> None:
        if slot < 0 or slot >= self.n_slots or not self._live[slot]:
            raise RuntimeError(f"slot {slot} is freed but not live")
        self._live[slot] = False
        self._free.append(slot)

    def live(self) -> set[int]:
        return {s for s, l in enumerate(self._live) if l}


class StateStore:
    """``tensors[run index][name]`` is ``[n_slots, *shape]`` on the device."""

    def __init__(self, n_slots: int, needs: dict[int, dict[str, StateNeed]], device):
        self.n_slots = n_slots
        self.tensors: dict[int, dict[str, torch.Tensor]] = {}
        for run, named in needs.items():
            self.tensors[run] = {
                name: torch.zeros((n_slots, *need.shape), dtype=need.dtype, device=device)
                for name, need in named.items()
            }

    def reset(self, slot: int) -> None:
        for named in self.tensors.values():
            for t in named.values():
                t[slot].zero_()

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for n in self.tensors.values() for t in n.values())
