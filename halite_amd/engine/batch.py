"""What one step runs: segments on the host, and their arrays on the device.

A *segment* is the next tokens of one request: a portion of its prompt, cut anywhere,
or one decoded token.  All segments of a step are one flat batch, as in the
reference's ``tokainfer`` engine (src/halite/transformers/tokainfer/types.py:521-553;
tokainfer/engine/input_building.py:138-306): token ids, positions, for every token the
segment it belongs to, per segment where its queries start and how many keys it has
after this step, the rows whose logits are wanted, and per cache group the block table
of the step's requests.  Everything is packed into one int32 buffer and copied to the
device once.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..kernels import attention as attention_kernels


@dataclass
class Segment:
    slot: int  # the request's slot in the cache manager
    start: int  # position of the first token == tokens already cached
    tokens: np.ndarray  # int32
    want: list[int] = field(default_factory=list)  # indices into tokens

    def __post_init__(self):
        self.tokens = np.asarray(self.tokens, dtype=np.int32).reshape(-1)


@dataclass
class GroupStep:
    group_id: int
    page_size: int
    window: int | None
    block_table: torch.Tensor  # [S, P] int32 on the device
    block_table_host: np.ndarray


class _Packer:
    def __init__(self):
        self.parts = []
        self.offsets = {}
        self.n = 0

    def add(self, name, arr, capacity: int | None = None):
        """Appends ``arr``; with ``capacity`` the piece takes that many ints whatever
        its length (so that later pieces keep their place from step to step)."""
        arr = np.ascontiguousarray(arr, dtype=np.int32).reshape(-1)
        room = arr.size if capacity is None else capacity
        if arr.size > room:
            raise ValueError(f"step array {name} has {arr.size} entries, room for {room}")
        room += (-room) % 4  # keep every piece 16-byte aligned
        self.offsets[name] = (self.n, arr.size)
        self.parts.append(arr)
        if room > arr.size:
            self.parts.append(np.zeros(room - arr.size, dtype=np.int32))
        self.n += room

    def flat(self):
        return np.concatenate(self.parts) if self.parts else np.zeros(0, dtype=np.int32)


class StaticLayout:
    """Fixed capacities and one persistent device buffer, so that every array of a
    step lies at the same address step after step: what a captured graph needs.
    Made for decode-only steps of ``n_segs`` requests."""

    def __init__(self, n_segs: int, bt_width: dict[int, int], device):
        self.n_segs = n_segs
        self.bt_width = dict(bt_width)
        self.device = device
        self.buffer: torch.Tensor | None = None
        self.size = 0

    def place(self, flat: np.ndarray, staging: "_Staging") -> torch.Tensor:
        if self.buffer is None:
            self.size = flat.size
            self.buffer = torch.zeros(flat.size, dtype=torch.int32, device=self.device)
        if flat.size != self.size:
            raise RuntimeError("a static step layout changed its size")
        self.buffer.copy_(staging.pinned(flat), non_blocking=True)
        staging.mark()
        return self.buffer


class _Staging:
    """A ring of pinned host buffers for the per-step copy."""

    def __init__(self, device, n=4):
        self.device = device
        self.bufs = [None] * n
        self.events = [None] * n
        self.i = 0
        self._last = 0

    def pinned(self, flat: np.ndarray) -> torch.Tensor:
        i = self.i
        self.i = (self.i + 1) % len(self.bufs)
        if self.events[i] is not None:
            self.events[i].synchronize()
        n = flat.size
        if self.bufs[i] is None or self.bufs[i].numel() < n:
            self.bufs[i] = torch.empty(max(n, 4096) * 2, dtype=torch.int32, pin_memory=True)
        self.bufs[i][:n].numpy()[:] = flat
        self._last = i
        return self.bufs[i][:n]

    def mark(self):
        ev = torch.cuda.Event()
        ev.record()
        self.events[self._last] = ev

    def upload(self, flat: np.ndarray) -> torch.Tensor:
        dev = self.pinned(flat).to(self.device, non_blocking=True)
        self.mark()
        return dev


class StepContext:
    """The device-side view of a step that the parts compute on."""

    def __init__(self, segments: list[Segment], cache, device, staging: _Staging | None = None,
                 static: StaticLayout | None = None):
        self.device = torch.device(device)
        self.segments = segments
        self.cache = cache
        self.static = static
        S = len(segments)
        self.n_segs = S
        lens = np.array([s.tokens.size for s in segments], dtype=np.int32)
        starts = np.array([s.start for s in segments], dtype=np.int32)
        self.seg_q_len_host = lens
        self.seg_pos0_host = starts
        self.seg_kv_len_host = starts + lens
        self.seg_q_start_host = np.concatenate(([0], np.cumsum(lens)[:-1])).astype(np.int32)
        self.seg_slot_host = np.array([s.slot for s in segments], dtype=np.int32)
        T = int(lens.sum())
        self.n_tokens = T
        tokens = np.concatenate([s.tokens for s in segments]) if S else np.zeros(0, np.int32)
        seg_of = np.repeat(np.arange(S, dtype=np.int32), lens)
        positions = np.arange(T, dtype=np.int32) - np.repeat(self.seg_q_start_host, lens) + np.repeat(starts, lens)
        rows = []
        for s, q0 in zip(segments, self.seg_q_start_host):
            for w in s.want:
                if not 0 <= w < s.tokens.size:
                    raise ValueError(f"wanted row {w} outside a segment of {s.tokens.size} tokens")
                rows.append(int(q0) + w)
        self.n_logit_rows = len(rows)
        self.max_position = int(self.seg_kv_len_host.max()) - 1 if S else 0
        self.positions_host = positions
        self.token_seg_host = seg_of
        if static is not None and not (S == T == len(rows) == static.n_segs):
            raise ValueError("a static layout serves decode-only steps of its own batch size")

        pk = _Packer()
        pk.add("tokens", tokens)
        pk.add("positions", positions)
        pk.add("token_seg", seg_of)
        pk.add("token_slot", np.repeat(self.seg_slot_host, lens))
        pk.add("logit_rows", np.array(rows, dtype=np.int32))
        pk.add("seg_q_start", self.seg_q_start_host)
        pk.add("seg_q_len", lens)
        pk.add("seg_kv_len", self.seg_kv_len_host)
        slots = [s.slot for s in segments]
        tables = {}
        for g in cache.groups:
            width = static.bt_width[g.group_id] if static is not None else None
            bt = cache.block_table(g.group_id, slots, width)
            tables[g.group_id] = bt
            pk.add(f"bt{g.group_id}", bt)
        self._packer = pk
        self._plans: dict = {}
        self._plan_host: dict = {}
        self._tables_host = tables
        self._staging = staging
        self._dev = None
        self._groups: dict[int, GroupStep] = {}
        self.empty_f32 = None

    # The plans of the attention kernel are part of the same upload, so they are
    # declared before the first device access.
    def plan_attention(self, group_id: int, n_heads: int, n_kv_heads: int, window: int,
                       head_dim: int, late=False) -> None:
        key = (group_id, n_heads // n_kv_heads, window)
        if key in self._plan_host:
            return
        if self._dev is not None and not late:
            return
        plan = attention_kernels.plan_items(
            self.seg_q_len_host, self.seg_kv_len_host, n_heads // n_kv_heads, n_kv_heads, window,
            attention_kernels.rows_per_big_item(head_dim),
        )
        self._plan_host[key] = plan
        plan.name = f"plan{len(self._plan_host)}"
        if self._dev is None:
            cap = None
            if self.static is not None:  # decode only: room for whatever the planner makes of these requests
                attention_kernels.fix_room_for_decode(plan, self.n_segs, n_heads // n_kv_heads, n_kv_heads)
                cap = plan.cap_items
            self._packer.add(plan.name + "_items", plan.items, None if cap is None else cap * attention_kernels.SMALL_ITEM_INTS)
            self._packer.add(plan.name + "_big", plan.big_items)
            self._packer.add(plan.name + "_merges", plan.merges, None if cap is None else plan.cap_merges * 8)
            self._packer.add(plan.name + "_counts", plan.counts())
        else:  # declared after the step's upload: a copy of its own
            if self.static is not None:
                raise RuntimeError("a static step needs its attention plans before the upload")
            self._plans[key] = attention_kernels.upload_plan(plan, self.device)

    def replace_tokens(self, tokens: np.ndarray) -> None:
        """Other token ids for a context that was put together before they were known
        (and has not been copied to the device yet)."""
        if self._dev is not None or tokens.size != self.n_tokens:
            raise RuntimeError("token ids can only be replaced, one for one, before the upload")
        self._packer.parts[0] = np.ascontiguousarray(tokens, dtype=np.int32).reshape(-1)

    def upload(self):
        if self._dev is not None:
            return
        flat = self._packer.flat()
        if self.static is not None:
            self._dev = self.static.place(flat, self._staging)
        elif self._staging is not None and self.device.type == "cuda":
            self._dev = self._staging.upload(flat)
        else:
            self._dev = torch.from_numpy(flat).to(self.device)
        self.empty_f32 = torch.empty((0, 0), dtype=torch.float32, device=self.device)

    def _view(self, name) -> torch.Tensor:
        self.upload()
        off, n = self._packer.offsets[name]
        return self._dev[off : off + n]

    tokens = property(lambda self: self._view("tokens"))
    positions = property(lambda self: self._view("positions"))
    token_seg = property(lambda self: self._view("token_seg"))
    token_slot = property(lambda self: self._view("token_slot"))
    logit_rows = property(lambda self: self._view("logit_rows"))
    seg_q_start = property(lambda self: self._view("seg_q_start"))
    seg_q_len = property(lambda self: self._view("seg_q_len"))
    seg_kv_len = property(lambda self: self._view("seg_kv_len"))

    def group(self, group_id: int) -> GroupStep:
        if group_id not in self._groups:
            host = self._tables_host[group_id]
            g = self.cache.groups[group_id]
            self._groups[group_id] = GroupStep(
                group_id, g.page_size, g.need.window, self._view(f"bt{group_id}").view(host.shape), host
            )
        return self._groups[group_id]

    def attention(self, q, q_row_stride, kv, group: GroupStep, n_heads, scale, window) -> torch.Tensor:
        """Attention of every token of the step over its request's cached keys."""
        return attention_kernels.paged_attention(self, q, q_row_stride, kv, group, n_heads, scale, window)

    def device_plan(self, group_id: int, group_size: int, window: int):
        key = (group_id, group_size, window)
        plan = self._plan_host.get(key)
        if plan is None:
            return None
        if key not in self._plans:
            self.upload()

            def piece(name, rows, ints=8):
                off, _ = self._packer.offsets[plan.name + name]
                return self._dev[off : off + rows * ints].view(rows, ints)

            counts = self._view(plan.name + "_counts")
            self._plans[key] = (plan, piece("_items", plan.cap_items, attention_kernels.SMALL_ITEM_INTS),
                                piece("_big", plan.cap_big, attention_kernels.BIG_ITEM_INTS),
                                piece("_merges", plan.cap_merges), counts)
        return self._plans[key]

    def fits_static(self) -> bool:
        """Whether every plan of this step fits the static layout's capacities."""
        return all(
            p.n_items <= p.cap_items and p.n_merges <= p.cap_merges and p.n_partials <= p.cap_partials and p.n_big == 0
            for p in self._plan_host.values()
        )
