"""Choice and planning of the paged-attention kernel for a step.

bfloat16 with a head size that is a multiple of 16 (up to 256) and pages of a multiple
of 8 tokens run on the matrix-core kernel; everything else (the 32-bit path, other
sizes) runs on the plain kernel.  The matrix-core kernel works through a list of
*items* that the host writes per step, once for all layers; the reference plans its
attention kernels per step in the same place
(src/halite/transformers/infer/engine/flashinfer_backend.py:182-261).
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass

import numpy as np
import torch

from . import library, ops

ROWS_PER_ITEM = 16
KEYS_PER_BLOCK = 32
MIN_SPLIT_KEYS = 128
TARGET_WAVES_LONG = 1024
WAVES_PER_GROUP = 4  # waves of a workgroup
SMALL_ITEM_INTS = 12  # an item of the kernel for one-tile segments: 8, then its tile's first partial slot and pieces
BIG_ITEM_INTS = 16  # an item of the kernel for long segments: 8, then what its workgroup would have to look up
# One-tile items: a tile's key range is cut into pieces, one per workgroup, of which there
# should be about one per compute unit (what a compute unit has in flight bounds what it
# reads a second, so an even share each counts for more than many waves: measured), and no
# piece shorter than this many keys (below, a second piece and the merge cost more than the
# shorter walk saves).
COMPUTE_UNITS = 256  # of the MI355X; the device that runs is asked (`compute_units`)
MIN_PIECE_KEYS = 384
# Up to this many pieces a tile the attention kernel merges the partial results itself (the
# workgroup that finishes a tile last does, in the same launch: 1 to 3 us less than a merge
# kernel behind it); more go to the merge kernel, which spreads a tile's partial results over
# many workgroups (16 and 32 pieces measured 1 to 2 us faster so).
MERGED_IN_KERNEL = 8
N_COUNTERS = 1 << 14  # one per (tile that the kernel merges, key/value head); a tile has pieces only while these are few


_compute_units: int | None = None


def compute_units() -> int:
    """Compute units of the device that runs the kernels, asked once (without a device,
    as where the planner is tested: the MI355X's)."""
    global _compute_units
    if _compute_units is None:
        if torch.cuda.is_available():
            _compute_units = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)
        else:
            _compute_units = COMPUTE_UNITS
    return _compute_units


def pieces_per_tile(n_tiles: int, n_kv_heads: int) -> int:
    """Into how many pieces, at most, the key range of each of ``n_tiles`` one-tile items
    is cut (every piece is one workgroup per key/value head)."""
    return max(1, compute_units() // max(1, n_tiles * n_kv_heads))


@dataclass
class AttentionPlan:
    """Work lists of the matrix-core kernel for one step (rows are (token, head of the
    group) pairs, token-major):
    ``items`` [n, 12]: segment, first row, first key, end key, partial slot or -1, then the
    segment's first token, number of tokens and number of keys — tiles of 16 rows of segments
    with at most 16 rows (decode tokens).  They come in runs of four, a workgroup's waves:
    one piece of a tile's key range cut in four (some may be empty), which the workgroup
    joins itself, into the output or, where the range has several pieces, into the run's
    partial slot.  Places 8 and 9: the tile's first partial slot and number of pieces if the
    kernel is to merge them itself (then the tile has no merge entry), else 0;
    ``big_items`` [n, 16] for longer segments: the first five the same, then the first rows
    of the item's further tiles (-1: none), ``rows_big`` rows per item; then the segment's
    first token, number of tokens and number of keys, and the first and end key of the walk
    of the item's run of four (a workgroup's waves), so that a workgroup knows all it needs
    after one trip to memory;
    ``merges`` [n, 8]: segment, first row of a 16-row tile, first partial slot, number of
    partials, slots between partials, the segment's first token and number of tokens.
    A segment's first token is the sum of the lengths of the segments before it."""

    items: np.ndarray
    big_items: np.ndarray
    merges: np.ndarray
    n_partials: int  # partial slots (one per 16 rows and piece)
    rows_big: int = 64
    name: str = ""
    # room in the device arrays (larger than the live counts under a static layout)
    cap_items: int = 0
    cap_big: int = 0
    cap_merges: int = 0
    cap_partials: int = 0
    # the most partial results that a merge item joins (under a static layout, whose kernel
    # launches are fixed while the plans change: the most that any of its plans could have)
    max_parts: int = 0
    # some one-tile items ask the kernel to merge their tile's pieces itself (it needs counters)
    merged_in_kernel: bool = False

    def __post_init__(self):
        if len(self.items) and int(self.items[:, 9].max()) > 1:
            self.merged_in_kernel = True
        if len(self.merges) and self.max_parts == 0:
            self.max_parts = int(self.merges[:, 3].max())
        self.cap_items = max(self.cap_items, len(self.items))
        self.cap_big = max(self.cap_big, len(self.big_items))
        self.cap_merges = max(self.cap_merges, len(self.merges))
        self.cap_partials = max(self.cap_partials, self.n_partials)

    @property
    def n_items(self):
        return len(self.items)

    @property
    def n_big(self):
        return len(self.big_items)

    @property
    def n_merges(self):
        return len(self.merges)

    def counts(self) -> np.ndarray:
        return np.array([self.n_items, self.n_big, self.n_merges], dtype=np.int32)


def fix_room_for_decode(plan: AttentionPlan, n_requests: int, group_size: int, n_kv_heads: int) -> None:
    """Gives ``plan``, of a step of one token for each of ``n_requests`` requests, the room
    that any such step's plan fits, whatever the requests' lengths, and says which way its
    tiles' pieces are merged: what launches that are recorded once for all later steps of
    this size need to know.  No plan cuts a key range into more pieces than
    ``pieces_per_tile`` allows (into none at all where the tiles are many), and by that
    number the attention kernel merges the pieces itself or leaves them to the merge kernel."""
    tiles = n_requests * -(-group_size // ROWS_PER_ITEM)
    most = pieces_per_tile(tiles, n_kv_heads)
    plan.cap_items = WAVES_PER_GROUP * tiles * most
    plan.cap_partials = tiles * most if most > 1 else 0
    plan.cap_merges = tiles if most > MERGED_IN_KERNEL else 0
    plan.merged_in_kernel = 1 < most <= MERGED_IN_KERNEL
    plan.max_parts = most


def mfma_supported(dtype: torch.dtype, head_dim: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 256 and page_size % 8 == 0


def rows_per_big_item(head_dim: int) -> int:
    """Rows that one wave takes of a long segment: the kernel library for this head size
    says how it was built."""
    return int(library.attention_library(head_dim).hal_attention_mfma_rows_per_big_item())


def _tiles(seg_q_len, seg_kv_len, group_size, window, rows_per_tile, pick):
    """The tiles of ``rows_per_tile`` rows of the segments whose row count ``pick``
    accepts: segment, first row, first and end key of each (arrays)."""
    ql = np.asarray(seg_q_len, dtype=np.int64)
    kl = np.asarray(seg_kv_len, dtype=np.int64)
    rows = ql * group_size
    chosen = np.nonzero(pick(rows, ql) & (rows > 0))[0] if len(ql) else np.zeros(0, dtype=np.int64)
    if len(chosen) == 0:
        z = np.zeros(0, dtype=np.int64)
        return z, z, z, z
    n_tiles = -(-rows[chosen] // rows_per_tile)
    seg_ids = np.repeat(chosen, n_tiles)
    first_tile = np.concatenate(([0], np.cumsum(n_tiles)[:-1]))
    r0 = (np.arange(int(n_tiles.sum())) - np.repeat(first_tile, n_tiles)) * rows_per_tile
    first_q = r0 // group_size
    last_q = np.minimum(rows[seg_ids] - 1, r0 + rows_per_tile - 1) // group_size
    pos0 = (kl - ql)[seg_ids]
    b = np.zeros_like(r0) if window <= 0 else np.maximum(0, pos0 + first_q - window + 1)
    e = pos0 + last_q + 1
    return seg_ids, r0, b, e


def _cut_long(seg_ids, rho0s, kv_b, kv_e, chunk, slots_per_tile, first_slot, seg_scalars, more_tiles):
    """Items and merge entries of the long segments' items, whose key ranges are cut into
    pieces of ``chunk`` keys (pieces end on multiples of 32 keys).  ``more_tiles`` [n, k]
    holds the first rows of an item's further 16-row tiles (-1: none); ``seg_scalars``
    [segments, 3] the segments' first token, tokens and keys."""
    n_tiles = len(seg_ids)
    if n_tiles == 0:
        return np.zeros((0, BIG_ITEM_INTS), np.int32), np.zeros((0, 8), np.int32), first_slot
    base = kv_b - kv_b % KEYS_PER_BLOCK
    n_pieces = np.maximum(1, -(-(kv_e - base) // chunk))
    n_items = int(n_pieces.sum())
    items = np.zeros((n_items, 8), dtype=np.int32)
    tile_of = np.repeat(np.arange(n_tiles), n_pieces)
    first_item = np.concatenate(([0], np.cumsum(n_pieces)[:-1]))
    piece = np.arange(n_items) - first_item[tile_of]
    items[:, 0] = seg_ids[tile_of]
    items[:, 1] = rho0s[tile_of]
    items[:, 2] = np.maximum(kv_b[tile_of], base[tile_of] + piece * chunk)
    items[:, 3] = np.minimum(kv_e[tile_of], base[tile_of] + (piece + 1) * chunk)
    items[:, 5:] = -1
    items[:, 5 : 5 + more_tiles.shape[1]] = more_tiles[tile_of]
    split = n_pieces[tile_of] > 1
    items[:, 4] = -1
    n_split = int(split.sum())
    items[split, 4] = first_slot + np.arange(n_split) * slots_per_tile
    # one merge entry per 16-row tile of every item that was cut
    cut = np.nonzero(n_pieces > 1)[0]
    firsts = np.concatenate((rho0s[cut][:, None], more_tiles[cut]), axis=1)
    sub = np.broadcast_to(np.arange(firsts.shape[1]), firsts.shape)
    keep = firsts >= 0
    rows_of = np.broadcast_to(cut[:, None], firsts.shape)[keep]
    merges = np.zeros((int(keep.sum()), 8), dtype=np.int32)
    merges[:, 0] = seg_ids[rows_of]
    merges[:, 1] = firsts[keep]
    merges[:, 2] = items[first_item[rows_of], 4] + sub[keep]
    merges[:, 3] = n_pieces[rows_of]
    merges[:, 4] = slots_per_tile
    merges[:, 5:7] = seg_scalars[merges[:, 0], :2]
    return _group_items(items, piece, WAVES_PER_GROUP, seg_scalars), merges, first_slot + n_split * slots_per_tile


def _cut_joined(seg_ids, rho0s, kv_b, kv_e, most_pieces, first_slot, seg_scalars):
    """Items and merge entries of one-tile items whose key ranges are cut into at most
    ``most_pieces`` pieces, one per workgroup, and every piece into four, one per wave (in
    blocks of 32 keys, as evenly as they go; where a piece is short some of the four are
    empty).  A piece's four items stand in a row and carry the piece's partial slot, or -1
    where the range is one piece; the longest pieces come first.  The pieces are merged by
    the kernel itself (no merge entries) unless ``most_pieces`` allows more of them than it
    takes."""
    n = len(seg_ids)
    if n == 0:
        return np.zeros((0, SMALL_ITEM_INTS), np.int32), np.zeros((0, 8), np.int32), first_slot
    base = kv_b - kv_b % KEYS_PER_BLOCK
    blocks = -(-(kv_e - base) // KEYS_PER_BLOCK)
    n_pieces = np.clip((kv_e - base) // MIN_PIECE_KEYS, 1, most_pieces)
    total = int(n_pieces.sum())
    tile_of = np.repeat(np.arange(n), n_pieces)
    first_item = np.concatenate(([0], np.cumsum(n_pieces)[:-1]))
    piece = np.arange(total) - first_item[tile_of]
    # wave w of all the range's waves takes the blocks from ceil(w * blocks / waves) on
    waves = (n_pieces * WAVES_PER_GROUP)[tile_of][:, None]
    w = piece[:, None] * WAVES_PER_GROUP + np.arange(WAVES_PER_GROUP + 1)[None, :]
    edge = base[tile_of][:, None] + -(-(w * blocks[tile_of][:, None]) // waves) * KEYS_PER_BLOCK
    b = np.maximum(kv_b[tile_of][:, None], edge[:, :-1])
    e = np.minimum(kv_e[tile_of][:, None], edge[:, 1:])
    empty = b >= e
    # (an empty item names the piece's first key twice: the kernel asks for the page of an
    # item's first key before it knows whether the item has any, and under a window the
    # pages before the piece may have been given back)
    items = np.zeros((total, WAVES_PER_GROUP, SMALL_ITEM_INTS), dtype=np.int32)
    items[:, :, 0] = seg_ids[tile_of][:, None]
    items[:, :, 1] = rho0s[tile_of][:, None]
    items[:, :, 2] = np.where(empty, b[:, :1], b)
    items[:, :, 3] = np.where(empty, b[:, :1], e)
    items[:, :, 5:8] = seg_scalars[seg_ids[tile_of]][:, None, :]
    split = n_pieces[tile_of] > 1
    n_split = int(split.sum())
    slots = np.full(total, -1, dtype=np.int64)
    slots[split] = first_slot + np.arange(n_split)
    items[:, :, 4] = slots[:, None]
    cut = np.nonzero(n_pieces > 1)[0]
    if most_pieces <= MERGED_IN_KERNEL:  # the kernel merges: the items say where and how many
        items[:, :, 8] = np.where(split, slots[first_item[tile_of]], 0)[:, None]
        items[:, :, 9] = np.where(split, n_pieces[tile_of], 0)[:, None]
        cut = cut[:0]
    merges = np.zeros((len(cut), 8), dtype=np.int32)
    merges[:, 0] = seg_ids[cut]
    merges[:, 1] = rho0s[cut]
    merges[:, 2] = slots[first_item[cut]]
    merges[:, 3] = n_pieces[cut]
    merges[:, 4] = 1
    merges[:, 5:7] = seg_scalars[seg_ids[cut], :2]
    keys = np.where(empty, 0, e).max(axis=1) - b[:, 0]  # a piece's first wave always has keys
    order = np.argsort(-keys, kind="stable")
    return items[order].reshape(total * WAVES_PER_GROUP, SMALL_ITEM_INTS), merges, first_slot + n_split


def _group_items(items: np.ndarray, piece: np.ndarray, group: int, seg_scalars: np.ndarray) -> np.ndarray:
    """Orders items so that every run of ``group`` items (a workgroup's waves) belongs to
    one segment and to the same piece of neighbouring tiles, i.e. walks nearly the same
    keys; a run that cannot be filled is padded with items that have no rows and no keys.
    The runs with the longest walk come first."""
    n = len(items)
    if n == 0:
        return np.zeros((0, BIG_ITEM_INTS), np.int32)
    order = np.lexsort((np.arange(n), piece, items[:, 0]))  # segment, then piece, then tile
    seg, pc = items[order, 0], piece[order]
    new_class = np.concatenate(([True], (seg[1:] != seg[:-1]) | (pc[1:] != pc[:-1])))
    class_start = np.nonzero(new_class)[0]
    class_len = np.diff(np.concatenate((class_start, [n])))
    padded_len = -(-class_len // group) * group
    padded_start = np.concatenate(([0], np.cumsum(padded_len)[:-1]))
    class_of = np.cumsum(new_class) - 1
    dest = padded_start[class_of] + (np.arange(n) - class_start[class_of])
    total = int(padded_len.sum())
    out = np.full((total, 8), -1, dtype=np.int32)
    out[:, 2:4] = 0
    out[:, 0] = np.repeat(seg[class_start], padded_len)  # the padding carries its run's segment
    out[dest] = items[order]
    runs = out.reshape(total // group, group, 8)
    live = runs[:, :, 3] > runs[:, :, 2]
    first_key = np.where(live, runs[:, :, 2], np.iinfo(np.int32).max).min(axis=1)
    end_key = np.where(live, runs[:, :, 3], 0).max(axis=1)
    walk = np.where(live.any(axis=1), end_key - first_key, 0)
    wide = np.zeros((total // group, group, BIG_ITEM_INTS), dtype=np.int32)
    wide[:, :, :8] = runs
    wide[:, :, 8:11] = seg_scalars[runs[:, 0, 0]][:, None, :]
    wide[:, :, 11] = np.where(live.any(axis=1), first_key, 0)[:, None]
    wide[:, :, 12] = end_key[:, None]
    return wide[np.argsort(-walk, kind="stable")].reshape(total, BIG_ITEM_INTS)


def _group_tiles(seg_ids, rho0s, kv_b, kv_e, per_item: int):
    """Groups neighbouring 16-row tiles of one segment into items of ``per_item`` tiles,
    which share nearly all of their keys.  (Pairing an early tile with a late one, which
    evens out the causal work per item, measured the same at 1,024 and 2,048 tokens and 5
    to 8% worse at 8,192 and 16,384: the item then walks the late tile's keys with the
    early tile idle most of the way.)"""
    out_seg, out_rho, out_b, out_e, more = [], [], [], [], []
    starts = np.nonzero(np.concatenate(([True], seg_ids[1:] != seg_ids[:-1])))[0]  # tiles are in segment order
    ends = np.concatenate((starts[1:], [len(seg_ids)]))
    for lo, hi in zip(starts.tolist(), ends.tolist()):
        n_items = -(-(hi - lo) // per_item)
        members = lo + np.arange(n_items * per_item).reshape(n_items, per_item)
        valid = members < hi
        members = np.minimum(members, hi - 1)
        out_seg.append(seg_ids[members[:, 0]])
        out_rho.append(rho0s[members[:, 0]])
        out_b.append(np.where(valid, kv_b[members], np.iinfo(np.int64).max).min(axis=1))
        out_e.append(np.where(valid, kv_e[members], 0).max(axis=1))
        more.append(np.where(valid[:, 1:], rho0s[members[:, 1:]], -1))
    cat = lambda x: np.concatenate(x).astype(np.int64)
    return cat(out_seg), cat(out_rho), cat(out_b), cat(out_e), np.concatenate(more).astype(np.int64).reshape(-1, per_item - 1)


def plan_items(seg_q_len, seg_kv_len, group_size: int, n_kv_heads: int, window: int,
               rows_big: int = 64) -> AttentionPlan:
    """Cuts the step's query rows into tiles of 16 rows.  A segment of at most 16 rows or
    of one token (decode tokens) gives one-tile items, four to a workgroup, which takes a
    piece of the tile's key range; a longer segment gives items of ``rows_big / 16`` tiles
    that share the keys a wave loads.  Where there are too few items to fill the GPU, a key range is cut
    into pieces whose partial results are merged."""
    ql = np.asarray(seg_q_len, dtype=np.int64).reshape(-1)
    seg_scalars = np.stack((np.cumsum(ql) - ql, ql, np.asarray(seg_kv_len, dtype=np.int64).reshape(-1)), axis=1)
    per_item = max(1, rows_big // ROWS_PER_ITEM)
    # (a single token is never a long segment, however many heads share its keys: a decode
    # step then has one-tile items only, whose room is known before the lengths are)
    short = lambda r, q: (r <= ROWS_PER_ITEM) | (q == 1) | (per_item == 1)
    small = _tiles(seg_q_len, seg_kv_len, group_size, window, ROWS_PER_ITEM, short)
    big = _tiles(seg_q_len, seg_kv_len, group_size, window, ROWS_PER_ITEM, lambda r, q: ~short(r, q))
    items, merges_s, slot = _cut_joined(*small, pieces_per_tile(len(small[0]), n_kv_heads), 0, seg_scalars)
    more = None
    if len(big[0]):
        *big, more = _group_tiles(*big, per_item)
    # the long segments' workgroups have eight waves each, and pieces cost a pass over
    # float32 partial results (prompt portions of 256 to 1,024 tokens measured 2 to 4% faster
    # as whole steps cut for this many waves than for twice as many)
    target = TARGET_WAVES_LONG
    if len(big[0]) * n_kv_heads * 2 >= target or len(big[0]) == 0:
        chunk = 1 << 30  # enough items to fill the GPU: nothing is cut
    else:
        total = int((big[3] - big[2]).sum()) * n_kv_heads
        chunk = -(-total // target)
        chunk = max(MIN_SPLIT_KEYS, -(-chunk // KEYS_PER_BLOCK) * KEYS_PER_BLOCK)
    big_items, merges_b, slot = _cut_long(*big, chunk, per_item, slot, seg_scalars, more)
    merges = np.concatenate((merges_s, merges_b)) if len(merges_s) or len(merges_b) else np.zeros((0, 8), np.int32)
    return AttentionPlan(items, big_items, merges, slot, rows_big)


_COUNTERS: dict = {}


def _counters(device) -> torch.Tensor:
    """The device's counters of the attention kernel: zero between its launches (the kernel
    sets back what it counts), so one array serves every launch of a stream, recorded ones
    included; launches that overlap on one device must not share it."""
    device = torch.device(device)
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
    if key not in _COUNTERS:
        _COUNTERS[key] = torch.zeros(N_COUNTERS, dtype=torch.int32, device=device)
    return _COUNTERS[key]


def reset_counters(device) -> None:
    """Sets the device's counters back to zero (a kernel on the current stream): after a
    step that raised, whose attention kernels may have counted pieces that nobody merged."""
    device = torch.device(device)
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
    if key in _COUNTERS:
        _COUNTERS[key].zero_()


def counters_idle(device) -> bool:
    """Whether every counter is zero, as it is between launches (a check for tests; it
    waits for the device)."""
    device = torch.device(device)
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
    return key not in _COUNTERS or int(_COUNTERS[key].abs().sum()) == 0


def attention_mfma(q, q_row_stride, plan_dev, ctx, group, kv, n_heads, scale, window):
    plan, items, big_items, merges, counts = plan_dev
    n_pages, n_kv, page_size, head_dim = kv.k.shape
    lib = library.attention_library(head_dim)
    n = ctx.n_tokens
    out = torch.empty((n, n_heads * head_dim), dtype=torch.bfloat16, device=q.device)
    part_o = part_ml = counters = None
    if plan.cap_partials:
        part_o = torch.empty((plan.cap_partials, n_kv, 16, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((plan.cap_partials, n_kv, 16, 2), dtype=torch.float32, device=q.device)
    if plan.merged_in_kernel:
        counters = _counters(q.device)
    P = ops._ptr
    rc = lib.hal_attention_mfma(
        P(q), q_row_stride, P(out), n_heads * head_dim,
        P(items), plan.cap_items, P(big_items), plan.cap_big, P(merges), plan.cap_merges, P(counts),
        P(ctx.seg_q_start), P(ctx.seg_q_len), P(ctx.seg_kv_len),
        P(group.block_table), group.block_table.shape[1], P(kv.k), P(kv.v), P(part_o), P(part_ml),
        P(counters), N_COUNTERS, n_heads, n_kv, head_dim, page_size, 1 if getattr(kv, "tiled", False) else 0,
        ctypes.c_float(scale), window, plan.max_parts, ops._stream(),
    )
    ops._check(lib, rc)
    return out


def upload_plan(plan: AttentionPlan, device):
    """A plan's arrays on the device, as ``attention_mfma`` takes them."""
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    return (plan, dev(plan.items), dev(plan.big_items), dev(plan.merges), dev(plan.counts()))


def paged_attention(ctx, q, q_row_stride, kv, group, n_heads, scale, window):
    n_pages, n_kv, page_size, head_dim = kv.k.shape
    if mfma_supported(q.dtype, head_dim, page_size) and q_row_stride % 8 == 0:
        plan_dev = ctx.device_plan(group.group_id, n_heads // n_kv, window)
        if plan_dev is None:
            ctx.plan_attention(group.group_id, n_heads, n_kv, window, head_dim, late=True)
            plan_dev = ctx.device_plan(group.group_id, n_heads // n_kv, window)
        return attention_mfma(q, q_row_stride, plan_dev, ctx, group, kv, n_heads, scale, window)
    if getattr(kv, "tiled", False):
        raise ops.KernelError(
            f"pages are kept in the matrix-core kernel's order, which only that kernel reads "
            f"(dtype {q.dtype}, head size {head_dim}, page size {page_size}, row stride {q_row_stride})"
        )
    # (a step whose launches are recorded serves other lengths later: the block table's width bounds them)
    known = ctx.static is None and len(ctx.seg_kv_len_host) > 0
    most = int(ctx.seg_kv_len_host.max()) if known else None
    fewest = int(ctx.seg_q_len_host.min()) if known else 1
    return ops.attention_simple(
        q, q_row_stride, ctx.positions, ctx.token_seg, group.block_table, kv.k, kv.v, n_heads, scale, window,
        max_kv_len=most, min_q_len=fewest,
    )
