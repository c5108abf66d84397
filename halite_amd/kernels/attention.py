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
MIN_SPLIT_KEYS = 256
TARGET_WAVES = 2048


@dataclass
class AttentionPlan:
    items: np.ndarray  # [n_items, 8] int32: segment, first row, first key, end key, partial, 0, 0, 0
    merges: np.ndarray  # [n_merges, 4] int32: segment, first row, first partial, count
    n_items: int
    n_merges: int
    n_partials: int
    name: str = ""
    # room in the device arrays (larger than the live counts under a static layout)
    cap_items: int = 0
    cap_merges: int = 0

    def __post_init__(self):
        self.cap_items = max(self.cap_items, self.n_items)
        self.cap_merges = max(self.cap_merges, self.n_merges)


def mfma_supported(dtype: torch.dtype, head_dim: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 256 and page_size % 8 == 0


def plan_items(seg_q_len, seg_kv_len, group_size: int, n_kv_heads: int, window: int) -> AttentionPlan:
    """Cuts the step's query rows into tiles of 16 rows (a row is a token and a head
    of the group, token-major) and, where there are too few tiles to fill the GPU,
    cuts a tile's key range into pieces whose partial results are merged."""
    seg_ids, rho0s, kv_b, kv_e = [], [], [], []
    for s, (ql, kl) in enumerate(zip(seg_q_len, seg_kv_len)):
        ql, kl = int(ql), int(kl)
        rows = ql * group_size
        r0 = np.arange(0, rows, ROWS_PER_ITEM, dtype=np.int64)
        first_q = r0 // group_size
        last_q = np.minimum(rows - 1, r0 + ROWS_PER_ITEM - 1) // group_size
        pos0 = kl - ql
        b = np.zeros_like(r0) if window <= 0 else np.maximum(0, pos0 + first_q - window + 1)
        e = pos0 + last_q + 1
        seg_ids.append(np.full(r0.shape, s, dtype=np.int64))
        rho0s.append(r0), kv_b.append(b), kv_e.append(e)
    if not seg_ids:
        z = np.zeros((0, 8), dtype=np.int32)
        return AttentionPlan(z, np.zeros((0, 4), dtype=np.int32), 0, 0, 0)
    seg_ids, rho0s = np.concatenate(seg_ids), np.concatenate(rho0s)
    kv_b, kv_e = np.concatenate(kv_b), np.concatenate(kv_e)
    span = kv_e - kv_b
    if len(span) * n_kv_heads * 2 >= TARGET_WAVES:
        chunk = 1 << 30  # enough tiles to fill the GPU: nothing is cut
    else:
        total = int(span.sum()) * n_kv_heads
        chunk = -(-total // TARGET_WAVES)
        chunk = max(MIN_SPLIT_KEYS, -(-chunk // KEYS_PER_BLOCK) * KEYS_PER_BLOCK)
    base = kv_b - kv_b % KEYS_PER_BLOCK  # pieces end on multiples of 32 keys
    n_pieces = np.maximum(1, -(-(kv_e - base) // chunk))

    n_items = int(n_pieces.sum())
    items = np.zeros((n_items, 8), dtype=np.int32)
    tile_of = np.repeat(np.arange(len(span)), n_pieces)
    first_item = np.concatenate(([0], np.cumsum(n_pieces)[:-1]))
    piece = np.arange(n_items) - first_item[tile_of]
    items[:, 0] = seg_ids[tile_of]
    items[:, 1] = rho0s[tile_of]
    items[:, 2] = np.maximum(kv_b[tile_of], base[tile_of] + piece * chunk)
    items[:, 3] = np.minimum(kv_e[tile_of], base[tile_of] + (piece + 1) * chunk)
    split = n_pieces[tile_of] > 1
    items[:, 4] = -1
    n_partials = int(split.sum())
    items[split, 4] = np.arange(n_partials)
    split_tiles = np.nonzero(n_pieces > 1)[0]
    merges = np.zeros((len(split_tiles), 4), dtype=np.int32)
    if len(split_tiles):
        merges[:, 0] = seg_ids[split_tiles]
        merges[:, 1] = rho0s[split_tiles]
        merges[:, 2] = items[first_item[split_tiles], 4]
        merges[:, 3] = n_pieces[split_tiles]
    return AttentionPlan(items, merges, n_items, len(split_tiles), n_partials)


def attention_mfma(q, q_row_stride, plan_dev, ctx, group, kv, n_heads, scale, window):
    plan, items, merges, counts = plan_dev
    n_pages, n_kv, page_size, head_dim = kv.k.shape
    lib = library.attention_library(head_dim)
    n = ctx.n_tokens
    out = torch.empty((n, n_heads * head_dim), dtype=torch.bfloat16, device=q.device)
    part_o = part_ml = None
    n_part = plan.cap_items if plan.cap_items > plan.n_items else plan.n_partials
    if n_part and plan.cap_merges:
        part_o = torch.empty((n_part, n_kv, 16, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_part, n_kv, 16, 2), dtype=torch.float32, device=q.device)
    P = ops._ptr
    rc = lib.hal_attention_mfma(
        P(q), q_row_stride, P(out), n_heads * head_dim,
        P(items), P(counts[0:1]), plan.cap_items, P(merges), P(counts[1:2]), plan.cap_merges,
        P(ctx.seg_q_start), P(ctx.seg_q_len), P(ctx.seg_kv_len),
        P(group.block_table), group.block_table.shape[1], P(kv.k), P(kv.v), P(part_o), P(part_ml),
        n_heads, n_kv, head_dim, page_size, ctypes.c_float(scale), window, ops._stream(),
    )
    ops._check(lib, rc)
    return out


def paged_attention(ctx, q, q_row_stride, kv, group, n_heads, scale, window):
    n_pages, n_kv, page_size, head_dim = kv.k.shape
    if mfma_supported(q.dtype, head_dim, page_size) and q_row_stride % 8 == 0:
        plan_dev = ctx.device_plan(group.group_id, n_heads // n_kv, window)
        if plan_dev is None:
            ctx.plan_attention(group.group_id, n_heads, n_kv, window, late=True)
            plan_dev = ctx.device_plan(group.group_id, n_heads // n_kv, window)
        return attention_mfma(q, q_row_stride, plan_dev, ctx, group, kv, n_heads, scale, window)
    return ops.attention_simple(
        q, q_row_stride, ctx.positions, ctx.token_seg, group.block_table, kv.k, kv.v, n_heads, scale, window
    )
