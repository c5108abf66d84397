"""The sampler on top of the sampling kernel
(src/halite/transformers/infer/engine/sampler.py:12-60)."""

from __future__ import annotations

import zlib

import numpy as np
import torch

from ..kernels import ops
from .params import SamplingParams

_MASK63 = (1 << 63) - 1


def request_seed(params: SamplingParams, request_id, engine_seed: int = 0) -> int:
    """The seed of a request's random stream: its own if given, else derived from
    the engine's seed and the request's id, so that it does not depend on what else
    runs."""
    if params.seed is not None:
        return int(params.seed) & _MASK63
    return (zlib.crc32(repr(request_id).encode()) * 2654435761 + engine_seed * 40503) & _MASK63


class Sampler:
    """``forward`` takes float32 logits ``[R, V]`` and, per row, the request's
    parameters, its seed and the index of the draw (how many tokens the request has
    sampled before); it returns int32 tokens and float32 log-probabilities on the
    device.  NaN logits count as -1e5 (sampler.py:21-26)."""

    RING = 4  # pinned staging buffers in turn; one is reused only after its copy is done

    def __init__(self, device):
        self.device = torch.device(device)
        self._staging: list[tuple[torch.Tensor, torch.cuda.Event | None]] = []
        self._turn = 0

    def _stage(self, words: int) -> torch.Tensor:
        """A pinned int32 buffer of at least ``words`` entries whose last copy has finished."""
        if len(self._staging) < self.RING:
            self._staging.append((torch.empty(max(words, 1024), dtype=torch.int32, pin_memory=True), None))
            self._turn = len(self._staging) - 1
        else:
            self._turn = (self._turn + 1) % self.RING
        buf, event = self._staging[self._turn]
        if event is not None:
            event.synchronize()
        if buf.numel() < words:
            buf = torch.empty(2 * words, dtype=torch.int32, pin_memory=True)
        self._staging[self._turn] = (buf, None)
        return buf

    def forward(self, logits: torch.Tensor, params: list[SamplingParams], seeds: list[int], draw_index: list[int]):
        n = logits.shape[0]
        if not (len(params) == len(seeds) == len(draw_index) == n):
            raise ValueError("one parameter set, seed and draw index per row of logits")
        if n == 0:
            e = torch.empty(0, device=self.device)
            return e.to(torch.int32), e.to(torch.float32)
        # all per-row parameters in one buffer, one copy: seeds (int64), then three float32
        # rows and two int32 rows
        host = self._stage(7 * n)
        words = host.numpy()
        words[: 2 * n].view(np.int64)[:] = seeds
        f = words[2 * n : 5 * n].view(np.float32).reshape(3, n)
        i = words[5 * n : 7 * n].reshape(2, n)
        for r, p in enumerate(params):
            f[0, r] = 0.0 if p.greedy else p.temperature
            f[1, r] = p.top_p
            f[2, r] = p.min_p
            i[0, r] = 1 if p.greedy else min(p.top_k, 2**31 - 1)
            i[1, r] = draw_index[r]
        dev = torch.empty(7 * n, dtype=torch.int32, device=self.device)
        dev.copy_(host[: 7 * n], non_blocking=True)
        if self.device.type == "cuda":
            event = torch.cuda.Event()
            event.record()
            self._staging[self._turn] = (self._staging[self._turn][0], event)
        fd = dev[2 * n : 5 * n].view(torch.float32).view(3, n)
        idv = dev[5 * n : 7 * n].view(2, n)
        sd = dev[: 2 * n].view(torch.int64)
        vocab = logits.shape[1]
        unfiltered = all(p.greedy or (not 0 < p.top_k < vocab and p.top_p >= 1.0 and p.min_p <= 0.0) for p in params)
        # top-k, top-p and min-p all at once in one row: top-p then refers to what top-k kept,
        # two searches one after the other
        late = any(not p.greedy and 0 < p.top_k < vocab and p.top_p < 1.0 and p.min_p > 0.0 for p in params)
        return ops.sample(logits.contiguous(), fd[0], idv[0], fd[1], fd[2], sd, idv[1],
                          all_greedy=all(p.greedy for p in params), unfiltered=unfiltered, spread=True, late=late)
