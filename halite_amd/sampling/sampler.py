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

    def __init__(self, device):
        self.device = torch.device(device)

    def forward(self, logits: torch.Tensor, params: list[SamplingParams], seeds: list[int], draw_index: list[int]):
        n = logits.shape[0]
        if not (len(params) == len(seeds) == len(draw_index) == n):
            raise ValueError("one parameter set, seed and draw index per row of logits")
        if n == 0:
            e = torch.empty(0, device=self.device)
            return e.to(torch.int32), e.to(torch.float32)
        f = np.empty((3, n), dtype=np.float32)
        i = np.empty((2, n), dtype=np.int32)
        for r, p in enumerate(params):
            f[0, r] = 0.0 if p.greedy else p.temperature
            f[1, r] = p.top_p
            f[2, r] = p.min_p
            i[0, r] = 1 if p.greedy else min(p.top_k, 2**31 - 1)
            i[1, r] = draw_index[r]
        fd = torch.from_numpy(f).to(self.device)
        idv = torch.from_numpy(i).to(self.device)
        sd = torch.tensor(seeds, dtype=torch.int64).to(self.device)
        return ops.sample(logits.contiguous(), fd[0], idv[0], fd[1], fd[2], sd, idv[1])
