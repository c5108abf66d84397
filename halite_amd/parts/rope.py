"""Rotary position encoding with the Llama 3 frequency scaling
(src/halite/transformers/position.py:90-210, 242-284)."""

from __future__ import annotations

import math

import torch
from typing import Literal

from pydantic import BaseModel, ConfigDict, Field, StrictBool, StrictInt, model_validator

from .base import POSITIONS, RotaryPositionEncoding


class BandedFrequencyScaling(BaseModel):
    """The frequency scaling of position.py:242-284, in the part's own terms: wavelengths
    longer than ``original_context_len / low_freq_factor`` are stretched by ``factor``,
    those shorter than ``original_context_len / high_freq_factor`` are kept, the band
    between is blended.  An architecture's description translates its own keys into these."""

    model_config = ConfigDict(extra="forbid")

    kind: Literal["banded"]
    factor: float = Field(gt=0)
    low_freq_factor: float
    high_freq_factor: float
    original_context_len: StrictInt = Field(gt=0)

    @model_validator(mode="after")
    def _check(self):
        if self.high_freq_factor == self.low_freq_factor:
            raise ValueError("frequency scaling: high_freq_factor equals low_freq_factor")
        return self


class RopeParams(BaseModel):
    head_dim: StrictInt = Field(gt=0)
    rotary_dim: StrictInt = Field(gt=0)
    theta: float = Field(gt=0)
    interleaved: StrictBool = False
    max_positions: StrictInt = Field(gt=0)
    scaling: BandedFrequencyScaling | None = None

    @model_validator(mode="after")
    def _check(self):
        if self.rotary_dim % 2 or self.rotary_dim > self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and <= head_dim {self.head_dim}")
        return self


def rope_inverse_frequencies(p: RopeParams) -> torch.Tensor:
    """float32 on the CPU, as position.py:129-138 computes them; with ``scaling``
    the three bands of position.py:264-284: wavelengths longer than
    ``original/low_freq_factor`` are stretched by ``factor``, shorter than
    ``original/high_freq_factor`` are kept, and between the two the stretched and
    the kept frequency are blended linearly in ``original/wavelength``."""
    exponent = torch.arange(0, p.rotary_dim, 2, dtype=torch.float32, device="cpu") / p.rotary_dim
    inv_freq = 1 / (p.theta**exponent)
    s = p.scaling
    if s is None:
        return inv_freq
    long_wavelen = s.original_context_len / s.low_freq_factor
    short_wavelen = s.original_context_len / s.high_freq_factor
    wavelen = 2 * math.pi / inv_freq
    stretched = torch.where(wavelen > long_wavelen, inv_freq / s.factor, inv_freq)
    blend = (s.original_context_len / wavelen - s.low_freq_factor) / (
        s.high_freq_factor - s.low_freq_factor
    )
    blended = (1 - blend) * stretched / s.factor + blend * stretched
    in_between = ~(wavelen < short_wavelen) & ~(wavelen > long_wavelen)
    return torch.where(in_between, blended, stretched)


@POSITIONS.register("rope")
class Rope(RotaryPositionEncoding):
    """Holds the float32 ``cos``/``sin`` table ``[positions, rotary_dim/2]`` on the
    device (position.py:140-167: outer product of float32 positions and
    frequencies).  The rotation itself happens in the kernel that also appends
    keys and values to the cache."""

    Params = RopeParams
    graph_safe = True

    def __init__(self, params, build):
        super().__init__(params, build)
        self.inv_freq = rope_inverse_frequencies(params)
        self._cos = self._sin = None

    @property
    def rotary_dim(self) -> int:
        return self.p.rotary_dim

    @property
    def interleaved(self) -> bool:
        return self.p.interleaved

    def tables(self, n_positions: int | None = None):
        """``(cos, sin)`` covering at least ``n_positions`` (default: all the model
        allows).  A position's values do not depend on the table's length."""
        n = n_positions or self.p.max_positions
        if self._cos is None or self._cos.shape[0] < n:
            n = max(n, min(self.p.max_positions, 4096))
            t = torch.arange(n, dtype=torch.float32, device="cpu")
            angles = torch.outer(t, self.inv_freq)
            self._cos = angles.cos().to(self.build.device).contiguous()
            self._sin = angles.sin().to(self.build.device).contiguous()
        return self._cos, self._sin
