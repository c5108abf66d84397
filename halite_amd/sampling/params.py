"""Sampling parameters under the reference's names
(src/halite/transformers/infer/engine/batch.py:19-78)."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SamplingParams:
    max_new_tokens: int = 128
    min_new_tokens: int = 0  # kept for the reference's signature; it never enforces it either
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int = -1  # -1: no limit (batch.py:48-49)
    min_p: float = 0.0
    n: int = 1
    stop: str | list[str] | None = None  # stop strings need a tokenizer
    stop_token_ids: list[int] | set[int] | None = None
    ignore_eos: bool = False
    seed: int | None = None  # the reference has no seed; None derives one from the request id

    def __post_init__(self):
        if self.max_new_tokens < 0:
            raise ValueError("max_new_tokens must not be negative")
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        if not 0 < self.top_p <= 1:
            raise ValueError("top_p must be in (0, 1]")
        if not 0 <= self.min_p <= 1:
            raise ValueError("min_p must be in [0, 1]")
        if self.top_k == 0 or self.top_k < -1:
            raise ValueError("top_k must be -1 (no limit) or positive")
        if self.n < 1:
            raise ValueError("n must be at least 1")
        self.stop_token_ids = set(self.stop_token_ids) if self.stop_token_ids else set()
        if isinstance(self.stop, str):
            self.stop = [self.stop]

    @property
    def greedy(self) -> bool:
        """The reference asks for greedy decoding with ``top_k == 1`` (batch.py:115);
        its second engine also with ``temperature == 0``
        (src/halite/transformers/tokainfer/types.py:480-490).  Both hold here."""
        return self.temperature == 0 or self.top_k == 1
